"""The layer calls under HIP graph capture (the role of crates/fe-exl3/src/bin/exl3-graphcheck.rs): forward calls of
both formats are recorded once on a stream of their own and replayed several times, with eager work and
synchronizations of the process in between; every replay must give the bits of the eager call. The calls allocate
nothing, clear nothing with a memset (arrival counters are re-armed by the kernels), and do not synchronize."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def test_forward_calls_replay_from_a_graph():
    import torch
    from ferrite_amd import _lib, exl3, fp4, synth
    lib, check = _lib.lib(), _lib.check
    kern, fk = exl3.Kernels.load(), fp4.Kernels.load()
    # the 300-row calls on the stream-K schedule: tiles shared between programs meet through the workspace, whose arrival
    # counters the kernels re-arm themselves
    kern.set_option("gemm_sk", 2)
    fk.set_option("gemm_sk", 2)
    t = synth.exl3_tensor(1024, 384, 4, 5)
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 64)  # column blocks shared by several programs
    uneven = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(7, 4, 4, 0))  # 7 uneven runs
    flin = synth.fp4_linear(384, 1024, 6).upload()
    # two more linears of the same input: with `lin` a grouped launch (the argument block is copied at capture)
    pair = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(1024, n, 4, 30 + n)), 64) for n in (256, 128)]
    group = [lin] + pair
    rows = [1, 16, 40, 300]
    ws = exl3.Workspace([lin, uneven] + pair, max(rows))
    assert exl3.forward_group_launches(group, 1, ws) in (1, 2) and exl3.forward_group_launches(group, 16, ws) in (1, 2)
    fws = fp4.Workspace(max(rows), 1024)
    xs = {m: dev_u16(torch, synth.activations(m, 1024, m)) for m in rows}

    def calls(stream, outs):
        for m in rows:
            lin.forward(xs[m], exl3.Dtype.Bf16, outs[("e", m)], exl3.Dtype.F32, m, ws, stream=stream)
            flin.forward(fk, fws, outs[("f", m)], 384, xs[m], 1024, m, stream=stream)
        uneven.forward(xs[16], exl3.Dtype.Bf16, outs[("s", 16)], exl3.Dtype.F32, 16, ws, stream=stream)
        for m in (1, 16):
            exl3.forward_group(group, xs[m], exl3.Dtype.Bf16, [outs[("g", m, i)] for i in range(3)], exl3.Dtype.F32, m, ws, stream=stream)

    def fresh():
        o = {("e", m): torch.zeros((m, 384), dtype=torch.float32, device="cuda") for m in rows}
        o.update({("f", m): torch.zeros((m, 384), dtype=torch.bfloat16, device="cuda") for m in rows})
        o[("s", 16)] = torch.zeros((16, 384), dtype=torch.float32, device="cuda")
        for m in (1, 16):
            for i, l in enumerate(group):
                o[("g", m, i)] = torch.zeros((m, l.n), dtype=torch.float32, device="cuda")
        return o

    eager = fresh()
    calls(None, eager)
    torch.cuda.synchronize()
    want = {k: v.clone() for k, v in eager.items()}
    assert torch.equal(want[("g", 16, 0)], want[("e", 16)])  # a member of a group has the bits of its own forward

    s = C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    outs = fresh()
    check(lib.fe_hip_graph_begin(s))
    calls(s, outs)
    g = C.c_void_p()
    check(lib.fe_hip_graph_end(s, C.byref(g)))
    for rep in range(4):
        for v in outs.values():
            v.fill_(7.0)
        torch.cuda.synchronize()
        check(lib.fe_hip_graph_launch(g, s))
        check(lib.fe_hip_stream_sync(s))
        for k, v in outs.items():
            assert torch.equal(v, want[k]), (rep, k)
        # eager work of the same linears between replays (shares the workspaces, stream-ordered by the syncs)
        calls(None, eager)
        torch.cuda.synchronize()
    check(lib.fe_hip_graph_destroy(g))
