"""The decode MLP block as one launch (fe_exl3_mlp_forward), through the C ABI: gate and up, then down on SwiGLU(gate, up)
(crates/fe-model/src/model.rs:3184-3199). The one launch must give the bits of its own fallback (the grouped gate + up
launch followed by down's forward_swiglu), which the other tests pin against the oracle; here it is also checked end to
end against the oracle's f64 linears, called again and again on one workspace, replayed from a graph, and driven into
its bounded wait's expiry from the host (every launch still ends, and the workspace reports it)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def bf16_to_f64(a):
    return (a.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def f64_to_bf16_bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def make(exl3, synth, kern, hidden, inter, bits, seed, blocks=None):
    ts = [synth.exl3_tensor(hidden, inter, bits, seed, "gate"), synth.exl3_tensor(hidden, inter, bits, seed + 1, "up"),
          synth.exl3_tensor(inter, hidden, bits, seed + 2, "down")]
    blocks = blocks or exl3.default_blocks(exl3.cu_count())
    return ts, [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), blocks) for t in ts]


def run(torch, exl3, lins, x, rows, y_dtype, ws, y0=None, stream=None):
    g, u, d = lins
    yg = torch.zeros((rows, g.n), dtype=torch.bfloat16, device="cuda")
    yu = torch.zeros((rows, g.n), dtype=torch.bfloat16, device="cuda")
    f32 = y_dtype in (exl3.Dtype.F32, exl3.Dtype.F32Add)
    y = torch.full((rows, d.n), 0.25 if y0 is None else y0, dtype=torch.float32 if f32 else torch.bfloat16, device="cuda")
    exl3.mlp_forward(g, u, d, x, exl3.Dtype.Bf16, yg, yu, y, y_dtype, rows, ws, stream=stream)
    return yg, yu, y


@pytest.mark.parametrize("bits,hidden,inter,rows,y_dtype", [
    (4, 512, 1536, 1, 0), (4, 1024, 2048, 1, 2), (3, 512, 1536, 2, 1), (5, 768, 1280, 1, 3), (2, 512, 1024, 1, 0),
    (6, 512, 1024, 1, 0), (8, 512, 1024, 1, 0), (4, 1024, 2048, 4, 0), (5, 512, 1536, 3, 2)])
def test_one_launch_has_the_bits_of_the_two_launches(bits, hidden, inter, rows, y_dtype):
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    _, lins = make(exl3, synth, kern, hidden, inter, bits, 40 + bits)
    ws = exl3.Workspace(lins, rows)
    x = dev_u16(torch, synth.activations(rows, hidden, 3))
    yd = exl3.Dtype(y_dtype)
    kern.set_option("mlp_chain", 0)
    assert exl3.mlp_forward_launches(*lins, rows, yd, ws) == 0
    want = [t.clone() for t in run(torch, exl3, lins, x, rows, yd, ws)]
    kern.set_option("mlp_chain", 1)
    assert exl3.mlp_forward_launches(*lins, rows, yd, ws) == 1, "the one launch does not apply to this case"
    for rep in range(4):  # the sequence number advances from call to call; nothing is cleared in between
        got = run(torch, exl3, lins, x, rows, yd, ws)
        torch.cuda.synchronize()
        for a, b, name in zip(got, want, ("gate", "up", "down")):
            assert torch.equal(a, b), (rep, name)
    assert ws.chain_status() == 0


def test_one_launch_against_the_oracle(oracle):
    """End to end against the CPU path: gate and up by linear_f64 on the bf16 input, SwiGLU in the reference's bf16
    arithmetic, down by linear_f64 on that activation."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    ts, lins = make(exl3, synth, kern, 512, 1536, 4, 77)
    ws = exl3.Workspace(lins, 1)
    xb = synth.activations(1, 512, 9)
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.F32, ws) == 1
    yg, yu, y = run(torch, exl3, lins, dev_u16(torch, xb), 1, exl3.Dtype.F32, ws)
    torch.cuda.synchronize()
    o = [oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh) for t in ts]
    x64 = bf16_to_f64(xb)
    rg, ru = oracle.linear_f64(o[0], x64), oracle.linear_f64(o[1], x64)
    bits_of = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)
    for got, ref in ((yg, rg), (yu, ru)):
        rms = np.sqrt((ref ** 2).mean())  # (bf16 outputs: half a bf16 step of the largest values is 1e-2 of the rms)
        assert (np.abs(bf16_to_f64(bits_of(got)) - ref) / np.maximum(np.abs(ref), rms)).max() < 1e-2
    # SwiGLU on the GPU's own bf16 gate / up (so that only the down projection is compared): bf16(bf16(silu(g)) * u)
    gb, ub = bf16_to_f64(bits_of(yg)), bf16_to_f64(bits_of(yu))
    silu = bf16_to_f64(f64_to_bf16_bits(gb / (1.0 + np.exp(-gb))))
    act = bf16_to_f64(f64_to_bf16_bits(silu * ub))
    ref = oracle.linear_f64(o[2], act)
    rms = np.sqrt((ref ** 2).mean())
    err = np.abs(y.cpu().numpy().astype(np.float64) - ref)
    # max relative error 1e-2 with the denominator floored at the rms (bf16 ties of the GPU's approximate exponential
    # against exp() can flip an activation by one bf16 step)
    assert (err / np.maximum(np.abs(ref), rms)).max() < 1e-2, err.max() / rms


def test_one_launch_replays_from_a_graph():
    import torch
    from ferrite_amd import _lib, exl3, synth
    lib, check = _lib.lib(), _lib.check
    kern = exl3.Kernels.load()
    _, lins = make(exl3, synth, kern, 1024, 2048, 4, 11)
    ws = exl3.Workspace(lins, 1)
    x = dev_u16(torch, synth.activations(1, 1024, 5))
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.Bf16, ws) == 1
    want = [t.clone() for t in run(torch, exl3, lins, x, 1, exl3.Dtype.Bf16, ws)]
    torch.cuda.synchronize()
    s, g = C.c_void_p(), C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    g_, u_, d_ = lins
    yg = torch.zeros((1, g_.n), dtype=torch.bfloat16, device="cuda")
    yu = torch.zeros((1, g_.n), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((1, d_.n), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    check(lib.fe_hip_graph_begin(s))
    exl3.mlp_forward(g_, u_, d_, x, exl3.Dtype.Bf16, yg, yu, y, exl3.Dtype.Bf16, 1, ws, stream=s)
    check(lib.fe_hip_graph_end(s, C.byref(g)))
    for rep in range(4):
        for t in (yg, yu, y):
            t.fill_(3.0)
        torch.cuda.synchronize()
        check(lib.fe_hip_graph_launch(g, s))
        check(lib.fe_hip_stream_sync(s))
        for a, b in zip((yg, yu, y), want):
            assert torch.equal(a, b), rep
        # an eager call between the replays moves the sequence number on; the replay must not mind
        got = run(torch, exl3, lins, x, 1, exl3.Dtype.Bf16, ws)
        torch.cuda.synchronize()
        assert torch.equal(got[2], want[2])
    check(lib.fe_hip_graph_destroy(g))
    check(lib.fe_hip_stream_destroy(s))
    assert ws.chain_status() == 0


def test_expired_wait_is_reported_and_every_launch_ends():
    """A spin limit of zero from the host: every program of the down stage gives up at once, sets the error word and goes
    on with whatever the outputs of gate and up hold at that moment; the launch ends normally. After chain_status() has
    reported and cleared the error the next launch is good again."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    _, lins = make(exl3, synth, kern, 512, 1536, 4, 21)
    ws = exl3.Workspace(lins, 1)
    x = dev_u16(torch, synth.activations(1, 512, 2))
    want = [t.clone() for t in run(torch, exl3, lins, x, 1, exl3.Dtype.Bf16, ws)]
    torch.cuda.synchronize()
    assert ws.chain_status() == 0
    kern.set_option("chain_spin", 0)
    run(torch, exl3, lins, x, 1, exl3.Dtype.Bf16, ws)
    torch.cuda.synchronize()
    assert ws.chain_status() != 0
    assert ws.chain_status() == 0  # cleared
    kern.set_option("chain_spin", 1 << 16)
    # ... and this workspace takes the two launches from now on; a new workspace takes the one launch again
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.Bf16, ws) == 0
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.Bf16, exl3.Workspace(lins, 1)) == 1
    got = run(torch, exl3, lins, x, 1, exl3.Dtype.Bf16, ws)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert ws.chain_status() == 0


def test_cases_the_one_launch_does_not_take_fall_back():
    """More rows than the fused rotation takes, a workspace made without down, mixed widths: two launches, same call."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    _, lins = make(exl3, synth, kern, 512, 1536, 4, 5)
    ws = exl3.Workspace(lins, 32)
    assert exl3.mlp_forward_launches(*lins, 32, exl3.Dtype.Bf16, ws) == 0
    x = dev_u16(torch, synth.activations(32, 512, 4))
    yg, yu, y = run(torch, exl3, lins, x, 32, exl3.Dtype.Bf16, ws, y0=0.0)
    torch.cuda.synchronize()
    # the same through the entry points it falls back to
    yg2 = torch.zeros_like(yg); yu2 = torch.zeros_like(yu); y2 = torch.zeros_like(y)
    exl3.forward_group(lins[:2], x, exl3.Dtype.Bf16, [yg2, yu2], exl3.Dtype.Bf16, 32, ws)
    lins[2].forward_swiglu(yg2, yu2, 1536, y2, exl3.Dtype.Bf16, 32, ws)
    torch.cuda.synchronize()
    assert torch.equal(yg, yg2) and torch.equal(yu, yu2) and torch.equal(y, y2)
    _, other = make(exl3, synth, kern, 512, 1536, 3, 6)
    ws2 = exl3.Workspace(lins + other, 1)
    assert exl3.mlp_forward_launches(lins[0], lins[1], other[2], 1, exl3.Dtype.Bf16, ws2) == 0  # widths differ


@pytest.mark.parametrize("down_units", [0, 4])
def test_a_row_has_the_same_bits_at_every_row_count(down_units):
    """Row r of a batch has the bits of the single-row call, with the one launch on or off
    (crates/fe-exl3/src/bin/exl3-rowcheck.rs:69-95, for the block): with down in its own partition (chain_down_units 0),
    and with down in programs of 4 units, where the call keeps that partition at every row count it sends through the
    GEMV, whatever plan the linear has of its own."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    kern.set_option("chain_down_units", down_units)  # (before the workspace is made)
    hidden, inter, bits = 512, 2048, 4
    ts = [synth.exl3_tensor(hidden, inter, bits, 31, "gate"), synth.exl3_tensor(hidden, inter, bits, 32, "up"),
          synth.exl3_tensor(inter, hidden, bits, 33, "down")]
    blocks = exl3.default_blocks(exl3.cu_count())
    lins = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), blocks) for t in ts[:2]]
    # down with a partition of its own that is not the one launch's: 6 programs over its 64 units (runs of 10 and 11)
    lins.append(exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(ts[2]), exl3.Plan(6, 1, 4, 4)))
    ws = exl3.Workspace(lins, 24)
    xb = synth.activations(24, hidden, 8)
    single = []
    for r in range(24):
        single.append(run(torch, exl3, lins, dev_u16(torch, xb[r:r + 1]), 1, exl3.Dtype.Bf16, ws)[2].clone())
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.Bf16, ws) == 1
    for chain in (1, 0):
        kern.set_option("mlp_chain", chain)
        for m in (1, 2, 3, 8, 17, 24):
            y = run(torch, exl3, lins, dev_u16(torch, xb[:m]), m, exl3.Dtype.Bf16, ws)[2]
            torch.cuda.synchronize()
            for r in range(m):
                assert torch.equal(y[r], single[r][0]), (chain, m, r)
    kern.set_option("mlp_chain", 1)
    kern.set_option("chain_down_units", 0)
    assert ws.chain_status() == 0


@pytest.mark.parametrize("option,value", [("fuse", 0), ("lds_pad", 0), ("chain_perm", 0), ("chain_down_units", 2),
                                          ("chain_down_units", 4), ("chain_down_units", 8), ("chain_rot_pairs", 8)])
def test_switches_of_the_launch_change_no_bit(option, value):
    """Every switch of the one launch (programs sharing a workgroup, the LDS request that sets the programs a CU, the order
    of the down stage, the length of down's programs, the rows it takes) against the same call with the one launch off:
    the same bits, whatever the launch looks like. The workspace is made after the switch is set, as the size of down's
    partition asks."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    defaults = {"fuse": 1, "lds_pad": 1, "chain_perm": 1, "chain_down_units": 0, "chain_rot_pairs": 32}
    try:
        kern.set_option(option, value)
        _, lins = make(exl3, synth, kern, 1024, 4096, 4, 90)
        for rows in (1, 2):
            ws = exl3.Workspace(lins, rows)
            x = dev_u16(torch, synth.activations(rows, 1024, 3))
            kern.set_option("mlp_chain", 0)
            want = [t.clone() for t in run(torch, exl3, lins, x, rows, exl3.Dtype.Bf16, ws)]
            kern.set_option("mlp_chain", 1)
            one = exl3.mlp_forward_launches(*lins, rows, exl3.Dtype.Bf16, ws)
            for rep in range(2):
                got = run(torch, exl3, lins, x, rows, exl3.Dtype.Bf16, ws)
                torch.cuda.synchronize()
                for a, b in zip(got, want):
                    assert torch.equal(a, b), (option, value, rows, one, rep)
            assert ws.chain_status() == 0
    finally:
        kern.set_option(option, defaults[option])
        kern.set_option("mlp_chain", 1)
