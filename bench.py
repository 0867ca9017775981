#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-prefill] [--no-sweep]

Workload (BASELINE.json configs[1]): the EXL3 decode MLP of a Qwen3.8-27B-shaped layer at M = 1, at 3, 4 and 5 bits per
weight: gate and up are K=5120 N=17408, down is K=17408 N=5120. One step = the forward (input rotation + trellis GEMV)
of all nine linears on seeded synthetic layers, inputs and weights resident in HBM, launched as the MLP block launches
them: gate and up, two linears of the same input, as one grouped call (fe_exl3_linear_forward_group), down as
Linear::forward. `value` is the trellis bytes streamed per second (the reference's numerator,
crates/fe-exl3/src/bin/exl3-bench.rs:104) over the whole step, launch gaps and input rotations included. The nine
weight sets total 401 MB, more than L2 plus the 256 MB Infinity Cache, so every step streams its weights from HBM.

`roofline` is the dominant kernel alone (the grouped 4-bit GEMV of the two 5120x17408 projections): its trellis bytes
over its average launch duration, measured with HIP event pairs on the launch stream around its launches inside the
timed region (the other launches of the timed region carry no events: every record is a packet of its own on the queue;
a pass after the timed region brackets all six launches for `per_launch`).
`cpu_baseline` times the CPU oracle (the reference's factored f64 linear, threaded over 128-column blocks) on the host.
`m2048` reports the prefill GEMMs (EXL3 4-bit and NVFP4, 5120x17408, M = 2048) in TFLOP/s against the bf16/f16 MFMA
peak; it is measured after the timed region and is not part of `value`.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes of one launch of the roofline kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE over
# `bench.py --traffic-pass` (profiles/exl3_gemv_group_b4_m1_hbm_traffic.md): 45202 KiB fetched x 2.0 (the factor that
# makes the counter read a streaming read and an elementwise update of known size correctly) + 799 KiB written x 1.0
ROOFLINE_TRAFFIC_BYTES = int((45202 * 2.0 + 799 * 1.0) * 1024)
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_FP8_PEAK_TFLOPS = 5000.0  # dense fp8 MFMA peak of MI355X
SEED = 20251
MLP = [("gate", 5120, 17408), ("up", 5120, 17408), ("down", 17408, 5120)]
BITS = [3, 4, 5]


class Events:
    """HIP events through the C ABI, on the stream the kernels are launched on."""

    def __init__(self, lib, check):
        self.lib, self.check = lib, check

    def new(self):
        e = C.c_void_p()
        self.check(self.lib.fe_hip_event_create(C.byref(e)))
        return e

    def record(self, e, stream):
        self.check(self.lib.fe_hip_event_record(e, stream))

    def ms(self, a, b):
        self.check(self.lib.fe_hip_event_sync(b))
        out = C.c_float()
        self.check(self.lib.fe_hip_event_elapsed_ms(C.byref(out), a, b))
        return out.value


def cpu_baseline(reps=12):
    """The CPU oracle on the workload's 4-bit MLP (gate, up, down at M = 1), all host cores, `reps` passes: a bounded
    sample of the step (the 3- and 5-bit thirds run the same code on 3/4 and 5/4 of the bytes)."""
    import numpy as np
    import oracle
    from ferrite_amd import synth
    cores = oracle.default_threads(64)
    layers, nbytes = [], 0
    for name, k, n in MLP:
        t = synth.exl3_tensor(k, n, 4, SEED, name)
        o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
        x = (synth.activations(1, k, SEED).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        layers.append((o, x))
        nbytes += t.trellis_bytes()
    y_gate = None
    t0 = time.perf_counter()
    for _ in range(reps):
        for i, (o, x) in enumerate(layers):
            y = oracle.linear_f64(o, x, threads=cores)
            if i == 0:
                y_gate = y
    dt = time.perf_counter() - t0
    return {"value": round(reps * nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"oracle linear_f64 (decode_tile + f64 factored linear, threaded over 128-column blocks) on the 4-bit "
                      f"gate, up and down projections at M=1, {reps} passes, {dt:.2f} s"}, y_gate


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--bracket-events", action="store_true",
                    help="time the roofline kernel with events recorded before and after its launch instead of events attached to its dispatch")
    ap.add_argument("--no-sweep", action="store_true", help="leave out the M = 1, 4, 8, 16 sweep (for a kernel trace of the step alone)")
    ap.add_argument("--traffic-pass", action="store_true",
                    help="for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: a streaming read and an elementwise update of "
                         "known size (the counters' calibration), then the roofline kernel, caches evicted in between")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the hot path on one GPU; --gpus must be 1 (no multi-GPU path exists)")

    import numpy as np
    import torch
    from ferrite_amd import _lib, exl3, fp4, synth

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU")
    if args.traffic_pass:
        return traffic_pass(torch, np, exl3, synth)
    cpu = None
    if not args.no_cpu:
        cpu, y_cpu = cpu_baseline()  # first, as the configuration asks

    kern = exl3.Kernels.load()
    lib = _lib.lib()
    ev = Events(lib, _lib.check)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    blocks = exl3.default_blocks(exl3.cu_count())

    # the nine linears, one device copy each
    linears = []
    for bits in BITS:
        for name, k, n in MLP:
            t = synth.exl3_tensor(k, n, bits, SEED, name)
            lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), blocks)
            x = torch.from_numpy(synth.activations(1, k, SEED).view(np.int16)).cuda()
            y = torch.zeros((1, n), dtype=torch.bfloat16, device="cuda")
            linears.append((name, bits, lin, x, y))
    ws = exl3.Workspace([l[2] for l in linears], 1)
    total_bytes = sum(l[2].weight_bytes() for l in linears)

    if cpu is not None:  # parity of the sampled layer on the GPU against the CPU result just computed
        name, bits, lin, x, _ = next(l for l in linears if l[0] == "gate" and l[1] == 4)
        yf = torch.zeros((1, lin.n), dtype=torch.float32, device="cuda")
        lin.forward(x, exl3.Dtype.Bf16, yf, exl3.Dtype.F32, 1, ws)
        torch.cuda.synchronize()
        got = yf.cpu().numpy().astype(np.float64)
        rel = float(np.abs(got - y_cpu).max() / np.sqrt((y_cpu ** 2).mean()))
        cpu["gpu_vs_cpu_max_err_over_rms"] = round(rel, 6)

    # The step's launches: per bit width, gate + up of one input as a grouped call, then down. Every argument of the calls
    # into the C ABI is prepared once.
    f_group, f_forward, f_rotate, f_rotated, f_record = (lib.fe_exl3_linear_forward_group, lib.fe_exl3_linear_forward,
                                                        lib.fe_exl3_linear_rotate_input, lib.fe_exl3_linear_gemv_rotated,
                                                        lib.fe_hip_event_record)
    bf16 = int(exl3.Dtype.Bf16)
    by = {(name, bits): (lin, x, y) for name, bits, lin, x, y in linears}
    launches = []  # (label, bytes, dominant, kernel launches, [(fn, args)...], keepalive)
    for bits in BITS:
        (g, xg, yg), (u, _, yu), (d, xd, yd) = by[("gate", bits)], by[("up", bits)], by[("down", bits)]
        hs = (C.c_void_p * 2)(g.h, u.h)
        ys = (C.c_uint64 * 2)(yg.data_ptr(), yu.data_ptr())
        n_launch = exl3.forward_group_launches([g, u], 1, ws)
        assert n_launch in (1, 2), "gate and up do not share a launch"
        launches.append((f"gate+up_b{bits}", g.weight_bytes() + u.weight_bytes(), bits == 4, n_launch,
                         [(f_group, (hs, 2, kern.h, stream, xg.data_ptr(), bf16, ys, bf16, 1, ws.h))], (hs, ys)))
        if d.forward_is_one_launch(1):  # forward() is the GEMV alone (it rotates its own input)
            calls = [(f_forward, (d.h, kern.h, stream, xd.data_ptr(), bf16, yd.data_ptr(), bf16, 1, ws.h))]
        else:
            calls = [(f_rotate, (d.h, kern.h, stream, xd.data_ptr(), bf16, 1, ws.h)),
                     (f_rotated, (d.h, stream, ws.xh_ptr, yd.data_ptr(), bf16, 1, ws.h))]
        launches.append((f"down_b{bits}", d.weight_bytes(), False, len(calls), calls, None))

    # Event pairs on the launch stream. In the timed region only the dominant kernel's launches carry them; one more pass
    # after the timed region times every launch for the per-launch table. A pair is attached to the dispatch of the
    # launch's last kernel (the GEMV), so it reads that kernel's own begin and end as a kernel trace does
    # (fe_hip_time_next_launch); with --bracket-events it is recorded before and after the launch instead, each record
    # a packet of its own on the queue, which adds the dispatch gap and the packets to the reading.
    attached = not args.bracket_events
    f_time_next = lib.fe_hip_time_next_launch
    events = [[(ev.new(), ev.new()) if la[2] else None for la in launches] for _ in range(args.steps)]
    table_events = [(ev.new(), ev.new()) for _ in launches]

    def step(pairs=None):
        rc = 0
        for li, la in enumerate(launches):
            calls = la[4]
            for fn, a in calls[:-1]:
                rc |= fn(*a)
            pair = pairs[li] if pairs is not None else None
            attach = pair is not None and attached and la[3] == len(calls)  # the last call is one kernel launch
            if attach:
                rc |= f_time_next(pair[0], pair[1])
            elif pair is not None:
                rc |= f_record(pair[0], stream)
            fn, a = calls[-1]
            rc |= fn(*a)
            if pair is not None and not attach:
                rc |= f_record(pair[1], stream)
        _lib.check(rc)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events[i])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    value = total_bytes / (dt / args.steps) / 1e9

    dom_ms = []
    for li, la in enumerate(launches):
        if la[2]:
            dom_ms += [ev.ms(*events[i][li]) for i in range(args.steps)]
            dom_bytes = la[1]
            dom_kernel = "exl3_gemv_group_b4"
    dom_avg_ms = sum(dom_ms) / len(dom_ms)
    achieved = dom_bytes / (dom_avg_ms * 1e-3) / 1e9

    # the dominant launch alone, back to back between one pair of events: its duration without the event packets and the
    # other launches' gaps (what a kernel trace reports for it inside the step; here the same 89 MB are read every time
    # and stay in the Infinity Cache, which does not help a kernel bound by its decode instructions)
    dom = next(la for la in launches if la[2])
    a, b = ev.new(), ev.new()
    rc = 0
    for fn, aa in dom[4]:
        rc |= fn(*aa)
    ev.record(a, stream)
    for _ in range(args.steps):
        for fn, aa in dom[4]:
            rc |= fn(*aa)
    ev.record(b, stream)
    _lib.check(rc)
    dom_b2b_us = ev.ms(a, b) * 1e3 / args.steps

    per, reps = {}, max(args.steps, 5)
    acc = [0.0] * len(launches)
    for _ in range(reps):  # after the timed region: every launch bracketed
        step(table_events)
        for li in range(len(launches)):
            acc[li] += ev.ms(*table_events[li])
    for li, la in enumerate(launches):
        us = acc[li] / reps * 1e3
        per[la[0]] = {"us": round(us, 2), "GB/s": round(la[1] / us / 1e3, 1), "launches": la[3]}

    out = {
        "metric": "quant linear GB/s (%HBM peak) at M=1; TFLOP/s (%MFMA peak) at M=2048",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "EXL3 decode MLP, Qwen3.8-27B-shaped layer, M=1, 3/4/5 bpw (gate, up 5120x17408; down 17408x5120)",
                   "linears_per_step": len(linears), "trellis_bytes_per_step": total_bytes, "seed": SEED,
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "kernel": f"{dom_kernel} (gate + up, 5120x17408 each, M=1)", "achieved": round(achieved, 2),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": ROOFLINE_TRAFFIC_BYTES,
                     "avg_launch_us": round(dom_avg_ms * 1e3, 3), "bytes_per_launch": dom_bytes, "launches": len(dom_ms),
                     "back_to_back_us": round(dom_b2b_us, 3),
                     "events": "recorded around the launch" if args.bracket_events else "attached to the kernel's dispatch"},
        "cpu_baseline": cpu,
        "per_launch": per,
    }

    out["graph_replay"] = graph_replay(lib, _lib.check, ev, launches, stream, total_bytes, args.steps, args.warmup)
    if not args.no_sweep:
        out["rows_sweep_b4"] = rows_sweep(torch, np, exl3, synth, kern, ev, stream, linears)
    if not args.no_prefill:
        out["m2048"] = prefill(torch, np, exl3, fp4, synth, kern, ev, stream)
    print(json.dumps(out))


def traffic_pass(torch, np, exl3, synth):
    """Three rounds of: evict (an elementwise update of 600 MiB: reads 600 MiB, writes 600 MiB), exl3_probe_v4 reading
    exactly the roofline kernel's algorithmic bytes, evict, the roofline kernel. Prints the known sizes."""
    kern = exl3.Kernels.load()
    k, n = 5120, 17408
    blocks = exl3.default_blocks(exl3.cu_count())
    lins = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, n, 4, SEED, name)), blocks) for name in ("gate", "up")]
    ws = exl3.Workspace(lins, 1)
    x = torch.from_numpy(synth.activations(1, k, SEED).view(np.int16)).cuda()
    ys = [torch.zeros((1, n), dtype=torch.bfloat16, device="cuda") for _ in lins]
    nbytes = sum(l.weight_bytes() for l in lins)
    buf = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    big = torch.zeros(600 << 20, dtype=torch.uint8, device="cuda")
    assert exl3.forward_group_launches(lins, 1, ws) == 1
    for _ in range(3):
        big.add_(1)
        kern.probe_stream_read(buf, 1024, 1)
        big.add_(1)
        exl3.forward_group(lins, x, exl3.Dtype.Bf16, ys, exl3.Dtype.Bf16, 1, ws)
    torch.cuda.synchronize()
    print(json.dumps({"exl3_probe_v4_reads_KiB": nbytes / 1024, "elementwise_reads_and_writes_KiB": (600 << 20) / 1024,
                      "roofline_kernel": "exl3_gemv_group_b4", "algorithmic_KiB": nbytes / 1024}))


def rows_sweep(torch, np, exl3, synth, kern, ev, stream, linears, reps=20):
    """The 4-bit MLP at M = 1, 4, 8, 16 (BASELINE's decode / speculative-verify row counts): microseconds per linear,
    launched back to back as the step launches them (gate + up grouped, then down), so that no weight is served from
    cache. Not part of `value`."""
    four = {name: lin for name, bits, lin, x, y in linears if bits == 4}
    g, u, d = four["gate"], four["up"], four["down"]
    res = {}
    for m in (1, 4, 8, 16):
        ws = exl3.Workspace([g, u, d], m)
        x = torch.from_numpy(synth.activations(m, g.k, SEED).view(np.int16)).cuda()
        xd = torch.from_numpy(synth.activations(m, d.k, SEED).view(np.int16)).cuda()
        yg, yu = (torch.zeros((m, g.n), dtype=torch.bfloat16, device="cuda") for _ in range(2))
        yd = torch.zeros((m, d.n), dtype=torch.bfloat16, device="cuda")

        def mlp():
            exl3.forward_group([g, u], x, exl3.Dtype.Bf16, [yg, yu], exl3.Dtype.Bf16, m, ws, stream=stream)
            d.forward(xd, exl3.Dtype.Bf16, yd, exl3.Dtype.Bf16, m, ws, stream=stream)

        mlp()
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        for _ in range(reps):
            mlp()
        ev.record(b, stream)
        us = ev.ms(a, b) * 1e3 / (reps * 3)
        nbytes = (g.weight_bytes() + u.weight_bytes() + d.weight_bytes()) / 3
        res[f"m{m}"] = {"us_per_linear": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                        "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                        "gate_up_launches": exl3.forward_group_launches([g, u], m, ws)}
        # the MLP block as the model runs it: down reads SwiGLU(gate, up) of the grouped launch's outputs and adds
        # into the residual stream
        resid = torch.zeros((m, d.n), dtype=torch.bfloat16, device="cuda")

        def block():
            exl3.forward_group([g, u], x, exl3.Dtype.Bf16, [yg, yu], exl3.Dtype.Bf16, m, ws, stream=stream)
            d.forward_swiglu(yg, yu, g.n, resid, exl3.Dtype.Bf16Add, m, ws, stream=stream)

        block()
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        for _ in range(reps):
            block()
        ev.record(b, stream)
        res[f"m{m}"]["mlp_block_us"] = round(ev.ms(a, b) * 1e3 / reps, 2)
    # the attention projections of the same layer (40 heads of 128, 8 KV heads): q, k, v of one input grouped, then o
    blocks = exl3.default_blocks(exl3.cu_count())
    q, kk, v, o = (exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(5120, n, 4, SEED, name)), blocks)
                   for name, n in (("q", 5120), ("k", 1024), ("v", 1024), ("o", 5120)))
    abytes = sum(l.weight_bytes() for l in (q, kk, v, o))
    for m in (1, 4, 8, 16):
        ws = exl3.Workspace([q, kk, v, o], m)
        x = torch.from_numpy(synth.activations(m, 5120, SEED).view(np.int16)).cuda()
        ys = [torch.zeros((m, l.n), dtype=torch.bfloat16, device="cuda") for l in (q, kk, v)]
        yo = torch.zeros((m, 5120), dtype=torch.bfloat16, device="cuda")

        def attn():
            exl3.forward_group([q, kk, v], x, exl3.Dtype.Bf16, ys, exl3.Dtype.Bf16, m, ws, stream=stream)
            o.forward(x, exl3.Dtype.Bf16, yo, exl3.Dtype.Bf16, m, ws, stream=stream)

        attn()
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        for _ in range(reps):
            attn()
        ev.record(b, stream)
        us = ev.ms(a, b) * 1e3 / reps
        res[f"m{m}"]["attn_qkv_o_us"] = round(us, 2)
        res[f"m{m}"]["attn_GB/s"] = round(abytes / us / 1e3, 1)
    return res


def graph_replay(lib, check, ev, launches, stream, total_bytes, steps, warmup):
    """The same step captured once into a HIP graph on a stream of its own and replayed: what the step costs when the
    host does not launch its kernels one by one. Reported beside `value`, which stays the eagerly launched step."""
    s = C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    check(lib.fe_hip_graph_begin(s))
    for la in launches:
        for fn, a in la[4]:
            check(fn(*[s if v is stream else v for v in a]))  # the prepared calls, on the capturing stream
    g = C.c_void_p()
    check(lib.fe_hip_graph_end(s, C.byref(g)))
    for _ in range(max(warmup, 2)):
        check(lib.fe_hip_graph_launch(g, s))
    a, b = ev.new(), ev.new()
    ev.record(a, s)
    for _ in range(steps):
        check(lib.fe_hip_graph_launch(g, s))
    ev.record(b, s)
    ms = ev.ms(a, b) / steps
    check(lib.fe_hip_graph_destroy(g))
    return {"ms_per_step": round(ms, 5), "GB/s": round(total_bytes / ms / 1e6, 1),
            "pct_hbm_peak": round(100 * total_bytes / ms / 1e6 / HBM_PEAK_GBS, 2)}


def prefill(torch, np, exl3, fp4, synth, kern, ev, stream, m=2048, k=5120, n=17408):
    """EXL3 4-bit and NVFP4 GEMMs at M = 2048 (activations N(0,1) with 1 % outlier channels x20 for EXL3)."""
    res = {}
    flops = 2.0 * m * n * k
    reps = 10
    # EXL3
    t = synth.exl3_tensor(k, n, 4, SEED, "gate")
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 1024)
    ws = exl3.Workspace([lin], m)
    x = torch.from_numpy(synth.activations(m, k, SEED, outliers=True).view(np.int16)).cuda()
    y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.rotate_input(x, exl3.Dtype.Bf16, m, ws)
    lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws)
    a, b = ev.new(), ev.new()
    ev.record(a, stream)
    for _ in range(reps):
        lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws)
    ev.record(b, stream)
    ms = ev.ms(a, b) / reps
    a2, b2 = ev.new(), ev.new()
    ev.record(a2, stream)
    for _ in range(reps):
        lin.rotate_input(x, exl3.Dtype.Bf16, m, ws)
    ev.record(b2, stream)
    rot_ms = ev.ms(a2, b2) / reps
    res["exl3_b4_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                                 "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "rot_in_ms": round(rot_ms, 4)}
    # the same with the weights decoded once and kept with the linear (2 bytes a weight): no decode launch per call
    lin.keep_decoded()
    lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws)
    a3, b3 = ev.new(), ev.new()
    ev.record(a3, stream)
    for _ in range(reps):
        lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws)
    ev.record(b3, stream)
    ms = ev.ms(a3, b3) / reps
    res["exl3_b4_5120x17408_decoded_kept"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                                              "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                                              "kept_bytes": ((n // 128 + 1) // 2) * 256 * k * 2}
    del lin, ws, y
    # NVFP4
    fk = fp4.Kernels.load()
    flin = synth.fp4_linear(n, k, SEED, input_scale=1.0).upload()
    fws = fp4.Workspace(m, k)
    xf = torch.from_numpy(synth.activations(m, k, SEED).view(np.int16)).cuda()
    yf = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    flin.forward(fk, fws, yf, n, xf, k, m)
    a, b = ev.new(), ev.new()
    ev.record(a, stream)
    for _ in range(reps):
        flin.gemm(fk, fws, yf, n, m)
    ev.record(b, stream)
    ms = ev.ms(a, b) / reps
    a2, b2 = ev.new(), ev.new()
    ev.record(a2, stream)
    for _ in range(reps):
        flin.quantize(fk, fws, xf, k, m)
    ev.record(b2, stream)
    q_ms = ev.ms(a2, b2) / reps
    res["nvfp4_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                               "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "quant_ms": round(q_ms, 4)}
    # NVFP4 at M = 1: the weight-read-bound GEMV over the same linear (codes + block scales = 9/16 byte a weight)
    flin.quantize(fk, fws, xf, k, 1)
    reps = 50
    pairs = [(ev.new(), ev.new()) for _ in range(reps)]
    flin.gemm(fk, fws, yf, n, 1)
    for a, b in pairs:
        ev.record(a, stream)
        flin.gemm(fk, fws, yf, n, 1)
        ev.record(b, stream)
    us = sum(ev.ms(a, b) for a, b in pairs) / reps * 1e3
    wbytes = n * k // 2 + n * k // 16
    res["nvfp4_5120x17408_m1"] = {"gemv_us": round(us, 2), "GB/s": round(wbytes / us / 1e3, 1),
                                  "frac_hbm_peak": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
    del flin, yf
    # the layer's other prefill shape, down (17408 x 5120): the same two GEMMs
    kd, nd = n, k
    flops_d = 2.0 * m * nd * kd

    def timed(fn):
        fn()
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        for _ in range(10):
            fn()
        ev.record(b, stream)
        return ev.ms(a, b) / 10

    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(kd, nd, 4, SEED, "down")), 1024)
    ws = exl3.Workspace([lin], m)
    x = torch.from_numpy(synth.activations(m, kd, SEED, outliers=True).view(np.int16)).cuda()
    y = torch.zeros((m, nd), dtype=torch.bfloat16, device="cuda")
    lin.rotate_input(x, exl3.Dtype.Bf16, m, ws)
    ms = timed(lambda: lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws))
    res["exl3_b4_17408x5120"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops_d / ms / 1e9, 1),
                                 "frac_mfma_peak": round(flops_d / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del lin, ws
    flin_d = synth.fp4_linear(nd, kd, SEED, input_scale=1.0).upload()
    fws_d = fp4.Workspace(m, kd)
    flin_d.quantize(fk, fws_d, x, kd, m)
    ms = timed(lambda: flin_d.gemm(fk, fws_d, y, nd, m))
    res["nvfp4_17408x5120"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops_d / ms / 1e9, 1),
                               "frac_mfma_peak": round(flops_d / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del flin_d, fws_d, x, y
    # the two neighbours of that GEMM in the prompt path: the fused gate|up front (SwiGLU + NVFP4 re-quantization in the
    # epilogue, 2 x 17408 output columns) and an FP8 linear of the same shape
    reps = 5
    gate, up = synth.fp4_linear(n, k, SEED, name="gate"), synth.fp4_linear(n, k, SEED + 1, name="up")
    pair = fp4.HostLinear.fuse([("gate", gate.codes, gate.sf, 1.0, 1.0), ("up", up.codes, up.sf, 1.0, 1.0)]).into_swiglu().upload()
    del gate, up
    act = fp4.Workspace(m, n)
    pair.forward_swiglu(fk, fws, act, xf, k, m, 1.0)
    a, b = ev.new(), ev.new()
    ev.record(a, stream)
    for _ in range(reps):
        pair.forward_swiglu(fk, fws, act, xf, k, m, 1.0)
    ev.record(b, stream)
    ms = ev.ms(a, b) / reps
    res["nvfp4_swiglu_front_5120x34816"] = {"quant_plus_gemm_ms": round(ms, 4), "TFLOP/s": round(2 * flops / ms / 1e9, 1),
                                            "frac_mfma_peak": round(2 * flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del pair, act
    f8 = synth.fp8_linear(n, k, SEED).upload()
    y8 = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    f8.forward(fk, fws, y8, n, xf, k, m)
    a, b = ev.new(), ev.new()
    ev.record(a, stream)
    for _ in range(reps):
        f8.gemm(fk, fws, y8, n, m)
    ev.record(b, stream)
    ms = ev.ms(a, b) / reps
    res["fp8_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1), "mfma": "f32_32x32x64_f8f6f4 (e4m3 x e4m3)",
                             "frac_mfma_fp8_peak": round(flops / ms / 1e9 / MFMA_FP8_PEAK_TFLOPS, 4)}
    del f8, y8
    # the plain bf16 weight form of the same linear (the caller's third form): GEMM at M = 2048 on the bf16 MFMA, GEMV
    # at 1 and 8 rows, which reads 2 bytes a weight and nothing else of size; three weight copies in turn, 535 MB, so
    # that no launch finds its weights in the 256 MB of last-level cache
    from ferrite_amd import bf16
    bk = bf16.Kernels.load()
    gen = torch.Generator(device="cuda").manual_seed(SEED)
    ws_b = [(torch.randn((n, k), generator=gen, device="cuda") * k ** -0.5).to(torch.bfloat16) for _ in range(3)]
    yb = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    ms = timed(lambda: bf16.gemm(bk, yb, n, xf, k, ws_b[0], m))
    res["bf16_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                              "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    wi = bf16.interleave_gu(bk, ws_b[0], ws_b[1])
    actb = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    ms = timed(lambda: bf16.gemm_swiglu(bk, actb, xf, k, wi, m))
    res["bf16_swiglu_front_5120x34816"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(2 * flops / ms / 1e9, 1),
                                           "frac_mfma_peak": round(2 * flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del wi, actb
    for rows in (1, 8):
        reps = 30
        pairs = [(ev.new(), ev.new()) for _ in range(reps)]
        bf16.gemv(bk, yb, n, xf, k, ws_b[0], rows)
        for i, (a, b) in enumerate(pairs):
            ev.record(a, stream)
            bf16.gemv(bk, yb, n, xf, k, ws_b[i % 3], rows)
            ev.record(b, stream)
        us = sum(ev.ms(a, b) for a, b in pairs) / reps * 1e3
        res[f"bf16_5120x17408_m{rows}"] = {"gemv_us": round(us, 2), "GB/s": round(2.0 * n * k / us / 1e3, 1),
                                          "frac_hbm_peak": round(2.0 * n * k / us / 1e3 / HBM_PEAK_GBS, 4)}
    return res


if __name__ == "__main__":
    main()
