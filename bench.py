#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-prefill] [--no-sweep] [--no-configs]

Workload (BASELINE.json configs[1]): the EXL3 decode MLP of a Qwen3.8-27B-shaped layer at M = 1, at 3, 4 and 5 bits per
weight: gate and up are K=5120 N=17408, down is K=17408 N=5120. One step = the forward (input rotation + trellis GEMV)
of all nine linears on seeded synthetic layers, inputs and weights resident in HBM, launched as the MLP block launches
them: per width one call of fe_exl3_mlp_forward, y = down(SwiGLU(gate(x), up(x))), which is one kernel launch (the
programs of down follow those of gate and up in the grid and wait for the column blocks they need). `value` is the
trellis bytes streamed per second (the reference's numerator, crates/fe-exl3/src/bin/exl3-bench.rs:104) over the whole
step, launch gaps and input rotations included. The nine weight sets total 401 MB, more than L2 plus the 256 MB Infinity
Cache, so every step streams its weights from HBM. `separate_launches` is the same nine linears launched as six kernels
(gate + up grouped, then down on an input of its own), the step of earlier versions of this bench.

`roofline` is the dominant kernel alone (exl3_mlp_b4, the three 4-bit projections in one launch): its trellis bytes
over its average launch duration, measured with HIP event pairs on the launch stream in a second pass of the same K
steps in which every launch carries such a pair (which is also where `per_launch` comes from; `value` is taken from the
first pass, without events: a pair costs the eager step 3.5 us a launch). It also carries the grouped gate + up launch
and the single 5120x17408 linear the target names, each timed alone, and the measured decode-only ceiling of the
vector ALUs (`alu_ceiling_*`), which splits the distance to the HBM roofline into "ceiling against HBM" and "kernel
against ceiling".
`cpu_baseline` times the CPU oracle (the reference's factored f64 linear, threaded over 128-column blocks) on the host;
`configs` holds, per BASELINE configuration, a CPU figure of the same kind and the parity of the GPU result against it
(W_hat mismatches on sampled tiles, max |y - ref| / rms(ref), max relative error with the denominator floored at the rms).
`m2048` reports the prefill GEMMs (EXL3 4-bit and NVFP4, 5120x17408, M = 2048) in TFLOP/s against the bf16/f16 MFMA
peak; it is measured after the timed region and is not part of `value`. Every timed figure cycles over enough copies of
its weights (at least 512 MB) that none is served from L2 or the Infinity Cache.
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
# `bench.py --traffic-pass`: KiB fetched x 2.0 (the factor that makes the counter read a streaming read and an
# elementwise update of known size correctly) + KiB written x 1.0
ROOFLINE_TRAFFIC_BYTES = int((69125 * 2.0 + 1632 * 1.0) * 1024)
ROOFLINE_TRAFFIC_SOURCE = "profiles/exl3_mlp_b4_m1_hbm_traffic.md (rocprofv3 --pmc, not measured by this run)"
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_FP8_PEAK_TFLOPS = 5000.0  # dense fp8 MFMA peak of MI355X
SEED = 20251
MLP = [("gate", 5120, 17408), ("up", 5120, 17408), ("down", 17408, 5120)]
BITS = [3, 4, 5]
COLD_BYTES = 512 << 20  # weights a timed loop cycles through: past the 256 MB Infinity Cache
ROW_SAMPLE = lambda m: sorted({0, 1, 17, 127, min(128, m - 1), m // 2, m - 1})  # crates/fe-fp4/src/bin/fp4-check.rs:96


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

    ramp_ms = 0.0  # untimed calls in front of every timed loop, until the GPU holds its clocks (set from --ramp-ms)

    def loop_us(self, stream, fn, reps, ramp_ms=None):
        """Microseconds per call of fn() over `reps` back-to-back calls between one pair of recorded events, after
        `ramp_ms` (default: self.ramp_ms) of the same calls untimed: host work in front of the loop leaves the GPU at idle
        clocks, and the first 30 ms of launches read 7-13 % slow."""
        def burst(n):
            a, b = self.new(), self.new()
            self.record(a, stream)
            for _ in range(n):
                fn()
            self.record(b, stream)
            return self.ms(a, b) * 1e3 / n
        fn()
        ramp_ms = self.ramp_ms if ramp_ms is None else ramp_ms
        if ramp_ms > 0:
            us = burst(8)
            burst(int(ramp_ms * 1e3 / max(us, 1.0)) + 1)
        return burst(reps)


def bf16_to_f64(np, bits):
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


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
        x = bf16_to_f64(np, synth.activations(1, k, SEED))
        layers.append((o, x))
        nbytes += t.trellis_bytes()
    t0 = time.perf_counter()
    for _ in range(reps):
        for o, x in layers:
            oracle.linear_f64(o, x, threads=cores)
    dt = time.perf_counter() - t0
    return {"value": round(reps * nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"oracle linear_f64 (decode_tile + f64 factored linear, threaded over 128-column blocks) on the 4-bit "
                      f"gate, up and down projections at M=1, {reps} passes, {dt:.2f} s"}


def cold_copies(torch, exl3, kern, lin_sets, total=COLD_BYTES):
    """lin_sets: a list of linears that one timed call uses together. Returns a list of such lists, the first the given
    one, the others over device copies of the same weights (plans and bits unchanged), enough of them that a loop over
    the list touches at least `total` bytes of trellis before it comes back to the first."""
    per = sum(l.weight_bytes() for l in lin_sets)
    out, keep = [list(lin_sets)], []
    while per * len(out) < total:
        cp = []
        for l in lin_sets:
            tr = torch.empty(l.weight_bytes() // 4, dtype=torch.int32, device="cuda")
            _copy_dtod(tr.data_ptr(), l.view.trellis, l.weight_bytes())
            v = exl3.Exl3View(l.k, l.n, l.bits, tr.data_ptr(), l.view.suh, l.view.svh, l.view.strips)
            cp.append(exl3.Linear.from_view(kern, l.name, v, l.plan))
            keep.append(tr)
        out.append(cp)
    return out, keep


def _copy_dtod(dst, src, nbytes):
    from ferrite_amd import _lib
    _lib.check(_lib.lib().fe_hip_memcpy_dtod_async(dst, src, nbytes, None))
    _lib.check(_lib.lib().fe_hip_synchronize())


def exl3_parity(torch, np, oracle, exl3, kern, t, x_bits, y_rows, rows, tiles=64):
    """Parity of one EXL3 linear on the GPU against the reference's CPU path restated in oracle/: W_hat on `tiles` sampled
    16x16 tiles, bit for bit, against decode_tile; outputs y_rows (f64, the rows `rows` of the batch x_bits) against
    linear_f64 on the same bf16 inputs. Returns the parity triple and the seconds the CPU linear took."""
    stored = exl3.DeviceExl3.upload(t)
    w = torch.zeros((t.k, t.n), dtype=torch.int16, device="cuda")
    kern.reconstruct_hat_f16(stored.view, w)
    torch.cuda.synchronize()
    rng = np.random.default_rng([SEED, t.k, t.n, t.bits])
    bad = 0
    for kt, nt in zip(rng.integers(0, t.k // 16, tiles), rng.integers(0, t.n // 16, tiles)):
        want = oracle.decode_tile(t.tile(int(kt), int(nt)), t.bits)
        got = w[kt * 16:kt * 16 + 16, nt * 16:nt * 16 + 16].cpu().numpy().view(np.uint16)
        bad += int((got != want).sum())
    del w, stored
    o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
    t0 = time.perf_counter()
    ref = oracle.linear_f64(o, bf16_to_f64(np, x_bits[rows]), threads=oracle.default_threads(64))
    dt = time.perf_counter() - t0
    rms = float(np.sqrt((ref ** 2).mean()))
    err = np.abs(y_rows - ref)
    return {"w_hat_mismatches": bad, "w_hat_values_checked": tiles * 256, "max_err_over_rms": round(float(err.max() / rms), 6),
            "max_rel_floored_at_rms": round(float((err / np.maximum(np.abs(ref), rms)).max()), 6), "rows_checked": len(rows)}, dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--ramp-ms", type=float, default=60.0,
                    help="untimed steps in front of the W + K steps of `value`, until the GPU holds its clocks (0: none)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="leave out the per-configuration CPU figures and parity")
    ap.add_argument("--bracket-events", action="store_true",
                    help="time the roofline kernel with events recorded before and after its launch instead of events attached to its dispatch")
    ap.add_argument("--separate", action="store_true",
                    help="the step as six launches (gate + up grouped, then down on an input of its own) instead of one launch per MLP")
    ap.add_argument("--step-only", action="store_true",
                    help="only the timed passes of the step (for a kernel trace in which every GEMV dispatch is one of the step's six launches)")
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
    cpu = None if args.no_cpu else cpu_baseline()  # first, as the configuration asks

    kern = exl3.Kernels.load()
    lib = _lib.lib()
    ev = Events(lib, _lib.check)
    ev.ramp_ms = args.ramp_ms
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    blocks = exl3.default_blocks(exl3.cu_count())

    # the nine linears, one device copy each
    linears, tensors = [], {}
    for bits in BITS:
        for name, k, n in MLP:
            t = synth.exl3_tensor(k, n, bits, SEED, name)
            tensors[(name, bits)] = t
            lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), blocks)
            x = torch.from_numpy(synth.activations(1, k, SEED).view(np.int16)).cuda()
            y = torch.zeros((1, n), dtype=torch.bfloat16, device="cuda")
            linears.append((name, bits, lin, x, y))
    ws = exl3.Workspace([l[2] for l in linears], 1)
    total_bytes = sum(l[2].weight_bytes() for l in linears)

    # The step's launches. Headline: per bit width one call of fe_exl3_mlp_forward, down on SwiGLU(gate(x), up(x)): one
    # kernel launch each. Beside it the step of earlier versions of this bench: gate + up of one input as a grouped call, then
    # down on an input of its own, six launches. Every argument of the calls into the C ABI is prepared once.
    f_group, f_forward, f_rotate, f_rotated, f_record, f_mlp = (lib.fe_exl3_linear_forward_group, lib.fe_exl3_linear_forward,
                                                               lib.fe_exl3_linear_rotate_input, lib.fe_exl3_linear_gemv_rotated,
                                                               lib.fe_hip_event_record, lib.fe_exl3_mlp_forward)
    bf16 = int(exl3.Dtype.Bf16)
    by = {(name, bits): (lin, x, y) for name, bits, lin, x, y in linears}
    launches = []  # (label, bytes, dominant, kernel launches, [(fn, args)...], keepalive)
    chain = []
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
        if exl3.mlp_forward_launches(g, u, d, 1, exl3.Dtype.Bf16, ws) == 1:
            chain.append((f"mlp_b{bits}", g.weight_bytes() + u.weight_bytes() + d.weight_bytes(), bits == 4, 1,
                          [(f_mlp, (g.h, u.h, d.h, kern.h, stream, xg.data_ptr(), bf16, yg.data_ptr(), yu.data_ptr(), yd.data_ptr(),
                                    bf16, 1, ws.h))], None))
    separate = launches
    one_launch_mlp = len(chain) == len(BITS) and not args.separate
    if one_launch_mlp:
        launches = chain

    # Event pairs on the launch stream, one per launch of a second pass of the same K steps. A pair is attached to the dispatch of the
    # launch's last kernel (the GEMV), so it reads that kernel's own begin and end as a kernel trace does and puts no
    # packets of its own on the queue (fe_hip_time_next_launch); every launch carries one, because a timed dispatch that
    # follows an untimed one takes its start when it is accepted, while the launch before it still drains (3-4 us too
    # long). With --bracket-events the pairs are recorded before and after the launch instead, each record a packet
    # of its own on the queue, which adds the dispatch gap and the packets to the reading.
    attached = not args.bracket_events
    f_time_next = lib.fe_hip_time_next_launch

    def measure(launches):
        """W + K steps right after the host work, the ramp, W + K steps again (`value`), then K steps with an event pair on
        every launch."""
        events = [[(ev.new(), ev.new()) for _ in launches] for _ in range(args.steps)]

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

        def timed_steps():  # W untimed steps, then exactly K steps between two synchronizations
            for _ in range(args.warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.steps):
                step()
            torch.cuda.synchronize()
            return time.perf_counter() - t0

        # The GPU comes out of the host work before this point (the CPU baseline, the uploads) at its idle clocks and takes
        # about 30 ms of continuous launches to reach the clocks it then holds: the same K steps read 2230 GB/s right after
        # idle, 2400 after 8 ms, 2500 after 16 ms and 2560 from 32 ms on (no further change up to 250 ms). A decode loop runs
        # in that steady state, so `value` is taken there: `after_idle` is the reading right after the host work, then the
        # steps run untimed for --ramp-ms, then W + K steps again.
        r = {}
        r["dt_idle"] = timed_steps()
        r["ramp_steps"] = int(args.ramp_ms * 1e-3 / (r["dt_idle"] / args.steps)) + 1 if args.ramp_ms > 0 else 0
        for _ in range(r["ramp_steps"]):
            step()
        r["dt"] = timed_steps() if r["ramp_steps"] else r["dt_idle"]
        # the same K steps once more with an event pair on every launch, for the roofline kernel's own duration and the
        # per-launch table (the pairs cost the eager step 3.5 us a launch, so `value` is taken without them)
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(events[i])
        torch.cuda.synchronize()
        r["ms_per_step_timed"] = (time.perf_counter() - t0) * 1e3 / args.steps
        r["dom_ms"] = []
        for li, la in enumerate(launches):
            if la[2]:
                r["dom_ms"] += [ev.ms(*events[i][li]) for i in range(args.steps)]
                r["dom_bytes"] = la[1]
        r["per"] = {}
        for li, la in enumerate(launches):  # every launch of the timed region, by its own events
            us = sum(ev.ms(*events[i][li]) for i in range(args.steps)) / args.steps * 1e3
            r["per"][la[0]] = {"us": round(us, 2), "GB/s": round(la[1] / us / 1e3, 1), "launches": la[3]}
        return r

    head = measure(launches)
    dt_idle, dt, ramp_steps, ms_per_step_timed, per = head["dt_idle"], head["dt"], head["ramp_steps"], head["ms_per_step_timed"], head["per"]
    ms_per_step = dt * 1e3 / args.steps
    value = total_bytes / (dt / args.steps) / 1e9
    dom_ms, dom_bytes = head["dom_ms"], head["dom_bytes"]
    dom_kernel = "exl3_mlp_b4" if one_launch_mlp else "exl3_gemvb_b4_r1"
    dom_avg_ms = sum(dom_ms) / len(dom_ms)
    achieved = dom_bytes / (dom_avg_ms * 1e-3) / 1e9
    if one_launch_mlp:
        assert ws.chain_status() == 0, "a bounded wait of the one-launch MLP ran out"

    if args.step_only:
        print(json.dumps({"metric": "quant linear GB/s (%HBM peak) at M=1; TFLOP/s (%MFMA peak) at M=2048", "value": round(value, 2),
                          "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "ms_per_step": round(ms_per_step, 5), "ramp_steps": ramp_steps,
                          "roofline": {"kernel": dom_kernel, "avg_launch_us": round(dom_avg_ms * 1e3, 3),
                                       "achieved": round(achieved, 2), "frac": round(achieved / HBM_PEAK_GBS, 4)},
                          "per_launch": per}))
        return
    # the six-launch step of earlier versions, measured the same way
    sep = measure(separate) if one_launch_mlp else head
    sep_value = total_bytes / (sep["dt"] / args.steps) / 1e9
    sep_dom_us = sum(sep["dom_ms"]) / len(sep["dom_ms"]) * 1e3

    # The dominant launch, the grouped gate + up launch and the single linear the target names, each alone: back to back
    # between one pair of events, eagerly launched and replayed from a graph (no host time between the launches), cycling
    # over weight copies past the caches. A launch period is an upper bound of the kernel's duration.
    g4, u4, d4 = by[("gate", 4)][0], by[("up", 4)][0], by[("down", 4)][0]
    x4 = by[("gate", 4)][1]
    mlp_sets, keep1 = cold_copies(torch, exl3, kern, [g4, u4, d4])
    ws_alone = exl3.Workspace([g4, u4, d4], 1)
    ys_pair = [by[("gate", 4)][2], by[("up", 4)][2]]
    y_down = by[("down", 4)][2]
    at = [0]

    def mlp_call(s=stream):
        g, u, d = mlp_sets[at[0] % len(mlp_sets)]
        exl3.mlp_forward(g, u, d, x4, exl3.Dtype.Bf16, ys_pair[0], ys_pair[1], y_down, exl3.Dtype.Bf16, 1, ws_alone, stream=s)
        at[0] += 1

    def pair_call(s=stream):
        exl3.forward_group(mlp_sets[at[0] % len(mlp_sets)][:2], x4, exl3.Dtype.Bf16, ys_pair, exl3.Dtype.Bf16, 1, ws_alone, stream=s)
        at[0] += 1

    def single_call(s=stream):
        mlp_sets[at[0] % len(mlp_sets)][0].forward(x4, exl3.Dtype.Bf16, ys_pair[0], exl3.Dtype.Bf16, 1, ws_alone, stream=s)
        at[0] += 1

    alone = {}
    for name, fn, nbytes in (("mlp_b4", mlp_call, dom_bytes if one_launch_mlp else g4.weight_bytes() + u4.weight_bytes() + d4.weight_bytes()),
                             ("gate_up_b4", pair_call, g4.weight_bytes() + u4.weight_bytes()),
                             ("single_5120x17408_b4", single_call, g4.weight_bytes())):
        eager_us = ev.loop_us(stream, fn, 4 * len(mlp_sets))
        replay_us = graph_us(lib, _lib.check, ev, fn, 2 * len(mlp_sets))
        alone[name] = {"bytes_per_launch": nbytes, "eager_period_us": round(eager_us, 3), "graph_replay_period_us": round(replay_us, 3),
                       "GB/s": round(nbytes / replay_us / 1e3, 1), "frac": round(nbytes / replay_us / 1e3 / HBM_PEAK_GBS, 4)}
    alone["mlp_b4"]["launches"] = 1 if one_launch_mlp else 2
    # ... and the single linear's kernel by events attached to its dispatch, every launch carrying a pair. The host cannot
    # keep the queue full at this pace (a launch with a pair costs it more than the kernel lasts), so each kernel starts on
    # an idle GPU and reads longer than the launch period above: reported, not used.
    one_pairs = [(ev.new(), ev.new()) for _ in range(2 * len(mlp_sets))]
    for a, b in one_pairs:
        _lib.check(f_time_next(a, b))
        single_call()
    alone["single_5120x17408_b4"]["attached_events_on_an_idle_queue_us"] = round(sum(ev.ms(a, b) for a, b in one_pairs) / len(one_pairs) * 1e3, 3)
    del mlp_sets, keep1, ws_alone

    # the decode-only ceiling of the vector ALUs: the GEMV's decode at the GEMV's occupancy with no memory traffic
    ceiling = {}
    for bits in BITS:
        grid, iters = 4 * exl3.cu_count(), 256
        if args.ramp_ms > 0:  # (the probes run at steady clocks like the kernel they bound)
            ms = kern.probe_decode(bits, grid, iters, 5)
            kern.probe_decode(bits, grid, iters, int(args.ramp_ms / max(ms, 1e-3)) + 1)
        ms = kern.probe_decode(bits, grid, iters, 20)
        ceiling[f"b{bits}"] = round(grid * 256 * 32 * iters * bits / 8 / (ms * 1e-3) / 1e9, 1)

    single, pair = alone["single_5120x17408_b4"], alone["gate_up_b4"]
    untimed = 2 * args.warmup + args.steps + ramp_steps  # steps in front of the K steps of `value`
    out = {
        "metric": "quant linear GB/s (%HBM peak) at M=1; TFLOP/s (%MFMA peak) at M=2048",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ramp_steps": ramp_steps, "untimed_steps_total": untimed,
        "after_idle_value": round(total_bytes / (dt_idle / args.steps) / 1e9, 2),
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "EXL3 decode MLP, Qwen3.8-27B-shaped layer, M=1, 3/4/5 bpw (gate, up 5120x17408; down 17408x5120)",
                   "linears_per_step": len(linears), "kernel_launches_per_step": sum(la[3] for la in launches),
                   "trellis_bytes_per_step": total_bytes, "seed": SEED,
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "untimed_steps_total": untimed, "ramp_steps": ramp_steps,
                   "after_idle_value": round(total_bytes / (dt_idle / args.steps) / 1e9, 2),
                   "separate_launches_value": round(sep_value, 2)},
        "roofline": {"bound": "hbm",
                     "kernel": (f"{dom_kernel} (gate, up and down of the 4-bit MLP in one launch, M=1)" if one_launch_mlp else
                                f"{dom_kernel} (gate + up in one launch, 5120x17408 each, 4 bits, M=1)"),
                     "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": ROOFLINE_TRAFFIC_BYTES if one_launch_mlp else None, "traffic_source": ROOFLINE_TRAFFIC_SOURCE,
                     "avg_launch_us": round(dom_avg_ms * 1e3, 3), "bytes_per_launch": dom_bytes, "launches": len(dom_ms),
                     "timed_in": f"a second pass of the {args.steps} steps with an event pair on every launch ({ms_per_step_timed:.5f} ms a step)",
                     "events": "recorded around the launch" if args.bracket_events else "attached to the kernel's dispatch",
                     "alu_ceiling_b3_GBs": ceiling["b3"], "alu_ceiling_b4_GBs": ceiling["b4"], "alu_ceiling_b5_GBs": ceiling["b5"],
                     "frac_of_alu_ceiling": round(achieved / ceiling["b4"], 4),
                     "graph_replay_period_us": alone["mlp_b4"]["graph_replay_period_us"],
                     "gate_up_launch_us": round(sep_dom_us, 3),
                     "gate_up_launch_frac": round(pair["bytes_per_launch"] / sep_dom_us / 1e3 / HBM_PEAK_GBS, 4),
                     "gate_up_launch_period_us": pair["graph_replay_period_us"],
                     "single_linear_us": single["graph_replay_period_us"], "single_linear_frac": single["frac"],
                     "alone": alone},
        "cpu_baseline": cpu,
        "per_launch": per,
        "after_idle": {"value": round(total_bytes / (dt_idle / args.steps) / 1e9, 2), "unit": "GB/s",
                       "ms_per_step": round(dt_idle * 1e3 / args.steps, 5),
                       "what": f"the same {args.warmup} + {args.steps} steps right after the host work, before the {ramp_steps} "
                               f"untimed steps ({args.ramp_ms:g} ms) that bring the GPU to the clocks it holds in a decode loop"},
        "separate_launches": {"value": round(sep_value, 2), "unit": "GB/s", "ms_per_step": round(sep["dt"] * 1e3 / args.steps, 5),
                              "kernel_launches_per_step": sum(la[3] for la in separate), "per_launch": sep["per"],
                              "what": "gate + up as one grouped launch, then down on an input of its own: the step of earlier "
                                      "versions of this bench"},
    }

    out["graph_replay"] = graph_replay(lib, _lib.check, ev, launches, stream, total_bytes, args.steps, args.warmup, ramp_steps)
    if not args.no_configs and not args.no_cpu:
        out["configs"] = configs(torch, np, exl3, fp4, synth, kern, ev, stream, tensors, by, ws)
    if not args.no_sweep:
        out["rows_sweep_b4"] = rows_sweep(torch, np, exl3, synth, kern, ev, stream, lib, _lib.check, linears)
    if not args.no_prefill:
        out["m2048"] = prefill(torch, np, exl3, fp4, synth, kern, ev, stream)
    print(json.dumps(out))


def configs(torch, np, exl3, fp4, synth, kern, ev, stream, tensors, by, ws):
    """Per BASELINE configuration: the CPU path (oracle/: the reference's CPU dequant + matmul restated) timed on the host
    cores, run before the GPU figure it stands beside, and the parity of the GPU result against it."""
    import oracle
    cores = oracle.default_threads(64)
    res = {"cpu_cores": cores}
    blocks = exl3.default_blocks(exl3.cu_count())

    # configs[0]: EXL3 4 bpw, K = N = 5120, M = 1; the CPU path first
    t = synth.exl3_tensor(5120, 5120, 4, SEED, "c1")
    xb = synth.activations(1, 5120, SEED)
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), blocks)
    w1 = exl3.Workspace([lin], 1)
    x = torch.from_numpy(xb.view(np.int16)).cuda()
    y = torch.zeros((1, 5120), dtype=torch.float32, device="cuda")
    o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
    t0 = time.perf_counter()
    for _ in range(5):
        oracle.linear_f64(o, bf16_to_f64(np, xb), threads=cores)
    cpu_s = (time.perf_counter() - t0) / 5
    lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 1, w1)
    torch.cuda.synchronize()
    par, _ = exl3_parity(torch, np, oracle, exl3, kern, t, xb, y.cpu().numpy().astype(np.float64), [0])
    sets, keep = cold_copies(torch, exl3, kern, [lin])
    yb = torch.zeros((1, 5120), dtype=torch.bfloat16, device="cuda")
    at = [0]

    def call():
        sets[at[0] % len(sets)][0].forward(x, exl3.Dtype.Bf16, yb, exl3.Dtype.Bf16, 1, w1, stream=stream)
        at[0] += 1

    us = ev.loop_us(stream, call, 2 * len(sets))
    nbytes = lin.weight_bytes()
    res["c1_exl3_b4_5120x5120_m1"] = {
        "cpu": {"seconds": round(cpu_s, 4), "GB/s": round(nbytes / cpu_s / 1e9, 4), "cores": cores, "kind": "port",
                "sample": "oracle linear_f64, whole linear, 5 passes"},
        "gpu": {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)},
        "gpu_over_cpu": round(cpu_s * 1e6 / us, 1), "parity": par}
    del sets, keep, lin, w1

    # configs[1]: every linear of the timed step against the CPU linear on the same input
    c2 = {}
    for (name, bits), t in tensors.items():
        lin, x, _ = by[(name, bits)]
        y = torch.zeros((1, t.n), dtype=torch.float32, device="cuda")
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 1, ws)
        torch.cuda.synchronize()
        par, cpu_s = exl3_parity(torch, np, oracle, exl3, kern, t, synth.activations(1, t.k, SEED), y.cpu().numpy().astype(np.float64), [0])
        par["cpu_linear_f64_seconds"] = round(cpu_s, 4)
        c2[f"{name}_b{bits}"] = par
    res["c2_decode_mlp_m1"] = c2

    # configs[3]: EXL3 4 bpw prefill, M = 2048, activations with 1 % outlier channels x20. The CPU figure is the f64 linear on
    # the reference's row sample and on one row: T(m) = a + b m (decode once, then the products), evaluated at 2048 rows.
    m = 2048
    c4 = {}
    for name, k, n in (("gate_up", 5120, 17408), ("down", 17408, 5120)):
        t = tensors[("gate" if name == "gate_up" else "down", 4)]
        xb = synth.activations(m, k, SEED, outliers=True)
        rows = ROW_SAMPLE(m)
        o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
        t0 = time.perf_counter()
        oracle.linear_f64(o, bf16_to_f64(np, xb[:1]), threads=cores)
        t1 = time.perf_counter() - t0
        lin = by[("gate" if name == "gate_up" else "down", 4)][0]
        wsm = exl3.Workspace([lin], m)
        x = torch.from_numpy(xb.view(np.int16)).cuda()
        y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.Bf16, m, wsm)
        torch.cuda.synchronize()
        got = y[rows].float().cpu().numpy().astype(np.float64)
        par, t7 = exl3_parity(torch, np, oracle, exl3, kern, t, xb, got, rows, tiles=16)
        b = max(t7 - t1, 0.0) / (len(rows) - 1)
        cpu_s = t1 + b * (m - 1)
        flops = 2.0 * m * n * k
        c4[f"exl3_b4_{k}x{n}"] = {
            "cpu": {"seconds_extrapolated": round(cpu_s, 2), "GFLOP/s": round(flops / cpu_s / 1e9, 2), "cores": cores, "kind": "port",
                    "sample": f"oracle linear_f64 on 1 row ({t1:.2f} s) and on rows {rows} ({t7:.2f} s), extrapolated linearly to {m} rows"},
            "parity": par}
        del wsm, x, y
    res["c4_exl3_prefill_m2048"] = c4

    # configs[4]: NVFP4, K = 5120, N = 17408, M = 1 and 2048: quantize the activations, dequantize both operands, f64 dot
    # products (crates/fe-fp4/src/format.rs:72-90, 136-142, 151-181), on the row sample; parity as fp4-check.rs:134-144
    k, n = 5120, 17408
    host = synth.fp4_linear(n, k, SEED, input_scale=1.0)
    fk = fp4.Kernels.load()
    flin = host.upload()
    t0 = time.perf_counter()
    wdq = oracle.dequant_fp4(host.codes, host.sf, 1.0)
    t_w = time.perf_counter() - t0
    c5 = {}
    for m in (1, 2048):
        xb = synth.activations(m, k, SEED)
        rows = ROW_SAMPLE(m) if m > 1 else [0]
        t0 = time.perf_counter()
        codes, sf = oracle.quant_fp4(xb[rows], host.g)
        ref = oracle.ref_gemm(oracle.dequant_fp4(codes, sf, 1.0), wdq).astype(np.float64) * host.alpha.astype(np.float64)
        t_rows = time.perf_counter() - t0
        cpu_s = t_w + t_rows / len(rows) * m
        fws = fp4.Workspace(m, k)
        x = torch.from_numpy(xb.view(np.int16)).cuda()
        y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        flin.forward(fk, fws, y, n, x, k, m)
        torch.cuda.synchronize()
        got = y[rows].float().cpu().numpy().astype(np.float64)
        gc, gsf_t = fws.read(m, k)
        gsf = oracle.untile_scales(gsf_t, m, k // 16).reshape(m, k // 16)
        scale = np.abs(ref).max(axis=1, keepdims=True).clip(1e-20)
        flops = 2.0 * m * n * k
        c5[f"m{m}"] = {
            "cpu": {"seconds" + ("_extrapolated" if m > 1 else ""): round(cpu_s, 3), "GFLOP/s": round(flops / cpu_s / 1e9, 2),
                    "cores": cores, "kind": "port",
                    "sample": f"oracle quant_fp4_row + dequant_fp4_row + ref_gemm on rows {rows} ({t_rows:.2f} s) plus the weight "
                              f"dequantization ({t_w:.2f} s)" + (f", scaled to {m} rows" if m > 1 else "")},
            "parity": {"activation_code_bytes_differing": int((gc[rows] != codes).sum()),
                       "activation_scale_bytes_differing": int((gsf[rows] != sf).sum()),
                       "max_err_over_row_max": round(float((np.abs(got - ref) / scale).max()), 6),
                       "max_rel_floored_at_1e-2_row_max": round(float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2 * scale)).max()), 6),
                       "rows_checked": len(rows)}}
        del fws, x, y
    res["c5_nvfp4_5120x17408"] = c5
    return res


def traffic_pass(torch, np, exl3, synth):
    """Three rounds of: evict (an elementwise update of 600 MiB: reads 600 MiB, writes 600 MiB), exl3_probe_v4 reading
    exactly the roofline kernel's algorithmic bytes, evict, the roofline kernel (the 4-bit MLP in one launch). Prints the
    known sizes."""
    kern = exl3.Kernels.load()
    blocks = exl3.default_blocks(exl3.cu_count())
    lins = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, n, 4, SEED, name)), blocks) for name, k, n in MLP]
    ws = exl3.Workspace(lins, 1)
    x = torch.from_numpy(synth.activations(1, 5120, SEED).view(np.int16)).cuda()
    ys = [torch.zeros((1, l.n), dtype=torch.bfloat16, device="cuda") for l in lins]
    nbytes = sum(l.weight_bytes() for l in lins)
    buf = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    big = torch.zeros(600 << 20, dtype=torch.uint8, device="cuda")
    assert exl3.mlp_forward_launches(*lins, 1, exl3.Dtype.Bf16, ws) == 1
    for _ in range(3):
        big.add_(1)
        kern.probe_stream_read(buf, 1024, 1)
        big.add_(1)
        exl3.mlp_forward(*lins, x, exl3.Dtype.Bf16, ys[0], ys[1], ys[2], exl3.Dtype.Bf16, 1, ws)
    torch.cuda.synchronize()
    print(json.dumps({"exl3_probe_v4_reads_KiB": nbytes / 1024, "elementwise_reads_and_writes_KiB": (600 << 20) / 1024,
                      "roofline_kernel": "exl3_mlp_b4", "algorithmic_KiB": nbytes / 1024}))


def graph_us(lib, check, ev, fn, inner, reps=5):
    """Microseconds per call of fn(stream) with `inner` calls captured into one HIP graph on a stream of its own and the
    graph replayed `reps` times."""
    s, g = C.c_void_p(), C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    fn(s)
    check(lib.fe_hip_stream_sync(s))
    check(lib.fe_hip_graph_begin(s))
    for _ in range(inner):
        fn(s)
    check(lib.fe_hip_graph_end(s, C.byref(g)))

    def burst(n):
        a, b = ev.new(), ev.new()
        ev.record(a, s)
        for _ in range(n):
            check(lib.fe_hip_graph_launch(g, s))
        ev.record(b, s)
        return ev.ms(a, b) * 1e3 / (n * inner)
    us = burst(1)
    if ev.ramp_ms > 0:  # (the capture is host work: back to steady clocks first)
        burst(int(ev.ramp_ms * 1e3 / max(us * inner, 1.0)) + 1)
    us = burst(reps)
    check(lib.fe_hip_graph_destroy(g))
    check(lib.fe_hip_stream_destroy(s))
    return us


def rows_sweep(torch, np, exl3, synth, kern, ev, stream, lib, check, linears):
    """The 4-bit MLP and the attention projections at M = 1, 4, 8, 16 (BASELINE's decode / speculative-verify row counts)
    and 32, 64 (the reference's all-linear times, crates/fe-exl3/BENCH.md:103):
    microseconds per linear, launched back to back as the step launches them (gate + up grouped, then down; q, k, v grouped,
    then o), cycling over weight copies of at least 512 MB in all, eagerly launched and replayed from a graph. Not part of
    `value`."""
    four = {name: lin for name, bits, lin, x, y in linears if bits == 4}
    g, u, d = four["gate"], four["up"], four["down"]
    mlp_sets, keep_a = cold_copies(torch, exl3, kern, [g, u, d])
    blocks = exl3.default_blocks(exl3.cu_count())
    q, kk, v, o = (exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(5120, n, 4, SEED, name)), blocks)
                   for name, n in (("q", 5120), ("k", 1024), ("v", 1024), ("o", 5120)))
    attn_sets, keep_b = cold_copies(torch, exl3, kern, [q, kk, v, o])
    abytes = sum(l.weight_bytes() for l in (q, kk, v, o))
    nbytes = (g.weight_bytes() + u.weight_bytes() + d.weight_bytes()) / 3
    res = {"weight_copies_cycled": {"mlp": len(mlp_sets), "attn": len(attn_sets)}}
    for m in (1, 4, 8, 16, 32, 64):
        ws = exl3.Workspace([g, u, d, q, kk, v, o], m)
        x = torch.from_numpy(synth.activations(m, g.k, SEED).view(np.int16)).cuda()
        xd = torch.from_numpy(synth.activations(m, d.k, SEED).view(np.int16)).cuda()
        yg, yu = (torch.zeros((m, g.n), dtype=torch.bfloat16, device="cuda") for _ in range(2))
        yd = torch.zeros((m, d.n), dtype=torch.bfloat16, device="cuda")
        resid = torch.zeros((m, d.n), dtype=torch.bfloat16, device="cuda")
        ys = [torch.zeros((m, l.n), dtype=torch.bfloat16, device="cuda") for l in (q, kk, v)]
        yo = torch.zeros((m, 5120), dtype=torch.bfloat16, device="cuda")
        at = [0]

        def mlp(s=stream):
            gg, uu, dd = mlp_sets[at[0] % len(mlp_sets)]
            at[0] += 1
            exl3.forward_group([gg, uu], x, exl3.Dtype.Bf16, [yg, yu], exl3.Dtype.Bf16, m, ws, stream=s)
            dd.forward(xd, exl3.Dtype.Bf16, yd, exl3.Dtype.Bf16, m, ws, stream=s)

        # the MLP block as the model runs it: down reads SwiGLU(gate, up) of the grouped launch's outputs and adds into the
        # residual stream
        def block(s=stream):
            gg, uu, dd = mlp_sets[at[0] % len(mlp_sets)]
            at[0] += 1
            exl3.mlp_forward(gg, uu, dd, x, exl3.Dtype.Bf16, yg, yu, resid, exl3.Dtype.Bf16Add, m, ws, stream=s)

        def attn(s=stream):
            qq, k2, vv, oo = attn_sets[at[0] % len(attn_sets)]
            at[0] += 1
            exl3.forward_group([qq, k2, vv], x, exl3.Dtype.Bf16, ys, exl3.Dtype.Bf16, m, ws, stream=s)
            oo.forward(x, exl3.Dtype.Bf16, yo, exl3.Dtype.Bf16, m, ws, stream=s)

        us = ev.loop_us(stream, mlp, 3 * len(mlp_sets)) / 3
        r = {"us_per_linear": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
             "gate_up_launches": exl3.forward_group_launches([g, u], m, ws),
             "mlp_block_is_one_launch": bool(exl3.mlp_forward_launches(g, u, d, m, exl3.Dtype.Bf16Add, ws))}
        r["mlp_block_us"] = round(ev.loop_us(stream, block, 3 * len(mlp_sets)), 2)
        r["mlp_block_graph_us"] = round(graph_us(lib, check, ev, block, 2 * len(mlp_sets)), 2)
        a_us = ev.loop_us(stream, attn, 2 * len(attn_sets))
        r["attn_qkv_o_us"] = round(a_us, 2)
        r["attn_GB/s"] = round(abytes / a_us / 1e3, 1)
        a_g = graph_us(lib, check, ev, attn, 2 * len(attn_sets))
        r["attn_qkv_o_graph_us"] = round(a_g, 2)
        r["attn_graph_GB/s"] = round(abytes / a_g / 1e3, 1)
        res[f"m{m}"] = r
    del mlp_sets, attn_sets, keep_a, keep_b
    return res


def graph_replay(lib, check, ev, launches, stream, total_bytes, steps, warmup, ramp_steps):
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
    for _ in range(max(warmup, 2) + ramp_steps):  # (the capture is host work: back to steady clocks first, as for `value`)
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
    # Steady state: a GEMM of this size runs against the board's power limit, and for the first 30-100 launches after an
    # idle stretch the clock has not settled (the same launch takes 350-400 us there and 300-340 us from about 0.1 s of
    # continuous work on). A prompt is a long run of such launches, so every figure is taken after 0.15 s of the same
    # launches, over 0.15 s more; `after_idle_ms` is the first ten launches after the preceding host work, for comparison.
    def timed(fn, reps=10, steady=True):
        first = ev.loop_us(stream, fn, reps, ramp_ms=0) / 1e3
        if not steady:
            return first
        n_warm = max(30, int(150.0 / first))
        ev.loop_us(stream, fn, n_warm, ramp_ms=0)
        timed.after_idle = first
        return ev.loop_us(stream, fn, n_warm, ramp_ms=0) / 1e3

    # What the matrix units sustain on this board with nothing else running: the register-only probe (4 x 4 independent
    # v_mfma_f32_32x32x16_f16 per wavefront, one wavefront a SIMD as in the GEMM core) after the same 0.15 s of launches, with
    # operands of 0.5 and 1 (the published peak's conditions: hardly a bit toggles), with random signs and mantissas (what
    # rotated activations and 11-bit codebook values feed the unit) and with five random mantissa bits (the six
    # significant bits of an NVFP4 operand). The clock is what rocm-smi reports during the sustained window.
    from ferrite_amd import probes
    fk = fp4.Kernels.load()
    peak = {}
    for label, kind, seed in (("f16_constant_operands", "f16", 0), ("f16_random_operands", "f16", 12345),
                              ("f16_five_mantissa_bits", "f16", 12346), ("f8_random_operands", "f8", 12345)):
        p = probes.mfma_peak(fk, kind, exl3.cu_count(), seed=seed)
        peak[label] = {"TFLOP/s": p["sustained_TFLOPs"], "burst_TFLOP/s": p["burst_TFLOPs"], "sclk_MHz": p.get("sclk_MHz_median")}
    res["mfma_sustained"] = peak
    sus16, sus16_5, sus8 = peak["f16_random_operands"]["TFLOP/s"], peak["f16_five_mantissa_bits"]["TFLOP/s"], peak["f8_random_operands"]["TFLOP/s"]

    # EXL3
    t = synth.exl3_tensor(k, n, 4, SEED, "gate")
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 1024)
    ws = exl3.Workspace([lin], m)
    x = torch.from_numpy(synth.activations(m, k, SEED, outliers=True).view(np.int16)).cuda()
    y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.rotate_input(x, exl3.Dtype.Bf16, m, ws)
    ms = timed(lambda: lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws))
    idle_ms = timed.after_idle
    rot_ms = timed(lambda: lin.rotate_input(x, exl3.Dtype.Bf16, m, ws), steady=False)
    res["exl3_b4_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                                 "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "rot_in_ms": round(rot_ms, 4),
                                 "after_idle_ms": round(idle_ms, 4)}
    # the same with the weights decoded once and kept with the linear (2 bytes a weight): no decode launch per call
    lin.keep_decoded()
    ms = timed(lambda: lin.gemv_rotated(ws.xh_ptr, y, exl3.Dtype.Bf16, m, ws))
    res["exl3_b4_5120x17408_decoded_kept"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                                              "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                                              "kept_bytes": ((n // 128 + 1) // 2) * 256 * k * 2}
    del lin, ws, y
    # yardstick: the vendor library's f16 GEMM (torch.matmul -> hipBLASLt) of the same shape on this box, same timing loop.
    # Launches of this size run against the board's power limit, not the MFMA's issue rate: the figure says what a tuned
    # plain GEMM sustains here.
    a16 = torch.randn((m, k), device="cuda", dtype=torch.float16)
    w16 = torch.randn((n, k), device="cuda", dtype=torch.float16)
    y16 = torch.empty((m, n), device="cuda", dtype=torch.float16)
    ms = timed(lambda: torch.matmul(a16, w16.T, out=y16))
    res["vendor_f16_gemm_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1), "after_idle_ms": round(timed.after_idle, 4),
                                         "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                                         "what": "torch.matmul (hipBLASLt), f16 x f16^T, random normal operands"}
    del a16, w16, y16
    # NVFP4
    flin = synth.fp4_linear(n, k, SEED, input_scale=1.0).upload()
    fws = fp4.Workspace(m, k)
    xf = torch.from_numpy(synth.activations(m, k, SEED).view(np.int16)).cuda()
    yf = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    flin.forward(fk, fws, yf, n, xf, k, m)
    ms = timed(lambda: flin.gemm(fk, fws, yf, n, m))
    idle_ms = timed.after_idle
    q_ms = timed(lambda: flin.quantize(fk, fws, xf, k, m), steady=False)
    res["nvfp4_5120x17408"] = {"gemm_ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                               "frac_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "quant_ms": round(q_ms, 4),
                               "after_idle_ms": round(idle_ms, 4),
                               # the quantizer leaves the activations as codes + scales (the format) and as the fp16 operand
                               # 2 * value * scale the GEMM reads: 2 bytes an element against the format's 9/16
                               "activation_operand_bytes": m * k * 2, "activation_format_bytes": m * k // 2 + m * k // 16}
    # NVFP4 at M = 1: the weight-read-bound GEMV over the same linear (codes + block scales = 9/16 byte a weight), cycling
    # over weight copies past the caches
    host1 = synth.fp4_linear(n, k, SEED, input_scale=1.0)
    wbytes = n * k // 2 + n * k // 16
    copies = [flin] + [host1.upload() for _ in range(max(1, COLD_BYTES // wbytes))]
    flin.quantize(fk, fws, xf, k, 1)
    at = [0]

    def gemv1():
        copies[at[0] % len(copies)].gemm(fk, fws, yf, n, 1)
        at[0] += 1

    us = ev.loop_us(stream, gemv1, 4 * len(copies))

    def gemv1_on(s):
        copies[at[0] % len(copies)].gemm(fk, fws, yf, n, 1, stream=s)
        at[0] += 1

    at[0] = 0
    from ferrite_amd import _lib
    us_graph = graph_us(_lib.lib(), _lib.check, ev, gemv1_on, 2 * len(copies))
    res["nvfp4_5120x17408_m1"] = {"gemv_us": round(us, 2), "GB/s": round(wbytes / us / 1e3, 1),
                                  "frac_hbm_peak": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                  # (the same launches replayed from a graph: the launch period without the eager loop's gaps)
                                  "graph_replay_us": round(us_graph, 2),
                                  "graph_replay_frac_hbm_peak": round(wbytes / us_graph / 1e3 / HBM_PEAK_GBS, 4),
                                  "weight_copies_cycled": len(copies)}
    del copies, flin, yf, host1
    # the layer's other prefill shape, down (17408 x 5120): the same two GEMMs
    kd, nd = n, k
    flops_d = 2.0 * m * nd * kd
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
                               "frac_mfma_peak": round(flops_d / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                               "schedule": "stream-K (160 tiles on %d CUs)" % exl3.cu_count()}
    # the same launch on the one-piece schedule (tiles cut three ways along K, partials added by a reduce kernel)
    fk.set_option("gemm_sk", 0)
    res["nvfp4_17408x5120"]["one_piece_schedule_ms"] = round(timed(lambda: flin_d.gemm(fk, fws_d, y, nd, m)), 4)
    fk.set_option("gemm_sk", 1)
    del flin_d, fws_d, x, y
    # the two neighbours of that GEMM in the prompt path: the fused gate|up front (SwiGLU + NVFP4 re-quantization in the
    # epilogue, 2 x 17408 output columns) and an FP8 linear of the same shape
    gate, up = synth.fp4_linear(n, k, SEED, name="gate"), synth.fp4_linear(n, k, SEED + 1, name="up")
    pair = fp4.HostLinear.fuse([("gate", gate.codes, gate.sf, 1.0, 1.0), ("up", up.codes, up.sf, 1.0, 1.0)]).into_swiglu().upload()
    del gate, up
    act = fp4.Workspace(m, n)
    ms = timed(lambda: pair.forward_swiglu(fk, fws, act, xf, k, m, 1.0), 5)
    res["nvfp4_swiglu_front_5120x34816"] = {"quant_plus_gemm_ms": round(ms, 4), "TFLOP/s": round(2 * flops / ms / 1e9, 1),
                                            "frac_mfma_peak": round(2 * flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del pair, act
    f8 = synth.fp8_linear(n, k, SEED).upload()
    y8 = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    f8.forward(fk, fws, y8, n, xf, k, m)
    ms = timed(lambda: f8.gemm(fk, fws, y8, n, m), 5)
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
    for rows in (1, 8):
        at = [0]

        def gv():
            bf16.gemv(bk, yb, n, xf, k, ws_b[at[0] % 3], rows)
            at[0] += 1

        us = ev.loop_us(stream, gv, 30)
        res[f"bf16_5120x17408_m{rows}"] = {"gemv_us": round(us, 2), "GB/s": round(2.0 * n * k / us / 1e3, 1),
                                          "frac_hbm_peak": round(2.0 * n * k / us / 1e3 / HBM_PEAK_GBS, 4)}
    # every GEMM against what the matrix units sustain alone on operands that toggle like its own
    for name, e in res.items():
        if isinstance(e, dict) and "TFLOP/s" in e and name != "mfma_sustained":
            ceiling = sus8 if name.startswith("fp8") else sus16_5 if name.startswith("nvfp4") else sus16
            e["frac_of_mfma_sustained"] = round(e["TFLOP/s"] / ceiling, 4)
    return res


if __name__ == "__main__":
    main()
