"""Ceilings of the MI355X the kernels are judged against, measured by register-only probes through the C ABI: the role of
the reference's crates/fe-fp4/src/bin/fp4-peak.rs (matrix-unit peak) and crates/fe-exl3/src/bin/exl3-probe.rs (issue rate
of the decode's instructions, streaming read roof).

    python -m ferrite_amd.probes mfma      # v_mfma 32x32x16 f16 / bf16, 32x32x64 f8: burst and sustained TFLOP/s, clock, power
    python -m ferrite_amd.probes valu      # issue rate of each vector instruction of the trellis decode
    python -m ferrite_amd.probes decode    # the whole decode of a load step at the GEMV's occupancy, 3 / 4 / 5 bits
    python -m ferrite_amd.probes stream    # streaming read of 1 GB

Every figure is printed as one JSON line per probe, so that a rocprofv3 run of the same command can be laid beside it.
"""
from __future__ import annotations

import json
import subprocess
import sys
import threading
import time


class Smi:
    """Shader clock and board power as `rocm-smi --showclocks --showpower --json` reports them, polled from a thread
    while a probe loops (the tool takes about 50 ms a reading)."""

    def __init__(self):
        self.samples, self._stop, self._t = [], False, None

    def _poll(self):
        while not self._stop:
            try:
                out = subprocess.run(["rocm-smi", "--showclocks", "--showpower", "--json"], capture_output=True, text=True, timeout=5).stdout
                card = next(iter(json.loads(out).values()))
                sclk = next((v for k, v in card.items() if "sclk" in k.lower()), None)
                power = next((v for k, v in card.items() if "power" in k.lower() and "(w)" in k.lower()), None)
                mhz = float(str(sclk).strip("()").lower().replace("mhz", "")) if sclk is not None else None
                self.samples.append((mhz, float(power) if power is not None else None))
            except Exception:  # no tool, no permission, another format: the probe figures stand without it
                return
            time.sleep(0.02)

    def __enter__(self):
        self._t = threading.Thread(target=self._poll, daemon=True)
        self._t.start()
        return self

    def __exit__(self, *a):
        self._stop = True
        self._t.join(timeout=6)

    def summary(self):
        def med(v):
            v = sorted(x for x in v if x is not None)
            return v[len(v) // 2] if v else None
        return {"sclk_MHz_median": med(s[0] for s in self.samples), "power_W_median": med(s[1] for s in self.samples),
                "samples": len(self.samples)}


def mfma_peak(fk, kind: str, grid: int, iters: int = 4096, ramp_s: float = 0.15, timed_s: float = 0.3, smi: bool = True, seed: int = 0):
    """Burst (the first five launches after the host work) and sustained (after ramp_s of the same launches, over
    timed_s) TFLOP/s of the register-only matrix probe, with clock and power during the sustained window. seed 0: operands
    of 0.5 and 1; otherwise random signs and mantissas (what a GEMM on real data feeds the unit)."""
    ms0, burst = fk.mfma_peak(kind, grid, iters, 5, seed)
    fk.mfma_peak(kind, grid, iters, max(1, int(ramp_s * 1e3 / ms0)), seed)
    n = max(1, int(timed_s * 1e3 / ms0))
    if smi:
        with Smi() as s:
            ms, tf = fk.mfma_peak(kind, grid, iters, n, seed)
        extra = s.summary()
    else:
        ms, tf = fk.mfma_peak(kind, grid, iters, n, seed)
        extra = {}
    what = "0.5 and 1" if not seed else "random signs and mantissas" if seed & 1 else "random signs, five random mantissa bits"
    return {"probe": f"mfma_{kind}", "operands": what, "grid": grid, "wavefronts_per_simd": max(1, grid // max(1, fk_cus())), "iters": iters,
            "burst_TFLOPs": round(burst, 1), "sustained_TFLOPs": round(tf, 1), "ms_per_launch": round(ms, 4), **extra}


def fk_cus():
    from . import exl3
    return exl3.cu_count()


def main(argv):
    import torch
    from . import exl3, fp4
    what = argv[1] if len(argv) > 1 else "mfma"
    assert torch.cuda.is_available(), "the probes need the GPU"
    cus = exl3.cu_count()
    if what == "mfma":
        fk = fp4.Kernels.load()
        for kind in ("f16", "bf16", "f8"):
            for seed in (0, 12345, 12346) if kind != "f8" else (0, 12345):
                time.sleep(0.5)  # (each probe from the same idle state)
                print(json.dumps(mfma_peak(fk, kind, cus, seed=seed, timed_s=1.0)), flush=True)
    elif what == "valu":
        kern = exl3.Kernels.load()
        grid, iters = 4 * cus, 4096
        base = None
        for op in exl3.Kernels.PROBE_OPS:
            kern.probe_op(op, grid, iters, 20)
            with Smi() as s:
                ms = kern.probe_op(op, grid, iters, 200)
            ops = grid * 256 * 8 * iters / (ms * 1e-3)
            base = base or ops
            clk = s.summary()["sclk_MHz_median"]
            print(json.dumps({"probe": f"valu_{op}", "Tlane_ops_per_s": round(ops / 1e12, 2), "relative_to_add": round(ops / base, 3),
                              "cycles_per_wave_instruction_per_simd": round(4 * cus * 64 * clk * 1e6 / ops, 2) if clk else None,
                              "sclk_MHz_median": clk}), flush=True)
    elif what == "decode":
        kern = exl3.Kernels.load()
        grid, iters = 4 * cus, 256
        for bits in (3, 4, 5):
            kern.probe_decode(bits, grid, iters, 200)
            ms = kern.probe_decode(bits, grid, iters, 100)
            w = grid * 256 * 32 * iters / (ms * 1e-3)
            print(json.dumps({"probe": f"decode_b{bits}", "Tweights_per_s": round(w / 1e12, 2), "trellis_GBs": round(w * bits / 8 / 1e9, 1),
                              "frac_hbm_peak": round(w * bits / 8 / 8e12, 4)}), flush=True)
    elif what == "stream":
        kern = exl3.Kernels.load()
        buf = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        for grid in (cus, 2 * cus, 4 * cus, 8 * cus):
            kern.probe_stream_read(buf, grid, 3)
            ms = kern.probe_stream_read(buf, grid, 10)
            print(json.dumps({"probe": "stream_read_1GB", "grid": grid, "GBs": round((1 << 30) / (ms * 1e-3) / 1e9, 1)}), flush=True)
    else:
        sys.exit(__doc__)


if __name__ == "__main__":
    main(sys.argv)
