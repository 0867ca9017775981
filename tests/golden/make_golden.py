"""Writes tests/golden/path_vectors.npz: small input/output vectors of the path, computed by the CPU oracle.

The reference holds no golden files for this path (its checks compute both sides at run time), so these vectors do not
pin the oracle against the reference: the closed-form and brute-force tests of tests/test_oracle_*.py do that. They pin
the oracle and the GPU kernels against change: a later edit of either that alters a bit of these outputs fails
tests/test_oracle_golden.py (CPU) or tests/test_gpu_golden.py (GPU).

    python tests/golden/make_golden.py        # from the repository root; rewrites the file
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from ferrite_amd import synth  # noqa: E402


def vectors():
    out = {}
    # decode_mul1 (cpu.rs:37-43): 256 states spread over the 16-bit range, plus the three known answers
    states = np.concatenate([np.arange(0, 65536, 257, dtype=np.uint32), np.array([0, 1, 0xFFFF], np.uint32)])
    out["mul1_states"] = states
    out["mul1_f16"] = np.array([oracle.decode_mul1(int(s)) for s in states], np.uint16)
    # one EXL3 tensor per bit width, 128 x 128: stored trellis, decoded W_hat (f16 bits; all of it at 4 bits, the first
    # 32 columns otherwise), reconstructed bf16 weights (4 bits), rotated input and the f64 linear of 3 rows
    x = synth.activations(3, 128, 5)
    out["exl3_x_bf16"] = x
    xf = (x.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    for bits in (2, 3, 4, 5, 6, 8):
        t = synth.exl3_tensor(128, 128, bits, 100 + bits)
        o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
        p = f"exl3_b{bits}_"
        out[p + "trellis"] = np.ascontiguousarray(t.trellis).view(np.uint32).reshape(-1)
        out[p + "suh"], out[p + "svh"] = np.asarray(t.suh, np.uint16), np.asarray(t.svh, np.uint16)
        out[p + "w_hat_f16"] = oracle.w_hat_f16(o) if bits == 4 else np.ascontiguousarray(oracle.w_hat_f16(o)[:, :32])
        if bits == 4:
            out[p + "weight_bf16"] = oracle.weight_bf16(o)
        out[p + "linear_f64"] = oracle.linear_f64(o, xf)
        out[p + "xh_f16"] = oracle.rotate_input_ref(o, xf)
    # NVFP4 quantizer (format.rs:72-90) and the f64 GEMM over quantized operands (format.rs:151-181)
    a = synth.activations(4, 256, 6)
    out["fp4_x_bf16"] = a
    for g in (1.0, 0.037, 2.5):
        codes, sf = oracle.quant_fp4(a, g)
        out[f"fp4_codes_g{g}"], out[f"fp4_sf_g{g}"] = codes, sf
    host = synth.fp4_linear(128, 256, 7)
    out["fp4_w_codes"], out["fp4_w_sf"], out["fp4_alpha"] = host.codes, host.sf, host.alpha
    codes, sf = oracle.quant_fp4(a, host.g)
    out["fp4_g"] = np.float32(host.g)
    out["fp4_ref_gemm"] = oracle.ref_gemm(oracle.dequant_fp4(codes, sf), oracle.dequant_fp4(host.codes, host.sf)) * host.alpha[None, :]
    # plain bf16 linear (gemm.rs:128-167) with and without the residual
    rng = np.random.default_rng(8)
    bits16 = lambda v: ((np.ascontiguousarray(v, np.float32).view(np.uint32) + 0x7FFF + ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)
    xb, wb, rb = bits16(rng.normal(size=(5, 256))), bits16(rng.normal(size=(64, 256)) / 16), bits16(rng.normal(size=(5, 64)))
    out["bf16_x"], out["bf16_w"], out["bf16_res"] = xb, wb, rb
    out["bf16_y"], out["bf16_acc"] = oracle.bf16_linear_ref(xb, wb)
    out["bf16_y_res"] = oracle.bf16_linear_ref(xb, wb, rb)[0]
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "path_vectors.npz")
    np.savez_compressed(path, **vectors())
    print(path, os.path.getsize(path), "bytes")
