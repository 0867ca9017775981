"""Seeded synthetic layers of the benchmark configurations: EXL3 tensors with uniform random trellis words and
fp16 sign-scale vectors sign * N(1, 0.05); NVFP4 linears with codes uniform over the 16 values and e4m3 block scales
|N(0,1)| * 0.1 clamped to the e4m3 range; bf16 activations N(0,1), optionally with 1% outlier channels scaled x20.
Every trellis bit pattern is a valid code stream, so random words are a legitimate tensor."""
from __future__ import annotations

import numpy as np

from .exl3 import Exl3Tensor
from .fp4 import HostLinear


def _bf16_bits(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bits, round to nearest even."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def exl3_tensor(k: int, n: int, bits: int, seed: int, name: str = "synthetic") -> Exl3Tensor:
    rng = np.random.default_rng([seed, k, n, bits])
    words = k // 16 * (n // 16) * 8 * bits
    trellis = rng.integers(0, 1 << 32, size=words, dtype=np.uint64).astype(np.uint32)
    suh = (rng.choice([-1.0, 1.0], size=k) * rng.normal(1.0, 0.05, size=k)).astype(np.float16).view(np.uint16)
    svh = (rng.choice([-1.0, 1.0], size=n) * rng.normal(1.0, 0.05, size=n)).astype(np.float16).view(np.uint16)
    return Exl3Tensor(name, k, n, bits, trellis, suh, svh)


def activations(m: int, k: int, seed: int, outliers: bool = False) -> np.ndarray:
    """bf16 bits [m][k], N(0,1); outliers: 1% of the channels scaled by 20."""
    rng = np.random.default_rng([seed, m, k, 7])
    x = rng.normal(size=(m, k)).astype(np.float32)
    if outliers:
        ch = rng.choice(k, size=max(1, k // 100), replace=False)
        x[:, ch] *= 20.0
    return _bf16_bits(x)


def e4m3_from_f32(v: np.ndarray) -> np.ndarray:
    """Positive f32 -> e4m3 codes, round to nearest even, saturating at 448 (vectorised)."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    out = np.empty(v.shape, np.uint8)
    sub = v < 2.0 ** -6
    out[sub] = np.rint(v[sub] * 512.0).astype(np.uint8)
    b = v[~sub].view(np.uint32).astype(np.uint64)
    b = b + 0x7FFFF + ((b >> 20) & 1)
    c = (((b >> 23) - 120) << 3) | ((b >> 20) & 7)
    out[~sub] = np.minimum(c, 0x7E).astype(np.uint8)
    out[v >= 448.0] = 0x7E
    return out


def fp4_linear(n: int, k: int, seed: int, input_scale: float = 1.0, name: str = "synthetic") -> HostLinear:
    """Codes uniform over the 16 e2m1 values, block scales e4m3(clamp(|N(0,1)| * 0.1, 2^-9, 448)), weight_scale_2 = 1.
    input_scale is pinned by the caller (1.0: alpha = 1, g = 1)."""
    rng = np.random.default_rng([seed, n, k, 4])
    codes = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    s = np.clip(np.abs(rng.normal(size=(n, k // 16))).astype(np.float32) * np.float32(0.1), 2.0 ** -9, 448.0)
    return HostLinear.fuse([(name, codes, e4m3_from_f32(s), 1.0, input_scale)])


def fp8_linear(n: int, k: int, seed: int, input_scale: float = 1.0, weight_scale: float = 1.0, name: str = "synthetic") -> HostLinear:
    """e4m3 codes of N(0, 1) weights scaled into the format's range, one weight scale for the tensor."""
    rng = np.random.default_rng([seed, n, k, 8])
    w = rng.normal(size=(n, k)).astype(np.float32) * np.float32(32.0)
    codes = e4m3_from_f32(np.abs(w)) | (np.signbit(w).astype(np.uint8) << 7)
    return HostLinear.fuse_fp8([(name, codes.astype(np.uint8), weight_scale, input_scale)])
