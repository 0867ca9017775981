"""The oracle's fp16/bf16 helpers against the reference's own unit tests (crates/fe-exl3/src/half.rs:104-123) and
against numpy's/torch's IEEE conversions, which are independent implementations of the same roundings."""
import numpy as np
import torch


def test_f16_roundtrip_all(oracle):
    # half.rs:105-113
    for h in range(0x10000):
        if (h >> 10) & 0x1F == 31:
            continue
        assert oracle.f64_to_f16(oracle.f16_to_f64(h)) == h, hex(h)


def test_f16_ties_to_even(oracle):
    # half.rs:116-123
    assert oracle.f64_to_f16(1.0 + 2.0 ** -11) == 0x3C00
    assert oracle.f64_to_f16(1.0 + 3.0 * 2.0 ** -11) == 0x3C02
    assert oracle.f64_to_f16(2.0 ** -25) == 0
    assert oracle.f64_to_f16(3.0 * 2.0 ** -25) == 2


def test_f16_to_f64_matches_numpy(oracle):
    codes = np.arange(0x10000, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float64)
    for h in range(0, 0x10000, 7):
        got = oracle.f16_to_f64(h)
        w = want[h]
        assert (np.isnan(got) and np.isnan(w)) or got == w, hex(h)


def test_f64_to_f16_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.normal(size=4000) * 10.0 ** rng.integers(-9, 6, size=4000),
        # exact midpoints between neighbouring fp16 values (normal and subnormal) and their neighbours
        np.array([(a.astype(np.float64) + b.astype(np.float64)) / 2
                  for a, b in zip(np.arange(0, 0x7BFF, 37, dtype=np.uint16).view(np.float16),
                                  np.arange(1, 0x7C00, 37, dtype=np.uint16).view(np.float16))]),
        np.array([65504.0, 65519.9, 65520.0, 65536.0, 1e10, -1e10, 0.0, -0.0, 2.0 ** -24, 2.0 ** -25 * 1.0000001]),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert oracle.f64_to_f16(float(x)) == int(w), x
    assert oracle.f64_to_f16(float("nan")) == 0x7E00


def test_f16_fma_single_rounding(oracle):
    # a*b+c evaluated exactly (python fractions) then rounded once by numpy
    from fractions import Fraction
    rng = np.random.default_rng(2)
    for _ in range(3000):
        a, b, c = (int(v) for v in rng.integers(0, 0x7C00, size=3))
        a |= int(rng.integers(0, 2)) << 15
        c |= int(rng.integers(0, 2)) << 15
        fa, fb, fc = (Fraction(float(np.uint16(v).view(np.float16))) for v in (a, b, c))
        exact = fa * fb + fc
        # nearest-even rounding of an exact rational to fp16 via float64 is safe when the rational is exactly
        # representable in float64: 22-bit product + aligned 11-bit addend within 2^±30
        if exact != 0 and not (Fraction(2) ** -40 < abs(exact) < Fraction(2) ** 40):
            continue
        f = float(exact)
        if Fraction(f) != exact:
            continue
        with np.errstate(over="ignore"):
            want = int(np.float64(f).astype(np.float16).view(np.uint16))
        got = oracle.f16_fma(a, b, c)
        if f == 0.0:
            assert got & 0x7FFF == 0
        else:
            assert got == want, (hex(a), hex(b), hex(c))


def test_bf16_matches_torch(oracle):
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.normal(size=5000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, size=5000),
                         np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for x, w in zip(xs, want):
        assert oracle.f32_to_bf16(x) == int(w), x
        assert oracle.bf16_to_f32(int(w)) == float(torch.tensor([int(w)], dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()[0]) \
            or np.isnan(oracle.bf16_to_f32(int(w)))
    # f64 -> bf16 the torch way: through f32
    ds = rng.normal(size=2000) * 10.0 ** rng.integers(-10, 10, size=2000)
    want = torch.from_numpy(ds).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for d, w in zip(ds, want):
        assert oracle.f64_to_bf16_torch(float(d)) == int(w)
    assert oracle.bf16_ulp_diff(0x3F80, 0x3F82) == 2
    assert oracle.bf16_ulp_diff(0x0001, 0x8001) == 2
