"""Pins the NVFP4/FP8 part of the CPU oracle: the reference's unit tests (crates/fe-fp4/src/format.rs:186-215,
crates/fe-fp4/src/lib.rs:583-589), exhaustive value tables and brute-force nearest-value search in float64."""
import numpy as np
import torch

E2M1_POS = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def e4m3_value(b):
    """OCP FP8 E4M3 (fn): bias 7, no infinities, only S.1111.111 is NaN."""
    s, e, m = b >> 7, (b >> 3) & 15, b & 7
    if e == 15 and m == 7:
        return float("nan")
    v = m / 8 * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
    return -v if s else v


def brute_nearest(table, a):
    """Index of the nearest table value in exact arithmetic; ties to the even index; saturate above."""
    best = None
    for i, v in enumerate(table):
        d = abs(a - v)
        if best is None or d < best[0] or (d == best[0] and i % 2 == 0 and best[1] % 2 == 1):
            best = (d, i)
    return best[1]


def test_e4m3_roundtrip(oracle):
    # format.rs:187-200
    for b in range(256):
        v = oracle.e4m3_to_f32(b)
        if np.isnan(v):
            assert b in (0x7F, 0xFF)
            continue
        assert v == e4m3_value(b)
        assert oracle.e4m3_to_f32(oracle.f32_to_e4m3(v)) == v, hex(b)
    assert oracle.f32_to_e4m3(1000.0) == 0x7E
    assert oracle.e4m3_to_f32(0x7E) == 448.0
    assert oracle.f32_to_e4m3(1.0625) == 0x38
    assert oracle.f32_to_e4m3(float("nan")) == 0x7F
    assert oracle.f32_to_e4m3(-0.0) == 0x80
    assert oracle.f32_to_e4m3(-1000.0) == 0xFE


def test_e4m3_matches_torch_and_brute_force(oracle):
    table = [e4m3_value(b) for b in range(127)]
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        np.abs(rng.normal(size=3000)).astype(np.float32) * np.float32(2.0) ** rng.integers(-12, 9, size=3000),
        np.array([(table[i] + table[i + 1]) / 2 for i in range(126)], np.float32),  # every tie
        np.array([448.0, 449.0, 464.0, 465.0, 1e9, 2.0 ** -10, 2.0 ** -11, 0.0], np.float32),
    ])
    for x in xs:
        want = brute_nearest(table, float(x))
        assert oracle.f32_to_e4m3(x) == want, x
        assert oracle.f32_to_e4m3(-x) == (want | 0x80)
    if hasattr(torch, "float8_e4m3fn"):
        ok = xs[xs <= 448.0]  # torch does not saturate above the range
        tw = torch.from_numpy(ok).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        got = np.array([oracle.f32_to_e4m3(x) for x in ok], np.uint8)
        assert np.array_equal(got, tw)


def test_e2m1_rounding(oracle):
    # format.rs:202-209
    assert oracle.f32_to_e2m1(0.25) == 0
    assert oracle.f32_to_e2m1(0.75) == 2
    assert oracle.f32_to_e2m1(2.5) == 4
    assert oracle.f32_to_e2m1(5.0) == 6
    assert oracle.f32_to_e2m1(7.0) == 7
    assert oracle.f32_to_e2m1(-3.2) == (8 | 5)
    assert list(oracle.E2M1[:8]) == E2M1_POS and list(oracle.E2M1[8:]) == [-v for v in E2M1_POS]
    rng = np.random.default_rng(1)
    for x in np.concatenate([rng.uniform(0, 8, size=2000), np.arange(0, 7, 0.125)]).astype(np.float32):
        want = brute_nearest(E2M1_POS, float(x))
        assert oracle.f32_to_e2m1(x) == want, x
        assert oracle.f32_to_e2m1(-x) == (want | 8)


def test_tiling_roundtrip(oracle):
    # format.rs:210-215
    rows, kb = 200, 24
    src = (np.arange(rows * kb) * 7 % 251).astype(np.uint8)
    tiled = oracle.tile_scales(src, rows, kb)
    assert tiled.size == 256 * kb
    assert np.array_equal(oracle.untile_scales(tiled, rows, kb), src)
    # layout: [rows/128][kb/8][128][8]
    t4 = tiled.reshape(2, kb // 8, 128, 8)
    s2 = src.reshape(rows, kb)
    for r, b in [(0, 0), (5, 9), (127, 23), (128, 0), (199, 17)]:
        assert t4[r // 128, b // 8, r % 128, b % 8] == s2[r, b]
        assert oracle.tiled_offset(r, b, kb) == ((r // 128) * (kb // 8) + b // 8) * 1024 + (r % 128) * 8 + b % 8
    assert t4[1, :, 72:, :].sum() == 0


def test_select_rows_and_cols(oracle):
    # lib.rs:583-589
    src = np.arange(40, dtype=np.uint8)
    assert list(oracle.select(src, 8, [(0, 1), (3, 5)], 2, 6)) == [2, 3, 4, 5, 26, 27, 28, 29, 34, 35, 36, 37]
    assert np.array_equal(oracle.select(src, 8, [(0, 5)], 0, 8), src)


def test_swiglu_perm_interleaves_by_eight(oracle):
    inter = 64
    got = [oracle.swiglu_perm(r, inter) for r in range(2 * inter)]
    assert sorted(got) == list(range(2 * inter))
    assert got[:16] == list(range(8)) + list(range(inter, inter + 8))
    assert got[16:24] == list(range(8, 16))


def bf16_bits(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_quant_fp4_row_against_first_principles(oracle):
    rng = np.random.default_rng(5)
    k = 256
    e4 = [e4m3_value(b) for b in range(127)]
    for g in (1.0, 0.37, 12.5):
        x = rng.normal(size=k).astype(np.float32) * np.float32(3.0)
        x[5] *= 20
        x[32:48] = 0.0  # an all-zero block: scale 0, codes 0
        xb = bf16_bits(x)
        xf = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).float().numpy()
        codes, sf = oracle.quant_fp4_row(xb, g)
        g32 = np.float32(g)
        for b in range(k // 16):
            blk = xf[b * 16:(b + 1) * 16]
            amax = np.float32(np.abs(blk).max())
            t = np.float32(np.float32(amax * np.float32(1.0 / 6.0)) * g32)
            s8 = brute_nearest(e4, float(t))
            assert sf[b] == s8
            sv = np.float32(e4[s8])
            mul = np.float32(g32 / sv) if sv > 0 else np.float32(0)
            for j in range(16):
                q = np.float32(blk[j] * mul)
                want = brute_nearest(E2M1_POS, abs(float(q))) | (8 if np.signbit(q) else 0)
                c = codes[b * 8 + j // 2]
                got = (c & 15) if j % 2 == 0 else (c >> 4)
                assert got == want, (g, b, j)
        assert sf[2] == 0 and not codes[16:24].any()
        # dequantised block reproduces x*g to e2m1 precision: |err| <= half an e2m1 step (1.0 at the top) * scale
        deq = oracle.dequant_fp4_row(codes, sf, 1.0)
        scale = np.repeat(np.array([e4[s] for s in sf], np.float32), 16)
        assert np.all(np.abs(deq - xf * g32) <= 1.0 * scale + 1e-6)


def test_dequant_and_ref_gemm(oracle):
    rng = np.random.default_rng(6)
    n, k, m = 24, 128, 3
    wc = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    ws = rng.integers(0x20, 0x48, size=(n, k // 16), dtype=np.uint8)
    ac = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    asf = rng.integers(0x20, 0x48, size=(m, k // 16), dtype=np.uint8)
    wf = oracle.dequant_fp4(wc, ws, 1.0)
    af = oracle.dequant_fp4(ac, asf, 0.5)
    # element 2i in the low nibble (format.rs:85, 139)
    lut = np.array(E2M1_POS + [-v for v in E2M1_POS])
    nib = np.stack([wc & 15, wc >> 4], axis=-1).reshape(n, k)
    want = lut[nib] * np.repeat(np.array([[e4m3_value(int(b)) for b in row] for row in ws]), 16, axis=1)
    assert np.array_equal(wf.astype(np.float64), want)  # products have <= 6 significant bits: exact
    assert np.array_equal(oracle.dequant_fp4(ac, asf, 1.0) * np.float32(0.5), af)
    y = oracle.ref_gemm(af, wf, threads=3)
    want_y = (af.astype(np.float64) @ wf.astype(np.float64).T).astype(np.float32)
    assert np.array_equal(y, want_y) or np.allclose(y, want_y, rtol=1e-6, atol=0)
    assert y.shape == (m, n)
    # a transposed operand would fail: n != k and rows distinct
    assert not np.allclose(y, (af.astype(np.float64)[:, ::-1] @ wf.astype(np.float64).T).astype(np.float32))


def test_fp8_row(oracle):
    x = bf16_bits(np.array([0.0, 1.0, -1.0625, 500.0, -0.001, 3.3], np.float32))
    q = oracle.quant_fp8_row(x, 2.0)
    assert list(q) == [oracle.f32_to_e4m3(v) for v in (0.0, 2.0, -2.125, 1000.0, float(np.float32(-0.001).astype(np.float32)) * 0 + oracle.bf16_to_f32(int(x[4])) * 2.0, oracle.bf16_to_f32(int(x[5])) * 2.0)]
    d = oracle.dequant_fp8_row(q, 0.5)
    assert d[1] == 1.0 and d[3] == 224.0
