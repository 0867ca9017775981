"""Pins the EXL3 part of the CPU oracle without importing the reference: its own unit tests
(crates/fe-exl3/src/format.rs:170-202), closed forms, brute force and explicit dense-matrix algebra."""
import numpy as np
import pytest

MUL1 = 0x83DCD12D


def synthetic(oracle, k, n, bits):
    """The reference's test generator, format.rs:162-168."""
    tw = 8 * bits
    cnt = k // 16 * (n // 16) * tw
    trellis = (np.arange(cnt, dtype=np.uint64) * 2654435761 & 0xFFFFFFFF).astype(np.uint32)
    suh = (0x3C00 | (np.arange(k) & 0x3FF)).astype(np.uint16)
    svh = (0xBC00 | (np.arange(n) & 0x3FF)).astype(np.uint16)
    return oracle.Exl3(k, n, bits, trellis, suh, svh)


def random_tensor(oracle, k, n, bits, seed):
    rng = np.random.default_rng(seed)
    trellis = rng.integers(0, 2 ** 32, size=k // 16 * (n // 16) * 8 * bits, dtype=np.uint64).astype(np.uint32)
    suh = (rng.choice([-1.0, 1.0], size=k) * rng.normal(1.0, 0.05, size=k)).astype(np.float16).view(np.uint16)
    svh = (rng.choice([-1.0, 1.0], size=n) * rng.normal(1.0, 0.05, size=n)).astype(np.float16).view(np.uint16)
    return oracle.Exl3(k, n, bits, trellis, suh, svh)


def f16(a):
    return np.asarray(a, np.uint16).view(np.float16).astype(np.float64)


def hadamard128():
    i = np.arange(128)
    pc = np.vectorize(lambda v: bin(v).count("1"))(i[:, None] & i[None, :])
    return np.where(pc % 2 == 0, 1.0, -1.0)


# ---- format.rs unit tests ------------------------------------------------------------------------------------
def test_slices_keep_tiles(oracle):
    t = synthetic(oracle, 256, 512, 3)
    c = oracle.slice_cols(t, [(128, 256), (384, 512)])
    assert (c.k, c.n) == (256, 256)
    for kt in range(16):
        assert np.array_equal(c.tile(kt, 0), t.tile(kt, 8))
        assert np.array_equal(c.tile(kt, 8), t.tile(kt, 24))
    assert np.array_equal(c.svh[:128], t.svh[128:256])
    r = oracle.slice_rows(t, 128, 256)
    assert (r.k, r.n) == (128, 512)
    assert np.array_equal(r.tile(0, 5), t.tile(8, 5))
    assert np.array_equal(r.suh, t.suh[128:256])
    with pytest.raises(ValueError):
        oracle.slice_cols(t, [(0, 100)])
    with pytest.raises(ValueError):
        oracle.slice_rows(t, 64, 128)


def test_strips_layout(oracle):
    t = synthetic(oracle, 256, 256, 2)
    s = oracle.strips(t)
    tw = t.tw
    for b in range(2):
        for kt in range(16):
            for j in range(8):
                at = ((b * 16 + kt) * 8 + j) * tw
                assert np.array_equal(s[at:at + tw], t.tile(kt, 8 * b + j))


# ---- fragment order -----------------------------------------------------------------------------------------
def test_value_map_is_the_b_fragment(oracle):
    seen = set()
    for lane in range(32):
        g, t4 = lane // 4, lane % 4
        for j in range(8):
            r, c = oracle.value_row(lane, j), oracle.value_col(lane, j)
            seen.add((r, c))
            # two m16n8k16 B fragments per tile (columns 0-7, then 8-15); inside one, b0 = (k 2t, 2t+1; col g),
            # b1 = (k 2t+8, 2t+9; col g)  (kernels/kcommon/src/mma.rs:3-8)
            frag, reg, half = j // 4, (j // 2) % 2, j % 2
            assert r == 2 * t4 + half + 8 * reg
            assert c == g + 8 * frag
    assert len(seen) == 256


# ---- tile_state ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", range(1, 9))
def test_tile_state_three_formulations_agree(oracle, bits):
    rng = np.random.default_rng(bits)
    for _ in range(3):
        tile = rng.integers(0, 2 ** 32, size=8 * bits, dtype=np.uint64).astype(np.uint32)
        for t in range(256):
            a = oracle.tile_state(tile, bits, t, "bits")
            assert a == oracle.tile_state(tile, bits, t, "funnel"), (bits, t)
            if 2 <= bits <= 5:  # the GEMV kernels exist for 2..5 bits (gemv.rs:875-878)
                assert a == oracle.tile_state(tile, bits, t, "lane"), (bits, t)


@pytest.mark.parametrize("bits", range(1, 9))
def test_tile_state_recovers_a_written_stream(oracle, bits):
    """Build the bit stream from its definition: position t contributes `bits` new bits, and the state is the last
    16 stream bits up to and including them (cyclic)."""
    rng = np.random.default_rng(100 + bits)
    sym = rng.integers(0, 2 ** bits, size=256)
    stream = np.zeros(256 * bits, np.uint8)
    for t in range(256):
        for b in range(bits):
            stream[t * bits + b] = (sym[t] >> (bits - 1 - b)) & 1
    words = np.zeros(8 * bits, np.uint32)
    for p, bit in enumerate(stream):
        words[p // 32] |= np.uint32(int(bit) << (31 - p % 32))
    for t in range(256):
        end = (t + 1) * bits
        want = 0
        for p in range(end - 16, end):
            want = (want << 1) | int(stream[p % (256 * bits)])
        assert oracle.tile_state(words, bits, t) == want


# ---- the mul1 codebook --------------------------------------------------------------------------------------
def test_decode_mul1_all_states(oracle):
    states = np.arange(65536, dtype=np.uint64)
    x = (states * MUL1) & 0xFFFFFFFF
    s = (x & 0xFF) + ((x >> 8) & 0xFF) + ((x >> 16) & 0xFF) + (x >> 24)
    c1 = float(np.uint16(0x1EEE).view(np.float16))
    c2 = float(np.uint16(0xC931).view(np.float16))
    assert c1 == 0.00676727294921875 and c2 == -10.3828125
    # (1024 + s) * c1 + c2 is exact in float64 (11-bit x 11-bit product, aligned addend); one rounding to fp16
    want = ((1024.0 + s.astype(np.float64)) * c1 + c2).astype(np.float16).view(np.uint16)
    got = np.array([oracle.decode_mul1(int(v)) for v in states], np.uint16)
    assert np.array_equal(got, want)
    # known answers (byte sums by hand: 1 * MUL1 = 0x83DCD12D -> 0x83+0xDC+0xD1+0x2D = 605)
    assert oracle.decode_mul1(0) == 0xC2E8 and float(np.uint16(0xC2E8).view(np.float16)) == -3.453125
    assert int(s[1]) == 605 and oracle.decode_mul1(1) == 0x3921
    assert int(s[0xFFFF]) == 414 and oracle.decode_mul1(0xFFFF) == 0xB936
    assert int(s.max()) <= 1020


def test_decode_tile_places_values(oracle):
    rng = np.random.default_rng(7)
    for bits in (2, 3, 4, 5, 6, 8):
        tile = rng.integers(0, 2 ** 32, size=8 * bits, dtype=np.uint64).astype(np.uint32)
        d = oracle.decode_tile(tile, bits)
        for lane in range(32):
            for j in range(8):
                v = oracle.decode_mul1(oracle.tile_state(tile, bits, 8 * lane + j))
                assert d[oracle.value_row(lane, j), oracle.value_col(lane, j)] == v


def test_w_hat_f16_is_tiles_side_by_side(oracle):
    t = random_tensor(oracle, 128, 256, 3, 11)
    w = oracle.w_hat_f16(t)
    for kt in range(8):
        for nt in range(16):
            assert np.array_equal(w[kt * 16:(kt + 1) * 16, nt * 16:(nt + 1) * 16], oracle.decode_tile(t.tile(kt, nt), 3))
    part = oracle.w_hat_f16(t, 128, 64)
    assert np.array_equal(part, w[:, 128:192])


# ---- Hadamard -----------------------------------------------------------------------------------------------
def test_fwht128_is_sylvester(oracle):
    H = hadamard128()
    assert np.array_equal(H @ H, 128.0 * np.eye(128))
    rng = np.random.default_rng(5)
    for i in (0, 1, 5, 64, 127):
        e = np.zeros(128)
        e[i] = 1.0
        assert np.array_equal(oracle.fwht128(e), H[:, i])
    v = rng.integers(-50, 50, size=128).astype(np.float64)
    assert np.array_equal(oracle.fwht128(v), H @ v)  # exact for small integers
    assert np.array_equal(oracle.fwht128(oracle.fwht128(v)), 128.0 * v)


# ---- dense-matrix algebra on small shapes -------------------------------------------------------------------
def dense_weight(oracle, t):
    """W = diag(suh) . Hk . W_hat . Hn . diag(svh) / 128 with explicit block-diagonal Hadamards."""
    H = hadamard128()
    Hk = np.kron(np.eye(t.k // 128), H)
    Hn = np.kron(np.eye(t.n // 128), H)
    what = f16(oracle.w_hat_f16(t))
    return (f16(t.suh)[:, None] * (Hk @ what @ Hn) * f16(t.svh)[None, :]) / 128.0


@pytest.mark.parametrize("k,n,bits", [(128, 128, 4), (256, 128, 3), (128, 256, 5), (256, 256, 2)])
def test_weight_and_linear_match_dense_algebra(oracle, k, n, bits):
    t = random_tensor(oracle, k, n, bits, 1000 + k + n + bits)
    W = dense_weight(oracle, t)
    for r0 in range(0, k, 128):
        blk = oracle.weight_block_f64(t, r0, 0, n)
        np.testing.assert_allclose(blk, W[r0:r0 + 128], rtol=1e-12, atol=1e-12)
    # bf16 rounding of the f64 weight, both layouts; an ulp of slack only where f64 summation order moves a tie
    import torch
    want = torch.from_numpy(W).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    kn = oracle.weight_bf16(t, layout="KN", threads=2)
    nk = oracle.weight_bf16(t, layout="NK", threads=3)
    assert np.array_equal(nk, kn.T)
    diff = np.array([oracle.bf16_ulp_diff(int(a), int(b)) for a, b in zip(kn.ravel(), want.ravel())])
    assert diff.max() <= 1 and (diff > 0).mean() < 1e-3
    # linear: x @ W, single- and multi-threaded (bit-identical), and a transposed-operand mistake would fail
    rng = np.random.default_rng(3)
    x = rng.normal(size=(3, k))
    y1 = oracle.linear_f64(t, x, threads=1)
    y2 = oracle.linear_f64(t, x, threads=2)
    assert np.array_equal(y1, y2)
    np.testing.assert_allclose(y1, x @ W, rtol=1e-10, atol=1e-10)
    # column sub-range of weight_block_f64
    if n > 128:
        np.testing.assert_array_equal(oracle.weight_block_f64(t, 0, 128, 128), oracle.weight_block_f64(t, 0, 0, n)[:, 128:256])


def test_rotate_input_and_gemv_ref(oracle):
    k, n, bits = 256, 256, 4
    t = random_tensor(oracle, k, n, bits, 77)
    H = hadamard128()
    Hk = np.kron(np.eye(k // 128), H)
    Hn = np.kron(np.eye(n // 128), H)
    rng = np.random.default_rng(9)
    x = rng.normal(size=(5, k)).astype(np.float32).astype(np.float64)
    xh = oracle.rotate_input_ref(t, x)
    exact = ((x * f16(t.suh)[None, :]) @ Hk) / np.sqrt(128.0)
    want = exact.astype(np.float16).view(np.uint16)
    ulp = np.abs(xh.astype(np.int32) - want.astype(np.int32))
    assert ulp.max() <= 1 and (ulp > 0).mean() < 1e-2  # ties only (f64 summation order)
    what = oracle.w_hat_f16(t)
    y = oracle.gemv_ref(t, what, xh)
    want_y = ((f16(xh) @ f16(what)) @ Hn) * f16(t.svh)[None, :] / np.sqrt(128.0)
    np.testing.assert_allclose(y, want_y, rtol=1e-10, atol=1e-10)
    # first-columns form (nc < n, a multiple of 128)
    y2 = oracle.gemv_ref(t, what[:, :128].copy(), xh)
    np.testing.assert_allclose(y2, want_y[:, :128], rtol=1e-10, atol=1e-10)
    # factored form == dense form: gemv_ref on exact-rotated input reproduces linear_f64 up to the fp16 rounding of xh
    ylin = oracle.linear_f64(t, x)
    assert np.abs(y - ylin).max() / np.sqrt((ylin ** 2).mean()) < 5e-3


def test_slices_are_exact_subtensors(oracle):
    """Column slices reproduce the matching output columns, row slices sum to the whole (format.rs:86-88, 112-114)."""
    t = random_tensor(oracle, 256, 384, 3, 21)
    rng = np.random.default_rng(4)
    x = rng.normal(size=(2, 256))
    y = oracle.linear_f64(t, x)
    c = oracle.slice_cols(t, [(0, 128), (256, 384)])
    yc = oracle.linear_f64(c, x)
    assert np.array_equal(yc, np.concatenate([y[:, :128], y[:, 256:]], axis=1))
    r0, r1 = oracle.slice_rows(t, 0, 128), oracle.slice_rows(t, 128, 256)
    ys = oracle.linear_f64(r0, x[:, :128]) + oracle.linear_f64(r1, x[:, 128:])
    np.testing.assert_allclose(ys, y, rtol=1e-12, atol=1e-12)
