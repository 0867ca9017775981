"""GPU parity of the plain bf16 linear (include/fe_bf16.h; kernels/k-core/src/gemm.rs, crates/fe-model/src/model.rs:310-345)
against the CPU oracle, through the C ABI: the two GEMV forms, the GEMM whole and cut along K, the residual epilogue (exact),
rows and columns past the end untouched, a row's bits independent of the batch, and the rule that routes the rows."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CANARY = 0xC040  # bf16 -3.0


@pytest.fixture(scope="module")
def env():
    import torch
    from ferrite_amd import bf16
    assert torch.cuda.is_available()
    return torch, bf16, bf16.Kernels.load()


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def host_u16(t):
    return t.cpu().numpy().view(np.uint16)


def f32(a):
    return (np.asarray(a, np.uint16).astype(np.uint32) << 16).view(np.float32)


def bits(x):
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def operands(n, k, m, seed, lda=None):
    rng = np.random.default_rng(seed)
    lda = lda or k
    x = bits(rng.normal(size=(m, lda)))
    w = bits(rng.normal(size=(n, k)) / np.sqrt(k))
    return x, w


def close(got_bits, acc):
    """bf16 of an f32-accumulated sum against the f64-accumulated one: half a bf16 step plus the f32 summation error.
    The bar of the path is max relative error 1e-2; this is tighter."""
    got, ref = f32(got_bits).astype(np.float64), acc.astype(np.float64)
    rms = np.sqrt((ref ** 2).mean())
    assert (np.abs(got - ref) <= np.abs(ref) / 256.0 + 1e-4 * rms).all()
    scale = np.abs(ref).max(axis=1, keepdims=True)
    assert (np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2 * scale)).max() < 1e-2


def call(torch, fn, kern, x, w, m, n, ldy=None, res=None, rows_alloc=None, lda=None, **kw):
    """Runs fn into a canary-filled [rows_alloc][ldy] buffer; returns the m x n block, checks the rest is untouched."""
    ldy = ldy or n
    rows_alloc = rows_alloc or m + 2
    y = dev_u16(torch, np.full((rows_alloc, ldy), CANARY, np.uint16))
    fn(kern, y, ldy, x, lda or x.shape[1], w, m, res=res, **kw)
    torch.cuda.synchronize()
    out = host_u16(y)
    assert (out[m:] == CANARY).all() and (out[:, n:] == CANARY).all()
    return out[:m, :n].copy()


@pytest.mark.parametrize("n,k,m", [(256, 512, 1), (1024, 1024, 3), (2048, 5120, 8), (96, 1024, 5), (48, 256, 1),
                                   (520, 768, 2), (1032, 2048, 7), (512, 512, 4), (528, 512, 6)])
def test_gemv(env, oracle, n, k, m):
    torch, bf16, kern = env
    xb, wb = operands(n, k, m, 7 + n)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)
    got = call(torch, bf16.gemv, kern, x, w, m, n, ldy=n + 12)
    want, acc = oracle.bf16_linear_ref(xb, wb)
    close(got, acc)
    assert (got != want).mean() < 0.02  # a different bf16 only where the f32 and f64 sums straddle a rounding boundary
    # a row's bits do not depend on the rows around it
    for r in {0, m - 1}:
        alone = call(torch, bf16.gemv, kern, x[r:r + 1].contiguous(), w, 1, n)
        assert np.array_equal(alone[0], got[r])
    # nor on how many columns a program takes (the "nc" option overrides the library's choice)
    for nc in (1, 2, 4, 8):
        kern.set_option("nc", nc)
        assert np.array_equal(call(torch, bf16.gemv, kern, x, w, m, n), got), nc
    kern.set_option("nc", -1)
    # residual: bf16(bf16(sum) + res), exact given the sums
    rb = bits(np.random.default_rng(3).normal(size=(m + 2, n)))
    with_res = call(torch, bf16.gemv, kern, x, w, m, n, res=dev_u16(torch, rb))
    assert np.array_equal(with_res, bits(f32(got) + f32(rb[:m])))


@pytest.mark.parametrize("n,k,m,lda", [(256, 512, 200, 512), (520, 768, 300, 776), (1024, 1024, 700, 1024), (96, 256, 33, 256),
                                       (768, 2048, 1, 2048)])
def test_gemm_whole_and_cut(env, oracle, n, k, m, lda):
    torch, bf16, kern = env
    xb, wb = operands(n, k, m, 11 + n, lda=lda)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)

    def run(res=None):
        return call(torch, bf16.gemm, kern, x, w, m, n, ldy=n + 8, res=res, lda=lda)

    cut = run()
    assert np.array_equal(cut, run())  # deterministic
    kern.set_option("gemm_splits", 1)
    whole = run()
    kern.set_option("gemm_splits", 8)
    want, acc = oracle.bf16_linear_ref(xb[:, :k], wb)
    close(cut, acc)
    close(whole, acc)
    rb = bits(np.random.default_rng(4).normal(size=(m + 2, n + 8)))
    got = run(res=dev_u16(torch, rb))
    assert np.array_equal(got, bits(f32(cut) + f32(rb[:m, :n])))
    # in place: res == y
    y = dev_u16(torch, rb)
    bf16.gemm(kern, y, n + 8, x, lda, w, m, res=y)
    torch.cuda.synchronize()
    out = host_u16(y)
    assert np.array_equal(out[:m, :n], got) and np.array_equal(out[m:], rb[m:]) and np.array_equal(out[:, n:], rb[:, n:])


def test_forward_routes_rows_as_the_reference(env, oracle):
    """Batches of up to 16 rows: every row through the GEMV in passes of 8; larger ones: the leading `dec` rows through
    the GEMV, the others through the GEMM (model.rs:310-345)."""
    torch, bf16, kern = env
    n, k = 640, 1024
    xb, wb = operands(n, k, 40, 5)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)

    def gemv_rows(r0, r1):
        out = [call(torch, bf16.gemv, kern, x[r:r + 8].contiguous(), w, min(8, r1 - r), n) for r in range(r0, r1, 8)]
        return np.concatenate(out)

    small = call(torch, bf16.forward, kern, x, w, 12, n)
    assert np.array_equal(small, gemv_rows(0, 12))
    mixed = call(torch, bf16.forward, kern, x, w, 40, n, dec=10)
    assert np.array_equal(mixed[:10], gemv_rows(0, 10))
    assert np.array_equal(mixed[10:], call(torch, bf16.gemm, kern, x[10:].contiguous(), w, 30, n))
    prompt = call(torch, bf16.forward, kern, x, w, 40, n, dec=0)
    assert np.array_equal(prompt, call(torch, bf16.gemm, kern, x, w, 40, n))
    # k % 256 != 0: no GEMV (model.rs:314)
    xb2, wb2 = operands(n, 320, 4, 6)
    x2, w2 = dev_u16(torch, xb2), dev_u16(torch, wb2)
    assert np.array_equal(call(torch, bf16.forward, kern, x2, w2, 4, n), call(torch, bf16.gemm, kern, x2, w2, 4, n))
    close(mixed, oracle.bf16_linear_ref(xb, wb)[1])


def test_route_linear_with_bf16_weights_only(env):
    torch, bf16, kern = env
    from ferrite_amd import route, _lib
    n, k, m = 384, 512, 24
    xb, wb = operands(n, k, m, 8)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)
    ctx = route.LinCtx()
    lin = route.Linear("plain", n, k, w=w.view(torch.bfloat16))
    y = dev_u16(torch, np.full((m, n), CANARY, np.uint16))
    with pytest.raises(_lib.FeError):
        lin.forward(ctx, y, n, x, k, m)  # no bf16 kernels in the context
    ctx.set_bf16(kern)
    ctx.dec = 5
    lin.forward(ctx, y, n, x, k, m)
    torch.cuda.synchronize()
    assert np.array_equal(host_u16(y), call(torch, bf16.forward, kern, x, w, m, n, dec=5))


def test_gemm_swiglu_over_interleaved_weights(env, oracle):
    """fe_interleave_gu + fe_gemm_swiglu (gemm.rs:264-296): the bits of the plain GEMM over the same interleaved weights
    followed by fe_silu_mul; against the oracle's sums and the exact formula within the bf16 steps of the two roundings."""
    torch, bf16, kern = env
    from ferrite_amd import route
    for inter, k, m in ((640, 512, 300), (136, 256, 40), (2048, 1024, 700)):
        rng = np.random.default_rng(inter)
        xb = bits(rng.normal(size=(m, k)))
        gb, ub = bits(rng.normal(size=(inter, k)) / np.sqrt(k) * 2), bits(rng.normal(size=(inter, k)) / np.sqrt(k) * 2)
        x, g, u = dev_u16(torch, xb), dev_u16(torch, gb), dev_u16(torch, ub)
        w = bf16.interleave_gu(kern, g, u)
        torch.cuda.synchronize()
        want_w = np.empty((2 * inter, k), np.uint16)
        r = np.arange(2 * inter)
        b, i = r // 16, r % 16
        want_w[i < 8] = gb[(b * 8 + i)[i < 8]]
        want_w[i >= 8] = ub[(b * 8 + i - 8)[i >= 8]]
        assert np.array_equal(host_u16(w), want_w)
        act = dev_u16(torch, np.full((m + 1, inter), CANARY, np.uint16))
        bf16.gemm_swiglu(kern, act, x, k, w, m)
        torch.cuda.synchronize()
        got = host_u16(act)
        assert (got[m:] == CANARY).all()
        # the plain GEMM over the interleaved weights, then fe_silu_mul on its gate and up columns
        y = call(torch, bf16.gemm, kern, x, w, m, 2 * inter)
        yb = y.reshape(m, inter // 8, 2, 8)
        gate, up = np.ascontiguousarray(yb[:, :, 0].reshape(m, inter)), np.ascontiguousarray(yb[:, :, 1].reshape(m, inter))
        gd, ud = dev_u16(torch, gate), dev_u16(torch, up)
        out = dev_u16(torch, np.zeros((m, inter), np.uint16))
        route.silu_mul(out, gd.data_ptr(), ud.data_ptr(), inter, inter, m)
        torch.cuda.synchronize()
        assert np.array_equal(got[:m], host_u16(out))
        # the formula on the oracle's sums
        _, ag = oracle.bf16_linear_ref(xb, gb)
        _, au = oracle.bf16_linear_ref(xb, ub)
        gq, uq = f32(bits(ag)).astype(np.float64), f32(bits(au)).astype(np.float64)
        ref = f32(bits(gq / (1.0 + np.exp(-gq)))).astype(np.float64) * uq
        gotf = f32(got[:m]).astype(np.float64)
        rms = np.sqrt((ref ** 2).mean())
        assert (np.abs(gotf - ref) <= np.abs(ref) * 2.0 ** -6 + 2e-2 * rms).all()
        assert np.median(np.abs(gotf - ref) / np.maximum(np.abs(ref), 1e-3 * rms)) < 2.0 ** -8


def test_mlp_block_with_bf16_weights(env):
    """The MLP block's second fused form (model.rs:3179-3188): more than 16 prompt rows take fe_gemm_swiglu over the
    interleaved gate|up weights and down's GEMM with the residual; the decode rows take the per-linear path. Each group of
    rows has the bits of the same steps called by hand."""
    torch, bf16, kern = env
    from ferrite_amd import route
    hidden, inter, rows, dec = 512, 1280, 60, 4
    rng = np.random.default_rng(17)
    xn_b, x_b = bits(rng.normal(size=(rows, hidden))), bits(rng.normal(size=(rows, hidden)))
    gb, ub = bits(rng.normal(size=(inter, hidden)) / np.sqrt(hidden) * 2), bits(rng.normal(size=(inter, hidden)) / np.sqrt(hidden) * 2)
    db = bits(rng.normal(size=(hidden, inter)) / np.sqrt(inter))
    xn, g, u, dn = dev_u16(torch, xn_b), dev_u16(torch, gb), dev_u16(torch, ub), dev_u16(torch, db)
    wi = bf16.interleave_gu(kern, g, u)
    ctx = route.LinCtx()
    ctx.set_bf16(kern)
    bf = torch.bfloat16
    gate_up = route.Proj([(route.Linear("gate", inter, hidden, w=g.view(bf)), [inter]), (route.Linear("up", inter, hidden, w=u.view(bf)), [inter])])
    down = route.Linear("down", hidden, inter, w=dn.view(bf))
    big = dev_u16(torch, np.zeros((rows, 2 * inter), np.uint16))
    act = dev_u16(torch, np.zeros((rows, inter), np.uint16))

    def run(nrows, d, fused):
        ctx.dec = d
        x = dev_u16(torch, x_b)
        route.mlp_forward(ctx, gate_up, down, x, xn, big, act, nrows, hidden, inter, swiglu_w=wi if fused else None)
        torch.cuda.synchronize()
        return host_u16(x)

    def by_hand_rows(r0, r1, gemv):
        """gate, up, fe_silu_mul, down + residual over rows [r0, r1), every linear through the GEMV or the GEMM."""
        m = r1 - r0
        fn = (lambda *a, **k: bf16.forward(*a, **k)) if gemv else bf16.gemm
        xs = xn[r0:r1].contiguous()
        yg, yu = call(torch, fn, kern, xs, g, m, inter), call(torch, fn, kern, xs, u, m, inter)
        a = dev_u16(torch, np.zeros((m, inter), np.uint16))
        gd, ud = dev_u16(torch, yg), dev_u16(torch, yu)
        route.silu_mul(a, gd.data_ptr(), ud.data_ptr(), inter, inter, m)
        return call(torch, fn, kern, a, dn, m, hidden, res=dev_u16(torch, x_b[r0:r1]))

    got = run(rows, dec, True)
    assert np.array_equal(got[:dec], by_hand_rows(0, dec, True))
    a = dev_u16(torch, np.zeros((rows - dec, inter), np.uint16))
    bf16.gemm_swiglu(kern, a, xn[dec:].contiguous(), hidden, wi, rows - dec)
    want = call(torch, bf16.gemm, kern, a, dn, rows - dec, hidden, res=dev_u16(torch, x_b[dec:]))
    assert np.array_equal(got[dec:], want)
    # without the interleaved weights: gate and up one by one, fe_silu_mul, down (the same sums: the same bits)
    plain = run(rows, dec, False)
    assert np.array_equal(plain[:dec], got[:dec])
    assert np.array_equal(plain[dec:], by_hand_rows(dec, rows, False))
    # a batch of up to 16 rows: all decode rows, the fused form is not used
    small = run(12, 0, True)
    assert np.array_equal(small[:12], by_hand_rows(0, 12, True)) and np.array_equal(small[12:], x_b[12:])


def test_events_attached_to_one_launch(env):
    """fe_hip_time_next_launch: the next launch carries the two events; the result is the launch's own, the reading a
    kernel duration, and the launch after it is an ordinary one again."""
    import ctypes as C
    torch, bf16, kern = env
    from ferrite_amd import _lib
    lib = _lib.lib()
    n, k = 4096, 2048
    xb, wb = operands(n, k, 1, 9)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)
    plain = call(torch, bf16.gemv, kern, x, w, 1, n)
    a, b = C.c_void_p(), C.c_void_p()
    _lib.check(lib.fe_hip_event_create(C.byref(a)))
    _lib.check(lib.fe_hip_event_create(C.byref(b)))
    for _ in range(2):
        _lib.check(lib.fe_hip_time_next_launch(a, b))
        timed = call(torch, bf16.gemv, kern, x, w, 1, n)
        assert np.array_equal(timed, plain)
        _lib.check(lib.fe_hip_event_sync(b))
        ms = C.c_float()
        _lib.check(lib.fe_hip_event_elapsed_ms(C.byref(ms), a, b))
        assert 1e-3 < ms.value < 5.0, ms.value  # 16 MB of weights: a few microseconds, not a host-side interval
        assert np.array_equal(call(torch, bf16.gemv, kern, x, w, 1, n), plain)
    _lib.check(lib.fe_hip_event_destroy(a))
    _lib.check(lib.fe_hip_event_destroy(b))


def test_argument_errors(env):
    torch, bf16, kern = env
    from ferrite_amd import _lib
    x = torch.zeros((9, 512), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((256, 512), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((9, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.FeError):
        bf16.gemv(kern, y, 256, x, 512, w, 9)  # more than 8 rows
    with pytest.raises(_lib.FeError):
        bf16.gemm(kern, y, 250, x, 512, w, 9)  # ldy < n
    with pytest.raises(_lib.FeError):
        bf16.gemm(kern, y, 256, x, 508, w, 9)  # lda < k
    with pytest.raises(_lib.FeError):
        bf16.gemm(kern, y, 256, x, 512, w[:, :500].contiguous(), 9)  # k % 64
    bf16.gemm(kern, y, 256, x, 512, w, 0)  # m == 0: nothing to do


def test_full_size_gate_up_shape(env, oracle):
    """5120 x 17408 at 1 row (GEMV) and 2048 rows (GEMM, the reference's sampled rows, fp4-check.rs:96)."""
    torch, bf16, kern = env
    n, k, m = 17408, 5120, 2048
    xb, wb = operands(n, k, m, 21)
    x, w = dev_u16(torch, xb), dev_u16(torch, wb)
    one = call(torch, bf16.gemv, kern, x, w, 1, n)
    close(one, oracle.bf16_linear_ref(xb[:1], wb)[1])
    y = dev_u16(torch, np.full((m, n), CANARY, np.uint16))
    bf16.gemm(kern, y, n, x, k, w, m)
    torch.cuda.synchronize()
    rows = [0, 1, 17, 127, 128, m // 2, m - 1]
    close(host_u16(y[rows]), oracle.bf16_linear_ref(xb[rows], wb)[1])
