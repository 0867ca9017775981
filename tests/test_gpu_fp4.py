"""GPU parity of the NVFP4 path against the CPU oracle, through the C ABI. Mirrors the reference's fp4-check
(crates/fe-fp4/src/bin/fp4-check.rs:30-208): activation quantizer bit-exact, GEMM vs an f64 GEMM over the same
quantized operands, the residual epilogue, the strided-output canary, and argument errors."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    from ferrite_amd import fp4
    assert torch.cuda.is_available()
    return torch, fp4, fp4.Kernels.load()


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def bf16_to_f32(a):
    return (a.astype(np.uint32) << 16).view(np.float32)


def bf16_bits(x):
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def fp4_check_activations(m, k, g, seed):
    """Gaussian with a few outliers, amax around the calibrated range 448 * 6 / g (fp4-check.rs:35-47)."""
    rng = np.random.default_rng(seed)
    sigma = 448.0 * 6.0 / g / 10.0
    x = rng.normal(size=m * k).astype(np.float32) * np.float32(sigma)
    x[::997] *= 6.0
    x = x.reshape(m, k)
    x[0, :16] = 0.0  # an all-zero block
    return bf16_bits(x)


@pytest.mark.parametrize("n,k,m,input_scale", [(256, 512, 200, 1.0), (128, 1024, 1, 0.037), (384, 256, 130, 2.5),
                                               (256, 512, 16, 1.0), (384, 1024, 37, 0.5), (640, 2048, 5, 1.0)])
def test_fp4_linear(env, oracle, n, k, m, input_scale):
    torch, fp4, kern = env
    from ferrite_amd import synth
    host = synth.fp4_linear(n, k, 11, input_scale=input_scale)
    host.alpha[:] = host.alpha * np.linspace(0.5, 2.0, n).astype(np.float32)  # distinct per-column scales
    lin = host.upload()
    ws = fp4.Workspace(m, k)
    xb = fp4_check_activations(m, k, lin.g, 3)
    xd = dev_u16(torch, xb)
    y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.forward(kern, ws, y, n, xd, k, m)
    torch.cuda.synchronize()
    yg = y.view(torch.int16).cpu().numpy().view(np.uint16)

    # (1) quantizer bit-exactness (fp4-check.rs:69-93); the reference tolerates < 0.1 % code bytes, here: none
    codes, sf_tiled = ws.read(m, k)
    sfa = oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16)
    want_codes, want_sf = oracle.quant_fp4(xb, lin.g)
    assert np.array_equal(sfa, want_sf)
    assert np.array_equal(codes, want_codes)
    assert want_sf[0, 0] == 0 and not want_codes[0, :8].any()

    # (2) GEMM vs the f64 reference over the same quantized operands (fp4-check.rs:95-144)
    rows = sorted({r for r in (0, 1, 17, 127, 128, m // 2, m - 1) if r < m})
    wf = oracle.dequant_fp4(host.codes, host.sf, 1.0)
    aq = oracle.dequant_fp4(codes[rows], sfa[rows], 1.0)
    refq = oracle.ref_gemm(aq, wf).astype(np.float64) * host.alpha.astype(np.float64)[None, :]
    got = bf16_to_f32(yg[rows]).astype(np.float64)
    scale = np.abs(refq).max(axis=1, keepdims=True).clip(1e-20)
    assert (np.abs(got - refq) / scale).max() < 8e-3
    # the north-star bar: max relative error 1e-2 (bf16 out), floored at 1e-2 of the row maximum
    assert (np.abs(got - refq) / np.maximum(np.abs(refq), 1e-2 * scale)).max() < 1e-2

    # (3) residual epilogue, in place: y2 = bf16(bf16(x.W) + res), exact (fp4-check.rs:160-173)
    res = bf16_bits(np.random.default_rng(5).normal(size=(m, n)).astype(np.float32))
    y2 = dev_u16(torch, res)
    lin.forward(kern, ws, y2, n, xd, k, m, res=y2)
    torch.cuda.synchronize()
    want = bf16_bits(bf16_to_f32(yg) + bf16_to_f32(res))
    assert np.array_equal(y2.cpu().numpy().view(np.uint16), want)

    # (4) canary: strided output inside a larger buffer, nothing outside rows < m, cols < n is written
    # (fp4-check.rs:175-191)
    ldy = n + 72
    yc = torch.full(((m + 3), ldy), -21555, dtype=torch.int16, device="cuda")
    lin.forward(kern, ws, yc, ldy, xd, k, m)
    lin.forward(kern, ws, yc, ldy, xd, k, m, res=yc)
    torch.cuda.synchronize()
    ych = yc.cpu().numpy()
    assert (ych[m:] == -21555).all() and (ych[:, n:] == -21555).all()
    assert np.array_equal(ych[:m, :n].view(np.uint16), bf16_bits(bf16_to_f32(yg) + bf16_to_f32(yg)))

    # (5) quantize once, gemm separately gives the same bits (lib.rs:518-543)
    y3 = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.quantize(kern, ws, xd, k, m)
    lin.gemm(kern, ws, y3, n, m)
    torch.cuda.synchronize()
    assert np.array_equal(y3.view(torch.int16).cpu().numpy().view(np.uint16), yg)


def test_fp4_gemm_tiles_cut_or_whole_and_views(env, oracle):
    """Several 256 x 256 output tiles with an odd count of 128-row weight tiles, computed whole (option gemm_splits = 1), cut
    along K with the reduce kernel (the default for a nearly empty last round), and from a row-major device view."""
    torch, fp4, kern = env
    from ferrite_amd import synth
    n, k, m = 640, 1024, 300
    host = synth.fp4_linear(n, k, 23, input_scale=1.0)
    host.alpha[:] = host.alpha * np.linspace(0.5, 2.0, n).astype(np.float32)
    lin = host.upload()
    ws = fp4.Workspace(m, k)
    xd = dev_u16(torch, fp4_check_activations(m, k, lin.g, 4))

    def run(l, res=None):
        y = torch.full((m + 2, n), -3.0, dtype=torch.bfloat16, device="cuda")
        l.forward(kern, ws, y, n, xd, k, m, res=res)
        torch.cuda.synchronize()
        out = y.view(torch.int16).cpu().numpy().view(np.uint16)
        assert (out[m:] == bf16_bits(np.float32([-3.0]))[0]).all()
        return out[:m]

    cut = run(lin)
    assert np.array_equal(cut, run(lin))  # deterministic
    kern.set_option("gemm_splits", 1)
    whole = run(lin)
    view = fp4.PromptLinear.from_view("view", n, k, torch.from_numpy(host.codes).cuda(), torch.from_numpy(host.sf).cuda(),
                                      torch.from_numpy(host.alpha).cuda(), host.g)
    assert np.array_equal(run(view), whole)
    kern.set_option("gemm_splits", 8)
    assert np.array_equal(run(view), cut)
    # cut and whole differ only by the order of the f32 sums: at most one bf16 step
    a, b = bf16_to_f32(cut).astype(np.float64), bf16_to_f32(whole).astype(np.float64)
    assert (np.abs(a - b) <= np.abs(b) / 128.0 + 1e-30).all()
    # against the f64 reference over the quantized operands
    codes, sf_tiled = ws.read(m, k)
    sfa = oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16)
    rows = [0, 127, 128, 255, 256, 299]
    refq = oracle.ref_gemm(oracle.dequant_fp4(codes[rows], sfa[rows], 1.0), oracle.dequant_fp4(host.codes, host.sf, 1.0))
    refq = refq.astype(np.float64) * host.alpha.astype(np.float64)[None, :]
    scale = np.abs(refq).max(axis=1, keepdims=True).clip(1e-20)
    for got in (a[rows], b[rows]):
        assert (np.abs(got - refq) / np.maximum(np.abs(refq), 1e-2 * scale)).max() < 1e-2
    # residual through the reduce kernel's epilogue
    res = dev_u16(torch, bf16_bits(np.random.default_rng(6).normal(size=(m + 2, n)).astype(np.float32)))
    got = run(lin, res=res)
    want = bf16_bits(bf16_to_f32(cut) + bf16_to_f32(res.cpu().numpy().view(np.uint16)[:m]))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,forced", [(2400, 3968, 2), (6600, 4096, 3)])
def test_gemm_on_the_stream_k_schedule(env, oracle, m, n, forced):
    """Stream-K: the GEMM walks the tiles' k tiles laid end to end, every program a contiguous run, and the pieces of a
    tile meet through the workspace with the last arriver adding them in piece order. Two cases the library picks the
    schedule for by itself on 256 CUs (option gemm_sk = 1 then gives the bits of the forced schedule): 2400 x 3968 over
    K = 1024 is 10 x 16 = 160 tiles of 16 k tiles (8 for FP8 codes), fewer tiles than CUs and no cut that fills its rounds
    (forced: 2, runs over all tiles; a ragged last row tile and a half last column tile); 6600 x 4096 is 26 x 16 = 416
    tiles, one whole round and runs of 10 k tiles over the other 160 (forced: 3; the library's choice for NVFP4 only). Repeats give the same bits (arrival
    order does not matter, counters are back at zero), the one-piece schedule (0) differs by the order of the f32 sums
    only; NVFP4 and both FP8 forms, the residual epilogue, rows past m untouched."""
    torch, fp4, kern = env
    from ferrite_amd import synth
    k = 1024
    rng = np.random.default_rng(12)
    res = dev_u16(torch, bf16_bits(rng.normal(size=(m + 2, n)).astype(np.float32)))
    for kind in ("nvfp4", "fp8", "fp8_f16"):
        host = synth.fp8_linear(n, k, 31, input_scale=0.05) if kind != "nvfp4" else synth.fp4_linear(n, k, 31, input_scale=1.0)
        host.alpha[:] = host.alpha * np.linspace(0.5, 2.0, n).astype(np.float32)
        lin = host.upload()
        ws = fp4.Workspace(m, k)
        xd = dev_u16(torch, fp4_check_activations(m, k, lin.g, 5))
        kern.set_option("fp8_f16", 1 if kind == "fp8_f16" else 0)

        def run(sk, r=None):
            kern.set_option("gemm_sk", sk)
            y = torch.full((m + 2, n), -3.0, dtype=torch.bfloat16, device="cuda")
            lin.forward(kern, ws, y, n, xd, k, m, res=r)
            torch.cuda.synchronize()
            out = y.view(torch.int16).cpu().numpy().view(np.uint16)
            assert (out[m:] == bf16_bits(np.float32([-3.0]))[0]).all()
            return out[:m]

        try:
            want = run(forced)
            for _ in range(4):
                assert np.array_equal(run(forced), want), kind
            # the library's own choice for this shape (whole rounds then runs: not for FP8, whose weight operand is large)
            assert np.array_equal(run(1), want if kind == "nvfp4" or forced == 2 else run(0)), kind
            a = bf16_to_f32(want).astype(np.float64)
            for other in (0, 2):
                b = bf16_to_f32(run(other)).astype(np.float64)
                assert (np.abs(a - b) <= np.abs(b) / 128.0 + 1e-4 * np.abs(b).max()).all(), (kind, other)
            got = run(forced, r=res)
            assert np.array_equal(got, bf16_bits(bf16_to_f32(want) + bf16_to_f32(res.cpu().numpy().view(np.uint16)[:m]))), kind
        finally:
            kern.set_option("gemm_sk", 1)
            kern.set_option("fp8_f16", 0)
        # against the f64 reference over the quantized operands
        rows = sorted({r for r in (0, 1, 17, 255, 256, 1023, 1024, 2047, 2048, 2303, 2304, m // 2, m - 1) if r < m})
        if kind == "nvfp4":
            codes, sf_tiled = ws.read(m, k)
            sfa = oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16)
            ref = oracle.ref_gemm(oracle.dequant_fp4(codes[rows], sfa[rows], 1.0), oracle.dequant_fp4(host.codes, host.sf, 1.0))
        else:
            codes = ws.read_fp8(m, k)
            ref = oracle.ref_gemm(np.stack([oracle.dequant_fp8_row(codes[r], 1.0) for r in rows]),
                                  np.stack([oracle.dequant_fp8_row(host.codes[c], 1.0) for c in range(n)]))
        ref = ref.astype(np.float64) * host.alpha.astype(np.float64)[None, :]
        scale = np.abs(ref).max(axis=1, keepdims=True).clip(1e-20)
        assert (np.abs(a[rows] - ref) / np.maximum(np.abs(ref), 1e-2 * scale)).max() < 1e-2, kind


def test_fp4_gemv_agrees_with_the_gemm(env, oracle):
    """Up to 64 rows run the weight-read-bound GEMV (up to 48 rows a pass, K cut over several programs); option gemv = 0
    sends the same rows through the GEMM. Both sum the same exact products in f32, in different orders; within the GEMV a
    row's bits do not depend on the rows around it."""
    torch, fp4, kern = env
    from ferrite_amd import synth
    n, k = 384, 2048
    host = synth.fp4_linear(n, k, 31, input_scale=1.0)
    host.alpha[:] = host.alpha * np.linspace(0.5, 2.0, n).astype(np.float32)
    lin = host.upload()
    view = fp4.PromptLinear.from_view("view", n, k, torch.from_numpy(host.codes).cuda(), torch.from_numpy(host.sf).cuda(),
                                      torch.from_numpy(host.alpha).cuda(), host.g)
    for m in (1, 3, 16, 17, 48, 64):
        ws = fp4.Workspace(m, k)
        xd = dev_u16(torch, fp4_check_activations(m, k, lin.g, 40 + m))
        res = dev_u16(torch, bf16_bits(np.random.default_rng(m).normal(size=(m + 1, n)).astype(np.float32)))

        def run(l, r=None):
            y = torch.full((m + 1, n), -3.0, dtype=torch.bfloat16, device="cuda")
            l.forward(kern, ws, y, n, xd, k, m, res=r)
            torch.cuda.synchronize()
            out = y.view(torch.int16).cpu().numpy().view(np.uint16)
            assert (out[m:] == bf16_bits(np.float32([-3.0]))[0]).all()
            return out[:m]

        gemv = run(lin)
        assert np.array_equal(gemv, run(lin)) and np.array_equal(gemv, run(view))
        with_res = run(lin, res)
        assert np.array_equal(with_res, bf16_bits(bf16_to_f32(gemv) + bf16_to_f32(res.cpu().numpy().view(np.uint16)[:m])))
        kern.set_option("gemv", 0)
        gemm = run(lin)
        kern.set_option("gemv", 1)
        a, b = bf16_to_f32(gemv).astype(np.float64), bf16_to_f32(gemm).astype(np.float64)
        assert (np.abs(a - b) <= np.abs(b) / 128.0 + 1e-30).all()
    # the same rows alone, in a pass of 16, 32 or 48 rows, and as the second pass of 64
    ws = fp4.Workspace(64, k)
    x64 = dev_u16(torch, fp4_check_activations(64, k, lin.g, 77))
    outs = {}
    for m, r0 in ((5, 0), (16, 0), (30, 0), (48, 0), (64, 0), (7, 48), (16, 48)):
        y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        lin.forward(kern, ws, y, n, x64[r0:], k, m)
        torch.cuda.synchronize()
        outs[(m, r0)] = y.view(torch.int16).cpu().numpy().view(np.uint16)
    for m in (16, 30, 48, 64):
        assert np.array_equal(outs[(m, 0)][:5], outs[(5, 0)])
    assert np.array_equal(outs[(64, 0)][48:55], outs[(7, 48)]) and np.array_equal(outs[(64, 0)][48:], outs[(16, 48)])


@pytest.mark.parametrize("n,k", [(384, 2048), (128, 256), (1024, 5120)])
def test_fp4_gemv_over_strips_agrees_with_the_weight_tiles(env, oracle, n, k):
    """The GEMV over strips of 16 weight rows (a workgroup a strip over all of K, activations staged in LDS, nothing
    handed between programs; option gemv_strips = 2 takes it wherever it fits, 0 never) against the GEMV over weight tiles
    and K splits: the same exact products summed in another order; both weight layouts; the residual epilogue; rows past m
    untouched; repeats bit-equal; and against the f64 reference over the dequantized operands (fp4-check.rs:134-144)."""
    torch, fp4, kern = env
    from ferrite_amd import synth
    host = synth.fp4_linear(n, k, 51, input_scale=1.0)
    lin = host.upload()
    view = fp4.PromptLinear.from_view("view", n, k, torch.from_numpy(host.codes).cuda(), torch.from_numpy(host.sf).cuda(),
                                      torch.from_numpy(host.alpha).cuda(), host.g)
    wdq = oracle.dequant_fp4(host.codes, host.sf, 1.0)
    try:
        for m in (1, 2, 4, 9, 16):
            if m * k * 2 > 48 * 1024:
                continue
            ws = fp4.Workspace(m, k)
            xb = fp4_check_activations(m, k, lin.g, 60 + m)
            xd = dev_u16(torch, xb)
            res = dev_u16(torch, bf16_bits(np.random.default_rng(m).normal(size=(m + 1, n)).astype(np.float32)))

            def run(l, strips, r=None, once=1):
                kern.set_option("gemv_strips", strips)
                kern.set_option("gemv_once", once)  # (1: every load of a workgroup issued at once, where K allows)
                y = torch.full((m + 1, n), -3.0, dtype=torch.bfloat16, device="cuda")
                l.forward(kern, ws, y, n, xd, k, m, res=r)
                torch.cuda.synchronize()
                out = y.view(torch.int16).cpu().numpy().view(np.uint16)
                assert (out[m:] == bf16_bits(np.float32([-3.0]))[0]).all()
                return out[:m]

            tiles, strips = run(lin, 0), run(lin, 2)
            assert np.array_equal(strips, run(lin, 2)) and np.array_equal(strips, run(view, 2))
            a, b = bf16_to_f32(strips).astype(np.float64), bf16_to_f32(tiles).astype(np.float64)
            assert (np.abs(a - b) <= np.abs(b) / 128.0 + 1e-30).all(), m
            looped = bf16_to_f32(run(lin, 2, once=0)).astype(np.float64)  # the looped form: other wavefront counts, other order
            assert (np.abs(looped - b) <= np.abs(b) / 128.0 + 1e-30).all(), m
            with_res = run(lin, 2, res)
            assert np.array_equal(with_res, bf16_bits(bf16_to_f32(strips) + bf16_to_f32(res.cpu().numpy().view(np.uint16)[:m])))
            codes, sf = oracle.quant_fp4(xb, host.g)
            ref = oracle.ref_gemm(oracle.dequant_fp4(codes, sf, 1.0), wdq).astype(np.float64) * host.alpha.astype(np.float64)[None, :]
            assert (np.abs(a - ref) / np.abs(ref).max(axis=1, keepdims=True)).max() < 8e-3, m
    finally:
        kern.set_option("gemv_strips", 1)
        kern.set_option("gemv_once", 1)


def test_quantizer_on_special_values(env, oracle):
    """Ties between codes, the saturation boundary, signed zeros, infinities and NaN (a NaN element has magnitude 0 and
    keeps its sign, format.rs:28-41, 66-69; it does not enter the block maximum, format.rs:76): codes and scales as the
    oracle's, bit for bit."""
    torch, fp4, kern = env
    k, m = 256, 3
    x = np.zeros((m, k), np.float32)
    ties = np.float32([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0])
    x[0, :16] = ties            # amax 7 -> scale e4m3(7/6); the elements land on and next to code boundaries
    x[0, 16:32] = ties * 0.5
    x[0, 32:48] = [0.0, -0.0, 1e-30, -1e-30, 3.0, -3.0, 6.0, -6.0, 1.0, 2.0, 4.0, 0.5, 1.5, -1.5, -0.5, -4.0]
    x[1, :16] = np.float32([np.nan, 1.0, -2.0, 3.0] * 4)
    x[1, 16:32] = np.float32([np.inf, 1.0, -np.inf, 2.0] * 4)
    x[1, 32:48] = np.float32([-np.nan, 6.0, 0.0, -6.0] * 4)
    x[2] = np.random.default_rng(2).normal(size=k).astype(np.float32) * 100
    xb = bf16_bits(x)
    xb[1, 0:16:4] = 0x7FC0      # bf16 NaN patterns survive the host-side rounding as NaN
    xb[1, 32:48:4] = 0xFFC0
    for g in (1.0, 0.3):
        ws = fp4.Workspace(m, k)
        lin = None
        from ferrite_amd import synth
        lin = synth.fp4_linear(128, k, 1, input_scale=1.0 / g).upload()
        lin.quantize(kern, ws, dev_u16(torch, xb), k, m)
        torch.cuda.synchronize()
        codes, sf_tiled = ws.read(m, k)
        want_codes, want_sf = oracle.quant_fp4(xb, lin.g)
        assert np.array_equal(oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16), want_sf)
        assert np.array_equal(codes, want_codes)


def test_fp4_argument_errors(env):
    torch, fp4, kern = env
    from ferrite_amd import synth
    from ferrite_amd._lib import FeError
    lin = synth.fp4_linear(128, 256, 1).upload()
    ws = fp4.Workspace(8, 256)
    x = dev_u16(torch, synth.activations(16, 256, 1))
    y = torch.zeros((16, 136), dtype=torch.bfloat16, device="cuda")
    lin.forward(kern, ws, y, 136, x, 256, 0)  # m == 0 is a no-op
    with pytest.raises(FeError):
        lin.forward(kern, ws, y, 136, x, 256, 9)  # workspace holds 8 rows
    with pytest.raises(FeError):
        lin.forward(kern, ws, y, 132, x, 256, 4)  # ldy % 8
    with pytest.raises(FeError):
        fp4.Workspace(8, 128) and lin.forward(kern, fp4.Workspace(8, 128), y, 136, x, 256, 4)  # k exceeds the workspace
    lin.forward(kern, ws, y, 136, x, 256, 8)
    torch.cuda.synchronize()
    assert torch.isfinite(y[:8, :128].float()).all()
