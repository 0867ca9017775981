"""Parity at the benchmark's own sizes, where the CPU oracle would take minutes per case: the kernels are checked through
properties that do not depend on the size.

EXL3: the GPU's W_hat (reconstruct_hat_f16, bit-exact against the oracle on whole small tensors in test_gpu_exl3.py) is
checked here against the oracle's decode_tile on sampled tiles of the full tensor; then every GEMV / GEMM output must
equal H(xh . W_hat) * svh / sqrt(128) computed by plain torch matmuls over that W_hat and the kernel's own rotated input
(f64 for decode-sized M, f32 for M = 2048), within the same bounds as the small cases. Rows of a batch must repeat the
bits of the single-row call (one summation order for 1..64 rows).

NVFP4: outputs against torch matmuls over the oracle's dequantization of the same quantized operands.

Shapes: hidden 5120, 40 heads x 128, 8 KV heads, MLP 17408 (q, o 5120x5120; k, v 5120x1024; gate, up 5120x17408; down
17408x5120), M in {1, 4, 8, 16, 2048}."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPES = {"qo": (5120, 5120), "kv": (5120, 1024), "gate_up": (5120, 17408), "down": (17408, 5120),
          "lm_head": (5120, 151936)}  # the largest linear of a decode step: 1187 column blocks


@pytest.fixture(scope="module")
def env():
    import torch
    from ferrite_amd import exl3
    assert torch.cuda.is_available()
    return torch, exl3, exl3.Kernels.load()


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def hadamard128(torch, dtype):
    i = torch.arange(128, device="cuda")
    bits = i[:, None] & i[None, :]
    pop = torch.zeros_like(bits)
    for b in range(7):
        pop += (bits >> b) & 1
    return (1 - 2 * (pop & 1)).to(dtype)  # H[i][j] = (-1)^popcount(i & j)


class Layer:
    """One EXL3 linear at full size with its GPU-reconstructed W_hat."""

    def __init__(self, env, oracle, k, n, bits, seed):
        torch, exl3, kern = env
        from ferrite_amd import synth
        self.t = synth.exl3_tensor(k, n, bits, seed)
        self.lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(self.t), exl3.default_blocks(exl3.cu_count()))
        stored = exl3.DeviceExl3.upload(self.t)
        w = torch.zeros((k, n), dtype=torch.int16, device="cuda")
        kern.reconstruct_hat_f16(stored.view, w)
        torch.cuda.synchronize()
        self.w_hat = w.view(torch.float16)
        # the decoder at this size: sampled tiles against the oracle, bit for bit
        rng = np.random.default_rng(seed)
        for kt, nt in zip(rng.integers(0, k // 16, 48), rng.integers(0, n // 16, 48)):
            want = oracle.decode_tile(self.t.tile(int(kt), int(nt)), bits)
            got = w[kt * 16:kt * 16 + 16, nt * 16:nt * 16 + 16].cpu().numpy().view(np.uint16)
            assert np.array_equal(got, want), (kt, nt)
        self.svh = torch.from_numpy(self.t.svh.view(np.float16).astype(np.float64)).cuda()

    def reference(self, torch, xh, dtype):
        """H(xh . W_hat) * svh / sqrt(128) from torch matmuls; xh: fp16 [m][k] on the device."""
        m, n = xh.shape[0], self.t.n
        s = xh.to(dtype) @ self.w_hat.to(dtype)
        s = (s.view(m, n // 128, 128) @ hadamard128(torch, dtype)).view(m, n)
        return (s.double() * self.svh / np.sqrt(128.0)).cpu().numpy()


def run_rows(env, layer, m, seed, outliers=False):
    torch, exl3, kern = env
    from ferrite_amd import synth
    lin = layer.lin
    ws = exl3.Workspace([lin], m)
    xd = dev_u16(torch, synth.activations(m, lin.k, seed, outliers=outliers))
    y = torch.full((m + 1, lin.n), float("nan"), dtype=torch.float32, device="cuda")
    lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
    yb = torch.zeros((m, lin.n), dtype=torch.bfloat16, device="cuda")
    lin.forward(xd, exl3.Dtype.Bf16, yb, exl3.Dtype.Bf16, m, ws)
    torch.cuda.synchronize()
    xh = torch.from_numpy(ws.xh(m, lin.k).view(np.int16)).cuda().view(torch.float16)
    got = y.cpu().numpy()
    assert np.isnan(got[m]).all()
    return xd, xh, got[:m].astype(np.float64), yb.float().cpu().numpy().astype(np.float64), ws


def check(got, got_bf16, ref, f32_bound):
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(got - ref).max() / rms < f32_bound
    # bf16 output: one rounding of the same sum
    assert np.all(np.abs(got_bf16 - ref) <= np.abs(ref) / 256.0 + f32_bound * rms)
    # the bar of the benchmark: max relative error 1e-2, denominators floored at the output's rms
    assert (np.abs(got_bf16 - ref) / np.maximum(np.abs(ref), rms)).max() < 1e-2


def end_to_end(oracle, layer, xd, rows, got_rows):
    """The whole linear against the reference's f64 linear on the bf16 inputs themselves (crates/fe-exl3/src/cpu.rs:180-215)
    for a subset of the rows: max |y - ref| / rms(ref). What separates the two is the fp16 rounding of the rotated inputs
    (the reference's GPU path has it too) and f32 sums."""
    t = layer.t
    o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
    xb = xd.cpu().numpy().view(np.uint16)[rows]
    x64 = (xb.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ref = oracle.linear_f64(o, x64, threads=oracle.default_threads(16))
    return np.abs(got_rows - ref).max() / np.sqrt((ref ** 2).mean())


@pytest.mark.parametrize("shape,bits", [("qo", 4), ("kv", 4), ("gate_up", 3), ("gate_up", 4), ("gate_up", 5), ("down", 3),
                                        ("down", 4), ("down", 5), ("lm_head", 6)])
def test_exl3_decode_rows_at_full_size(env, oracle, shape, bits):
    torch, exl3, kern = env
    k, n = SHAPES[shape]
    layer = Layer(env, oracle, k, n, bits, 500 + bits)
    single = None
    for m in (1, 4, 8, 16):
        xd, xh, got, got_bf16, ws = run_rows(env, layer, m, 9)
        check(got, got_bf16, layer.reference(torch, xh, torch.float64), 1e-4)
        if m == 1 and shape != "lm_head":  # end to end against the reference's CPU linear
            assert end_to_end(oracle, layer, xd, [0], got[:1]) < 2e-3
        if m == 16:  # each row of the batch has the bits of the single-row call
            for r in (0, 7, 15):
                y1 = torch.zeros((1, n), dtype=torch.float32, device="cuda")
                layer.lin.forward(xd[r:r + 1], exl3.Dtype.Bf16, y1, exl3.Dtype.F32, 1, ws)
                torch.cuda.synchronize()
                assert np.array_equal(y1.cpu().numpy()[0].astype(np.float64), got[r])


@pytest.mark.parametrize("shapes,bits", [(("gate_up", "gate_up"), 4), (("qo", "kv", "kv"), 4), (("gate_up", "gate_up"), 3)])
def test_exl3_grouped_projections_at_full_size(env, shapes, bits):
    """The projections of one input (gate, up; q, k, v) as one grouped launch at the benchmark's sizes: every member's
    output has the bits of the member's own forward (checked against the reference above), at 1..16 rows."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    k = SHAPES[shapes[0]][0]
    blocks = exl3.default_blocks(exl3.cu_count())
    lins = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, SHAPES[s][1], bits, 900 + i)), blocks)
            for i, s in enumerate(shapes)]
    ws = exl3.Workspace(lins, 16)
    xd = dev_u16(torch, synth.activations(16, k, 3, outliers=True))
    for m in (1, 4, 8, 16):
        assert exl3.forward_group_launches(lins, m, ws) in (1, 2)
        want = [torch.zeros((m, l.n), dtype=torch.bfloat16, device="cuda") for l in lins]
        got = [torch.ones((m, l.n), dtype=torch.bfloat16, device="cuda") for l in lins]
        for l, y in zip(lins, want):
            l.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.Bf16, m, ws)
        exl3.forward_group(lins, xd, exl3.Dtype.Bf16, got, exl3.Dtype.Bf16, m, ws)
        torch.cuda.synchronize()
        for a, b in zip(want, got):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), m


def test_exl3_decode_mlp_back_to_back_is_deterministic(env):
    """The decode MLP's launches (gate + up grouped, then down) 240 times back to back on one workspace without a
    synchronization in between, the row count changing from call to call (the role of
    crates/fe-exl3/src/bin/exl3-stress.rs): partial sums and arrival counters of one launch must never leak into the
    next, so every call has the bits of the first call with its row count."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    blocks = exl3.default_blocks(exl3.cu_count())
    g, u = (exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(5120, 17408, 4, 40 + i)), blocks) for i in range(2))
    d = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(17408, 5120, 4, 42)), blocks)
    ws = exl3.Workspace([g, u, d], 16)
    x = dev_u16(torch, synth.activations(16, 5120, 5))
    xd = dev_u16(torch, synth.activations(16, 17408, 6))
    rows_list = (1, 16, 4, 8, 2, 13)
    outs = []
    for it in range(240):
        m = rows_list[it % len(rows_list)]
        ys = [torch.empty((m, 17408), dtype=torch.bfloat16, device="cuda") for _ in range(2)]
        yd = torch.empty((m, 5120), dtype=torch.bfloat16, device="cuda")
        exl3.forward_group([g, u], x, exl3.Dtype.Bf16, ys, exl3.Dtype.Bf16, m, ws)
        d.forward(xd, exl3.Dtype.Bf16, yd, exl3.Dtype.Bf16, m, ws)
        outs.append((m, ys[0], ys[1], yd))
    torch.cuda.synchronize()
    first = {}
    for it, (m, a, b, c) in enumerate(outs):
        if m not in first:
            first[m] = (a, b, c)
            continue
        for want, got in zip(first[m], (a, b, c)):
            assert torch.equal(want.view(torch.int16), got.view(torch.int16)), (it, m)
    # rows of a batch have the bits of the same rows in a smaller batch
    assert torch.equal(first[16][0][:4].view(torch.int16), first[4][0].view(torch.int16))
    assert torch.equal(first[16][2][:1].view(torch.int16), first[1][2].view(torch.int16))


@pytest.mark.parametrize("bits,down_units", [(3, 0), (4, 0), (5, 0), (4, 4), (5, 8)])
def test_exl3_decode_mlp_in_one_launch_at_full_size(env, oracle, bits, down_units):
    """The decode MLP block of the benchmark (gate, up 5120 x 17408, down 17408 x 5120) through fe_exl3_mlp_forward: gate's
    and up's outputs have the bits of their grouped launch (checked against the reference above); down is checked
    against H(xh . W_hat) * svh / sqrt(128) over the activation the GPU formed, SwiGLU restated in numpy on gate's and
    up's bf16 outputs and rotated by the oracle; the one launch and its two-launch form agree bit for bit at 1..16 rows,
    and row r of every batch has the bits of the single-row call."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    blocks = exl3.default_blocks(exl3.cu_count())
    g, u = (exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(5120, 17408, bits, 70 + i, nm)), blocks)
            for i, nm in enumerate(("gate", "up")))
    down = Layer(env, oracle, 17408, 5120, bits, 72)
    lins = [g, u, down.lin]
    kern.set_option("chain_down_units", down_units)  # (down in its own partition, or in shorter programs; before the workspace)
    ws = exl3.Workspace(lins, 16)
    xd = dev_u16(torch, synth.activations(16, 5120, 4))

    def run(m, x=None):
        yg, yu = (torch.zeros((m, 17408), dtype=torch.bfloat16, device="cuda") for _ in range(2))
        y = torch.zeros((m, 5120), dtype=torch.float32, device="cuda")
        exl3.mlp_forward(g, u, down.lin, xd[:m] if x is None else x, exl3.Dtype.Bf16, yg, yu, y, exl3.Dtype.F32, m, ws)
        torch.cuda.synchronize()
        return yg, yu, y

    try:
        assert exl3.mlp_forward_launches(g, u, down.lin, 1, exl3.Dtype.F32, ws) == 1
        one = {m: run(m) for m in (1, 3, 8, 16)}
        kern.set_option("mlp_chain", 0)
        for m, got in one.items():
            assert exl3.mlp_forward_launches(g, u, down.lin, m, exl3.Dtype.F32, ws) == 0
            for a, b in zip(got, run(m)):
                assert torch.equal(a, b), m
        kern.set_option("mlp_chain", 1)
        # gate and up: the grouped launch's bits
        want = [torch.zeros((3, 17408), dtype=torch.bfloat16, device="cuda") for _ in range(2)]
        exl3.forward_group([g, u], xd[:3], exl3.Dtype.Bf16, want, exl3.Dtype.Bf16, 3, ws)
        torch.cuda.synchronize()
        assert torch.equal(one[3][0], want[0]) and torch.equal(one[3][1], want[1])
        # rows of a batch against the single-row call
        for r in (0, 2, 7, 15):
            single = run(1, xd[r:r + 1])
            for m in (3, 8, 16):
                if r < m:
                    assert all(torch.equal(a[r], b[0]) for a, b in zip(one[m], single)), (m, r)
        # down against the reference over the activation the GPU formed
        yg, yu, y = one[3]
        f64 = lambda t: (t.view(torch.int16).cpu().numpy().view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        def bf16r(a):
            w = np.ascontiguousarray(a, np.float32).view(np.uint32)
            return (((w + 0x7FFF + ((w >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32).astype(np.float64)
        gq, uq = f64(yg), f64(yu)
        act = bf16r(bf16r(gq / (1.0 + np.exp(-gq))) * uq)
        o = oracle.Exl3(down.t.k, down.t.n, down.t.bits, down.t.trellis, down.t.suh, down.t.svh)
        xh = oracle.rotate_input_ref(o, act)  # fp16 bits [m][k]
        ref = down.reference(torch, torch.from_numpy(np.ascontiguousarray(xh).view(np.int16)).cuda().view(torch.float16), torch.float64)
        got = y.cpu().numpy().astype(np.float64)
        rms = np.sqrt((ref ** 2).mean())
        # (the GPU's exponential is the hardware's approximate one: an activation can land on the other side of a bf16
        # tie, which moves an output by about 1e-3 of the rms; the stage-wise bound of the plain linear is 1e-4)
        assert np.abs(got - ref).max() / rms < 5e-3
        assert ws.chain_status() == 0
    finally:
        kern.set_option("mlp_chain", 1)
        kern.set_option("chain_down_units", 0)


@pytest.mark.parametrize("shape", ["gate_up", "down"])
@pytest.mark.parametrize("m", [128, 300, 512, 1024, 2048, 3072])
def test_exl3_prefill_at_full_size(env, oracle, shape, m):
    """Prompt rows with 1 % outlier channels x20 through the MFMA GEMM, including the tiles cut along K and the reduce
    kernel: 3072 rows run over tiles decoded once per call; 128, 300, 512 (the chunks a prompt usually comes in) and 2048
    rows decode inside the GEMM, at the real strides and with the schedule the launcher picks: a K cut for one or two
    rows of output tiles (512 rows x 17408 columns, 136 tiles: stream-K), at 1024 rows x 17408 columns equal runs of 85 k
    tiles over all 272 tiles, at 2048 rows runs of 170 over all 544 tiles for 5120 x 17408, stream-K over all 160
    tiles for 17408 x 5120.
    Stage by stage against the GPU's own rotated input (1e-4 of the rms), and end to end against the reference's f64
    linear on the bf16 inputs for the reference's row sample (crates/fe-fp4/src/bin/fp4-check.rs:96)."""
    torch, exl3, kern = env
    k, n = SHAPES[shape]
    layer = Layer(env, oracle, k, n, 4, 77)
    xd, xh, got, got_bf16, ws = run_rows(env, layer, m, 11, outliers=True)
    check(got, got_bf16, layer.reference(torch, xh, torch.float32), 1e-4)
    again = run_rows(env, layer, m, 11, outliers=True)[2]
    assert np.array_equal(again, got)  # deterministic
    rows = sorted({0, 1, 17, 127, min(128, m - 1), m // 2, m - 1})
    assert end_to_end(oracle, layer, xd, rows, got[rows]) < 2e-3


@pytest.mark.parametrize("m,shape", [(1, "gate_up"), (16, "gate_up"), (1, "down"), (40, "down"), (64, "gate_up"),
                                     (1024, "gate_up"), (2048, "gate_up"), (2048, "down")])
def test_nvfp4_at_full_size(env, oracle, m, shape):
    """The NVFP4 linear at the layer's shapes: the GEMV at 1, 16, 40 rows (three groups of 16 in a pass, K cut 12 ways on
    17408 x 5120) and 64 rows (two passes); at 1024 rows on 5120 x 17408 the GEMM as equal runs of 85 k tiles over all 272 tiles; at 2048
    rows the GEMM on the stream-K schedule
    (5120 x 17408: runs of 170 k tiles over all 544 tiles; 17408 x 5120: stream-K over all 160 tiles, 272 k tiles each)."""
    torch, exl3, kern = env
    from ferrite_amd import fp4, synth
    k, n = SHAPES[shape]
    fk = fp4.Kernels.load()
    host = synth.fp4_linear(n, k, 20251, input_scale=1.0)
    lin = host.upload()
    ws = fp4.Workspace(m, k)
    xd = dev_u16(torch, synth.activations(m, k, 5))
    y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.forward(fk, ws, y, n, xd, k, m)
    torch.cuda.synchronize()
    codes, sf_tiled = ws.read(m, k)
    sfa = oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16)
    # the quantizer at this size, bit for bit on sampled rows
    xb = synth.activations(m, k, 5)
    for r in sorted({0, m // 2, m - 1}):
        wc, wsf = oracle.quant_fp4(xb[r:r + 1], lin.g)
        assert np.array_equal(codes[r:r + 1], wc) and np.array_equal(sfa[r:r + 1], wsf)
    a = torch.from_numpy(oracle.dequant_fp4(codes, sfa, 1.0)).cuda()
    w = torch.from_numpy(oracle.dequant_fp4(host.codes, host.sf, 1.0)).cuda()
    ref = ((a.double() if m <= 64 else a) @ (w.double().T if m <= 64 else w.T)).double().cpu().numpy() * host.alpha.astype(np.float64)
    got = y.float().cpu().numpy().astype(np.float64)
    scale = np.abs(ref).max(axis=1, keepdims=True).clip(1e-20)
    assert (np.abs(got - ref) / scale).max() < 8e-3  # fp4-check.rs:134-144
    assert (np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2 * scale)).max() < 1e-2


@pytest.mark.parametrize("shape", ["gate_up", "down"])
def test_fp8_at_full_size(env, oracle, shape):
    """The FP8 linear on the 8-bit matrix instruction at 2048 rows and the layer's shapes (one piece a program with a K cut
    for 5120 x 17408, stream-K over all 160 tiles for 17408 x 5120): quantizer bit for bit on sampled rows, the GEMM
    against an f64 product over the same codes on the reference's row sample (crates/fe-fp4/src/bin/fp4-check.rs:96)."""
    torch, exl3, kern = env
    from ferrite_amd import fp4, synth
    k, n = SHAPES[shape]
    m = 2048
    fk = fp4.Kernels.load()
    host = synth.fp8_linear(n, k, 20252, input_scale=0.05, weight_scale=0.003)
    lin = host.upload()
    ws = fp4.Workspace(m, k)
    xb = synth.activations(m, k, 6)
    y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    lin.forward(fk, ws, y, n, dev_u16(torch, xb), k, m)
    torch.cuda.synchronize()
    codes = ws.read_fp8(m, k)
    rows = sorted({0, 1, 17, 127, 128, m // 2, m - 1})
    for r in rows[:3]:
        assert np.array_equal(codes[r], oracle.quant_fp8_row(xb[r], lin.g))
    a = np.stack([oracle.dequant_fp8_row(codes[r], 1.0) for r in rows])
    w = np.stack([oracle.dequant_fp8_row(host.codes[c], 1.0) for c in range(n)])
    ref = oracle.ref_gemm(a, w).astype(np.float64) * host.alpha.astype(np.float64)[None, :]
    got = y[rows].float().cpu().numpy().astype(np.float64)
    scale = np.abs(ref).max(axis=1, keepdims=True).clip(1e-20)
    assert (np.abs(got - ref) / scale).max() < 8e-3
    assert (np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2 * scale)).max() < 1e-2


def test_swiglu_front_at_full_size(env, oracle):
    """The fused gate|up front at the layer's size (2048 rows, 2 x 17408 columns over K = 5120): SwiGLU and the NVFP4
    re-quantization in the GEMM's epilogue against the same steps done on the host from the unfused bf16 output of the
    same linear, on sampled rows. silu runs on the hardware exponential and reciprocal, so a bf16 rounding of it may
    fall on the other side of a tie: such flips are counted, and dequantized the two agree to one step of an element."""
    torch, exl3, kern = env
    from ferrite_amd import fp4, synth
    k, inter = SHAPES["gate_up"]
    m = 2048
    fk = fp4.Kernels.load()
    g, u = synth.fp4_linear(inter, k, 1, name="gate"), synth.fp4_linear(inter, k, 2, name="up")
    fused = fp4.HostLinear.fuse([("gate", g.codes, g.sf, 1.0, 1.0), ("up", u.codes, u.sf, 1.0, 1.0)])
    fused.alpha[:] = fused.alpha * np.float32(0.01)  # outputs of order 1, where silu bends
    sw = fused.into_swiglu().upload()
    del g, u, fused
    ws, act = fp4.Workspace(m, k), fp4.Workspace(m, inter)
    xd = dev_u16(torch, synth.activations(m, k, 9))
    yi = torch.zeros((m, 2 * inter), dtype=torch.bfloat16, device="cuda")
    sw.forward(fk, ws, yi, 2 * inter, xd, k, m)
    down_g = 0.5
    sw.forward_swiglu(fk, ws, act, xd, k, m, down_g)
    torch.cuda.synchronize()
    rows = sorted({0, 1, 17, 127, 128, 255, 256, m // 2, m - 1})
    bits = yi[rows].view(torch.int16).cpu().numpy().view(np.uint16)
    y = (bits.astype(np.uint32) << 16).view(np.float32).reshape(len(rows), inter // 8, 2, 8)
    gate, up = y[:, :, 0, :].reshape(len(rows), inter).astype(np.float64), y[:, :, 1, :].reshape(len(rows), inter)

    def bf16_round(x):
        b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
        return (((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint32) << 16).view(np.float32)

    want_act = bf16_round(bf16_round((gate / (1.0 + np.exp(-gate))).astype(np.float32)) * up)
    want_bits = (want_act.view(np.uint32) >> 16).astype(np.uint16)
    want_codes, want_sf = oracle.quant_fp4(want_bits, down_g)
    codes, sf_tiled = act.read(m, inter)
    sfa = oracle.untile_scales(sf_tiled, m, inter // 16).reshape(m, inter // 16)
    bad_sf, bad_codes = (sfa[rows] != want_sf).mean(), (codes[rows] != want_codes).mean()
    assert bad_sf < 2e-3 and bad_codes < 5e-3, (bad_sf, bad_codes)
    a_got, a_want = oracle.dequant_fp4(codes[rows], sfa[rows], 1.0), oracle.dequant_fp4(want_codes, want_sf, 1.0)
    assert np.abs(a_got - a_want).max() <= 0.26 * np.abs(a_want).max()
