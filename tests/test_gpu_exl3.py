"""GPU parity of the EXL3 path against the CPU oracle, through the C ABI. Mirrors the reference's check binaries:
exl3-gpucheck (reconstruct), exl3-gemvcheck (rot_in, GEMV at rows 1..64, untouched rows, row invariance, fused
residual add), exl3-tpcheck (slices) and exl3-detcheck (determinism with a shared workspace)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 5, 8, 9, 16, 17, 33, 64]  # crates/fe-exl3/src/bin/exl3-gemvcheck.rs:53


@pytest.fixture(scope="module")
def env():
    import torch
    from ferrite_amd import exl3
    assert torch.cuda.is_available()
    kern = exl3.Kernels.load()
    return torch, exl3, kern


def to_oracle(oracle, t):
    return oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def bf16_to_f64(a):
    return (a.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_reconstruct_hat_is_bit_exact(env, oracle, bits):
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(256, 384, bits, 100 + bits)
    d = exl3.DeviceExl3.upload(t)
    out = torch.zeros((t.k, t.n), dtype=torch.int16, device="cuda")
    kern.reconstruct_hat_f16(d.view, out)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    want = oracle.w_hat_f16(to_oracle(oracle, t))
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} values differ"


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("strips", [True, False])
def test_hot_loop_decoder_is_bit_exact(env, oracle, bits, strips):
    """The decoder of the hot loops (decode_lane: boundary windows, one extract per state; the GEMV, the decoding GEMM
    and exl3_hat_tiles_b* all run it) bit for bit against decode_tile (crates/fe-exl3/src/cpu.rs:57-69): the tiles that
    exl3_hat_tiles_b* leaves with the linear are exactly decode_lane's fp16 values, read back and un-swizzled. An odd
    count of column blocks (the last 256-column tile half empty) and both trellis layouts."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(384, 384, bits, 300 + bits)
    d = exl3.DeviceExl3.upload_strips(t) if strips else exl3.DeviceExl3.upload(t)
    lin = exl3.Linear.new(kern, d, 64)
    lin.keep_decoded()
    got = lin.decoded_w_hat()
    want = oracle.w_hat_f16(to_oracle(oracle, t))
    assert got.shape == want.shape
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} values differ"


@pytest.mark.parametrize("bits", [3, 4, 5])
def test_fenced_handoff_gives_the_same_bits(env, bits):
    """The hand-off of segment sums between programs is written with write-through stores, acknowledged, a relaxed
    agent-scope arrival, and loads that pass the L2. Option handoff_fenced runs the same partition with the memory model's
    own means instead (plain stores, release fence, arrival, acquire fence, plain loads): slow, and required to give the
    same bits, single linears and grouped launches, call after call on one workspace."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    ts = [synth.exl3_tensor(1024, n, bits, 500 + bits + i) for i, n in enumerate((640, 384))]
    lins = [exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(11 + 4 * i, 1, 4, 4)) for i, t in enumerate(ts)]  # uneven runs
    ws = exl3.Workspace(lins, 16)
    try:
        for rows in (1, 5, 16):
            x = dev_u16(torch, synth.activations(rows, 1024, rows))
            outs = {}
            for fenced in (0, 1, 0, 1):
                kern.set_option("handoff_fenced", fenced)
                ys = [torch.zeros((rows, l.n), dtype=torch.float32, device="cuda") for l in lins]
                single = torch.zeros((rows, lins[0].n), dtype=torch.float32, device="cuda")
                lins[0].forward(x, exl3.Dtype.Bf16, single, exl3.Dtype.F32, rows, ws)
                exl3.forward_group(lins, x, exl3.Dtype.Bf16, ys, exl3.Dtype.F32, rows, ws)
                torch.cuda.synchronize()
                got = [single.cpu()] + [y.cpu() for y in ys]
                if fenced in outs:
                    assert all(torch.equal(a, b) for a, b in zip(got, outs[fenced]))
                outs[fenced] = got
            assert all(torch.equal(a, b) for a, b in zip(outs[0], outs[1])), rows
            assert torch.equal(outs[0][0], outs[0][1])  # a member of a group has the bits of its own forward
    finally:
        kern.set_option("handoff_fenced", 0)


def test_reconstruct_bf16_within_one_ulp(env, oracle):
    """crates/fe-exl3/src/bin/exl3-gpucheck.rs:58-98: GPU f32 math vs the f64 reference: at most 1 bf16 ulp apart, more
    only as f32 cancellation noise near zero (absolute error below 1e-4 of the tensor's rms); [n][k] is the exact
    transpose of [k][n]."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(384, 256, 4, 7)
    d = exl3.DeviceExl3.upload(t)
    res = {}
    for layout in ("KN", "NK"):
        out = torch.zeros(t.k * t.n, dtype=torch.int16, device="cuda")
        # a scratch of 128 columns forces the column-sliced path
        scratch = torch.empty(t.k * 128, dtype=torch.float32, device="cuda")
        kern.reconstruct_bf16(d.view, out, layout, scratch)
        torch.cuda.synchronize()
        res[layout] = out.cpu().numpy().view(np.uint16).reshape((t.k, t.n) if layout == "KN" else (t.n, t.k))
    got = res["KN"]
    assert np.array_equal(res["NK"], got.T)
    want = oracle.weight_bf16(to_oracle(oracle, t), layout="KN")
    ordered = lambda h: np.where(h & 0x8000, -(h & 0x7FFF).astype(np.int32), h.astype(np.int32))
    ulp = np.abs(ordered(got) - ordered(want))
    rms = np.sqrt((bf16_to_f64(want) ** 2).mean())
    err = np.abs(bf16_to_f64(got) - bf16_to_f64(want)) / rms
    assert np.all((ulp <= 1) | (err < 1e-4))
    assert (ulp > 0).mean() < 0.02


def run_forward(torch, exl3, lin, ws, xd, rows, y_dtype, prefill=None):
    f32 = y_dtype in (exl3.Dtype.F32, exl3.Dtype.F32Add)
    if prefill is None:
        y = torch.full((64 if rows <= 64 else rows, lin.n), float("nan"), dtype=torch.float32 if f32 else torch.bfloat16, device="cuda")
    else:
        y = prefill
    lin.forward(xd, exl3.Dtype.Bf16, y, y_dtype, rows, ws)
    torch.cuda.synchronize()
    return y


def check_linear(env, oracle, t, plan, strips, rows_list=ROWS, seed=1):
    torch, exl3, kern = env
    from ferrite_amd import synth
    o = to_oracle(oracle, t)
    mr = 64
    xb = synth.activations(mr, t.k, seed)
    x64 = bf16_to_f64(xb)
    d = exl3.DeviceExl3(t, strips)
    lin = exl3.Linear.with_plan(kern, d, plan)
    ws = exl3.Workspace([lin], mr)
    xd = dev_u16(torch, xb)
    # rot_in alone vs the f64 reference: a rare 1-ulp tie flip allowed (exl3-gemvcheck.rs:79-88)
    lin.rotate_input(xd, exl3.Dtype.Bf16, mr, ws)
    torch.cuda.synchronize()
    xh_gpu = ws.xh(mr, t.k)
    xh_ref = oracle.rotate_input_ref(o, x64)
    # (more than one ulp apart only where cancellation leaves a value near zero: the f32 butterflies' rounding, 1e-7 of the
    # inputs, is then several ulps of the result)
    gv, rv = xh_gpu.view(np.float16).astype(np.float64), xh_ref.view(np.float16).astype(np.float64)
    far = (np.abs(xh_gpu.astype(np.int32) - xh_ref.astype(np.int32)) > 1) & (np.abs(gv - rv) > 1e-6 * np.sqrt((rv ** 2).mean()))
    assert not far.any() and (xh_gpu != xh_ref).mean() < 2e-3
    hat = oracle.w_hat_f16(o)
    yref = oracle.gemv_ref(o, hat, xh_gpu)  # on the GPU's own rotated input: what is left is fp32 summation order
    first5 = {}
    for rows in rows_list:
        y = run_forward(torch, exl3, lin, ws, xd, rows, exl3.Dtype.F32).cpu().numpy().astype(np.float64)
        yb = run_forward(torch, exl3, lin, ws, xd, rows, exl3.Dtype.Bf16).view(torch.int16).cpu().numpy().view(np.uint16)
        ref = yref[:rows]
        rms = np.sqrt((ref ** 2).mean())
        rel_max = np.abs(y[:rows] - ref).max() / rms
        assert rel_max < 1e-4, (rows, rel_max)  # exl3-gemvcheck.rs:117-121
        # the north-star bar: max relative error 1e-2 (floored at 1e-2 of the rms)
        assert (np.abs(y[:rows] - ref) / np.maximum(np.abs(ref), 1e-2 * rms)).max() < 1e-2
        # bf16 output within one rounding of the exact value (exl3-gemvcheck.rs:106-110)
        e = np.abs(bf16_to_f64(yb[:rows]) - ref)
        assert np.all(e <= np.abs(ref) / 256.0 + 1e-5 * rms), rows
        # rows past `rows` untouched (exl3-gemvcheck.rs:113-116)
        if rows < 64:
            assert np.isnan(y[rows:]).all()
        if rows >= 5:  # row invariance (exl3-gemvcheck.rs:124-141): a row's bits do not depend on the row count
            if 0 not in first5:
                first5[0] = y[:5].copy()
            else:
                assert np.array_equal(first5[0].view(np.uint64), y[:5].view(np.uint64)), rows
    # fused residual add: y (bf16, prefilled with 1.5) += x @ W, 5 rows (exl3-gemvcheck.rs:142-168)
    rows = 5
    pre = torch.full((mr, t.n), 1.5, dtype=torch.bfloat16, device="cuda")
    ya = run_forward(torch, exl3, lin, ws, xd, rows, exl3.Dtype.Bf16Add, prefill=pre).view(torch.int16).cpu().numpy().view(np.uint16)
    want = 1.5 + yref[:rows]
    rms = np.sqrt((yref[:rows] ** 2).mean())
    assert np.all(np.abs(bf16_to_f64(ya[:rows]) - want) <= np.abs(want) / 256.0 + 1e-5 * rms)
    assert (ya[rows:] == 0x3FC0).all()
    pre32 = torch.full((mr, t.n), 0.25, dtype=torch.float32, device="cuda")
    y32 = run_forward(torch, exl3, lin, ws, xd, rows, exl3.Dtype.F32Add, prefill=pre32).cpu().numpy().astype(np.float64)
    assert np.abs(y32[:rows] - 0.25 - yref[:rows]).max() / rms < 1e-4 and (y32[rows:] == 0.25).all()
    return lin, ws, xd, yref


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("ver", [1, 3])
def test_gemv_all_bit_widths(env, oracle, bits, ver):
    """ver 1: sk programs per column block; ver 3: occ programs per CU over the whole tensor."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(512, 256, bits, 20 + bits)
    check_linear(env, oracle, t, exl3.Plan(2, 4, ver, 2), strips=True, rows_list=[1, 5, 16, 17, 64])


@pytest.mark.parametrize("programs,strips", [(1, True), (2, False), (5, True), (7, False), (13, True), (24, False), (1000, True)])
def test_gemv_any_partition(env, oracle, programs, strips):
    """The GEMV cuts the tensor's 24 work units (3 column blocks x 8 blocks of 128 channels) into runs of any length: runs
    that start and end inside a column block, cover whole blocks or several, or are a single unit (plan ver 4: that many
    programs; more programs than units: one a unit)."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(1024, 384, 4, 77)
    check_linear(env, oracle, t, exl3.Plan(programs, 4, 4, 0), strips=strips, rows_list=[1, 2, 5, 8, 9, 16, 17, 64])


def test_programs_sharing_a_workgroup_keep_their_bits(env, oracle):
    """A launch with more programs than the CUs hold at once runs consecutive programs of the partition in one workgroup
    (up to 4 rows). Every program still flushes its own sums to its own slot, so the bits are those of the launch with a
    workgroup per program; both against the oracle."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(4096, 4224, 3, 91)  # 32 x 33 = 1056 units
    plan = exl3.Plan(1056, 1, 4, 0)           # a program a unit: more than 4 per CU
    check_linear(env, oracle, t, plan, strips=True, rows_list=[1, 3, 4])
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), plan)
    ws = exl3.Workspace([lin], 4)
    x = torch.from_numpy(synth.activations(4, t.k, 3).view(np.int16)).cuda()
    outs = []
    try:
        for fuse in (1, 0):
            kern.set_option("fuse", fuse)
            for rows in (1, 4):
                y = torch.full((rows, t.n), float("nan"), dtype=torch.float32, device="cuda")
                lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, rows, ws)
                outs.append(y)
    finally:
        kern.set_option("fuse", 1)
    torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int32), outs[2].view(torch.int32))
    assert torch.equal(outs[1].view(torch.int32), outs[3].view(torch.int32))


@pytest.mark.parametrize("sk,strips", [(1, True), (1, False), (4, True), (8, False), (16, True)])
def test_gemv_splits_and_layouts(env, oracle, sk, strips):
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(1024, 384, 4, 31)
    check_linear(env, oracle, t, exl3.Plan(sk), strips=strips)


def test_gemv_long_k_streams_inputs_in_chunks(env, oracle):
    """K long enough that 64 rows of inputs do not fit LDS at once (one split, 68 load steps, chunks of 4)."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(4352, 128, 3, 5)
    check_linear(env, oracle, t, exl3.Plan(1), strips=True, rows_list=[1, 16, 64])


def test_plan_for_default_and_determinism_with_shared_workspace(env, oracle):
    """crates/fe-exl3/src/bin/exl3-detcheck.rs:36-70: repeated forwards interleaved with a second linear that shares the
    workspace give identical bits."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    a = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(1024, 256, 4, 1)), exl3.default_blocks(exl3.cu_count()))
    b = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(1024, 384, 3, 2)), exl3.default_blocks(exl3.cu_count()))
    assert a.plan.sk > 1 and b.plan.sk > 1
    ws = exl3.Workspace([a, b], 16)
    xa, xb = dev_u16(torch, synth.activations(16, 1024, 3)), dev_u16(torch, synth.activations(16, 1024, 4))
    ya = torch.empty((16, 256), dtype=torch.float32, device="cuda")
    yb = torch.empty((16, 384), dtype=torch.float32, device="cuda")
    first = None
    for it in range(40):
        rows = 1 + (it * 7) % 16
        a.forward(xa, exl3.Dtype.Bf16, ya, exl3.Dtype.F32, 16, ws)
        b.forward(xb, exl3.Dtype.Bf16, yb, exl3.Dtype.F32, rows, ws)
        torch.cuda.synchronize()
        cur = ya.cpu().numpy().copy()
        if first is None:
            first = cur
        assert np.array_equal(first.view(np.uint32), cur.view(np.uint32)), it


def test_tp_slices_match_the_whole(env, oracle):
    """crates/fe-exl3/src/bin/exl3-tpcheck.rs: column slices reproduce their columns, row slices sum to the whole."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(512, 512, 4, 9)
    xb = synth.activations(4, 512, 9)
    xd = dev_u16(torch, xb)

    def fwd(tt, x):
        lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(tt), exl3.Plan(2))
        ws = exl3.Workspace([lin], 4)
        y = torch.empty((4, tt.n), dtype=torch.float32, device="cuda")
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 4, ws)
        torch.cuda.synchronize()
        return y.cpu().numpy().astype(np.float64)

    whole = fwd(t, xd)
    rms = np.sqrt((whole ** 2).mean())
    cols = fwd(t.slice_cols([(128, 256), (384, 512)]), xd)
    assert np.array_equal(cols, np.concatenate([whole[:, 128:256], whole[:, 384:512]], axis=1))
    parts = fwd(t.slice_rows(0, 256), dev_u16(torch, xb[:, :256])) + fwd(t.slice_rows(256, 512), dev_u16(torch, xb[:, 256:]))
    assert np.abs(parts - whole).max() / rms < 2e-5  # exl3-tpcheck.rs:103-105


@pytest.mark.parametrize("bits,m", [(4, 200), (3, 129), (5, 65), (2, 300), (6, 257), (8, 70)])
def test_prefill_gemm_matches_the_oracle(env, oracle, bits, m):
    """More than 64 rows take the LDS-staged MFMA GEMM; same contract as the GEMV (f64 reference on the GPU's own xh)."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(512, 256, bits, 40 + bits)
    o = to_oracle(oracle, t)
    xb = synth.activations(m, t.k, 3, outliers=True)
    for strips in (True, False):
        lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3(t, strips), exl3.Plan(2))
        ws = exl3.Workspace([lin], m)
        xd = dev_u16(torch, xb)
        y = torch.full((m + 3, t.n), float("nan"), dtype=torch.float32, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
        yb = torch.zeros((m, t.n), dtype=torch.bfloat16, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, yb, exl3.Dtype.Bf16, m, ws)
        torch.cuda.synchronize()
        xh = ws.xh(m, t.k)
        ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), xh)
        got = y.cpu().numpy().astype(np.float64)
        rms = np.sqrt((ref ** 2).mean())
        assert np.abs(got[:m] - ref).max() / rms < 1e-4
        assert np.isnan(got[m:]).all()
        e = np.abs(bf16_to_f64(yb.view(torch.int16).cpu().numpy().view(np.uint16)) - ref)
        assert np.all(e <= np.abs(ref) / 256.0 + 1e-5 * rms)
        # end to end against the reference linear on the bf16 inputs themselves (f64 all the way; this adds the fp16
        # rounding of the rotated inputs, which the reference's GPU path has too): max relative error 1e-2, with the
        # denominator floored at the output's rms so that sums that cancel to ~0 do not define the scale
        lin64 = oracle.linear_f64(o, bf16_to_f64(xb), threads=4)
        assert (np.abs(got[:m] - lin64) / np.maximum(np.abs(lin64), np.sqrt((lin64 ** 2).mean()))).max() < 1e-2


@pytest.mark.parametrize("m,n,forced", [(2400, 3968, 2), (6600, 4096, 3)])
def test_prefill_on_the_stream_k_schedule(env, oracle, m, n, forced):
    """Stream-K: the prefill GEMM walks the tiles' k tiles laid end to end, every program a contiguous run; the pieces of
    a tile meet through the workspace and the last arriver adds them in piece order. 2400 x 3968 over K = 1024: 10 x 16 =
    160 tiles of 16 k tiles on 256 CUs (forced: 2, runs over all tiles), the last row tile ragged, the last column tile
    half; the library picks the schedule for it by itself (option gemm_sk = 1 gives the bits of the forced schedule).
    6600 x 4096: 416 tiles, one whole round and runs of 10 k tiles over the other 160 (forced: 3): its own choice for the
    decoding GEMM, not for the GEMM over decoded tiles, whose programs would stream the fp16 weights past the L2 (there
    gemm_sk = 1 gives the bits of the one-piece schedule). Repeats give the same bits (arrival order does not matter,
    counters return to zero); the one-piece schedule (0) differs by the order of the f32 sums; an add output mode;
    against the oracle."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(1024, n, 4, 77)
    xd = dev_u16(torch, synth.activations(m, t.k, 8, outliers=True))
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 256)
    kern.set_option("hat_rows", 65)
    ws = exl3.Workspace([lin], m)

    def run(sk, hat, dt=exl3.Dtype.F32, pre=float("nan")):
        kern.set_option("gemm_sk", sk)
        kern.set_option("hat_rows", 65 if hat else 0)
        y = torch.full((m + 1, t.n), pre, dtype=torch.float32, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, y, dt, m, ws)
        torch.cuda.synchronize()
        out = y.cpu().numpy()
        assert np.array_equal(out[m].view(np.uint32), np.full(t.n, pre, dtype=np.float32).view(np.uint32))
        return out[:m]

    try:
        o = to_oracle(oracle, t)
        ref = None
        for hat in (False, True):
            want = run(forced, hat)
            for _ in range(4):
                assert np.array_equal(run(forced, hat).view(np.uint32), want.view(np.uint32)), hat
            pieces = run(0, hat)
            own = pieces if hat and forced == 3 else want
            assert np.array_equal(run(1, hat).view(np.uint32), own.view(np.uint32)), hat
            rms = np.sqrt((pieces.astype(np.float64) ** 2).mean())
            assert np.abs(want.astype(np.float64) - pieces).max() < 2e-6 * rms, hat
            added = run(forced, hat, exl3.Dtype.F32Add, 0.25)
            plus = want.astype(np.float64) + 0.25  # (the add is fused into the last product: one rounding, not two)
            assert (np.abs(added - plus) <= (np.abs(plus) + np.abs(want)) * 2.0 ** -23).all(), hat
            rows = sorted({r for r in (0, 1, 17, 255, 256, 1023, 1024, 2047, 2048, 2303, 2304, m // 2, m - 1) if r < m})
            if ref is None:
                ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), ws.xh(m, t.k)[rows])
            assert np.abs(want[rows].astype(np.float64) - ref).max() / np.sqrt((ref ** 2).mean()) < 1e-4, hat
    finally:
        kern.set_option("gemm_sk", 1)
        kern.set_option("hat_rows", 3072)


def test_argument_errors_are_results_not_crashes(env):
    torch, exl3, kern = env
    from ferrite_amd import synth
    from ferrite_amd._lib import FeError
    t = synth.exl3_tensor(256, 128, 4, 1)
    d = exl3.DeviceExl3.upload_strips(t)
    with pytest.raises(FeError):
        exl3.Linear.with_plan(kern, d, exl3.Plan(3))  # 4 load steps do not divide by 3
    with pytest.raises(FeError):
        exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(256, 128, 7, 1)), exl3.Plan(1))
    lin = exl3.Linear.with_plan(kern, d, exl3.Plan(2))
    ws = exl3.Workspace([lin], 4)
    x = dev_u16(torch, synth.activations(8, 256, 1))
    y = torch.zeros((8, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(FeError):
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 0, ws)
    with pytest.raises(FeError):
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 5, ws)  # workspace holds 4 rows
    small = exl3.Workspace([exl3.Linear.with_plan(kern, d, exl3.Plan(1))], 4)
    with pytest.raises(FeError):
        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 4, small)  # no room for split partials
    with pytest.raises(FeError):
        kern.reconstruct_hat_f16(d.view, y)  # strips layout
    lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 4, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y[:4]).all()


def test_prefill_gemm_tiles_cut_or_whole(env, oracle):
    """Several 256 x 256 tiles with an odd count of 128-column blocks: computed whole (option gemm_splits = 1) and cut along K
    with the reduce kernel (the default for a nearly empty last round)."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    m = 300
    t = synth.exl3_tensor(1024, 384, 4, 77)
    o = to_oracle(oracle, t)
    xb = synth.activations(m, t.k, 5, outliers=True)
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 256)
    ws = exl3.Workspace([lin], m)
    xd = dev_u16(torch, xb)

    def run():
        y = torch.full((m + 2, t.n), float("nan"), dtype=torch.float32, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
        torch.cuda.synchronize()
        out = y.cpu().numpy().astype(np.float64)
        assert np.isnan(out[m:]).all()
        return out[:m]

    cut = run()
    assert np.array_equal(cut, run())
    kern.set_option("gemm_splits", 1)
    whole = run()
    kern.set_option("gemm_splits", 8)
    ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), ws.xh(m, t.k))
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(cut - ref).max() / rms < 1e-4
    assert np.abs(whole - ref).max() / rms < 1e-4
    # accumulate into y (y dtype flag 3: f32, add)
    y = torch.ones((m, t.n), dtype=torch.float32, device="cuda")
    lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32Add, m, ws)
    torch.cuda.synchronize()
    assert np.abs(y.cpu().numpy().astype(np.float64) - 1.0 - ref).max() / rms < 1e-4


def test_tuner_returns_a_fitting_plan(env):
    """ferrite_amd.exl3.tune (the role of exl3-tune): every candidate is timed at 1 and 16 rows, the best one fits."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    t = synth.exl3_tensor(1024, 512, 4, 3)
    best, table = exl3.tune(kern, t, iters=2, copies_bytes=1 << 20)
    assert best.ver == 3 and best.occ in (2, 3, 4, 5) and len(table) >= 4
    assert all(us1 > 0 and us16 > 0 for _, us1, us16 in table)
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), best)
    assert lin.plan.occ == best.occ


@pytest.mark.parametrize("k,sk", [(1024, 1), (1024, 4), (2048, 16), (1024, 8), (1024, 16), (1280, 2), (1280, 4)])
def test_forward_rotates_inside_the_gemv_or_before_it(env, oracle, k, sk):
    """forward() for few rows is one launch (the GEMV rotates its own input and leaves it in the workspace) while a
    program's share of the rotation stays small, two launches otherwise (and always with the "fused_rot" option off). Both
    give the same bits, in y and in the workspace's rotated input, for bf16 and f32 inputs."""
    torch, exl3, kern = env
    from ferrite_amd import _lib, synth
    from ferrite_amd._lib import check
    t = synth.exl3_tensor(k, 384, 4, 70 + sk)
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(sk=sk, wk=1, ver=1, occ=2))
    # one launch while a program's share of the rotation stays small: rows x 128-channel blocks of its run <= 16
    programs = min(3 * sk, 3 * (k // 128))
    for rows in (1, 4, 7, 16, 33, 64, 65):
        assert lin.forward_is_one_launch(rows) == (rows <= 64 and rows * -(-(3 * (k // 128)) // programs) <= 16), rows
    ws = exl3.Workspace([lin], 64)
    xb = synth.activations(64, k, 8, outliers=True)
    xd = dev_u16(torch, xb)
    xf = xd.view(torch.bfloat16).float().contiguous()
    for rows in (1, 7, 16, 33, 64):
        for x, xdt in ((xd, exl3.Dtype.Bf16), (xf, exl3.Dtype.F32)):
            out = {}
            for mode in ("fused", "separate"):
                kern.set_option("fused_rot", 0 if mode == "separate" else 1)
                check(_lib.lib().fe_hip_memset_d8(ws.xh_ptr, 0x7e, 64 * k * 2, None))  # fp16 NaNs: stale inputs would show
                y = torch.full((65, lin.n), float("nan"), dtype=torch.float32, device="cuda")
                lin.forward(x, xdt, y, exl3.Dtype.F32, rows, ws)
                torch.cuda.synchronize()
                out[mode] = (y.cpu().numpy(), ws.xh(rows, k))
                kern.set_option("fused_rot", 1)
            assert np.array_equal(out["fused"][1], out["separate"][1]), (rows, xdt)
            assert np.array_equal(out["fused"][0][:rows].view(np.uint32), out["separate"][0][:rows].view(np.uint32)), (rows, xdt)
            assert np.isnan(out["fused"][0][rows:]).all()
    # the rotated input the fused launch leaves behind is the oracle's (as for the separate kernel)
    # (outlier channels: the f32 butterflies leave an absolute error, so small results may be off by more than an ulp)
    want = oracle.rotate_input_ref(to_oracle(oracle, t), bf16_to_f64(xb)).view(np.float16).astype(np.float64)
    got = out["fused"][1].view(np.float16).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) / 1024.0 + 1e-5 * np.sqrt((want ** 2).mean()))


@pytest.mark.parametrize("k,sk", [(1024, 2), (1280, 2), (2048, 16)])
def test_forward_on_swiglu_of_gate_and_up(env, k, sk):
    """The down projection of the MLP block takes SwiGLU(gate, up) as its input without the activation being stored:
    the bits of fe_silu_mul into a buffer followed by forward() on it, for every row count (inside the GEMV, in the
    rotation kernel in front of the GEMV, in front of the GEMM) and output mode, gate and up being column ranges of one
    wider array."""
    torch, exl3, kern = env
    from ferrite_amd import route, synth
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, 384, 4, 90 + sk)), exl3.Plan(sk=sk, wk=1, ver=1, occ=2))
    mr = 130
    ws = exl3.Workspace([lin], mr)
    ld = 2 * k + 8
    gu = dev_u16(torch, synth.activations(mr, ld, 21, outliers=True))  # [gate | up | 8 unused columns]
    gate_ptr, up_ptr = gu.data_ptr(), gu.data_ptr() + 2 * k
    seen = set()
    for rows in (1, 3, 16, 40, 64, 65, 130):
        act = torch.zeros((rows, k), dtype=torch.bfloat16, device="cuda")
        route.silu_mul(act, gate_ptr, up_ptr, ld, k, rows)
        seen.add(lin.forward_is_one_launch(rows))
        for ydt, tdt in ((exl3.Dtype.F32, torch.float32), (exl3.Dtype.Bf16Add, torch.bfloat16)):
            want = torch.full((rows + 1, 384), 0.5, dtype=tdt, device="cuda")
            got = torch.full((rows + 1, 384), 0.5, dtype=tdt, device="cuda")
            lin.forward(act.view(torch.int16), exl3.Dtype.Bf16, want, ydt, rows, ws)
            torch.cuda.synchronize()
            xh_want = ws.xh(rows, k).copy()
            lin.forward_swiglu(gate_ptr, up_ptr, ld, got, ydt, rows, ws)
            torch.cuda.synchronize()
            assert np.array_equal(ws.xh(rows, k), xh_want), rows
            a, b = want.view(torch.int32 if tdt == torch.float32 else torch.int16), got.view(torch.int32 if tdt == torch.float32 else torch.int16)
            assert torch.equal(a, b), (rows, ydt)
            assert float(got[rows].float().abs().max()) == 0.5  # the row after the batch is untouched
    assert seen == {True, False}
    from ferrite_amd._lib import FeError
    with pytest.raises(FeError):
        lin.forward_swiglu(gate_ptr, up_ptr, k - 4, got, exl3.Dtype.F32, 1, ws)
    with pytest.raises(FeError):
        lin.forward_swiglu(gate_ptr + 2, up_ptr, ld, got, exl3.Dtype.F32, 1, ws)


@pytest.mark.parametrize("bits,k,ns,sks", [(4, 1024, (384, 128, 256), (2, 4, 1)), (3, 1280, (256, 640), (2, 1)),
                                           (5, 1024, (128, 128, 384, 256), (8, 1, 2, 4)), (4, 2048, (512, 384), (16, 4))])
def test_group_forward_has_the_bits_of_each_members_forward(env, bits, k, ns, sks):
    """Linears of one input (q, k, v; gate, up) in one GEMV launch: every member's programs are those of its own launch,
    so each output has the bits of the member's forward(), for every row count, input and output type, with the input
    rotated inside the GEMV (one launch) or by one launch for all members (two). Groups that cannot share a launch
    (different bits, a workspace without the room) run member by member."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    lins = []
    for i, (n, sk) in enumerate(zip(ns, sks)):
        t = synth.exl3_tensor(k, n, bits, 300 + 7 * i + bits)
        lins.append(exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t) if i % 2 == 0 else exl3.DeviceExl3(t, False),
                                          exl3.Plan(sk=sk, wk=1, ver=1, occ=2)))
    ws = exl3.Workspace(lins, 64)
    xb = synth.activations(64, k, 11, outliers=True)
    xd = dev_u16(torch, xb)
    xf = xd.view(torch.bfloat16).float().contiguous()
    seen = set()
    assert exl3.forward_group_launches(lins, 65, exl3.Workspace(lins, 65)) == 0  # more than a GEMV pass: member by member
    for rows in (1, 3, 8, 16, 17, 40, 64):
        launches = exl3.forward_group_launches(lins, rows, ws)
        assert launches == (1 if all(l.forward_is_one_launch(rows) for l in lins) else 2), rows
        seen.add(launches)
        for x, xdt in ((xd, exl3.Dtype.Bf16), (xf, exl3.Dtype.F32)):
            for ydt, tdt in ((exl3.Dtype.F32, torch.float32), (exl3.Dtype.Bf16, torch.bfloat16), (exl3.Dtype.Bf16Add, torch.bfloat16)):
                fill = 1.5 if ydt == exl3.Dtype.Bf16Add else float("nan")
                want = [torch.full((65, n), fill, dtype=tdt, device="cuda") for n in ns]
                got = [torch.full((65, n), fill, dtype=tdt, device="cuda") for n in ns]
                for lin, y in zip(lins, want):
                    lin.forward(x, xdt, y, ydt, rows, ws)
                exl3.forward_group(lins, x, xdt, got, ydt, rows, ws)
                torch.cuda.synchronize()
                for a, b in zip(want, got):
                    ia, ib = (a.view(torch.int32), b.view(torch.int32)) if tdt == torch.float32 else (a.view(torch.int16), b.view(torch.int16))
                    assert torch.equal(ia, ib), (rows, xdt, ydt)
    assert 1 in seen
    # twice in a row on the same workspace: the arrival counters are back at zero after each launch
    y1 = [torch.zeros((4, n), dtype=torch.float32, device="cuda") for n in ns]
    y2 = [torch.zeros((4, n), dtype=torch.float32, device="cuda") for n in ns]
    exl3.forward_group(lins, xd, exl3.Dtype.Bf16, y1, exl3.Dtype.F32, 4, ws)
    exl3.forward_group(lins, xd, exl3.Dtype.Bf16, y2, exl3.Dtype.F32, 4, ws)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(y1, y2))
    # member by member: switched off, one member alone, a member of other bits, a workspace made for one small linear
    kern.set_option("group", 0)
    assert exl3.forward_group_launches(lins, 1, ws) == 0
    y3 = [torch.zeros((4, n), dtype=torch.float32, device="cuda") for n in ns]
    exl3.forward_group(lins, xd, exl3.Dtype.Bf16, y3, exl3.Dtype.F32, 4, ws)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(y1, y3))
    kern.set_option("group", 1)
    assert exl3.forward_group_launches(lins[:1], 1, ws) == 0
    other = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, 128, bits + 1, 5)), exl3.Plan(sk=1, wk=1, ver=1, occ=2))
    mixed = [lins[0], other]
    ws_mixed = exl3.Workspace(mixed, 16)
    assert exl3.forward_group_launches(mixed, 1, ws_mixed) == 0
    y4 = [torch.zeros((4, ns[0]), dtype=torch.float32, device="cuda"), torch.zeros((4, 128), dtype=torch.float32, device="cuda")]
    exl3.forward_group(mixed, xd, exl3.Dtype.Bf16, y4, exl3.Dtype.F32, 4, ws_mixed)
    torch.cuda.synchronize()
    assert torch.equal(y4[0], y1[0])
    small = exl3.Workspace([min(lins, key=lambda l: l.n * l.plan.sk)], 16)  # no room for every member's partial sums
    assert exl3.forward_group_launches(lins, 16, small) == 0


@pytest.mark.parametrize("bits,n,strips", [(2, 384, True), (3, 256, False), (4, 640, True), (5, 384, False), (6, 128, True),
                                           (8, 384, True), (4, 2304, True), (3, 4224, False)])
def test_prefill_over_decoded_tiles_has_the_bits_of_the_decoding_gemm(env, oracle, bits, n, strips):
    """Many rows: the trellis is decoded once into fp16 tiles (the GEMM's own LDS images) and the GEMM copies them instead
    of decoding per output tile row. Same fragments and MFMA order, so with whole tiles the same bits in every output
    mode; the two forms walk the tiles in different orders, so with a last round cut along K other tiles are the cut
    ones and those differ by the order of their f32 sums (so do the tiles that the stream-K schedule shares between
    programs, which is forced here for the pass that compares within a tolerance). The "hat_rows" option moves the row
    count from which this form runs (0: never). 2304 and 4224 columns: 9 and 17 column tiles, dealt to the XCDs in bands
    of 8."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    m = 600
    t = synth.exl3_tensor(1024, n, bits, 90 + bits)
    xd = dev_u16(torch, synth.activations(m, t.k, 6, outliers=True))
    lin = exl3.Linear.new(kern, exl3.DeviceExl3(t, strips), 256)
    kern.set_option("hat_rows", 65)
    ws = exl3.Workspace([lin], m)  # created for the decoded form

    def run(rows, dt, torch_dt, pre):
        y = torch.full((m + 1, t.n), pre, dtype=torch_dt, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, y, dt, rows, ws)
        torch.cuda.synchronize()
        return y.view(torch.int16 if torch_dt == torch.bfloat16 else torch.int32).cpu().numpy()

    for splits in (None, "1"):
        kern.set_option("gemm_splits", int(splits) if splits else 8)
        kern.set_option("gemm_sk", 0 if splits else 2)
        for rows in (65, 300, 600):
            for dt, tdt, pre in ((exl3.Dtype.F32, torch.float32, float("nan")), (exl3.Dtype.Bf16, torch.bfloat16, 7.0),
                                 (exl3.Dtype.Bf16Add, torch.bfloat16, 1.5), (exl3.Dtype.F32Add, torch.float32, 0.25)):
                kern.set_option("hat_rows", 65)
                tiles = run(rows, dt, tdt, pre)
                kern.set_option("hat_rows", 0)
                fused = run(rows, dt, tdt, pre)
                if splits:
                    assert np.array_equal(tiles, fused), (splits, rows, dt)
                else:
                    as_f = lambda a: (a.astype(np.int32) << 16).view(np.float32) if a.dtype == np.int16 else a.view(np.float32)
                    a, b = as_f(tiles[:rows]).astype(np.float64), as_f(fused[:rows]).astype(np.float64)
                    rms = np.sqrt((b ** 2).mean())
                    assert np.all(np.abs(a - b) <= np.abs(b) / 128.0 + 1e-4 * rms), (rows, dt)
                assert (tiles[rows:] == tiles[m]).all()  # rows past `rows` keep the prefill
    kern.set_option("gemm_splits", 8)
    kern.set_option("gemm_sk", 1)
    # and against the oracle
    kern.set_option("hat_rows", 65)
    y = torch.zeros((m, t.n), dtype=torch.float32, device="cuda")
    lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
    torch.cuda.synchronize()
    o = to_oracle(oracle, t)
    ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), ws.xh(m, t.k))
    assert np.abs(y.cpu().numpy().astype(np.float64) - ref).max() / np.sqrt((ref ** 2).mean()) < 1e-4
    kern.set_option("hat_rows", 3072)


def test_prefill_over_kept_decoded_weights(env, oracle):
    """keep_decoded: the fp16 tiles stay with the linear, every call above 64 rows runs the GEMM over them (no decode
    launch, any workspace). Whole tiles have the bits of the decoding GEMM; decode-sized calls are untouched."""
    torch, exl3, kern = env
    from ferrite_amd import synth
    m = 300
    t = synth.exl3_tensor(1024, 384, 4, 123)
    xd = dev_u16(torch, synth.activations(m, t.k, 4, outliers=True))
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), 256)
    ws = exl3.Workspace([lin], m)  # not created for the decoded form

    def run(rows):
        y = torch.full((m + 1, t.n), float("nan"), dtype=torch.float32, device="cuda")
        lin.forward(xd, exl3.Dtype.Bf16, y, exl3.Dtype.F32, rows, ws)
        torch.cuda.synchronize()
        out = y.cpu().numpy()
        assert np.isnan(out[rows:]).all()
        return out[:rows]

    kern.set_option("gemm_splits", 1)
    before = {rows: run(rows) for rows in (1, 16, 64, 65, 300)}
    lin.keep_decoded()
    lin.keep_decoded()  # a second call keeps what is there
    for rows, want in before.items():
        assert np.array_equal(run(rows).view(np.uint32), want.view(np.uint32)), rows
    kern.set_option("gemm_splits", 8)
    cut = run(300)  # a last round cut along K: other tiles are the cut ones, sums in another order
    rms = np.sqrt((before[300].astype(np.float64) ** 2).mean())
    assert np.abs(cut.astype(np.float64) - before[300]).max() / rms < 1e-4
    lin.keep_decoded(False)
    assert np.array_equal(run(300).view(np.uint32), run(300).view(np.uint32))
