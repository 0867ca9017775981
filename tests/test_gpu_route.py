"""GPU tests of the layer that routes the rows of a batch to the two quantized linears (include/fe_route.h), the role of
fe_model::Linear::forward, Proj::forward and the MLP block (crates/fe-model/src/model.rs:260-403, 3160-3203): decode rows
take the trellis GEMV whatever the batch size, so each routed row must have the bits of the direct call of the layer it
is routed to; prompt rows take the prompt linear; the fused forms place their outputs where the reference does."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HIDDEN, INTER = 512, 1024


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def bf16_to_f32(a):
    return (a.astype(np.uint32) << 16).view(np.float32)


def bf16_bits(x):
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def bits(t):
    import torch
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.fixture(scope="module")
def env():
    import torch
    from ferrite_amd import exl3, fp4, route, synth
    assert torch.cuda.is_available()

    class E:
        pass

    e = E()
    e.torch, e.exl3, e.fp4, e.route, e.synth = torch, exl3, fp4, route, synth
    e.xk, e.fk = exl3.Kernels.load(), fp4.Kernels.load()
    blocks = exl3.default_blocks(exl3.cu_count())

    def q(name, k, n, seed):
        t = synth.exl3_tensor(k, n, 4, seed, name)
        return t, exl3.Linear.new(e.xk, exl3.DeviceExl3.upload_strips(t), blocks)

    e.t_gate, e.q_gate = q("gate", HIDDEN, INTER, 1)
    e.t_up, e.q_up = q("up", HIDDEN, INTER, 2)
    e.t_down, e.q_down = q("down", INTER, HIDDEN, 3)
    e.max_rows = 320
    e.xws = exl3.Workspace([e.q_gate, e.q_up, e.q_down], e.max_rows)
    g, u = synth.fp4_linear(INTER, HIDDEN, 1, name="gate"), synth.fp4_linear(INTER, HIDDEN, 2, name="up")
    e.h_gate, e.h_up = g, u
    e.h_gu = fp4.HostLinear.fuse([("gate", g.codes, g.sf, 1.0, 1.0), ("up", u.codes, u.sf, 1.0, 1.0)])
    e.h_gu.alpha[:] = e.h_gu.alpha * np.float32(0.02)  # outputs of order 1, where silu bends
    e.p_gu = e.h_gu.upload()
    e.p_sw = e.h_gu.into_swiglu().upload()
    e.h_down = synth.fp4_linear(HIDDEN, INTER, 3, input_scale=0.5, name="down")
    e.p_down = e.h_down.upload()
    e.p_gate = g.upload()
    e.fws = fp4.Workspace(e.max_rows, max(HIDDEN, INTER))
    e.act_ws = fp4.Workspace(e.max_rows, INTER)
    e.ctx = route.LinCtx((e.xk, e.xws), (e.fk, e.fws), None, max_proj=2 * INTER)
    return e


def x3_direct(e, lin, x, rows, add_to=None):
    """The EXL3 layer called directly, in passes of 64 rows."""
    torch, exl3 = e.torch, e.exl3
    y = torch.zeros((rows, lin.n), dtype=torch.bfloat16, device="cuda") if add_to is None else add_to.clone()
    for r in range(0, rows, 64):
        n = min(64, rows - r)
        lin.forward(x[r:r + n], exl3.Dtype.Bf16, y[r:r + n], exl3.Dtype.Bf16 if add_to is None else exl3.Dtype.Bf16Add, n, e.xws)
    torch.cuda.synchronize()
    return bits(y)


def test_linear_routes_decode_rows_to_the_trellis_and_prompt_rows_to_the_prompt_linear(env):
    e = env
    torch, route = e.torch, e.route
    from ferrite_amd._lib import FeError
    lin = route.Linear("gate", INTER, HIDDEN, q=e.q_gate, p=e.p_gate)
    c = e.ctx
    m = 40
    x = dev_u16(torch, e.synth.activations(m, HIDDEN, 5))
    want_q = x3_direct(e, e.q_gate, x, m)
    yp = torch.zeros((m, INTER), dtype=torch.bfloat16, device="cuda")

    # up to 16 rows: every row through the trellis, whatever dec says
    for rows, dec in ((1, 0), (5, 0), (16, 3)):
        c.dec = dec
        y = torch.full((m, INTER), 9.0, dtype=torch.bfloat16, device="cuda")
        lin.forward(c, y, INTER, x, HIDDEN, rows)
        torch.cuda.synchronize()
        got = bits(y)
        assert np.array_equal(got[:rows], want_q[:rows]) and (got[rows:] == bf16_bits(np.float32([9.0]))[0]).all()

    # 40 rows, the first 8 of them decode rows: trellis bits for those, the prompt linear's for the other 32
    c.dec = 8
    y = torch.zeros((m, INTER), dtype=torch.bfloat16, device="cuda")
    lin.forward(c, y, INTER, x, HIDDEN, m)
    e.p_gate.forward(e.fk, e.fws, yp[8:], INTER, x[8:], HIDDEN, m - 8)
    torch.cuda.synchronize()
    got = bits(y)
    assert np.array_equal(got[:8], want_q[:8])
    assert np.array_equal(got[8:], bits(yp)[8:])
    assert not np.array_equal(got[8:], want_q[8:])  # two different weights: the routing shows

    # residual in place: decode rows y = bf16(f32(y) + x.W) in the GEMV's epilogue, prompt rows bf16(bf16(x.W) + res)
    res = dev_u16(torch, bf16_bits(np.random.default_rng(1).normal(size=(m, INTER)).astype(np.float32)))
    y = res.clone()
    lin.forward(c, y, INTER, x, HIDDEN, m, res=y)
    torch.cuda.synchronize()
    got = bits(y)
    assert np.array_equal(got[:8], x3_direct(e, e.q_gate, x, 8, add_to=res.view(torch.bfloat16)[:8]))
    assert np.array_equal(got[8:], bf16_bits(bf16_to_f32(bits(yp)[8:]) + bf16_to_f32(bits(res)[8:])))
    with pytest.raises(FeError, match="in place"):
        lin.forward(c, y, INTER, x, HIDDEN, m, res=res)

    # a row stride the trellis layer does not take: every row to the prompt linear
    c.dec = 8
    wide = torch.zeros((m, INTER + 64), dtype=torch.bfloat16, device="cuda")
    lin.forward(c, wide, INTER + 64, x, HIDDEN, m)
    e.p_gate.forward(e.fk, e.fws, yp, INTER, x, HIDDEN, m)
    torch.cuda.synchronize()
    assert np.array_equal(bits(wide)[:, :INTER], bits(yp)) and not bits(wide)[:, INTER:].any()
    c.dec = 0


def test_linear_without_prompt_weights(env):
    """model.rs:305-309: no prompt form, so every row takes the trellis linear: in passes of 64 rows through the GEMV (the
    reference's way, each row with its decode bits), or in one call, which above 64 rows is this library's GEMM."""
    e = env
    torch, route = e.torch, e.route
    from ferrite_amd._lib import FeError
    lin = route.Linear("down", HIDDEN, INTER, q=e.q_down)
    c = e.ctx
    m = 150
    x = dev_u16(torch, e.synth.activations(m, INTER, 6))
    c.dec = 0
    c.set_x3_gemm(False)
    y = torch.zeros((m, HIDDEN), dtype=torch.bfloat16, device="cuda")
    lin.forward(c, y, HIDDEN, x, INTER, m)
    torch.cuda.synchronize()
    passes = bits(y)
    assert np.array_equal(passes, x3_direct(e, e.q_down, x, m))
    c.set_x3_gemm(True)
    y2 = torch.zeros((m, HIDDEN), dtype=torch.bfloat16, device="cuda")
    lin.forward(c, y2, HIDDEN, x, INTER, m)
    yd = torch.zeros((m, HIDDEN), dtype=torch.bfloat16, device="cuda")
    e.q_down.forward(x, e.exl3.Dtype.Bf16, yd, e.exl3.Dtype.Bf16, m, e.xws)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y2), bits(yd))
    a, b = bf16_to_f32(bits(y2)).astype(np.float64), bf16_to_f32(passes).astype(np.float64)
    assert np.all(np.abs(a - b) <= np.abs(b) / 128.0 + 1e-3 * np.sqrt((b ** 2).mean()))  # the same sums in another order
    # a linear with no weights at all
    empty = route.Linear("none", HIDDEN, INTER)
    with pytest.raises(FeError, match="no bf16 weights"):
        empty.forward(c, y, HIDDEN, x, INTER, 4)
    # shapes are checked when the linear is made
    with pytest.raises(FeError):
        route.Linear("bad", HIDDEN, HIDDEN, q=e.q_down)


def test_linear_with_trellis_and_bf16_weights(env):
    """model.rs:305, 664-684: a linear that holds the trellis (q) and plain bf16 weights (w): decode rows take the trellis
    GEMV, the prompt rows after them the bf16 linear, never the trellis again."""
    e = env
    torch, route = e.torch, e.route
    from ferrite_amd import bf16
    bk = bf16.Kernels.load()
    wb = bf16_bits(np.random.default_rng(5).normal(size=(HIDDEN, INTER)) / 32)
    w = dev_u16(torch, wb)
    lin = route.Linear("down", HIDDEN, INTER, q=e.q_down, w=w)
    c = e.ctx
    c.set_bf16(bk)
    try:
        m, dec = 150, 5
        x = dev_u16(torch, e.synth.activations(m, INTER, 9))
        c.dec = dec
        y = torch.zeros((m, HIDDEN), dtype=torch.bfloat16, device="cuda")
        lin.forward(c, y, HIDDEN, x, INTER, m)
        torch.cuda.synchronize()
        got = bits(y)
        assert np.array_equal(got[:dec], x3_direct(e, e.q_down, x, dec))
        want = torch.zeros((m - dec, HIDDEN), dtype=torch.bfloat16, device="cuda")
        bf16.forward(bk, want, HIDDEN, x[dec:], INTER, w, m - dec, dec=0)
        torch.cuda.synchronize()
        assert np.array_equal(got[dec:], bits(want))
        # no decode rows announced: all 150 rows are prompt rows of the bf16 linear
        c.dec = 0
        lin.forward(c, y, HIDDEN, x, INTER, m)
        allw = torch.zeros((m, HIDDEN), dtype=torch.bfloat16, device="cuda")
        bf16.forward(bk, allw, HIDDEN, x, INTER, w, m, dec=0)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), bits(allw))
        # a small batch is all decode rows: the trellis
        lin.forward(c, y, HIDDEN, x, INTER, 7)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y)[:7], x3_direct(e, e.q_down, x, 7))
    finally:
        c.dec = 0
        c.set_bf16(None)


def test_proj_places_parts_as_the_reference(env):
    e = env
    torch, route = e.torch, e.route
    c = e.ctx
    g, u = route.Linear("gate", INTER, HIDDEN, q=e.q_gate), route.Linear("up", INTER, HIDDEN, q=e.q_up)
    proj = route.Proj([(g, [INTER]), (u, [INTER])], prompt=(e.p_gu, 2))
    assert proj.total_n() == 2 * INTER
    m = 48
    x = dev_u16(torch, e.synth.activations(m, HIDDEN, 7))
    want_g, want_u = x3_direct(e, e.q_gate, x, m), x3_direct(e, e.q_up, x, m)

    # a small batch: no fused GEMM, each linear writes its own [m][n] block
    c.dec = 0
    out = torch.zeros((m, 2 * INTER), dtype=torch.bfloat16, device="cuda")
    parts = proj.forward(c, out, x, HIDDEN, 10)
    torch.cuda.synchronize()
    assert parts == [(out.data_ptr(), INTER), (out.data_ptr() + 10 * INTER * 2, INTER)]
    flat = bits(out).reshape(-1)
    assert np.array_equal(flat[:10 * INTER].reshape(10, INTER), want_g[:10])
    assert np.array_equal(flat[10 * INTER:20 * INTER].reshape(10, INTER), want_u[:10])

    # 48 rows, 6 decode rows: one fused GEMM for rows 6.., the linears' own GEMVs copied into the fused layout for 0..5
    c.dec = 6
    out = torch.zeros((m, 2 * INTER), dtype=torch.bfloat16, device="cuda")
    parts = proj.forward(c, out, x, HIDDEN, m)
    yp = torch.zeros((m, 2 * INTER), dtype=torch.bfloat16, device="cuda")
    e.p_gu.forward(e.fk, e.fws, yp[6:], 2 * INTER, x[6:], HIDDEN, m - 6)
    torch.cuda.synchronize()
    assert parts == [(out.data_ptr(), 2 * INTER), (out.data_ptr() + INTER * 2, 2 * INTER)]
    got = bits(out)
    assert np.array_equal(got[:6, :INTER], want_g[:6]) and np.array_equal(got[:6, INTER:], want_u[:6])
    assert np.array_equal(got[6:], bits(yp)[6:])

    # no fused prompt linear, 40 rows that are all decode / verify rows: one GEMV pass, the two linears as one grouped
    # launch, each writing its own [m][n] block
    plain = route.Proj([(g, [INTER]), (u, [INTER])])
    assert e.exl3.forward_group_launches([e.q_gate, e.q_up], 40, e.xws) in (1, 2)
    c.dec = 40
    out = torch.zeros((40, 2 * INTER), dtype=torch.bfloat16, device="cuda")
    parts = plain.forward(c, out, x, HIDDEN, 40)
    torch.cuda.synchronize()
    assert parts == [(out.data_ptr(), INTER), (out.data_ptr() + 40 * INTER * 2, INTER)]
    flat = bits(out).reshape(-1)
    assert np.array_equal(flat[:40 * INTER].reshape(40, INTER), want_g[:40])
    assert np.array_equal(flat[40 * INTER:].reshape(40, INTER), want_u[:40])
    c.dec = 0


def test_silu_mul_and_copy2d(env):
    e = env
    torch, route = e.torch, e.route
    rng = np.random.default_rng(3)
    rows, inter, ld = 7, 770, 1600
    gu = bf16_bits(rng.normal(size=(rows, ld)).astype(np.float32) * 3.0)
    gu[0, :6] = bf16_bits(np.float32([0.0, -0.0, 80.0, -80.0, 1e-20, -30.0]))
    d = dev_u16(torch, gu)
    out = torch.full((rows + 1, inter), 5.0, dtype=torch.bfloat16, device="cuda")
    route.silu_mul(out, d.data_ptr(), d.data_ptr() + 800 * 2, ld, inter, rows)
    torch.cuda.synchronize()
    g = bf16_to_f32(gu[:, :inter]).astype(np.float64)
    u = bf16_to_f32(gu[:, 800:800 + inter])
    silu = bf16_to_f32(bf16_bits((g / (1.0 + np.exp(-g))).astype(np.float32)))
    want = bf16_to_f32(bf16_bits(silu * u)).astype(np.float64)
    got = bf16_to_f32(bits(out)).astype(np.float64)
    # the hardware exponential and reciprocal: silu may land on the other side of a bf16 rounding tie
    assert np.all(np.abs(got[:rows] - want) <= np.abs(want) / 64.0 + 1e-30)
    assert (got[:rows] != want).mean() < 0.02
    assert (got[rows] == 5.0).all() and got[0, 0] == 0.0 and got[0, 1] == 0.0
    # copy2d
    dst = torch.zeros((rows, 900), dtype=torch.int16, device="cuda")
    route.copy2d(dst.data_ptr() + 20 * 2, 900, d.data_ptr() + 6 * 2, ld, 300, rows - 1)
    torch.cuda.synchronize()
    got = dst.cpu().numpy().view(np.uint16)
    assert np.array_equal(got[:rows - 1, 20:320], gu[:rows - 1, 6:306])
    assert not got[rows - 1].any() and not got[:, :20].any() and not got[:, 320:].any()


def test_mlp_block_routes_as_the_reference(env, oracle):
    """x += down(SwiGLU(gate(xn), up(xn))): the decode rows through the three trellis linears and fe_silu_mul, the prompt
    rows through the fused gate|up front and down's GEMM on the quantized activation. Each group of rows must have the
    bits of the same steps called by hand, and the decode rows must agree with the f64 reference of the trellis MLP."""
    e = env
    torch, route, exl3 = e.torch, e.route, e.exl3
    c = e.ctx
    g, u = route.Linear("gate", INTER, HIDDEN, q=e.q_gate), route.Linear("up", INTER, HIDDEN, q=e.q_up)
    gate_up = route.Proj([(g, [INTER]), (u, [INTER])], prompt=(e.p_gu, 2))
    down = route.Linear("down", HIDDEN, INTER, q=e.q_down, p=e.p_down)
    rows, dec = 300, 5
    xn_b = e.synth.activations(rows, HIDDEN, 11)
    x_b = bf16_bits(np.random.default_rng(12).normal(size=(rows, HIDDEN)).astype(np.float32))
    xn = dev_u16(torch, xn_b)
    big = torch.zeros((rows, 2 * INTER), dtype=torch.bfloat16, device="cuda")
    act = torch.zeros((rows, INTER), dtype=torch.bfloat16, device="cuda")

    def run(nrows, d, swiglu):
        c.dec = d
        x = dev_u16(torch, x_b)
        route.mlp_forward(c, gate_up, down, x, xn, big, act, nrows, HIDDEN, INTER, swiglu=swiglu, act_ws=e.act_ws if swiglu else None)
        torch.cuda.synchronize()
        return bits(x)

    # by hand, decode rows
    def by_hand_decode(n):
        yg, yu = x3_direct(e, e.q_gate, xn, n), x3_direct(e, e.q_up, xn, n)
        a = torch.zeros((n, INTER), dtype=torch.bfloat16, device="cuda")
        gu = dev_u16(torch, np.concatenate([yg, yu], axis=1))
        route.silu_mul(a, gu.data_ptr(), gu.data_ptr() + INTER * 2, 2 * INTER, INTER, n)
        return x3_direct(e, e.q_down, a.view(torch.int16), n, add_to=dev_u16(torch, x_b[:n]).view(torch.bfloat16)), bits(a)

    # by hand, prompt rows [d, rows)
    def by_hand_prompt(d):
        x = dev_u16(torch, x_b)
        e.p_sw.forward_swiglu(e.fk, e.fws, e.act_ws, xn[d:], HIDDEN, rows - d, e.p_down.g)
        e.p_down.gemm(e.fk, e.act_ws, x[d:], HIDDEN, rows - d, res=x[d:])
        torch.cuda.synchronize()
        return bits(x)[d:]

    got = run(rows, dec, e.p_sw)
    hand_dec, act_dec = by_hand_decode(dec)
    assert np.array_equal(got[:dec], hand_dec)
    assert np.array_equal(got[dec:], by_hand_prompt(dec))
    assert not np.array_equal(got[dec:], x_b[dec:])

    # a small batch: every row is a decode row, the fused front is not used
    got12 = run(12, 0, e.p_sw)
    assert np.array_equal(got12[:12], by_hand_decode(12)[0]) and np.array_equal(got12[12:], x_b[12:])
    assert np.array_equal(got12[:dec], got[:dec])  # a decode row's bits do not depend on the batch around it

    # a single decode row: the three trellis linears as one launch (fe_exl3_mlp_forward), the bits of the steps by hand
    assert exl3.mlp_forward_launches(e.q_gate, e.q_up, e.q_down, 1, exl3.Dtype.Bf16Add, e.xws) == 1
    got1 = run(1, 0, e.p_sw)
    assert np.array_equal(got1[:1], by_hand_decode(1)[0]) and np.array_equal(got1[1:], x_b[1:])
    assert np.array_equal(got1[:1], got[:1])
    assert e.xws.chain_status() == 0

    # without the fused front: prompt rows through the fused gate|up GEMM, fe_silu_mul and down's prompt linear
    got_unfused = run(rows, dec, None)
    assert np.array_equal(got_unfused[:dec], hand_dec)
    a, b = bf16_to_f32(got_unfused[dec:]).astype(np.float64), bf16_to_f32(got[dec:]).astype(np.float64)
    # (the unfused path rounds the activation to bf16 before it is quantized for down, the fused one does the same in
    # its epilogue: the two agree up to rounding flips of single activations)
    assert np.abs(a - b).max() <= 0.1 * np.abs(b).max()

    # the decode rows against the f64 reference of the trellis MLP on the same inputs
    og, ou, od = (oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh) for t in (e.t_gate, e.t_up, e.t_down))
    xn64 = bf16_to_f32(xn_b[:dec]).astype(np.float64)
    yg, yu = oracle.linear_f64(og, xn64), oracle.linear_f64(ou, xn64)
    ref_act = yg / (1.0 + np.exp(-yg)) * yu
    ref = bf16_to_f32(x_b[:dec]).astype(np.float64) + oracle.linear_f64(od, ref_act)
    gotf = bf16_to_f32(got[:dec]).astype(np.float64)
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(gotf - ref).max() / rms < 3e-2  # three bf16 roundings on the way (gate/up, silu, act) and the fp16 rotation
    c.dec = 0
