"""The GPU path against the committed vectors of tests/golden/path_vectors.npz, inputs and expected outputs both taken
from the file: dequantized weights and quantizer codes bit-exact, rotated input within one fp16 step, outputs within the
path's bar (max relative error 1e-2)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "path_vectors.npz")


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def f32(a):
    return (np.asarray(a, np.uint16).astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_exl3_vectors(bits):
    import torch
    from ferrite_amd import exl3
    g = np.load(GOLD)
    p = f"exl3_b{bits}_"
    t = exl3.Exl3Tensor("golden", 128, 128, bits, g[p + "trellis"], g[p + "suh"], g[p + "svh"])
    kern = exl3.Kernels.load()
    d = exl3.DeviceExl3.upload(t)
    hat = torch.zeros((t.k, t.n), dtype=torch.int16, device="cuda")
    kern.reconstruct_hat_f16(d.view, hat)
    torch.cuda.synchronize()
    want = g[p + "w_hat_f16"]
    assert np.array_equal(hat.cpu().numpy().view(np.uint16)[:, :want.shape[1]], want)
    ordered = lambda h: np.where(h & 0x8000, -(h & 0x7FFF).astype(np.int32), h.astype(np.int32))
    if bits == 4:
        out = torch.zeros(t.k * t.n, dtype=torch.int16, device="cuda")
        kern.reconstruct_bf16(d.view, out, "KN", torch.empty(t.k * 128, dtype=torch.float32, device="cuda"))
        torch.cuda.synchronize()
        got, wb = out.cpu().numpy().view(np.uint16).reshape(t.k, t.n), g[p + "weight_bf16"]
        rms = np.sqrt((f32(wb).astype(np.float64) ** 2).mean())
        far = np.abs(ordered(got) - ordered(wb)) > 1
        assert (np.abs(f32(got).astype(np.float64) - f32(wb))[far] < 1e-4 * rms).all()  # f32 against f64: one bf16 step
    lin = exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(t), exl3.default_blocks(exl3.cu_count()))
    ws = exl3.Workspace([lin], 3)
    y = torch.zeros((3, t.n), dtype=torch.float32, device="cuda")
    lin.forward(dev_u16(torch, g["exl3_x_bf16"]), exl3.Dtype.Bf16, y, exl3.Dtype.F32, 3, ws)
    torch.cuda.synchronize()
    xh, xh_want = ws.xh(3, t.k), g[p + "xh_f16"]
    assert (np.abs(ordered(xh) - ordered(xh_want)) <= 1).all()
    ref = g[p + "linear_f64"]
    got = y.cpu().numpy().astype(np.float64)
    # max relative error 1e-2, the denominator floored at the output's rms (sums that cancel to ~0 do not define the
    # scale); the difference is the fp16 rounding of the rotated input, which the f64 reference does not have
    rms = np.sqrt((ref ** 2).mean())
    assert (np.abs(got - ref) / np.maximum(np.abs(ref), rms)).max() < 1e-2
    assert np.abs(got - ref).max() / rms < 2e-3


def test_fp4_vectors():
    import torch
    from ferrite_amd import fp4
    g = np.load(GOLD)
    kern = fp4.Kernels.load()
    x = dev_u16(torch, g["fp4_x_bf16"])
    n, k, m = 128, 256, 4
    alpha = g["fp4_alpha"]
    for gs in (1.0, 0.037, 2.5, float(g["fp4_g"])):
        lin = fp4.PromptLinear.from_view("golden", n, k, torch.from_numpy(g["fp4_w_codes"]).cuda(),
                                         torch.from_numpy(g["fp4_w_sf"]).cuda(), torch.from_numpy(alpha).cuda(), gs)
        ws = fp4.Workspace(m, k)
        y = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        lin.forward(kern, ws, y, n, x, k, m)
        torch.cuda.synchronize()
        key = f"fp4_codes_g{gs}"
        if key in g.files:
            import oracle
            codes, sf_tiled = ws.read(m, k)
            assert np.array_equal(codes, g[key])
            assert np.array_equal(oracle.untile_scales(sf_tiled, m, k // 16).reshape(m, k // 16), g[f"fp4_sf_g{gs}"])
        else:
            ref = g["fp4_ref_gemm"].astype(np.float64)
            got = y.float().cpu().numpy().astype(np.float64)
            assert (np.abs(got - ref) / np.abs(ref).max(axis=1, keepdims=True)).max() < 8e-3


def test_bf16_vectors():
    import torch
    from ferrite_amd import bf16
    g = np.load(GOLD)
    kern = bf16.Kernels.load()
    x, w, res = dev_u16(torch, g["bf16_x"]), dev_u16(torch, g["bf16_w"]), dev_u16(torch, g["bf16_res"])
    acc = g["bf16_acc"].astype(np.float64)
    for fn in (bf16.gemv, bf16.gemm):
        y = dev_u16(torch, np.zeros((5, 64), np.uint16))
        fn(kern, y, 64, x, 256, w, 5)
        torch.cuda.synchronize()
        got = y.cpu().numpy().view(np.uint16)
        assert (np.abs(f32(got) - acc) <= np.abs(acc) / 256 + 1e-6).all()
        assert (got != g["bf16_y"]).mean() < 0.02
        fn(kern, y, 64, x, 256, w, 5, res=res)
        torch.cuda.synchronize()
        b = np.ascontiguousarray(f32(got) + f32(g["bf16_res"]), np.float32).view(np.uint32)
        assert np.array_equal(y.cpu().numpy().view(np.uint16), ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16))
