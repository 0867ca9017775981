"""The entry point that allocates nothing (fe_exl3_linear_forward_static): its output has the bits of
fe_exl3_linear_forward over a workspace object, call after call on the shared static scratch array, and shapes beyond
the array are refused with an error."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def both(torch, exl3, synth, kern, k, n, bits, rows, seed, y_dtype, sk=None):
    t = synth.exl3_tensor(k, n, bits, seed)
    w = exl3.DeviceExl3.upload_strips(t)
    lin = exl3.Linear.new(kern, w, exl3.default_blocks(exl3.cu_count())) if sk is None else exl3.Linear.with_plan(kern, w, exl3.Plan(sk))
    x = dev_u16(torch, synth.activations(rows, k, seed + 1))
    tdt = torch.float32 if y_dtype == exl3.Dtype.F32 else torch.bfloat16
    want = torch.full((rows + 1, n), float("nan"), dtype=tdt, device="cuda")
    got = torch.full((rows + 1, n), float("nan"), dtype=tdt, device="cuda")
    ws = exl3.Workspace([lin], rows)
    lin.forward(x, exl3.Dtype.Bf16, want, y_dtype, rows, ws)
    lin.forward_static(x, exl3.Dtype.Bf16, got, y_dtype, rows)
    torch.cuda.synchronize()
    return lin, got, want


def same_bits(torch, got, want, rows):
    as_int = torch.int32 if got.dtype == torch.float32 else torch.int16
    assert torch.equal(got[:rows].view(as_int), want[:rows].view(as_int))
    assert torch.isnan(got[rows:]).all()  # rows past the call stay untouched


def test_two_calls_in_a_row_the_second_smaller():
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    # split K (partials and counters in the static array), 7 rows, f32 out
    lin, got, want = both(torch, exl3, synth, kern, 2048, 1024, 4, 7, 11, exl3.Dtype.F32, sk=4)
    assert lin.plan.sk == 4
    assert torch.isfinite(want[:7]).all()
    same_bits(torch, got, want, 7)
    # straight after it on the same array: a smaller linear, fewer rows, bf16 out, another bit width
    _, got, want = both(torch, exl3, synth, kern, 1024, 256, 3, 2, 12, exl3.Dtype.Bf16, sk=2)
    same_bits(torch, got, want, 2)
    # and the first shape again: what the smaller call left behind does not show
    _, got, want = both(torch, exl3, synth, kern, 2048, 1024, 4, 7, 11, exl3.Dtype.F32, sk=4)
    same_bits(torch, got, want, 7)


def test_the_benchmark_shape_at_one_and_sixteen_rows():
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    for rows in (16, 1):
        _, got, want = both(torch, exl3, synth, kern, 5120, 17408, 4, rows, 13, exl3.Dtype.Bf16)
        same_bits(torch, got, want, rows)


def test_sizes_beyond_the_array_are_errors():
    import torch
    from ferrite_amd import exl3, synth
    from ferrite_amd._lib import FeError
    kern = exl3.Kernels.load()
    t = synth.exl3_tensor(1024, 256, 4, 14)
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(2))
    x = torch.zeros((64, 1024), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((64, 256), dtype=torch.float32, device="cuda")
    for rows in (0, 17, 64):
        with pytest.raises(FeError) as e:
            lin.forward_static(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, rows)
        assert e.value.code == 10002  # FE_ERR_WORKSPACE
    # partial sums of 2048 programs over 256 column blocks at 16 rows: 2304 slots x 16 x 512 B = 18 MiB, more than the
    # array holds
    t = synth.exl3_tensor(1024, 32768, 2, 15)
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(8))
    x = torch.zeros((16, 1024), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((16, 32768), dtype=torch.float32, device="cuda")
    with pytest.raises(FeError) as e:
        lin.forward_static(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 16)
    assert e.value.code == 10002 and "partial sums" in str(e.value)
    lin.forward_static(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, 8)  # half the rows fit
    torch.cuda.synchronize()
