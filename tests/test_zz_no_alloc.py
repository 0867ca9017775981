"""The entry point that allocates nothing (fe_exl3_linear_forward_static): its output has the bits of
fe_exl3_linear_forward over a workspace object, call after call on the shared static scratch array; the free device
memory does not move across its calls; it records into a HIP graph and replays; and shapes beyond the array are refused
with an error."""
import ctypes as C

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


def test_no_device_memory_moves_and_the_widest_plan_fits():
    """Free device memory (hipMemGetInfo) reads the same before and after a run of calls; 5120 x 17408 at 16 rows under a
    plan of 5 programs a CU (1280 programs: the most room a tuned shape asks of the array) is served."""
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    t = synth.exl3_tensor(5120, 17408, 4, 13)
    w = exl3.DeviceExl3.upload_strips(t)
    lin5 = exl3.Linear.with_plan(kern, w, exl3.Plan(10, 4, 3, 5))
    lin = exl3.Linear.new(kern, w, exl3.default_blocks(exl3.cu_count()))
    x = dev_u16(torch, synth.activations(16, 5120, 3))
    want = torch.zeros((16, 17408), dtype=torch.bfloat16, device="cuda")
    got = torch.zeros((16, 17408), dtype=torch.bfloat16, device="cuda")
    ws = exl3.Workspace([lin5], 16)
    lin5.forward(x, exl3.Dtype.Bf16, want, exl3.Dtype.Bf16, 16, ws)
    lin5.forward_static(x, exl3.Dtype.Bf16, got, exl3.Dtype.Bf16, 16)  # (first call: any lazy set-up is behind us)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    free0 = torch.cuda.mem_get_info()[0]
    for rows in (1, 16, 3, 16, 1):
        lin5.forward_static(x, exl3.Dtype.Bf16, got, exl3.Dtype.Bf16, rows)
        lin.forward_static(x, exl3.Dtype.Bf16, got, exl3.Dtype.Bf16, rows)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "a forward_static call changed the free device memory"


def test_records_into_a_graph_and_replays():
    import torch
    from ferrite_amd import _lib, exl3, synth
    lib, check = _lib.lib(), _lib.check
    kern = exl3.Kernels.load()
    t = synth.exl3_tensor(2048, 1024, 4, 21)
    lin = exl3.Linear.with_plan(kern, exl3.DeviceExl3.upload_strips(t), exl3.Plan(4))  # split K: counters and partial sums in use
    x = dev_u16(torch, synth.activations(5, 2048, 22))
    ws = exl3.Workspace([lin], 5)
    want = torch.zeros((5, 1024), dtype=torch.float32, device="cuda")
    lin.forward(x, exl3.Dtype.Bf16, want, exl3.Dtype.F32, 5, ws)
    got = torch.zeros((5, 1024), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    s, g = C.c_void_p(), C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    check(lib.fe_hip_graph_begin(s))
    lin.forward_static(x, exl3.Dtype.Bf16, got, exl3.Dtype.F32, 5, stream=s)
    check(lib.fe_hip_graph_end(s, C.byref(g)))
    for rep in range(3):
        got.fill_(9.0)
        torch.cuda.synchronize()
        check(lib.fe_hip_graph_launch(g, s))
        check(lib.fe_hip_stream_sync(s))
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), rep
        # an eager call on the same array between the replays
        lin.forward_static(x, exl3.Dtype.Bf16, got, exl3.Dtype.F32, 2)
        torch.cuda.synchronize()
    check(lib.fe_hip_graph_destroy(g))
    check(lib.fe_hip_stream_destroy(s))


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
