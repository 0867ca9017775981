"""Stress of the EXL3 decode path, of the prefill GEMMs' schedules and of the NVFP4 GEMV, bounded so that it runs in
seconds: random shapes, bit widths, plans, layouts and row counts against the oracle (each case stops at its first
mismatch and names itself), and thousands of random (linear, rows) calls on one shared workspace without a
synchronization in between, every one compared bit for bit with the first result of its kind (the role of
crates/fe-exl3/src/bin/exl3-stress.rs:62-98, which runs 256k such calls)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 33, 48, 63, 64]


def dev_u16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def random_plan(rng, exl3, k, n):
    kind = int(rng.integers(0, 3))
    if kind == 0:  # sk programs per column block
        steps = k // 64
        return exl3.Plan(int(rng.choice([d for d in range(1, steps + 1) if steps % d == 0])), 1, 1, 0)
    if kind == 1:  # occ programs per CU, runs of at least wk units
        return exl3.Plan(1, int(rng.choice([1, 2, 4])), 3, int(rng.integers(1, 6)))
    return exl3.Plan(int(rng.integers(1, (k // 128) * (n // 128) + 3)), 1, 4, 0)  # that many programs in all


def test_random_shapes_against_the_oracle(oracle):
    import torch
    from ferrite_amd import exl3, route, synth
    kern = exl3.Kernels.load()
    rng = np.random.default_rng(20251)
    for case in range(48):
        k = int(rng.integers(1, 17)) * 128
        bits = int(rng.choice([2, 3, 4, 5, 6, 8]))
        ns = [int(rng.integers(1, 7)) * 128 for _ in range(int(rng.integers(1, 4)))]
        rows = int(rng.choice(ROWS))
        lins, ts = [], []
        for i, n in enumerate(ns):
            t = synth.exl3_tensor(k, n, bits, 1000 + case * 10 + i)
            strips = bool(rng.integers(0, 2))
            lins.append(exl3.Linear.with_plan(kern, exl3.DeviceExl3(t, strips), random_plan(rng, exl3, k, n)))
            ts.append(t)
        ws = exl3.Workspace(lins, 64)
        xb = synth.activations(rows, k, case, outliers=bool(rng.integers(0, 2)))
        x = dev_u16(torch, xb)
        what = f"case {case}: k {k} bits {bits} ns {ns} plans {[l.plan for l in lins]} rows {rows}"
        ys = [torch.full((rows + 1, n), float("nan"), dtype=torch.float32, device="cuda") for n in ns]
        for l, y in zip(lins, ys):
            l.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, rows, ws)
        torch.cuda.synchronize()
        for l, t, y in zip(lins, ts, ys):
            o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
            l.rotate_input(x, exl3.Dtype.Bf16, rows, ws)
            torch.cuda.synchronize()
            ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), ws.xh(rows, k))
            got = y.cpu().numpy()
            assert np.abs(got[:rows] - ref).max() / max(np.sqrt((ref ** 2).mean()), 1e-30) < 1e-4, what
            assert np.isnan(got[rows]).all(), what
        if len(lins) >= 2:  # the same linears as one launch: the bits of each one's own forward
            gs = [torch.full((rows + 1, n), float("nan"), dtype=torch.float32, device="cuda") for n in ns]
            exl3.forward_group(lins, x, exl3.Dtype.Bf16, gs, exl3.Dtype.F32, rows, ws)
            torch.cuda.synchronize()
            for a, b in zip(ys, gs):
                assert torch.equal(a[:rows].view(torch.int32), b[:rows].view(torch.int32)) and torch.isnan(b[rows]).all(), what
        # SwiGLU of two arrays as the input: the bits of fe_silu_mul followed by forward
        gu = dev_u16(torch, synth.activations(rows, 2 * k, case + 7))
        act = torch.zeros((rows, k), dtype=torch.bfloat16, device="cuda")
        route.silu_mul(act, gu.data_ptr(), gu.data_ptr() + 2 * k, 2 * k, k, rows)
        a = torch.zeros((rows, ns[0]), dtype=torch.float32, device="cuda")
        b = torch.zeros_like(a)
        lins[0].forward(act.view(torch.int16), exl3.Dtype.Bf16, a, exl3.Dtype.F32, rows, ws)
        lins[0].forward_swiglu(gu.data_ptr(), gu.data_ptr() + 2 * k, 2 * k, b, exl3.Dtype.F32, rows, ws)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), what


def test_random_calls_on_a_shared_workspace_repeat_their_bits():
    import torch
    from ferrite_amd import exl3, synth
    kern = exl3.Kernels.load()
    blocks = exl3.default_blocks(exl3.cu_count())
    shapes = [(1024, 2048, 4), (2048, 1024, 3), (5120, 1024, 4), (1024, 384, 5), (3072, 640, 2), (512, 4096, 6)]
    lins = [exl3.Linear.new(kern, exl3.DeviceExl3.upload_strips(synth.exl3_tensor(k, n, b, 70 + i)), blocks)
            for i, (k, n, b) in enumerate(shapes)]
    ws = exl3.Workspace(lins, 64)
    xs = [dev_u16(torch, synth.activations(64, k, 80 + i)) for i, (k, n, b) in enumerate(shapes)]
    rows_list = [1, 2, 4, 8, 16, 17, 33, 64]
    want = {}
    for li, l in enumerate(lins):
        for m in rows_list:
            y = torch.zeros((m, l.n), dtype=torch.float32, device="cuda")
            l.forward(xs[li], exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
            want[(li, m)] = y
    torch.cuda.synchronize()
    rng = np.random.default_rng(7)
    calls, batches, bad = 400, 24, 0
    for bi in range(batches):
        picks = [(int(rng.integers(0, len(lins))), int(rng.choice(rows_list))) for _ in range(calls)]
        outs = []
        for li, m in picks:
            y = torch.empty((m, lins[li].n), dtype=torch.float32, device="cuda")
            lins[li].forward(xs[li], exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
            outs.append(y)
        torch.cuda.synchronize()
        for (li, m), y in zip(picks, outs):
            if not torch.equal(y.view(torch.int32), want[(li, m)].view(torch.int32)):
                bad += 1
        assert bad == 0, f"batch {bi}: {bad} of {calls} calls differ from their first result"


def test_random_prefill_shapes_on_both_schedules(oracle):
    """The prefill GEMMs (EXL3 decoding in the GEMM and over decoded tiles, NVFP4) on random shapes of 65..1500 rows under
    the one-piece schedule and both forced stream-K forms: every schedule against the oracle (EXL3) or within the order
    of the f32 sums of the one-piece result (NVFP4, which the other tests pin to its reference), and a repeat of every
    stream-K launch bit for bit (pieces of a tile arrive in whatever order; tiles of up to eight and more pieces occur
    here). Each case names itself."""
    import torch
    from ferrite_amd import exl3, fp4, synth
    kern, fk = exl3.Kernels.load(), fp4.Kernels.load()
    rng = np.random.default_rng(77)
    try:
        for case in range(20):
            k = int(rng.integers(2, 13)) * 128
            n = int(rng.integers(1, 17)) * 128
            m = int(rng.integers(65, 1500))
            bits = int(rng.choice([3, 4, 5]))
            what = f"case {case}: m {m} k {k} n {n} bits {bits}"
            t = synth.exl3_tensor(k, n, bits, 3000 + case)
            lin = exl3.Linear.new(kern, exl3.DeviceExl3(t, bool(rng.integers(0, 2))), 64)
            kern.set_option("hat_rows", 65)
            ws = exl3.Workspace([lin], m)
            x = dev_u16(torch, synth.activations(m, k, case, outliers=True))
            o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
            rows = sorted({0, 1, m // 3, m // 2, m - 2, m - 1})
            ref = None
            for hat in (0, 65):
                kern.set_option("hat_rows", hat)
                for sk in (0, 2, 3):
                    kern.set_option("gemm_sk", sk)
                    outs = []
                    for rep in range(2 if sk else 1):
                        y = torch.full((m + 1, n), float("nan"), dtype=torch.float32, device="cuda")
                        lin.forward(x, exl3.Dtype.Bf16, y, exl3.Dtype.F32, m, ws)
                        torch.cuda.synchronize()
                        outs.append(y.cpu().numpy())
                    if ref is None:
                        ref = oracle.gemv_ref(o, oracle.w_hat_f16(o), ws.xh(m, k)[rows])
                    err = np.abs(outs[0][rows] - ref).max() / max(np.sqrt((ref ** 2).mean()), 1e-30)
                    assert err < 1e-4, (what, hat, sk, err)
                    assert np.isnan(outs[0][m]).all(), (what, hat, sk)
                    if sk:
                        assert np.array_equal(outs[0][:m].view(np.uint32), outs[1][:m].view(np.uint32)), (what, hat, sk)
            kern.set_option("gemm_sk", 1)
            kern.set_option("hat_rows", 3072)
            host = synth.fp4_linear(n, k, 4000 + case, input_scale=1.0)
            flin = host.upload()
            fws = fp4.Workspace(m, k)
            got = {}
            for sk in (0, 2, 3):
                fk.set_option("gemm_sk", sk)
                for rep in range(2 if sk else 1):
                    yb = torch.full((m + 1, n), -3.0, dtype=torch.bfloat16, device="cuda")
                    flin.forward(fk, fws, yb, n, x, k, m)
                    torch.cuda.synchronize()
                    out = yb.float().cpu().numpy()
                    assert (out[m] == -3.0).all(), (what, sk)
                    if rep:
                        assert np.array_equal(out[:m], got[sk]), (what, sk)
                    got[sk] = out[:m]
                if sk:
                    a, b = got[sk].astype(np.float64), got[0].astype(np.float64)
                    assert (np.abs(a - b) <= np.abs(b) / 128.0 + 1e-4 * np.abs(b).max()).all(), (what, sk)
            fk.set_option("gemm_sk", 1)
    finally:
        kern.set_option("gemm_sk", 1)
        kern.set_option("hat_rows", 3072)
        fk.set_option("gemm_sk", 1)


def test_random_nvfp4_gemv_shapes_rows_and_splits():
    """The NVFP4 GEMV on random shapes, 1..64 rows (one to three groups of 16 rows, and two passes) and forced K splits of
    1..16 (the partials of a split meet through the workspace): every case against the GEMM over the same rows (the same
    exact products, summed in another order), the row after the batch untouched, a repeat bit for bit. Each case names
    itself."""
    import torch
    from ferrite_amd import fp4, synth
    fk = fp4.Kernels.load()
    rng = np.random.default_rng(3)
    try:
        for case in range(60):
            n, k = int(rng.integers(1, 17)) * 128, int(rng.integers(2, 33)) * 128
            m, sk = int(rng.integers(1, 65)), int(rng.choice([0, 1, 2, 3, 5, 8, 16]))
            what = f"case {case}: n {n} k {k} rows {m} split {sk}"
            lin = synth.fp4_linear(n, k, 100 + case, input_scale=1.0).upload()
            ws = fp4.Workspace(m, k)
            x = dev_u16(torch, synth.activations(m, k, case))

            def run():
                y = torch.full((m + 1, n), -3.0, dtype=torch.bfloat16, device="cuda")
                lin.forward(fk, ws, y, n, x, k, m)
                torch.cuda.synchronize()
                return y.float().cpu().numpy()

            fk.set_option("gemv_sk", sk)
            a, again = run(), run()
            fk.set_option("gemv", 0)
            b = run()
            fk.set_option("gemv", 1)
            assert np.array_equal(a, again) and (a[m] == -3.0).all(), what
            a, b = a[:m].astype(np.float64), b[:m].astype(np.float64)
            assert (np.abs(a - b) <= np.abs(b) / 100.0 + 1e-3 * np.abs(b).max()).all(), what
    finally:
        fk.set_option("gemv", 1)
        fk.set_option("gemv_sk", 0)
