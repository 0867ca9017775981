"""CPU-side checks of the product: the C-ABI library loads and exports every symbol include/*.h declares, and the
host logic of the Python mirror (layouts, slices, plans, fused linears) agrees with the reference's unit tests and the
oracle. No compute call is made here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for h in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(fe_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from ferrite_amd import _lib
    L = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 60
    for n in names:
        assert hasattr(L, n), n
    # and the ctypes table covers exactly the header
    assert sorted(_lib.SYMBOLS) == names


def test_embedded_code_objects_are_gfx950_elf():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(ROOT, "ferrite_amd", "libferrite_amd.so")],
                         stdout=subprocess.PIPE, text=True).stdout
    # the code objects are private data of the library; check them through the build directory instead
    for k in ("k_exl3", "k_fp4", "k_route", "k_bf16"):
        p = os.path.join(ROOT, "ferrite_amd", "_build", k + ".hsaco")
        if os.path.exists(p):
            head = open(p, "rb").read(20)
            assert head[:4] == b"\x7fELF" and head[18] == 0xE0  # EM_AMDGPU
    assert "fe_exl3_linear_forward" in out and "fe_fp4_linear_forward" in out and "fe_bf16_linear_forward" in out


def synthetic(k, n, bits):
    """crates/fe-exl3/src/format.rs:162-168"""
    from ferrite_amd.exl3 import Exl3Tensor
    tw = 8 * bits
    cnt = k // 16 * (n // 16) * tw
    trellis = (np.arange(cnt, dtype=np.uint64) * 2654435761 & 0xFFFFFFFF).astype(np.uint32)
    suh = (0x3C00 | (np.arange(k) & 0x3FF)).astype(np.uint16)
    svh = (0xBC00 | (np.arange(n) & 0x3FF)).astype(np.uint16)
    return Exl3Tensor("t", k, n, bits, trellis, suh, svh)


def test_host_slices_keep_tiles():
    # crates/fe-exl3/src/format.rs:170-186
    t = synthetic(256, 512, 3)
    c = t.slice_cols([(128, 256), (384, 512)])
    assert (c.k, c.n) == (256, 256)
    for kt in range(16):
        assert np.array_equal(c.tile(kt, 0), t.tile(kt, 8))
        assert np.array_equal(c.tile(kt, 8), t.tile(kt, 24))
    assert np.array_equal(c.svh[:128], t.svh[128:256])
    r = t.slice_rows(128, 256)
    assert (r.k, r.n) == (128, 512)
    assert np.array_equal(r.tile(0, 5), t.tile(8, 5))
    assert np.array_equal(r.suh, t.suh[128:256])
    with pytest.raises(ValueError):
        t.slice_cols([(0, 100)])
    with pytest.raises(ValueError):
        t.slice_rows(64, 128)


def test_host_strips_layout():
    # crates/fe-exl3/src/format.rs:188-202
    t = synthetic(256, 256, 2)
    s = t.strips()
    tw = t.tile_words()
    for b in range(2):
        for kt in range(16):
            for j in range(8):
                at = ((b * 16 + kt) * 8 + j) * tw
                assert np.array_equal(s[at:at + tw], t.tile(kt, 8 * b + j))


def test_host_layouts_match_the_oracle(oracle):
    from ferrite_amd import synth
    t = synth.exl3_tensor(256, 384, 5, 3)
    o = oracle.Exl3(t.k, t.n, t.bits, t.trellis, t.suh, t.svh)
    assert np.array_equal(t.strips(), oracle.strips(o))
    c, oc = t.slice_cols([(128, 384)]), oracle.slice_cols(o, [(128, 384)])
    assert np.array_equal(c.trellis, oc.trellis) and np.array_equal(c.svh, oc.svh)
    r, orr = t.slice_rows(128, 256), oracle.slice_rows(o, 128, 256)
    assert np.array_equal(r.trellis, orr.trellis) and np.array_equal(r.suh, orr.suh)
    assert t.trellis_bytes() == 256 * 384 * 5 // 8


def test_exl3_tensor_rejects_bad_shapes():
    from ferrite_amd.exl3 import Exl3Tensor
    with pytest.raises(ValueError):
        Exl3Tensor("x", 128, 128, 9, np.zeros(8 * 8 * 72, np.uint32), np.zeros(128, np.uint16), np.zeros(128, np.uint16))
    with pytest.raises(ValueError):
        Exl3Tensor("x", 128, 128, 4, np.zeros(10, np.uint32), np.zeros(128, np.uint16), np.zeros(128, np.uint16))
    with pytest.raises(ValueError):
        Exl3Tensor("x", 128, 128, 4, np.zeros(8 * 8 * 32, np.uint32), np.zeros(64, np.uint16), np.zeros(128, np.uint16))


def test_plans():
    from ferrite_amd.exl3 import Linear, Plan
    assert Plan.parse("2,8") == Plan(2, 8, 1, 0)
    assert Plan.parse("10,4,9,2") == Plan(10, 4, 9, 2)
    assert Plan.parse("x") is None
    # plan_for: whole programs per CU (the target `blocks` rounded, 1..5 a CU; 256 CUs where no device is bound), runs
    # of at least wk units of 128 channels x 128 columns, never more programs than that leaves; sk records the K splits
    # per column block this amounts to. Shapes in the tuned table take its occ and wk instead.
    os.environ["FE_EXL3_UNTUNED"] = "1"
    try:
        for k, n in [(5120, 17408), (17408, 5120), (5120, 5120), (5120, 1024), (128, 128), (1024, 256), (512, 384)]:
            for blocks in (256, 704, 1024, 0):
                p = Linear.plan_for(k, n, 4, blocks)
                occ = min(5, max(1, (blocks + 128) // 256)) if blocks else 4
                units, nb = (k // 128) * (n // 128), n // 128
                programs = max(1, min(occ * 256, units // p.wk))
                assert (p.ver, p.occ, p.wk) == (3, occ, 4) and p.sk == -(-programs // nb)
        assert Linear.plan_for(5120, 17408, 4, 1024).sk == 8 and Linear.plan_for(5120, 1024, 4, 1024).sk == 10
    finally:
        del os.environ["FE_EXL3_UNTUNED"]
    os.environ["FE_EXL3_NOSPLIT"] = "1"
    try:
        assert Linear.plan_for(5120, 1024, 4, 1024).sk == 1
    finally:
        del os.environ["FE_EXL3_NOSPLIT"]
    from ferrite_amd._lib import FeError
    with pytest.raises(FeError):
        Linear.plan_for(100, 128, 4, 1024)


def test_fused_host_linear(oracle):
    from ferrite_amd.fp4 import HostLinear
    rng = np.random.default_rng(0)
    k = 256
    mk = lambda n: (rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8), rng.integers(1, 0x7E, size=(n, k // 16), dtype=np.uint8))
    (gc, gs), (uc, us) = mk(128), mk(128)
    h = HostLinear.fuse([("gate", gc, gs, 0.5, 0.02), ("up", uc, us, 0.25, 0.04)])
    # crates/fe-fp4/src/lib.rs:344-348, 378-383: activation scale = max input_scale; alpha = weight scale * that
    assert h.n == 256 and h.k == k and h.g == float(np.float32(1) / np.float32(0.04))
    assert np.all(h.alpha[:128] == np.float32(0.5) * np.float32(0.04)) and np.all(h.alpha[128:] == np.float32(0.25) * np.float32(0.04))
    assert np.array_equal(h.codes[128:], uc) and np.array_equal(h.sf[:128], gs)
    s = h.into_swiglu()
    perm = [oracle.swiglu_perm(r, 128) for r in range(256)]
    assert np.array_equal(s.codes, h.codes[perm]) and np.array_equal(s.sf, h.sf[perm]) and np.array_equal(s.alpha, h.alpha[perm])
    with pytest.raises(ValueError):
        HostLinear.fuse([("a", gc[:100], gs[:100], 1.0, 1.0)])
    with pytest.raises(ValueError):
        HostLinear.fuse([("a", gc, gs, 1.0, 0.0)])


def test_synthetic_scales_are_e4m3_nearest(oracle):
    from ferrite_amd import synth
    v = np.abs(np.random.default_rng(1).normal(size=4000)).astype(np.float32) * np.float32(0.1)
    v = np.concatenate([np.clip(v, 2.0 ** -9, 448.0), np.array([448.0, 500.0, 2.0 ** -9, 0.0156, 0.015625], np.float32)])
    got = synth.e4m3_from_f32(v)
    want = np.array([oracle.f32_to_e4m3(x) for x in v], np.uint8)
    assert np.array_equal(got, want)
    x = synth.activations(3, 128, 5)
    assert np.array_equal(x, np.array([[oracle.f32_to_bf16(f) for f in row] for row in
                                       np.random.default_rng([5, 3, 128, 7]).normal(size=(3, 128)).astype(np.float32)], np.uint16))


def test_compute_calls_fail_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from ferrite_amd import _lib
    with pytest.raises(_lib.FeError):
        _lib.check(_lib.lib().fe_hip_init(0))


def gemm_schedule(tiles, ktiles, cus=256, mode=1, small_b=True):
    from ferrite_amd import _lib
    out = [C.c_uint32(0) for _ in range(6)]
    _lib.check(_lib.lib().fe_gemm_schedule_query(tiles, ktiles, cus, mode, int(small_b), *[C.byref(o) for o in out]))
    return dict(zip(("stream_k", "programs", "whole", "splits", "run", "run_rem"), (o.value for o in out)))


def test_gemm_schedule_choice():
    """Host arithmetic of the schedule the GEMMs share (no GPU call): stream-K only where its runs have the shape that was
    measured faster, the one-piece schedule with its K cut everywhere else; every schedule covers each k tile once."""
    # 2048 rows x 5120 columns: 160 tiles on 256 CUs, no cut fills its rounds -> runs of 5/8 of a tile over all tiles
    s = gemm_schedule(160, 272)
    assert s == {"stream_k": 1, "programs": 256, "whole": 0, "splits": 1, "run": 170, "run_rem": 0}
    assert gemm_schedule(160, 80)["run"] == 50 and gemm_schedule(160, 80, small_b=False)["stream_k"] == 1
    # 2048 x 17408: 544 tiles = two whole rounds and 32 tiles, which would be 8 pieces each as runs behind them: short K and
    # at most 2 1/8 rounds -> equal runs of 170 k tiles over all tiles (in step), for a small weight operand; else one piece
    # a program, the last 32 cut 7 ways. 2304 x 16384 (576 tiles, 2 1/4 rounds): one whole round and runs of 100 over the
    # other 320. 4096 x 17408: three whole rounds + runs of 100. Whole rounds only, or long K with no whole round in front:
    # one piece
    s = gemm_schedule(544, 80)
    assert s == {"stream_k": 1, "programs": 256, "whole": 0, "splits": 1, "run": 170, "run_rem": 0}
    s = gemm_schedule(576, 80)
    assert s == {"stream_k": 1, "programs": 256, "whole": 256, "splits": 1, "run": 100, "run_rem": 0}
    for tiles, run in ((320, 100), (384, 120), (416, 130)):  # between one and two rounds, a last round of up to 5/8 of the CUs
        s = gemm_schedule(tiles, 80)
        assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 0, run, 0)
    for tiles in (448, 480):  # a fuller last round that runs whole: left alone
        assert gemm_schedule(tiles, 80)["stream_k"] == 0
    s = gemm_schedule(544, 80, small_b=False)
    assert (s["stream_k"], s["programs"], s["whole"], s["splits"]) == (0, 512 + 32 * 7, 512, 7)
    assert gemm_schedule(1088, 80)["whole"] == 768 and gemm_schedule(1088, 80)["run"] == 100
    assert gemm_schedule(320, 272)["stream_k"] == 0 and gemm_schedule(512, 80)["stream_k"] == 0
    # whole rounds in front of a last round of 160 tiles
    s = gemm_schedule(416, 16)
    assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 256, 10, 0)
    # 129..160 tiles, where the one-piece schedule's three pieces a tile leave its second round half empty: runs over all
    # tiles even though they are not in step, for a small weight operand only
    s = gemm_schedule(136, 80)
    assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 0, 42, 128)
    assert gemm_schedule(136, 80, small_b=False)["stream_k"] == 0 and gemm_schedule(148, 64)["run"] == 37
    # the same for the last round of a larger launch: 1536 x 17408 is 408 tiles = one whole round + runs over the other 152
    s = gemm_schedule(408, 80)
    assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 256, 47, 128)
    assert gemm_schedule(408, 80, small_b=False)["stream_k"] == 0 and gemm_schedule(680, 80)["stream_k"] == 0
    # one whole round and a last round of an eighth of the CUs or fewer, too short for runs behind the whole round: equal
    # runs of at least a tile over all tiles, the programs of an XCD at no more than two depths of K (small weight operand)
    s = gemm_schedule(272, 80)
    assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 0, 85, 0)
    assert gemm_schedule(288, 80)["run"] == 90 and gemm_schedule(272, 80, small_b=False)["stream_k"] == 0
    for tiles, ktiles in ((280, 80), (528, 80), (272, 16), (296, 80)):  # unequal runs; a second whole round; short runs; 40 tiles
        assert gemm_schedule(tiles, ktiles)["stream_k"] == 0, (tiles, ktiles)
    # tile counts that a K cut balances, or that run whole in one round, or whose runs would not be in step, or with many
    # pieces a tile: one piece a program
    for tiles, ktiles in ((128, 80), (192, 80), (224, 80), (240, 272), (120, 272), (32, 80), (8, 80), (256, 80), (512, 80)):
        assert gemm_schedule(tiles, ktiles)["stream_k"] == 0, (tiles, ktiles)
    assert gemm_schedule(160, 272, mode=0)["stream_k"] == 0
    # forced: runs over all tiles (2) / as many whole rounds as leave good runs (3)
    s = gemm_schedule(544, 80, mode=2)
    assert (s["stream_k"], s["whole"], s["run"], s["run_rem"]) == (1, 0, 170, 0)
    assert gemm_schedule(544, 80, mode=3, small_b=False)["whole"] == 256
    s = gemm_schedule(27, 16, mode=2)  # 432 k tiles on 256 programs: 176 runs of 2, 80 of 1
    assert (s["stream_k"], s["run"], s["run_rem"]) == (1, 1, 176)
    # every k tile exactly once
    for tiles, ktiles, mode in ((160, 272, 1), (544, 80, 1), (27, 16, 2), (1088, 80, 1), (416, 16, 1), (408, 80, 1), (136, 80, 1),
                                (272, 80, 1)):
        s = gemm_schedule(tiles, ktiles, mode=mode)
        assert s["stream_k"] == 1
        assert s["whole"] % s["programs"] == 0
        assert s["whole"] * ktiles + s["programs"] * s["run"] + s["run_rem"] == tiles * ktiles


def test_gemm_schedule_covers_every_k_tile_once():
    """Whatever the policy picks (every tile count up to five rounds, several K lengths, both kinds of weight operand, all
    modes): a stream-K schedule's whole rounds and runs add up to tiles x k tiles, whole rounds are a multiple of the
    grid, and a one-piece schedule's cut tiles fit one launch."""
    for ktiles in (16, 40, 64, 80, 128, 272):
        for tiles in list(range(1, 1300, 7)) + [160, 256, 272, 288, 320, 384, 416, 448, 480, 512, 528, 544, 576, 640, 1088]:
            for small_b in (True, False):
                for mode in (0, 1, 2, 3):
                    s = gemm_schedule(tiles, ktiles, mode=mode, small_b=small_b)
                    what = (tiles, ktiles, small_b, mode, s)
                    if s["stream_k"]:
                        assert mode != 0 and s["programs"] <= 256 and s["whole"] % s["programs"] == 0 and s["whole"] <= tiles, what
                        assert s["whole"] * ktiles + s["programs"] * s["run"] + s["run_rem"] == tiles * ktiles, what
                        assert s["run_rem"] < s["programs"] and s["run"] + (1 if s["run_rem"] else 0) > 0, what
                    else:
                        assert s["whole"] <= tiles and s["splits"] >= 1, what
                        assert s["programs"] == s["whole"] + (tiles - s["whole"]) * s["splits"], what
                        assert s["splits"] == 1 or s["splits"] * 4 <= ktiles, what

