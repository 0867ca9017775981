"""ctypes/numpy front end of the CPU oracle (``oracle/libfe_oracle.so``).

TEST INFRASTRUCTURE ONLY: a restatement of the reference's CPU algorithms (crates/fe-exl3/src/{half,format,cpu}.rs,
crates/fe-fp4/src/format.rs).  Only the tests, ``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of ``bench.py``
may import this package; the product library never does.

How each function is pinned (tests/test_oracle_*.py):

* half: the reference's own unit tests (half.rs:104-123) + numpy's float16/float32 conversions over all codes.
* tile_state: three independent formulations (cpu.rs:14-23, recon.rs:12-22, gemv.rs:184-208) agree for bits 1..8,
  and write-then-recover of known states.
* decode_mul1: all 65536 states against numpy float64 -> float16 (single rounding) of the closed form.
* value_row/value_col: bijection onto 16x16 and the m16n8k16 B-fragment map (kernels/kcommon/src/mma.rs:3-8).
* fwht128: H[i][j] = (-1)^popcount(i & j) as an explicit matrix, H.H = 128 I.
* weight_block_f64 / weight_bf16 / linear_f64 / gemv_ref / rotate_input_ref: explicit dense-matrix algebra in numpy
  on k = n = 128 / 256.
* strips / slices: the reference's unit tests (format.rs:170-202) with its synthetic generator.
* e4m3 / e2m1 / quant_fp4_row / tiling / ref_gemm: the reference's unit tests (crates/fe-fp4/src/format.rs:186-215,
  lib.rs:583-589), exhaustive tables and brute-force nearest-value search in float64.

Parity with exllamav3 on real checkpoints is not pinned here (no checkpoint, no exllamav3 in this image); the
synthetic configurations define correctness against the reference's own decoder, which is what this restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfe_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds). Returns the library path."""
    srcs = [os.path.join(_HERE, f) for f in ("half.c", "exl3.c", "fp4.c", "fe_oracle.h", "Makefile")]
    if force or not os.path.exists(_SO) or any(os.path.getmtime(s) > os.path.getmtime(_SO) for s in srcs):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libfe_oracle.so"])
    return _SO


_lib = None


class _Exl3(C.Structure):
    _fields_ = [("k", C.c_size_t), ("n", C.c_size_t), ("bits", C.c_uint32), ("trellis", C.c_void_p),
                ("suh", C.c_void_p), ("svh", C.c_void_p)]


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.or_f16_to_f64.restype = C.c_double
        L.or_f16_to_f64.argtypes = [C.c_uint16]
        L.or_f64_to_f16.restype = C.c_uint16
        L.or_f64_to_f16.argtypes = [C.c_double]
        L.or_f16_fma.restype = C.c_uint16
        L.or_f16_fma.argtypes = [C.c_uint16] * 3
        L.or_f32_to_bf16.restype = C.c_uint16
        L.or_f32_to_bf16.argtypes = [C.c_float]
        L.or_bf16_to_f32.restype = C.c_float
        L.or_bf16_to_f32.argtypes = [C.c_uint16]
        L.or_f64_to_bf16_torch.restype = C.c_uint16
        L.or_f64_to_bf16_torch.argtypes = [C.c_double]
        L.or_bf16_ulp_diff.restype = C.c_uint32
        L.or_bf16_ulp_diff.argtypes = [C.c_uint16, C.c_uint16]
        for f in ("or_value_row", "or_value_col"):
            getattr(L, f).restype = C.c_size_t
            getattr(L, f).argtypes = [C.c_size_t, C.c_size_t]
        for f in ("or_tile_state", "or_tile_state_funnel", "or_tile_state_lane"):
            getattr(L, f).restype = C.c_uint32
            getattr(L, f).argtypes = [C.c_void_p, C.c_uint32, C.c_size_t]
        L.or_decode_mul1.restype = C.c_uint16
        L.or_decode_mul1.argtypes = [C.c_uint32]
        L.or_decode_tile.restype = None
        L.or_decode_tile.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p]
        L.or_strips.restype = None
        L.or_strips.argtypes = [C.POINTER(_Exl3), C.c_void_p]
        L.or_slice_cols.restype = C.c_size_t
        L.or_slice_cols.argtypes = [C.POINTER(_Exl3), C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
        L.or_slice_rows.restype = C.c_size_t
        L.or_slice_rows.argtypes = [C.POINTER(_Exl3), C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p]
        L.or_w_hat_f16.restype = None
        L.or_w_hat_f16.argtypes = [C.POINTER(_Exl3), C.c_size_t, C.c_size_t, C.c_void_p]
        L.or_fwht128.restype = None
        L.or_fwht128.argtypes = [C.c_void_p]
        L.or_weight_block_f64.restype = None
        L.or_weight_block_f64.argtypes = [C.POINTER(_Exl3), C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        L.or_weight_bf16.restype = None
        L.or_weight_bf16.argtypes = [C.POINTER(_Exl3), C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
        L.or_linear_f64.restype = None
        L.or_linear_f64.argtypes = [C.POINTER(_Exl3), C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.or_rotate_input_ref.restype = None
        L.or_rotate_input_ref.argtypes = [C.POINTER(_Exl3), C.c_void_p, C.c_size_t, C.c_void_p]
        L.or_gemv_ref.restype = None
        L.or_gemv_ref.argtypes = [C.POINTER(_Exl3), C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]
        L.or_e4m3_to_f32.restype = C.c_float
        L.or_e4m3_to_f32.argtypes = [C.c_uint8]
        L.or_f32_to_e4m3.restype = C.c_uint8
        L.or_f32_to_e4m3.argtypes = [C.c_float]
        L.or_f32_to_e2m1.restype = C.c_uint8
        L.or_f32_to_e2m1.argtypes = [C.c_float]
        L.or_quant_fp4_row.restype = None
        L.or_quant_fp4_row.argtypes = [C.c_void_p, C.c_size_t, C.c_float, C.c_void_p, C.c_void_p]
        L.or_quant_fp8_row.restype = None
        L.or_quant_fp8_row.argtypes = [C.c_void_p, C.c_size_t, C.c_float, C.c_void_p]
        L.or_tiled_offset.restype = C.c_size_t
        L.or_tiled_offset.argtypes = [C.c_size_t] * 3
        L.or_tile_scales.restype = None
        L.or_tile_scales.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.or_untile_scales.restype = None
        L.or_untile_scales.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.or_dequant_fp4_row.restype = None
        L.or_dequant_fp4_row.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_size_t]
        L.or_dequant_fp8_row.restype = None
        L.or_dequant_fp8_row.argtypes = [C.c_void_p, C.c_float, C.c_void_p, C.c_size_t]
        L.or_ref_gemm.restype = None
        L.or_ref_gemm.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_void_p]
        L.or_select.restype = C.c_size_t
        L.or_select.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        L.or_swiglu_perm.restype = C.c_size_t
        L.or_swiglu_perm.argtypes = [C.c_size_t, C.c_size_t]
        L.or_default_threads.restype = C.c_int
        L.or_default_threads.argtypes = [C.c_int]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


class Exl3:
    """A borrowed EXL3 tensor in the stored layout (format.rs:17-30): trellis u32 [k/16 * n/16 * 8*bits]."""

    def __init__(self, k, n, bits, trellis, suh, svh):
        self.k, self.n, self.bits = int(k), int(n), int(bits)
        self.trellis = _c(trellis, np.uint32).reshape(-1)
        self.suh = _c(suh, np.uint16).reshape(-1)
        self.svh = _c(svh, np.uint16).reshape(-1)
        assert self.trellis.size == self.k // 16 * (self.n // 16) * 8 * self.bits
        assert self.suh.size == self.k and self.svh.size == self.n
        self._s = _Exl3(self.k, self.n, self.bits, self.trellis.ctypes.data, self.suh.ctypes.data, self.svh.ctypes.data)

    @property
    def ref(self):
        return C.byref(self._s)

    @property
    def tw(self):
        return 8 * self.bits

    def tile(self, kt, nt):
        i = (kt * (self.n // 16) + nt) * self.tw
        return self.trellis[i:i + self.tw]


# ---- half ---------------------------------------------------------------------------------------------------
def f16_to_f64(h): return lib().or_f16_to_f64(int(h))
def f64_to_f16(x): return lib().or_f64_to_f16(float(x))
def f16_fma(a, b, c): return lib().or_f16_fma(int(a), int(b), int(c))
def f32_to_bf16(x): return lib().or_f32_to_bf16(float(np.float32(x)))
def bf16_to_f32(h): return lib().or_bf16_to_f32(int(h))
def f64_to_bf16_torch(x): return lib().or_f64_to_bf16_torch(float(x))
def bf16_ulp_diff(a, b): return lib().or_bf16_ulp_diff(int(a), int(b))


# ---- EXL3 ---------------------------------------------------------------------------------------------------
def value_row(lane, j): return lib().or_value_row(lane, j)
def value_col(lane, j): return lib().or_value_col(lane, j)


def tile_state(tile, bits, t, form="bits"):
    tile = _c(tile, np.uint32)
    f = {"bits": lib().or_tile_state, "funnel": lib().or_tile_state_funnel, "lane": lib().or_tile_state_lane}[form]
    return f(_p(tile), bits, t)


def decode_mul1(state): return lib().or_decode_mul1(int(state))


def decode_tile(tile, bits):
    tile = _c(tile, np.uint32)
    out = np.empty((16, 16), np.uint16)
    lib().or_decode_tile(_p(tile), bits, _p(out))
    return out


def strips(t: Exl3):
    out = np.empty_like(t.trellis)
    lib().or_strips(t.ref, _p(out))
    return out


def slice_cols(t: Exl3, ranges):
    r = _c(np.array(ranges, dtype=np.uint64).reshape(-1), np.uint64)
    cols = sum(max(0, b - a) for a, b in ranges)
    tr = np.empty(t.k // 16 * max(cols, 16) // 16 * t.tw, np.uint32)
    sv = np.empty(max(cols, 1), np.uint16)
    got = lib().or_slice_cols(t.ref, _p(r), len(ranges), _p(tr), _p(sv))
    if got == 0:
        raise ValueError(f"column ranges {ranges} not 128-aligned in 0..{t.n}")
    return Exl3(t.k, got, t.bits, tr[: t.k // 16 * got // 16 * t.tw], t.suh.copy(), sv[:got])


def slice_rows(t: Exl3, k0, k1):
    if not (0 <= k0 < k1 <= t.k) or k0 % 128 or k1 % 128:
        raise ValueError(f"row range {k0}..{k1} not 128-aligned in 0..{t.k}")
    tr = np.empty((k1 - k0) // 16 * (t.n // 16) * t.tw, np.uint32)
    su = np.empty(k1 - k0, np.uint16)
    got = lib().or_slice_rows(t.ref, k0, k1, _p(tr), _p(su))
    assert got == k1 - k0
    return Exl3(got, t.n, t.bits, tr, su, t.svh.copy())


def w_hat_f16(t: Exl3, n0=0, ns=None):
    ns = t.n - n0 if ns is None else ns
    assert n0 % 16 == 0 and ns % 16 == 0 and n0 + ns <= t.n
    w = np.empty((t.k, ns), np.uint16)
    lib().or_w_hat_f16(t.ref, n0, ns, _p(w))
    return w


def fwht128(v):
    v = _c(v, np.float64).copy()
    assert v.size == 128
    lib().or_fwht128(_p(v))
    return v


def weight_block_f64(t: Exl3, r0, n0, ns):
    assert r0 % 128 == 0 and n0 % 128 == 0 and ns % 128 == 0 and n0 + ns <= t.n
    w = np.empty((128, ns), np.float64)
    lib().or_weight_block_f64(t.ref, r0, n0, ns, _p(w))
    return w


def weight_bf16(t: Exl3, n0=0, ns=None, layout="KN", threads=0):
    ns = t.n - n0 if ns is None else ns
    out = np.empty((t.k, ns) if layout == "KN" else (ns, t.k), np.uint16)
    lib().or_weight_bf16(t.ref, n0, ns, 0 if layout == "KN" else 1, threads, _p(out))
    return out


def linear_f64(t: Exl3, x, threads=1):
    x = _c(x, np.float64).reshape(-1, t.k)
    y = np.empty((x.shape[0], t.n), np.float64)
    lib().or_linear_f64(t.ref, _p(x), x.shape[0], threads, _p(y))
    return y


def rotate_input_ref(t: Exl3, x):
    x = _c(x, np.float64).reshape(-1, t.k)
    xh = np.empty(x.shape, np.uint16)
    lib().or_rotate_input_ref(t.ref, _p(x), x.shape[0], _p(xh))
    return xh


def gemv_ref(t: Exl3, w_hat, xh):
    w_hat = _c(w_hat, np.uint16)
    xh = _c(xh, np.uint16).reshape(-1, t.k)
    nc = w_hat.shape[1]
    assert w_hat.shape[0] == t.k
    y = np.empty((xh.shape[0], nc), np.float64)
    lib().or_gemv_ref(t.ref, _p(w_hat), nc, _p(xh), xh.shape[0], _p(y))
    return y


# ---- FP4 ----------------------------------------------------------------------------------------------------
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32)


def e4m3_to_f32(b): return lib().or_e4m3_to_f32(int(b))
def f32_to_e4m3(x): return lib().or_f32_to_e4m3(float(np.float32(x)))
def f32_to_e2m1(x): return lib().or_f32_to_e2m1(float(np.float32(x)))


def quant_fp4_row(x, g):
    x = _c(x, np.uint16).reshape(-1)
    codes = np.empty(x.size // 2, np.uint8)
    sf = np.empty(x.size // 16, np.uint8)
    lib().or_quant_fp4_row(_p(x), x.size, float(np.float32(g)), _p(codes), _p(sf))
    return codes, sf


def quant_fp4(x, g):
    """Row-wise quant_fp4_row over x [m][k] bf16 bits -> (codes [m][k/2], sf [m][k/16])."""
    x = _c(x, np.uint16)
    m, k = x.shape
    codes = np.empty((m, k // 2), np.uint8)
    sf = np.empty((m, k // 16), np.uint8)
    for r in range(m):
        lib().or_quant_fp4_row(_p(x[r]), k, float(np.float32(g)), _p(codes[r]), _p(sf[r]))
    return codes, sf


def quant_fp8_row(x, g):
    x = _c(x, np.uint16).reshape(-1)
    out = np.empty(x.size, np.uint8)
    lib().or_quant_fp8_row(_p(x), x.size, float(np.float32(g)), _p(out))
    return out


def tiled_offset(r, b, kb): return lib().or_tiled_offset(r, b, kb)


def tile_scales(src, rows, kb):
    src = _c(src, np.uint8).reshape(-1)
    assert kb % 8 == 0 and src.size == rows * kb
    out = np.empty((rows + 127) // 128 * 128 * kb, np.uint8)
    lib().or_tile_scales(_p(src), rows, kb, _p(out))
    return out


def untile_scales(t, rows, kb):
    t = _c(t, np.uint8).reshape(-1)
    out = np.empty(rows * kb, np.uint8)
    lib().or_untile_scales(_p(t), rows, kb, _p(out))
    return out


def dequant_fp4_row(codes, sf, gs=1.0):
    codes = _c(codes, np.uint8).reshape(-1)
    sf = _c(sf, np.uint8).reshape(-1)
    out = np.empty(codes.size * 2, np.float32)
    lib().or_dequant_fp4_row(_p(codes), _p(sf), float(np.float32(gs)), _p(out), out.size)
    return out


def dequant_fp4(codes, sf, gs=1.0):
    codes = _c(codes, np.uint8)
    sf = _c(sf, np.uint8)
    out = np.empty((codes.shape[0], codes.shape[1] * 2), np.float32)
    for r in range(codes.shape[0]):
        lib().or_dequant_fp4_row(_p(codes[r]), _p(sf[r]), float(np.float32(gs)), _p(out[r]), out.shape[1])
    return out


def dequant_fp8_row(codes, gs=1.0):
    codes = _c(codes, np.uint8).reshape(-1)
    out = np.empty(codes.size, np.float32)
    lib().or_dequant_fp8_row(_p(codes), float(np.float32(gs)), _p(out), out.size)
    return out


def ref_gemm(a, w, threads=0):
    """a [rows][k] f32, w [n][k] f32 -> [rows][n] f32 (f64 accumulation)."""
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    rows, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k
    y = np.empty((rows, n), np.float32)
    lib().or_ref_gemm(_p(a), rows, _p(w), n, k, threads, _p(y))
    return y


def bf16_linear_ref(x_bits, w_bits, res_bits=None, threads=0):
    """The plain bf16 linear of the caller (kernels/k-core/src/gemm.rs:128-167): x [m][k], w [n][k] as bf16 bit
    patterns (uint16) -> (y bits [m][n], the f64-accumulated sums as f32). y = bf16(sum); with res: bf16(bf16(sum) + res),
    two roundings (gemm.rs:152-158). Pinned in tests/test_oracle_bf16.py by one-hot weights (y == x), all-ones operands
    (y == k), a brute-force loop on a tiny case and a residual whose two roundings differ from one."""
    x = (np.ascontiguousarray(x_bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    w = (np.ascontiguousarray(w_bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    acc = ref_gemm(x, w, threads)

    def rne(f):
        b = np.ascontiguousarray(f, np.float32).view(np.uint32)
        return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)

    y = rne(acc)
    if res_bits is not None:
        r = (np.ascontiguousarray(res_bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
        y = rne((y.astype(np.uint32) << 16).view(np.float32) + r)
    return y, acc


def select(src, row_len, keep, c0, c1):
    src = _c(src, np.uint8).reshape(-1)
    kp = _c(np.array(keep, dtype=np.uint64).reshape(-1), np.uint64)
    out = np.empty(sum(b - a for a, b in keep) * (c1 - c0), np.uint8)
    w = lib().or_select(_p(src), row_len, _p(kp), len(keep), c0, c1, _p(out))
    assert w == out.size
    return out


def swiglu_perm(r, inter): return lib().or_swiglu_perm(r, inter)


def default_threads(cap=0): return lib().or_default_threads(cap)
