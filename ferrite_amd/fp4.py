"""Python mirror of the reference's fe-fp4 NVFP4 layer API over the C ABI (include/fe_fp4.h).

`HostLinear` (fused parts, alpha, g), `PromptLinear::{forward, quantize, gemm}`, `Workspace` and `Kernels` follow
crates/fe-fp4/src/lib.rs. torch tensors hold device memory; every compute call goes to libferrite_amd.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import _lib
from ._lib import check
from .exl3 import _stream

TILE = 128  # crates/fe-fp4/src/lib.rs:28


@dataclass
class Part:
    """One logical checkpoint tensor inside a fused linear (lib.rs:234-243)."""
    name: str
    n0: int
    n: int
    alpha: float
    input_scale: float


@dataclass
class HostLinear:
    """An NVFP4 linear in host memory (lib.rs:285-301): codes [n][k/2] (element 2i in the low nibble), e4m3 scales
    row-major [n][k/16], alpha per output column, g = 1 / max(input_scale)."""
    n: int
    k: int
    name: str
    parts: list
    codes: np.ndarray
    sf: np.ndarray
    alpha: np.ndarray
    g: float
    swiglu: bool = False
    kind: str = "nvfp4"  # or "fp8": e4m3 codes [n][k], no block scales (Kind, lib.rs:229-233)

    @staticmethod
    def fuse(parts):
        """Fuse tensors along N (lib.rs:305-384). parts: (name, codes [n][k/2], scales [n][k/16], weight_scale_2,
        input_scale). The activation scale is the parts' max input_scale; alpha = that times each weight scale."""
        if not parts:
            raise ValueError("no parts")
        k = parts[0][1].shape[1] * 2
        ps, n = [], 0
        for name, codes, sf, wscale, in_scale in parts:
            pn, pk = codes.shape[0], codes.shape[1] * 2
            if pk != k:
                raise ValueError(f"{name}: k {pk} != {k}")
            if pn % TILE or n % TILE:
                raise ValueError(f"{name}: n {pn} not a multiple of {TILE}")
            if sf.shape != (pn, k // 16):
                raise ValueError(f"{name}: weight_scale bytes")
            ps.append(Part(name, n, pn, float(wscale), float(in_scale)))
            n += pn
        if k % 128:
            raise ValueError(f"{parts[0][0]}: k {k} not a multiple of 128")
        in_scale = max(np.float32(p.input_scale) for p in ps)
        if not in_scale > 0:
            raise ValueError(f"{parts[0][0]}: input_scale 0")
        alpha = np.empty(n, np.float32)
        for p in ps:
            p.alpha = float(np.float32(p.alpha) * in_scale)
            alpha[p.n0:p.n0 + p.n] = p.alpha
        return HostLinear(n, k, "+".join(p.name for p in ps), ps,
                          np.ascontiguousarray(np.concatenate([c for _, c, _, _, _ in parts]), dtype=np.uint8),
                          np.ascontiguousarray(np.concatenate([s for _, _, s, _, _ in parts]), dtype=np.uint8), alpha,
                          float(np.float32(1.0) / in_scale))

    @staticmethod
    def fuse_fp8(parts):
        """The same for FP8 parts: (name, codes [n][k] e4m3, weight_scale, input_scale)."""
        if not parts:
            raise ValueError("no parts")
        k = parts[0][1].shape[1]
        ps, n = [], 0
        for name, codes, wscale, in_scale in parts:
            pn, pk = codes.shape
            if pk != k:
                raise ValueError(f"{name}: k {pk} != {k}")
            if pn % TILE or n % TILE:
                raise ValueError(f"{name}: n {pn} not a multiple of {TILE}")
            ps.append(Part(name, n, pn, float(wscale), float(in_scale)))
            n += pn
        if k % 128:
            raise ValueError(f"{parts[0][0]}: k {k} not a multiple of 128")
        in_scale = max(np.float32(p.input_scale) for p in ps)
        if not in_scale > 0:
            raise ValueError(f"{parts[0][0]}: input_scale 0")
        alpha = np.empty(n, np.float32)
        for p in ps:
            p.alpha = float(np.float32(p.alpha) * in_scale)
            alpha[p.n0:p.n0 + p.n] = p.alpha
        return HostLinear(n, k, "+".join(p.name for p in ps), ps,
                          np.ascontiguousarray(np.concatenate([c for _, c, _, _ in parts]), dtype=np.uint8),
                          np.zeros((0,), np.uint8), alpha, float(np.float32(1.0) / in_scale), False, "fp8")

    def into_swiglu(self):
        """gate|up rows interleaved in blocks of 8 (lib.rs:386-417)."""
        if self.kind != "nvfp4" or len(self.parts) != 2 or self.parts[0].n != self.parts[1].n:
            raise ValueError(f"{self.name}: not an NVFP4 gate|up pair")
        if self.n % 256:
            raise ValueError(f"{self.name}: n {self.n}")
        inter = self.n // 2
        r = np.arange(self.n)
        blk, w = r // 16, r % 16
        perm = np.where(w < 8, blk * 8 + w, inter + blk * 8 + w - 8)
        return HostLinear(self.n, self.k, f"{self.name}(swiglu)", self.parts, self.codes[perm].copy(), self.sf[perm].copy(),
                          self.alpha[perm].copy(), self.g, True)

    def upload(self):
        return PromptLinear(self)


class Kernels:
    """The gfx950 code object of the NVFP4 kernels (lib.rs:30-117)."""

    def __init__(self):
        _lib.init()
        self.h = C.c_void_p()
        check(_lib.lib().fe_fp4_kernels_load(C.byref(self.h)))

    @classmethod
    def load(cls):
        return cls()

    def set_option(self, name: str, value: int):
        """A switch of the launch paths, by name (the header lists them)."""
        check(_lib.lib().fe_fp4_kernels_set_option(self.h, name.encode(), int(value)))

    MFMA_KINDS = {"f16": (0, 16), "bf16": (1, 16), "f8": (2, 64)}  # kind, k of the instruction (32 x 32 x k)

    def mfma_peak(self, kind: str, grid: int, iters: int, launches: int, seed: int = 0, stream=None):
        """(milliseconds per launch, TFLOP/s) of the register-only matrix-unit probe (fp4-peak.rs:11-31): grid x 4 wavefronts
        x iters x 16 independent v_mfma_f32_32x32x{16,64} of the given operand kind; seed 0: operands of 0.5 and 1, else
        random signs and mantissas."""
        from .exl3 import _stream
        code, k = self.MFMA_KINDS[kind]
        ms = C.c_float()
        check(_lib.lib().fe_fp4_mfma_peak(self.h, _stream(stream), code, seed, grid, iters, launches, C.byref(ms)))
        flops = grid * 4 * iters * 16 * 2.0 * 32 * 32 * k
        return ms.value, flops / (ms.value * 1e-3) / 1e12

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_fp4_kernels_destroy(self.h)
            self.h = None


class Workspace:
    """Quantized-activation scratch shared by all prompt linears (lib.rs:213-226)."""

    def __init__(self, max_rows: int, max_k: int):
        _lib.init()
        self.h = C.c_void_p()
        check(_lib.lib().fe_fp4_workspace_create(C.byref(self.h), max_rows, max_k))
        self.max_rows, self.max_k = max_rows, max_k
        c, s = C.c_uint64(), C.c_uint64()
        check(_lib.lib().fe_fp4_workspace_buffers(self.h, C.byref(c), C.byref(s), None, None))
        self.codes_ptr, self.sf_ptr = c.value, s.value
        a = C.c_uint64()
        check(_lib.lib().fe_fp4_workspace_operand(self.h, C.byref(a)))
        self.operand_ptr = a.value

    def read_fp8(self, m, k):
        """e4m3 codes [m][k] as a host array."""
        codes = np.empty((m, k), np.uint8)
        check(_lib.lib().fe_hip_memcpy_dtoh(codes.ctypes.data_as(C.c_void_p), self.codes_ptr, codes.size))
        return codes

    def read(self, m, k):
        """(codes [m][k/2], tiled scale bytes of ceil(m/128)*128 rows) as host arrays."""
        codes = np.empty((m, k // 2), np.uint8)
        check(_lib.lib().fe_hip_memcpy_dtoh(codes.ctypes.data_as(C.c_void_p), self.codes_ptr, codes.size))
        rp = (m + TILE - 1) // TILE * TILE
        sf = np.empty(rp * k // 16, np.uint8)
        check(_lib.lib().fe_hip_memcpy_dtoh(sf.ctypes.data_as(C.c_void_p), self.sf_ptr, sf.size))
        return codes, sf

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_fp4_workspace_destroy(self.h)
            self.h = None


class PromptLinear:
    """y[M][N] = x[M][K] . W[N][K]^T for an NVFP4 weight (lib.rs:264-283, 457-543)."""

    def __init__(self, host: HostLinear):
        _lib.init()
        self.n, self.k, self.name, self.parts, self.g, self.swiglu = host.n, host.k, host.name, host.parts, host.g, host.swiglu
        self.kind = host.kind
        self.h = C.c_void_p()
        alpha = np.ascontiguousarray(host.alpha, dtype=np.float32)
        if host.kind == "fp8":
            check(_lib.lib().fe_fp8_linear_upload(C.byref(self.h), host.name.encode(), host.n, host.k,
                                                  host.codes.ctypes.data_as(C.c_void_p), alpha.ctypes.data_as(C.c_void_p),
                                                  host.g))
            return
        check(_lib.lib().fe_fp4_linear_upload(C.byref(self.h), host.name.encode(), host.n, host.k,
                                              host.codes.ctypes.data_as(C.c_void_p), host.sf.ctypes.data_as(C.c_void_p),
                                              alpha.ctypes.data_as(C.c_void_p), host.g))

    @classmethod
    def from_view(cls, name: str, n: int, k: int, codes, scales, alpha, g: float) -> "PromptLinear":
        """A linear over device tensors in the format's own layout (codes [n][k/2], scales [n][k/16] row-major, alpha
        f32 [n]); nothing is copied, the tensors are kept alive (place + set_views, lib.rs:445, 486)."""
        _lib.init()
        self = cls.__new__(cls)
        self.n, self.k, self.name, self.parts, self.g, self.swiglu = n, k, name, [], g, False
        self._keep = (codes, scales, alpha)
        self.h = C.c_void_p()
        if scales is None:  # FP8: e4m3 codes [n][k]
            self.kind = "fp8"
            check(_lib.lib().fe_fp8_linear_from_view(C.byref(self.h), name.encode(), n, k, codes.data_ptr(), alpha.data_ptr(), g))
            return self
        self.kind = "nvfp4"
        check(_lib.lib().fe_fp4_linear_from_view(C.byref(self.h), name.encode(), n, k, codes.data_ptr(), scales.data_ptr(),
                                                 alpha.data_ptr(), g))
        return self

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_fp4_linear_destroy(self.h)
            self.h = None

    def forward(self, kern, ws, y, ldy, x, lda, m, res=None, stream=None):
        check(_lib.lib().fe_fp4_linear_forward(self.h, kern.h, _stream(stream), ws.h, y.data_ptr(), ldy, x.data_ptr(), lda, m,
                                               res.data_ptr() if res is not None else 0))

    def forward_swiglu(self, kern, ws, act, x, lda, m, down_g, stream=None):
        """act = SwiGLU(x . [gate|up]^T), NVFP4-quantized with down_g into the workspace `act` (lib.rs:496-508); then
        down.gemm(kern, act, y, ldy, m, res) finishes the MLP."""
        check(_lib.lib().fe_fp4_linear_forward_swiglu(self.h, kern.h, _stream(stream), ws.h, act.h, x.data_ptr(), lda, m,
                                                      down_g))

    def quantize(self, kern, ws, x, lda, m, stream=None):
        check(_lib.lib().fe_fp4_linear_quantize(self.h, kern.h, _stream(stream), ws.h, x.data_ptr(), lda, m))

    def gemm(self, kern, ws, y, ldy, m, res=None, stream=None):
        check(_lib.lib().fe_fp4_linear_gemm(self.h, kern.h, _stream(stream), ws.h, y.data_ptr(), ldy, m,
                                            res.data_ptr() if res is not None else 0))
