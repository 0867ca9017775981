"""Python mirror of the plain bf16 linear (include/fe_bf16.h): the GEMM and the two decode-sized GEMVs of
kernels/k-core/src/gemm.rs and the rule of crates/fe-model/src/model.rs:310-345 that picks among them. torch tensors hold
device memory; every compute call goes to libferrite_amd.so.
"""
from __future__ import annotations

import ctypes as C

from . import _lib
from ._lib import check
from .exl3 import _stream


class Kernels:
    """The gfx950 code object of the bf16 kernels and the GEMM's partial-sum buffer (model.rs:20-24, 75-77)."""

    def __init__(self):
        _lib.init()
        self.h = C.c_void_p()
        check(_lib.lib().fe_bf16_kernels_load(C.byref(self.h)))

    @classmethod
    def load(cls):
        return cls()

    def set_option(self, name: str, value: int):
        """A switch of the launch paths, by name (the header lists them)."""
        check(_lib.lib().fe_bf16_kernels_set_option(self.h, name.encode(), int(value)))

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_bf16_kernels_destroy(self.h)
            self.h = None


def _args(y, ldy, x, lda, w, res, m):
    n, k = w.shape
    assert w.is_contiguous() and w.element_size() == 2
    return (y.data_ptr(), ldy, x.data_ptr(), lda, w.data_ptr(), res.data_ptr() if res is not None else 0, m, n, k)


def gemv(kern: Kernels, y, ldy: int, x, lda: int, w, m: int, res=None, stream=None):
    """y[r] = bf16(x[r] . W^T) (+ res) for r < m <= 8 (gemm.rs:172-262)."""
    check(_lib.lib().fe_bf16_gemv(kern.h, _stream(stream), *_args(y, ldy, x, lda, w, res, m)))


def gemm(kern: Kernels, y, ldy: int, x, lda: int, w, m: int, res=None, stream=None):
    """y = bf16(x . W^T) (+ res) for any m (gemm.rs:128-167)."""
    check(_lib.lib().fe_bf16_gemm(kern.h, _stream(stream), *_args(y, ldy, x, lda, w, res, m)))


def forward(kern: Kernels, y, ldy: int, x, lda: int, w, m: int, res=None, dec: int = 0, stream=None):
    """The bf16 branch of Linear::forward (model.rs:310-345)."""
    check(_lib.lib().fe_bf16_linear_forward(kern.h, _stream(stream), *_args(y, ldy, x, lda, w, res, m), dec))


def interleave_gu(kern: Kernels, gate, up, stream=None):
    """gate, up [inter][k] bf16 -> [2 inter][k], rows interleaved in blocks of 8 (fe_interleave_gu, gemm.rs:281-296)."""
    import torch
    inter, k = gate.shape
    assert up.shape == gate.shape and gate.is_contiguous() and up.is_contiguous()
    dst = torch.empty((2 * inter, k), dtype=gate.dtype, device=gate.device)
    check(_lib.lib().fe_bf16_interleave_gu(kern.h, _stream(stream), dst.data_ptr(), gate.data_ptr(), up.data_ptr(), inter, k))
    return dst


def gemm_swiglu(kern: Kernels, act, x, lda: int, w, m: int, stream=None):
    """act[m][inter] = SwiGLU(x . W^T) over interleaved gate|up weights W [2 inter][k] (fe_gemm_swiglu, gemm.rs:264-279)."""
    n, k = w.shape
    assert w.is_contiguous() and w.element_size() == 2
    check(_lib.lib().fe_bf16_gemm_swiglu(kern.h, _stream(stream), act.data_ptr(), x.data_ptr(), lda, w.data_ptr(), m, n // 2, k))
