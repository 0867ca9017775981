"""Python mirror of the layer that routes the rows of a batch to the two quantized linears (include/fe_route.h):
`LinCtx`, `Linear::forward`, `Proj::forward` and the MLP block of crates/fe-model/src/model.rs:172-203, 260-403,
3160-3203. torch tensors hold device memory; every compute call goes to libferrite_amd.so.
"""
from __future__ import annotations

import ctypes as C

from . import _lib
from ._lib import check
from .exl3 import _stream

X3_ROWS, X3_PASS, DEC_MAX = 16, 64, 64  # model.rs:172, 179, 203


class LinCtx:
    """The EXL3 kernels + workspace, the prompt kernels + workspace (either pair may be None), the stream, the scratch for
    decode rows of fused prompt projections ([DEC_MAX][max_proj] bf16), and `dec` (model.rs:189-200)."""

    def __init__(self, x3=None, fp4=None, stream=None, max_proj: int = 0):
        _lib.init()
        self._keep = (x3, fp4)
        xk, xws = (x3[0].h, x3[1].h) if x3 else (None, None)
        fk, fws = (fp4[0].h, fp4[1].h) if fp4 else (None, None)
        self.h = C.c_void_p()
        check(_lib.lib().fe_route_ctx_create(C.byref(self.h), xk, xws, fk, fws, _stream(stream), max_proj))
        self._dec = 0

    @property
    def dec(self) -> int:
        return self._dec

    @dec.setter
    def dec(self, d: int):
        check(_lib.lib().fe_route_ctx_set_dec(self.h, d))
        self._dec = d

    def set_bf16(self, kernels):
        """LinCtx::k: the plain bf16 kernels (ferrite_amd.bf16.Kernels), or None."""
        self._bf16 = kernels
        check(_lib.lib().fe_route_ctx_set_bf16(self.h, kernels.h if kernels is not None else None))

    def set_x3_gemm(self, on: bool):
        check(_lib.lib().fe_route_ctx_set_x3_gemm(self.h, int(on)))

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_route_ctx_destroy(self.h)
            self.h = None


class Linear:
    """y[M][N] = x[M][K] . W[N][K]^T with q = the EXL3 linear, p = the prompt linear, w = bf16 weights [n][k] (a torch
    tensor on the device); any of them may be None (model.rs:260-346)."""

    def __init__(self, name: str, n: int, k: int, q=None, p=None, w=None):
        _lib.init()
        self.name, self.n, self.k, self.q, self.p, self.w = name, n, k, q, p, w
        self.h = C.c_void_p()
        check(_lib.lib().fe_route_linear_create(C.byref(self.h), name.encode(), n, k, q.h if q is not None else None,
                                                p.h if p is not None else None))
        if w is not None:
            assert tuple(w.shape) == (n, k) and w.is_contiguous() and w.element_size() == 2
            check(_lib.lib().fe_route_linear_set_bf16(self.h, w.data_ptr()))

    def forward(self, c: LinCtx, y, ldy: int, x, lda: int, m: int, res=None):
        check(_lib.lib().fe_route_linear_forward(self.h, c.h, y.data_ptr(), ldy, x.data_ptr(), lda, m,
                                                 res.data_ptr() if res is not None else 0))

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_route_linear_destroy(self.h)
            self.h = None


class Proj:
    """Several logical outputs of one input; lins = [(Linear, [widths])], prompt = (PromptLinear fused over the first
    `cover` linears, cover) (model.rs:349-403)."""

    def __init__(self, lins, prompt=None):
        _lib.init()
        self.lins, self.prompt = lins, prompt
        n = len(lins)
        handles = (C.c_void_p * n)(*[l.h for l, _ in lins])
        rows = [(C.c_uint32 * len(w))(*w) for _, w in lins]
        widths = (C.POINTER(C.c_uint32) * n)(*[C.cast(r, C.POINTER(C.c_uint32)) for r in rows])
        lens = (C.c_uint32 * n)(*[len(w) for _, w in lins])
        self.parts = sum(len(w) for _, w in lins)
        self.h = C.c_void_p()
        check(_lib.lib().fe_route_proj_create(C.byref(self.h), handles, widths, lens, n,
                                              prompt[0].h if prompt else None, prompt[1] if prompt else 0))

    def total_n(self) -> int:
        return _lib.lib().fe_route_proj_total_n(self.h)

    def forward(self, c: LinCtx, out, x, lda: int, m: int):
        """Returns [(device pointer, row stride in elements)] of every logical part, in order."""
        ptr, ld, got = (C.c_uint64 * self.parts)(), (C.c_uint32 * self.parts)(), C.c_size_t()
        check(_lib.lib().fe_route_proj_forward(self.h, c.h, out.data_ptr(), x.data_ptr(), lda, m, ptr, ld, self.parts,
                                               C.byref(got)))
        return [(ptr[i], ld[i]) for i in range(got.value)]

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_route_proj_destroy(self.h)
            self.h = None


def silu_mul(out, gate_ptr: int, up_ptr: int, ld: int, inter: int, rows: int, stream=None):
    """out[r][c] = bf16(bf16(silu(gate)) * up) (kernels/k-core/src/misc.rs:58-71)."""
    check(_lib.lib().fe_route_silu_mul(_stream(stream), out.data_ptr(), gate_ptr, up_ptr, ld, inter, rows))


def copy2d(dst_ptr: int, ldd: int, src_ptr: int, lds: int, cols: int, rows: int, stream=None):
    check(_lib.lib().fe_route_copy2d(_stream(stream), dst_ptr, ldd, src_ptr, lds, cols, rows))


def mlp_forward(c: LinCtx, gate_up: Proj, down: Linear, x, xn, big, act, rows: int, hidden: int, inter: int, swiglu=None,
                act_ws=None, swiglu_w=None):
    """x += down(SwiGLU(gate(xn), up(xn))) with the reference's routing of decode and prompt rows (model.rs:3160-3203).
    swiglu / act_ws: the fused NVFP4 front; swiglu_w: interleaved bf16 gate|up weights [2 inter][hidden] (its second form)."""
    check(_lib.lib().fe_route_mlp_forward_w(c.h, gate_up.h, down.h, swiglu.h if swiglu is not None else None,
                                            act_ws.h if act_ws is not None else None,
                                            swiglu_w.data_ptr() if swiglu_w is not None else 0, x.data_ptr(), xn.data_ptr(),
                                            big.data_ptr(), act.data_ptr(), rows, hidden, inter))
