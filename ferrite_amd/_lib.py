"""ctypes loader of libferrite_amd.so (the C ABI declared in include/*.h). There is no CPU fallback: without the built
library, or without a GPU, the calls raise."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libferrite_amd.so")

_lib = None
_inited = False


class FeError(RuntimeError):
    """A non-zero return of the C ABI; `code` is the HIP error or an FE_ERR_* value."""

    def __init__(self, code, text):
        super().__init__(f"[{code}] {text}")
        self.code = code


class View(C.Structure):  # fe_exl3_view
    _fields_ = [("k", C.c_uint32), ("n", C.c_uint32), ("bits", C.c_uint32), ("trellis", C.c_uint64), ("suh", C.c_uint64),
                ("svh", C.c_uint64), ("strips", C.c_uint32)]


class PlanC(C.Structure):  # fe_exl3_plan
    _fields_ = [("sk", C.c_uint32), ("wk", C.c_uint32), ("ver", C.c_uint32), ("occ", C.c_uint32)]


# name -> (restype, argtypes); every symbol include/*.h declares
P, U32, U64, I, SZ, F = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int, C.c_size_t, C.c_float
PP = C.POINTER(C.c_void_p)
SYMBOLS = {
    # fe_hip.h
    "fe_hip_init": (I, [I]),
    "fe_hip_cu_count": (I, [C.POINTER(I)]),
    "fe_hip_device_name": (I, [C.c_char_p, SZ]),
    "fe_hip_synchronize": (I, []),
    "fe_hip_last_error": (C.c_char_p, []),
    "fe_hip_malloc": (I, [C.POINTER(U64), SZ]),
    "fe_hip_free": (I, [U64]),
    "fe_hip_canary_on": (I, []),
    "fe_hip_zero_alloc_on": (I, []),
    "fe_hip_canary_tails": (I, [P, SZ, C.POINTER(SZ)]),
    "fe_hip_memset_d8": (I, [U64, C.c_uint8, SZ, P]),
    "fe_hip_memset_d32": (I, [U64, U32, SZ, P]),
    "fe_hip_memcpy_htod": (I, [U64, P, SZ]),
    "fe_hip_memcpy_dtoh": (I, [P, U64, SZ]),
    "fe_hip_memcpy_dtod_async": (I, [U64, U64, SZ, P]),
    "fe_hip_module_load": (I, [PP, P, SZ]),
    "fe_hip_module_load_file": (I, [PP, C.c_char_p]),
    "fe_hip_module_unload": (I, [P]),
    "fe_hip_module_get_function": (I, [PP, P, C.c_char_p]),
    "fe_hip_func_set_max_dyn_lds": (I, [P, U32]),
    "fe_hip_launch": (I, [P, U32, U32, U32, U32, U32, U32, U32, P, PP]),
    "fe_hip_stream_create": (I, [PP]),
    "fe_hip_stream_destroy": (I, [P]),
    "fe_hip_stream_sync": (I, [P]),
    "fe_hip_time_next_launch": (I, [P, P]),
    "fe_hip_event_create": (I, [PP]),
    "fe_hip_event_destroy": (I, [P]),
    "fe_hip_event_record": (I, [P, P]),
    "fe_hip_event_sync": (I, [P]),
    "fe_hip_event_elapsed_ms": (I, [C.POINTER(F), P, P]),
    "fe_hip_graph_begin": (I, [P]),
    "fe_hip_graph_end": (I, [P, PP]),
    "fe_hip_graph_launch": (I, [P, P]),
    "fe_hip_graph_destroy": (I, [P]),
    # fe_exl3.h
    "fe_exl3_kernels_load": (I, [PP]),
    "fe_exl3_kernels_destroy": (I, [P]),
    "fe_exl3_kernels_set_option": (I, [P, C.c_char_p, U32]),
    "fe_exl3_plan_for": (I, [U32, U32, U32, U32, C.POINTER(PlanC)]),
    "fe_exl3_plan_parse": (I, [C.c_char_p, C.POINTER(PlanC)]),
    "fe_exl3_linear_from_view": (I, [PP, P, C.c_char_p, C.POINTER(View), C.POINTER(PlanC)]),
    "fe_exl3_linear_upload": (I, [PP, P, C.c_char_p, U32, U32, U32, P, P, P, I, C.POINTER(PlanC), U32]),
    "fe_exl3_linear_destroy": (I, [P]),
    "fe_exl3_linear_view": (I, [P, C.POINTER(View), C.POINTER(PlanC)]),
    "fe_exl3_linear_weight_bytes": (SZ, [P]),
    "fe_exl3_workspace_create": (I, [PP, PP, SZ, U32]),
    "fe_exl3_workspace_destroy": (I, [P]),
    "fe_exl3_workspace_xh": (I, [P, C.POINTER(U64), C.POINTER(U32), C.POINTER(U32)]),
    "fe_exl3_linear_forward": (I, [P, P, P, U64, I, U64, I, U32, P]),
    "fe_exl3_linear_forward_static": (I, [P, P, P, U64, I, U64, I, U32]),
    "fe_exl3_linear_forward_is_one_launch": (I, [P, U32]),
    "fe_exl3_linear_keep_decoded": (I, [P, P, I]),
    "fe_exl3_linear_decoded": (I, [P, C.POINTER(U64), C.POINTER(SZ)]),
    "fe_exl3_linear_forward_swiglu": (I, [P, P, P, U64, U64, U32, U64, I, U32, P]),
    "fe_exl3_linear_forward_group": (I, [PP, SZ, P, P, U64, I, C.POINTER(U64), I, U32, P]),
    "fe_exl3_linear_forward_group_launches": (I, [PP, SZ, U32, P]),
    "fe_exl3_mlp_forward": (I, [P, P, P, P, P, U64, I, U64, U64, U64, I, U32, P]),
    "fe_exl3_mlp_forward_launches": (I, [P, P, P, U32, I, P]),
    "fe_exl3_workspace_chain_status": (I, [P, C.POINTER(U32)]),
    "fe_exl3_linear_rotate_input": (I, [P, P, P, U64, I, U32, P]),
    "fe_exl3_linear_gemv_rotated": (I, [P, P, U64, U64, I, U32, P]),
    "fe_exl3_reconstruct_hat_f16": (I, [P, P, C.POINTER(View), U64]),
    "fe_exl3_reconstruct_bf16": (I, [P, P, C.POINTER(View), U64, I, U64, SZ]),
    "fe_exl3_probe_stream_read": (I, [P, P, U64, SZ, U32, U32, C.POINTER(F)]),
    "fe_exl3_probe_decode": (I, [P, P, U32, U32, U32, U32, C.POINTER(F)]),
    "fe_exl3_probe_op": (I, [P, P, C.c_char_p, U32, U32, U32, C.POINTER(F)]),
    # fe_fp4.h
    "fe_fp4_kernels_load": (I, [PP]),
    "fe_fp4_kernels_destroy": (I, [P]),
    "fe_fp4_kernels_set_option": (I, [P, C.c_char_p, C.c_int32]),
    "fe_gemm_schedule_query": (I, [U32, U32, U32, C.c_int32, C.c_int32] + [C.POINTER(U32)] * 6),
    "fe_fp4_linear_upload": (I, [PP, C.c_char_p, U32, U32, P, P, P, F]),
    "fe_fp4_linear_from_view": (I, [PP, C.c_char_p, U32, U32, U64, U64, U64, F]),
    "fe_fp8_linear_upload": (I, [PP, C.c_char_p, U32, U32, P, P, F]),
    "fe_fp8_linear_from_view": (I, [PP, C.c_char_p, U32, U32, U64, U64, F]),
    "fe_fp4_linear_destroy": (I, [P]),
    "fe_fp4_linear_shape": (I, [P, C.POINTER(U32), C.POINTER(U32), C.POINTER(F)]),
    "fe_fp4_workspace_create": (I, [PP, U32, U32]),
    "fe_fp4_workspace_destroy": (I, [P]),
    "fe_fp4_workspace_buffers": (I, [P, C.POINTER(U64), C.POINTER(U64), C.POINTER(U32), C.POINTER(U32)]),
    "fe_fp4_workspace_operand": (I, [P, C.POINTER(U64)]),
    "fe_fp4_linear_forward": (I, [P, P, P, P, U64, U32, U64, U32, U32, U64]),
    "fe_fp4_linear_quantize": (I, [P, P, P, P, U64, U32, U32]),
    "fe_fp4_linear_gemm": (I, [P, P, P, P, U64, U32, U32, U64]),
    "fe_fp4_linear_forward_swiglu": (I, [P, P, P, P, P, U64, U32, U32, F]),
    "fe_fp4_mfma_peak": (I, [P, P, I, U32, U32, U32, U32, C.POINTER(F)]),
    # fe_route.h
    "fe_route_ctx_create": (I, [PP, P, P, P, P, P, U32]),
    "fe_route_ctx_destroy": (I, [P]),
    "fe_route_ctx_set_dec": (I, [P, U32]),
    "fe_route_ctx_set_x3_gemm": (I, [P, I]),
    "fe_route_ctx_set_bf16": (I, [P, P]),
    "fe_route_linear_set_bf16": (I, [P, U64]),
    # fe_bf16.h
    "fe_bf16_kernels_load": (I, [PP]),
    "fe_bf16_kernels_destroy": (I, [P]),
    "fe_bf16_kernels_set_option": (I, [P, C.c_char_p, C.c_int32]),
    "fe_bf16_gemv": (I, [P, P, U64, U32, U64, U32, U64, U64, U32, U32, U32]),
    "fe_bf16_gemm": (I, [P, P, U64, U32, U64, U32, U64, U64, U32, U32, U32]),
    "fe_bf16_interleave_gu": (I, [P, P, U64, U64, U64, U32, U32]),
    "fe_bf16_gemm_swiglu": (I, [P, P, U64, U64, U32, U64, U32, U32, U32]),
    "fe_route_mlp_forward_w": (I, [P, P, P, P, P, U64, U64, U64, U64, U64, U32, U32, U32]),
    "fe_bf16_linear_forward": (I, [P, P, U64, U32, U64, U32, U64, U64, U32, U32, U32, U32]),
    "fe_route_linear_create": (I, [PP, C.c_char_p, U32, U32, P, P]),
    "fe_route_linear_destroy": (I, [P]),
    "fe_route_linear_forward": (I, [P, P, U64, U32, U64, U32, U32, U64]),
    "fe_route_proj_create": (I, [PP, PP, C.POINTER(C.POINTER(U32)), C.POINTER(U32), SZ, P, U32]),
    "fe_route_proj_destroy": (I, [P]),
    "fe_route_proj_total_n": (U32, [P]),
    "fe_route_proj_forward": (I, [P, P, U64, U64, U32, U32, C.POINTER(U64), C.POINTER(U32), SZ, C.POINTER(SZ)]),
    "fe_route_silu_mul": (I, [P, U64, U64, U64, U32, U32, U32]),
    "fe_route_copy2d": (I, [P, U64, U32, U64, U32, U32, U32]),
    "fe_route_mlp_forward": (I, [P, P, P, P, P, U64, U64, U64, U64, U32, U32, U32]),
}


def lib():
    """The loaded library. torch is imported first so that both bind the same HIP runtime (one libamdhip64.so.7)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FeError(-1, f"{LIB_PATH} is not built: run `python -m ferrite_amd.build`")
        import torch  # noqa: F401  (loads torch's libamdhip64 before ours resolves the same soname)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(code):
    if code:
        raise FeError(code, lib().fe_hip_last_error().decode(errors="replace"))


def init(ordinal: int = 0):
    """Bind device `ordinal` (Context::new, crates/fe-cuda/src/lib.rs:112-126). Raises without a GPU."""
    global _inited
    if not _inited:
        check(lib().fe_hip_init(ordinal))
        _inited = True
