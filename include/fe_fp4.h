/*
 * fe_fp4: the NVFP4 prompt linear (e2m1 codes, e4m3 scale per 16 along K, fp32 scale per output column) over fe_hip,
 * with the FP8 (e4m3, per-tensor scale) linears and the fused gate|up SwiGLU front of the same layer API.
 *
 * C ABI of the reference's fe-fp4 layer API for its NVFP4 path (crates/fe-fp4/src/lib.rs): HostLinear-style inputs
 * (codes [n][k/2], row-major scales [n][k/16], alpha[n], g), PromptLinear::{forward, quantize, gemm}, Workspace.
 * Requirements as in the reference (lib.rs:156-157, 521-537): N % 128 == 0, K % 128 == 0, ldy % 8 == 0, y and res
 * 16-byte aligned, m == 0 is a no-op, m <= ws.max_rows, k <= ws.max_k. Errors are return codes, as in fe_exl3.h.
 */
#ifndef FE_FP4_H
#define FE_FP4_H

#include "fe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct fe_fp4_kernels fe_fp4_kernels;     /* Kernels, crates/fe-fp4/src/lib.rs:30-117 */
typedef struct fe_fp4_linear fe_fp4_linear;       /* PromptLinear, crates/fe-fp4/src/lib.rs:265-283 */
typedef struct fe_fp4_workspace fe_fp4_workspace; /* Workspace, crates/fe-fp4/src/lib.rs:215-226 */

/* Kernels::load (lib.rs:65-117): the embedded gfx950 code object, or the file named by FE_FP4_HSACO.
 * FE_FP4_GROUP sets the raster group height in row tiles (default 8, 0 = all). */
int fe_fp4_kernels_load(fe_fp4_kernels **out);
int fe_fp4_kernels_destroy(fe_fp4_kernels *k);
/* Switches of the launch paths, by name (the environment variable that sets the same switch when the kernels are loaded):
 * "group_m" (FE_FP4_GROUP), "gemv" 0/1 (FE_FP4_NO_GEMV), "gemv_sk" (FE_FP4_GEMV_SK; 0 = automatic), "gemv_strips" 0/1/2 (FE_FP4_NO_STRIPS: the GEMV over strips of 16
 * weight rows never / where it pays / wherever it fits), "gemv_once" 0/1 (FE_FP4_NO_ONCE: the strips kernel that issues all of a workgroup's loads
 * before it waits, where a wavefront's share of K is short enough; same bits), "gemv_waves" (FE_FP4_GEMV_WAVES: wavefronts of a strip's workgroup; 0 = automatic), "xcd" -1/0/1
 * (FE_FP4_XCD), "fp8_f16" 0/1 (FE_FP8_F16), "gemm_splits" (FE_GEMM_SPLITS), "gemm_sk" 0..3 (FE_GEMM_SK: the stream-K schedule of the
 * GEMM never / where it is the faster one / over all tiles / whole rounds then runs, the last two for tests). forward() reads no environment variable. No
 * counterpart in the reference (its FE_FP4_GROUP is read at load too, crates/fe-fp4/src/lib.rs:31-32, 68). */
int fe_fp4_kernels_set_option(fe_fp4_kernels *k, const char *name, int32_t value);
/* How a GEMM launch of `tiles` 256 x 256 output tiles, `ktiles` k tiles each, would be spread over `cus` CUs under
 * gemm_sk = mode (the schedule the EXL3, NVFP4 and FP8 GEMMs share; small_b: packed weights of a few KB a k tile), with a
 * workspace of two partial slots a CU and enough counters: stream_k 0 = one piece a program (whole = tiles computed
 * whole, splits = pieces of each remaining tile, added by a reduce launch), 1 = stream-K (whole = tiles computed whole in
 * rounds, then runs of run (+ 1 for the first run_rem programs) k tiles over the rest). Pure host arithmetic, no GPU
 * call. No counterpart in the reference; for tests and tuners. */
int fe_gemm_schedule_query(uint32_t tiles, uint32_t ktiles, uint32_t cus, int32_t mode, int32_t small_b, uint32_t *stream_k,
                           uint32_t *programs, uint32_t *whole, uint32_t *splits, uint32_t *run, uint32_t *run_rem);

/* HostLinear::upload (lib.rs:425-440) of an NVFP4 linear already fused on the host: codes [n][k/2], scales row-major
 * [n][k/16] (e4m3), alpha[n] = max(input_scale) * weight_scale_2 of the column's part, g = 1 / max(input_scale). */
int fe_fp4_linear_upload(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, const uint8_t *codes,
                         const uint8_t *scales, const float *alpha, float g);
/* A linear over device buffers the caller owns (the reference's streamed form, PromptLinear::set_views lib.rs:485-494). */
int fe_fp4_linear_from_view(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, fe_devptr_t codes,
                            fe_devptr_t scales, fe_devptr_t alpha, float g);
/* The same for an FP8 linear (Kind::Fp8, lib.rs:229-233, 305-384): e4m3 codes [n][k], no block scales,
 * alpha[n] = max(input_scale) * weight_scale. forward / quantize / gemm below take either kind. */
int fe_fp8_linear_upload(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, const uint8_t *codes,
                         const float *alpha, float g);
int fe_fp8_linear_from_view(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, fe_devptr_t codes,
                            fe_devptr_t alpha, float g);
int fe_fp4_linear_destroy(fe_fp4_linear *l);
int fe_fp4_linear_shape(const fe_fp4_linear *l, uint32_t *n, uint32_t *k, float *g);

/* Workspace::new(max_rows, max_k) (lib.rs:221-226): quantized activations: codes, tiled scales
 * ([rows/128][k/128][128][8], crates/fe-fp4/src/format.rs:98-111), and the fp16 operand the GEMM reads. */
int fe_fp4_workspace_create(fe_fp4_workspace **out, uint32_t max_rows, uint32_t max_k);
int fe_fp4_workspace_destroy(fe_fp4_workspace *ws);
int fe_fp4_workspace_buffers(const fe_fp4_workspace *ws, fe_devptr_t *codes, fe_devptr_t *sf, uint32_t *max_rows,
                             uint32_t *max_k);

/* The fp16 operand [rows][k] the quantizer leaves beside the codes (what the GEMM kernels read): a small power of two
 * times the quantized value, exact. No counterpart in the reference, whose tensor cores read the codes. */
int fe_fp4_workspace_operand(const fe_fp4_workspace *ws, fe_devptr_t *aq);

/* PromptLinear::forward (lib.rs:510-516): y (row stride ldy) = x (bf16, row stride lda) . W^T for m rows; with res
 * (stride ldy, may equal y): y = bf16(bf16(x . W^T) + res). res == 0: none. */
int fe_fp4_linear_forward(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                          fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda, uint32_t m, fe_devptr_t res);
/* PromptLinear::quantize (lib.rs:518-530). */
int fe_fp4_linear_quantize(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                           fe_devptr_t x, uint32_t lda, uint32_t m);
/* PromptLinear::gemm (lib.rs:532-543) over activations already quantized into ws by a linear with the same k and g. */
int fe_fp4_linear_gemm(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                       fe_devptr_t y, uint32_t ldy, uint32_t m, fe_devptr_t res);

/* PromptLinear::forward_swiglu (lib.rs:496-508): the fused MLP front for prompt rows. l = gate and up fused with their
 * rows interleaved in blocks of 8 (HostLinear::into_swiglu, lib.rs:386-417), n = 2 * inter, n % 256 == 0. Quantizes x
 * into ws, then act = SwiGLU(x . [gate|up]^T) is written NVFP4-quantized with global scale down_g (the down
 * projection's g) into the workspace `act` (rows <= act.max_rows, inter <= act.max_k), ready for
 * fe_fp4_linear_gemm(down, kern, s, act, y, ldy, m, res). */
int fe_fp4_linear_forward_swiglu(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s,
                                 const fe_fp4_workspace *ws, const fe_fp4_workspace *act, fe_devptr_t x, uint32_t lda,
                                 uint32_t m, float down_g);

/* Matrix-unit peak probe (fe_fp4_peak, kernels/k-fp4/src/lib.rs:866-916, driven by crates/fe-fp4/src/bin/fp4-peak.rs):
 * grid x 4 wavefronts issue iters x 16 independent matrix instructions each on register operands, no memory traffic.
 * kind 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_32x32x16_bf16, 2: v_mfma_f32_32x32x64_f8f6f4 (e4m3 x e4m3).
 * seed 0: operands of 0.5 and 1 (few bits toggle, the reference's kind of pattern); otherwise random signs and mantissas, as
 * a GEMM on real data toggles its operands (the clock held under the board's power limit depends on it).
 * ms: average milliseconds of `launches` launches; flops of one = grid * 4 * iters * 16 * 2 * 32 * 32 * (kind == 2 ? 64 : 16). */
int fe_fp4_mfma_peak(const fe_fp4_kernels *kern, fe_stream_t s, int kind, uint32_t seed, uint32_t grid, uint32_t iters,
                     uint32_t launches, float *ms);

#ifdef __cplusplus
}
#endif
#endif
