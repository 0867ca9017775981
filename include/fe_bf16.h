/*
 * fe_bf16: the plain bf16 weight form of the caller's linear, y[M][N] = x[M][K] . W[N][K]^T (+ residual), W row-major
 * bf16, f32 sums, bf16 out: what the reference's model layer runs for a linear that has neither a trellis nor a prompt
 * form (the reconstructed bf16 weights of its prefill fallback, the narrow GDN projections). C ABI of the kernels
 * of kernels/k-core/src/gemm.rs (fe_gemm_bf16 :128-167, fe_gemv_bf16 :172-208, fe_gemv_bf16_kw :210-262, fe_gemm_swiglu
 * :264-279, fe_interleave_gu :281-296) and of the rule that picks among the first three,
 * crates/fe-model/src/model.rs:310-345.
 *
 * Activations are bf16, row-major, rows 16-byte aligned (lda % 8 == 0); y / res rows 8-byte aligned (ldy % 4 == 0).
 * K % 64 == 0, N % 8 == 0. Errors are return codes as in fe_exl3.h (fe_hip_last_error() has the text).
 */
#ifndef FE_BF16_H
#define FE_BF16_H

#include "fe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The loaded kernels (LinKernels { gemm, gemv, gemv_kw }, model.rs:20-24, 75-77) plus the device buffer the GEMM leaves
 * the partial sums of its last, K-split round of tiles in: calls that share one object must be stream-ordered. */
typedef struct fe_bf16_kernels fe_bf16_kernels;
int fe_bf16_kernels_load(fe_bf16_kernels **out);
int fe_bf16_kernels_destroy(fe_bf16_kernels *k);
/* Switches by name: "nc" columns a GEMV program takes (FE_BF16_NC; -1 = by the shape), "raster_group" (FE_BF16_GROUP;
 * -1 = by the shape), "gemm_splits" (FE_GEMM_SPLITS). Read from the environment once, at load; no call reads it later. */
int fe_bf16_kernels_set_option(fe_bf16_kernels *k, const char *name, int32_t value);

/* fe_gemv_bf16 / fe_gemv_bf16_kw (gemm.rs:172-262): m <= 8 rows. One kernel family here: a program takes 1, 2, 4
 * or 8 columns by the width of the linear and the row count (model.rs:316-322 picks between the two kernels by the shape), and a row's bits
 * depend neither on that nor on m. res (stride ldy) may be 0; with it y = bf16(bf16(x . W) + res), res may be y. */
int fe_bf16_gemv(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda,
                 fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k);
/* fe_gemm_bf16 (gemm.rs:128-167): any m. */
int fe_bf16_gemm(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda,
                 fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k);
/* fe_interleave_gu (gemm.rs:281-296): dst [2 inter][k] = gate and up rows ([inter][k] each) interleaved in blocks of 8,
 * the weight layout of fe_bf16_gemm_swiglu (what fuse_swiglu builds at load, model.rs:1118-1140). */
int fe_bf16_interleave_gu(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t dst, fe_devptr_t gate, fe_devptr_t up,
                          uint32_t inter, uint32_t k);
/* fe_gemm_swiglu (gemm.rs:264-279): act[m][inter] = bf16(bf16(silu(bf16(g))) * bf16(u)) with g | u = x . W^T over the
 * interleaved weights W [2 inter][k]; act rows have stride inter. inter % 8 == 0. */
int fe_bf16_gemm_swiglu(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t act, fe_devptr_t x, uint32_t lda,
                        fe_devptr_t w, uint32_t m, uint32_t inter, uint32_t k);
/* The bf16 branch of Linear::forward (model.rs:310-345): all rows of a batch of <= 16, else the leading `dec` rows, go
 * through the GEMV in passes of 8 rows (when k % 256 == 0); the rows after them through the GEMM. */
int fe_bf16_linear_forward(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x,
                           uint32_t lda, fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k, uint32_t dec);

#ifdef __cplusplus
}
#endif
#endif
