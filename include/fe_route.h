/*
 * fe_route: the caller of the two quantized linears, i.e. how the reference's model layer routes the rows of a batch to
 * them: decode / verify rows through the EXL3 trellis GEMV (whatever the batch size, so a row's bits do not depend on
 * the batch), prompt rows through the NVFP4 / FP8 prompt linear, fused prompt projections, and the MLP block built from
 * them. C ABI of crates/fe-model/src/model.rs:172-203 (constants, LinCtx), :260-346 (Linear::forward), :349-403 (Proj),
 * :3160-3203 (the MLP block). A linear with none of the three weight forms (trellis, prompt, plain bf16) fails as the
 * reference does for a linear without weights.
 *
 * All activations are bf16, row-major. Errors are return codes as in fe_exl3.h (fe_hip_last_error() has the text).
 */
#ifndef FE_ROUTE_H
#define FE_ROUTE_H

#include "fe_bf16.h"
#include "fe_exl3.h"
#include "fe_fp4.h"

#ifdef __cplusplus
extern "C" {
#endif

#define FE_X3_ROWS 16 /* batches up to this many rows run the trellis GEMV for every row (model.rs:172) */
#define FE_X3_PASS 64 /* rows of one GEMV call (model.rs:179) */
#define FE_DEC_MAX 64 /* most decode / verify rows of a batch (model.rs:203) */

typedef struct fe_route_ctx fe_route_ctx;       /* LinCtx, model.rs:189-200 */
typedef struct fe_route_linear fe_route_linear; /* Linear, model.rs:260-273 */
typedef struct fe_route_proj fe_route_proj;     /* Proj, model.rs:351-359 */

/* LinCtx: the EXL3 kernels + workspace (either may be NULL: no trellis path), the prompt kernels + workspace (NULL: no
 * prompt path), the stream, and scratch for the decode rows of fused prompt projections, [FE_DEC_MAX][max_proj] bf16
 * (model.rs:195, 1517). Everything is borrowed; the caller keeps it alive. */
int fe_route_ctx_create(fe_route_ctx **out, const fe_exl3_kernels *xk, const fe_exl3_workspace *xws,
                        const fe_fp4_kernels *fk, const fe_fp4_workspace *fws, fe_stream_t s, uint32_t max_proj);
int fe_route_ctx_destroy(fe_route_ctx *c);
/* LinCtx::dec (model.rs:197-199): the first `dec` rows of the next batches are decode / verify rows. */
int fe_route_ctx_set_dec(fe_route_ctx *c, uint32_t dec);
/* LinCtx::k (model.rs:191): the plain bf16 kernels, NULL (default) = no bf16 path. Borrowed. */
int fe_route_ctx_set_bf16(fe_route_ctx *c, const fe_bf16_kernels *bk);
/* What prompt rows of a linear without prompt weights run on: 1 (default) = one call of the trellis linear with all of
 * them, which above 64 rows is the MFMA GEMM (needs an EXL3 workspace for that many rows); 0 = passes of FE_X3_PASS rows
 * through the GEMV as the reference (model.rs:305-309). No counterpart in the reference, which has no trellis GEMM. */
int fe_route_ctx_set_x3_gemm(fe_route_ctx *c, int on);

/* Linear { n, k, q, p } (model.rs:262-273): q = the EXL3 linear, p = the NVFP4 / FP8 prompt linear; either may be NULL.
 * Borrowed. */
int fe_route_linear_create(fe_route_linear **out, const char *name, uint32_t n, uint32_t k, const fe_exl3_linear *q,
                           const fe_fp4_linear *p);
/* Linear::w (model.rs:265): bf16 weights [n][k] on the device (0 = none). They take the rows that neither the trellis GEMV
 * (decode rows of a linear with q) nor p takes; a linear that holds q and w (the loader's bf16 + exl3_decode form,
 * model.rs:664-684) never sends prompt rows back through the trellis (model.rs:305). Borrowed. */
int fe_route_linear_set_bf16(fe_route_linear *l, fe_devptr_t w);
int fe_route_linear_destroy(fe_route_linear *l);
/* Linear::forward (model.rs:275-346): y (row stride ldy) = x (row stride lda) . W^T for m rows; with res (stride ldy):
 * y = bf16(bf16(x . W) + res). On the trellis path res must be y itself (the add happens in the GEMV's epilogue). */
int fe_route_linear_forward(const fe_route_linear *l, const fe_route_ctx *c, fe_devptr_t y, uint32_t ldy, fe_devptr_t x,
                            uint32_t lda, uint32_t m, fe_devptr_t res);

/* Proj { lins: [(Linear, widths)], prompt: (PromptLinear, cover) } (model.rs:351-359): several logical outputs of one
 * input. widths[i] lists the logical parts of linear i side by side (they sum to its n); widths_len[i] their count.
 * prompt (may be NULL) is one fused prompt linear over the first `cover` linears. Borrowed. */
int fe_route_proj_create(fe_route_proj **out, const fe_route_linear *const *lins, const uint32_t *const *widths,
                         const uint32_t *widths_len, size_t count, const fe_fp4_linear *prompt, uint32_t cover);
int fe_route_proj_destroy(fe_route_proj *p);
/* Proj::total_n (model.rs:361-363). */
uint32_t fe_route_proj_total_n(const fe_route_proj *p);
/* Proj::forward (model.rs:365-403): every linear writes its own [m][n] block of `out` (prompt rows of the covered
 * linears: one fused GEMM into [m][prompt n]; their decode rows: the linear's own GEMV into the context's scratch, then
 * copied into the fused layout). Returns (pointer, row stride in elements) of every logical part, in order:
 * part_ptr / part_ld have room for parts_cap entries, *parts_n receives the count. */
int fe_route_proj_forward(const fe_route_proj *p, const fe_route_ctx *c, fe_devptr_t out, fe_devptr_t x, uint32_t lda,
                          uint32_t m, fe_devptr_t *part_ptr, uint32_t *part_ld, size_t parts_cap, size_t *parts_n);

/* fe_silu_mul (kernels/k-core/src/misc.rs:58-71): out[r][c] = bf16(bf16(silu(gate[r][c])) * up[r][c]), gate / up rows
 * share stride ld, out is [rows][inter]. inter % 2 == 0. */
int fe_route_silu_mul(fe_stream_t s, fe_devptr_t out, fe_devptr_t gate, fe_devptr_t up, uint32_t ld, uint32_t inter,
                      uint32_t rows);
/* fe_copy2d (kernels/k-core/src/misc.rs:164-171): dst[r][0..cols) = src[r][0..cols), row strides ldd / lds, cols % 2 == 0. */
int fe_route_copy2d(fe_stream_t s, fe_devptr_t dst, uint32_t ldd, fe_devptr_t src, uint32_t lds, uint32_t cols,
                    uint32_t rows);

/* The MLP block after its norm (model.rs:3160-3203): x [rows][hidden] += down(SwiGLU(gate(xn), up(xn))), xn [rows][hidden]
 * the normed input. gate_up: a Proj whose first two parts are gate and up (each `inter` wide); down: hidden x inter.
 * Prompt rows [d, rows) with more than FE_X3_ROWS of them take the fused front when swiglu (gate|up interleaved by 8,
 * NVFP4), down's prompt form and act_ws (a prompt workspace for [rows][inter]) are given: forward_swiglu, then down's
 * GEMM on the quantized activation with the residual in place. The other rows: gate_up, fe_silu_mul, down with the
 * residual; where all of them go through down's trellis GEMV in one pass, SwiGLU is applied as that GEMV's input
 * rotation reads gate and up (fe_exl3_linear_forward_swiglu: the same bits, act is not written).
 * big: scratch for gate_up's outputs ([rows][total n]); act: scratch [rows][inter]. */
int fe_route_mlp_forward(const fe_route_ctx *c, const fe_route_proj *gate_up, const fe_route_linear *down,
                         const fe_fp4_linear *swiglu, const fe_fp4_workspace *act_ws, fe_devptr_t x, fe_devptr_t xn,
                         fe_devptr_t big, fe_devptr_t act, uint32_t rows, uint32_t hidden, uint32_t inter);

/* The same with the block's second fused form (model.rs:3179-3188): swiglu_w = bf16 gate|up weights [2 inter][hidden]
 * interleaved in blocks of 8 (fe_bf16_interleave_gu), 0 = none. Taken for more than FE_X3_ROWS prompt rows when the NVFP4
 * front does not apply and the context has the bf16 kernels: fe_bf16_gemm_swiglu into act, then down with the residual. */
int fe_route_mlp_forward_w(const fe_route_ctx *c, const fe_route_proj *gate_up, const fe_route_linear *down,
                           const fe_fp4_linear *swiglu, const fe_fp4_workspace *act_ws, fe_devptr_t swiglu_w, fe_devptr_t x,
                           fe_devptr_t xn, fe_devptr_t big, fe_devptr_t act, uint32_t rows, uint32_t hidden, uint32_t inter);

#ifdef __cplusplus
}
#endif
#endif
