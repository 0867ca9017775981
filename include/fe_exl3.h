/*
 * fe_exl3: the EXL3 (trellis-coded, Hadamard-rotated) linear layer over fe_hip.
 *
 * C ABI of the reference's fe-exl3 layer API: the same packed-weight layout (trellis words in the stored
 * [k/16][n/16][8*bits] layout or the "strips" relayout, fp16 suh[k] / svh[n] sign-scale vectors), the same launch-plan
 * and workspace objects and the same call signatures, so that fe-model's `Linear::forward`
 * (crates/fe-model/src/model.rs:275-346) can bind it in place of `fe_exl3::linear` + `fe_exl3::gpu`.
 *
 * All functions return 0 or an error code (HIP's, or FE_ERR_*); fe_hip_last_error() gives the text. Shape and
 * workspace violations are errors, never aborts (crates/fe-exl3/src/linear.rs:291-307). Calls that share a workspace
 * must be ordered on one stream. No call synchronizes the host; forward/rotate_input/gemv_rotated only enqueue.
 */
#ifndef FE_EXL3_H
#define FE_EXL3_H

#include "fe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define FE_ERR_SHAPE 10001     /* shape does not fit the kernel or plan */
#define FE_ERR_WORKSPACE 10002 /* rows or sizes exceed the workspace */
#define FE_ERR_ARG 10003       /* null or inconsistent argument */
#define FE_ERR_UNSUPPORTED 10004

/* Activation / output element type; the *_ADD forms are outputs only: y += x @ W, bf16 adds in f32 and rounds once.
 * Values are the kernels' flag (crates/fe-exl3/src/linear.rs:15-31). */
enum { FE_DTYPE_BF16 = 0, FE_DTYPE_F32 = 1, FE_DTYPE_BF16_ADD = 2, FE_DTYPE_F32_ADD = 3 };

/* Device pointers of one EXL3 tensor (Exl3View, crates/fe-exl3/src/gpu/mod.rs:17-34). strips != 0: trellis is in the
 * strips layout [n/128][k/16][8][8*bits] (crates/fe-exl3/src/format.rs:70-84). */
typedef struct {
    uint32_t k, n, bits;
    fe_devptr_t trellis, suh, svh;
    uint32_t strips;
} fe_exl3_view;

/* Launch plan (Plan, crates/fe-exl3/src/linear.rs:33-43), the reference's plan strings "sk,wk[,ver[,occ]]". The gfx950
 * decode GEMV deals 128-channel x 128-column units of the tensor to its programs in equal contiguous runs; a plan says how
 * many programs. ver 1 (the reference's meaning): sk programs per 128-column block, i.e. sk K splits (needs k / 64
 * divisible by sk). ver 2, 3 (what fe_exl3_plan_for returns): occ programs per CU, each a run of at least wk units; sk then
 * records the K splits per column block this amounts to. ver 4: sk programs in all (any partition: tests and tuners). */
typedef struct {
    uint32_t sk, wk, ver, occ;
} fe_exl3_plan;

typedef struct fe_exl3_kernels fe_exl3_kernels;     /* Kernels, crates/fe-exl3/src/gpu/mod.rs:78-102 */
typedef struct fe_exl3_linear fe_exl3_linear;       /* Linear, crates/fe-exl3/src/linear.rs:163-176 */
typedef struct fe_exl3_workspace fe_exl3_workspace; /* Workspace, crates/fe-exl3/src/linear.rs:137-161 */

/* Kernels::load: the embedded gfx950 code object, or the file named by FE_EXL3_HSACO (the reference's FE_EXL3_CUBIN,
 * crates/fe-exl3/src/gpu/mod.rs:88-93). */
int fe_exl3_kernels_load(fe_exl3_kernels **out);
int fe_exl3_kernels_destroy(fe_exl3_kernels *k);
/* Switches of the launch paths, by name (the environment variable that sets the same switch when the kernels are loaded):
 * "fused_rot" 0/1 (FE_EXL3_NO_FUSED_ROT), "fused_rot_pairs" (FE_EXL3_FUSED_ROT_PAIRS), "group" 0/1 (FE_EXL3_NO_GROUP),
 * "hat_rows" (FE_EXL3_HAT_ROWS; 0 = never), "lds_pad" 0/1 (FE_EXL3_NO_LDS_PAD), "fuse" 0/1 (FE_EXL3_NO_FUSE), "gemm_group_m" (FE_EXL3_GROUP),
 * "gemm_splits" (FE_GEMM_SPLITS), "mlp_chain" 0/1 (FE_EXL3_NO_CHAIN), "chain_spin" (FE_EXL3_CHAIN_SPIN),
 * "handoff_fenced" 0/1 (the decode GEMV for 1..16 rows with its hand-off between programs written with release / acquire fences
 * at agent scope and plain accesses instead of write-through stores and loads that pass the L2: several times slower, a cross-check), "gemm_sk" 0..3 (FE_GEMM_SK: the stream-K schedule of the prefill GEMM never / where it
 * is the faster one / over all tiles / whole rounds then runs, the last two for tests). forward() reads no environment variable; tests and tuners flip a switch here. Not for
 * use while launches with this handle are being issued from another thread. No counterpart in the reference, which reads
 * its switches (FE_EXL3_NOSPLIT, FE_EXL3_UNTUNED, ...) from the environment at plan time. */
int fe_exl3_kernels_set_option(fe_exl3_kernels *k, const char *name, uint32_t value);

/* Linear::plan_for (crates/fe-exl3/src/linear.rs:217-233): the tuned plan of the shape where the table has one for this
 * CU count (plans::tuned; FE_EXL3_UNTUNED=1 skips the table), else the rule: `blocks` is the program target (4 per CU is the
 * default, default_blocks linear.rs:132-134), rounded to whole programs per CU. Honours FE_EXL3_NOSPLIT=1 / FE_EXL3_SPLIT=0. */
int fe_exl3_plan_for(uint32_t k, uint32_t n, uint32_t bits, uint32_t blocks, fe_exl3_plan *out);
/* Plan::parse "sk,wk[,ver[,occ]]" (linear.rs:47-55). */
int fe_exl3_plan_parse(const char *s, fe_exl3_plan *out);

/* Linear::from_view (linear.rs:242-266): a linear over device buffers the caller owns and keeps alive. */
int fe_exl3_linear_from_view(fe_exl3_linear **out, const fe_exl3_kernels *kern, const char *name, const fe_exl3_view *view,
                             const fe_exl3_plan *plan);
/* Linear::new(DeviceExl3::upload_strips(tensor)) (linear.rs:212-215, gpu/mod.rs:52-70): host tensor in the stored
 * layout (trellis words, fp16 suh/svh); the linear owns the device copy. plan == NULL: plan_for(blocks). */
int fe_exl3_linear_upload(fe_exl3_linear **out, const fe_exl3_kernels *kern, const char *name, uint32_t k, uint32_t n,
                          uint32_t bits, const uint32_t *trellis, const uint16_t *suh, const uint16_t *svh, int strips,
                          const fe_exl3_plan *plan, uint32_t blocks);
int fe_exl3_linear_destroy(fe_exl3_linear *l);
int fe_exl3_linear_view(const fe_exl3_linear *l, fe_exl3_view *view, fe_exl3_plan *plan);
/* Trellis bytes streamed per call (linear.rs:268-271). */
size_t fe_exl3_linear_weight_bytes(const fe_exl3_linear *l);

/* Workspace::new(&[&Linear], max_rows) (linear.rs:147-160): xh fp16 [max_rows][max k], f32 split partials, split
 * arrival counters (zero at rest; each call re-arms them). */
int fe_exl3_workspace_create(fe_exl3_workspace **out, fe_exl3_linear *const *linears, size_t count, uint32_t max_rows);
int fe_exl3_workspace_destroy(fe_exl3_workspace *ws);
int fe_exl3_workspace_xh(const fe_exl3_workspace *ws, fe_devptr_t *xh, uint32_t *max_rows, uint32_t *max_k);

/* Linear::forward (linear.rs:274-287): y[rows][n] = x[rows][k] @ W; x bf16 or f32, y bf16 or f32 (+ the add forms),
 * both row-major and contiguous. rows <= 64 run the decode GEMV (HBM-bound); more rows run the LDS-staged MFMA GEMM.
 * The workspace's xh holds the rotated input afterwards, as after rotate_input. */
int fe_exl3_linear_forward(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype,
                           fe_devptr_t y, int y_dtype, uint32_t rows, const fe_exl3_workspace *ws);
/* Prefill over weights decoded once: decodes the trellis into fp16 tiles (2 bytes a weight, in the rotated basis) that
 * stay with the linear, and from then on every call with more than 64 rows runs the GEMM over them without decoding
 * (same bits as the decoding GEMM for whole tiles). The role of the reference's dequantized prompt weights
 * (reconstruct_bf16 into Linear.w, crates/fe-model/src/model.rs:262-266), for callers that have the memory: 178 MB for
 * 5120 x 17408. on == 0 frees them. Stream-ordered; the first GEMM may follow on the same stream. */
int fe_exl3_linear_keep_decoded(fe_exl3_linear *l, fe_stream_t s, int on);
/* The kept tiles (null / 0 when there are none), for checks of the decoder that runs in the hot loops against
 * decode_tile (crates/fe-exl3/src/cpu.rs:57-69): fp16 W_hat, block (tn, kt) of 32 KB at ((tn * (k / 64)) + kt) * 32768 =
 * columns 256 tn .. + 255 of channels 64 kt .. + 63, 128 bytes a column r, the 16-byte chunk c (channels 8 c .. 8 c + 7)
 * of column r at byte r * 128 + 16 * (c ^ (r & 7) ^ ((r >> 3) & 1)). */
int fe_exl3_linear_decoded(const fe_exl3_linear *l, fe_devptr_t *tiles, size_t *bytes);
/* 1 if forward() with this many rows is a single launch (the decode GEMV rotates its own input: every program's K range
 * is whole 128-element Hadamard blocks), 0 if it is rotate_input followed by gemv_rotated. Same bits either way. */
int fe_exl3_linear_forward_is_one_launch(const fe_exl3_linear *l, uint32_t rows);
/* forward() on SwiGLU(gate, up) without the activation ever being stored: y = act @ W with
 * act[r][c] = bf16(bf16(silu(gate[r][c])) * up[r][c]) (the arithmetic of fe_silu_mul, kernels/k-core/src/misc.rs:58-71),
 * computed as the input rotation reads it, inside the GEMV for few rows. gate and up are bf16 [rows][>= k] with row
 * stride ld elements, 8-byte aligned, ld % 4 == 0. Same bits as fe_silu_mul into a buffer followed by
 * fe_exl3_linear_forward on it. This is the down projection of the MLP block (crates/fe-model/src/model.rs:3184-3199),
 * where the reference launches fe_silu_mul and Linear::forward one after the other. */
int fe_exl3_linear_forward_swiglu(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t gate,
                                  fe_devptr_t up, uint32_t ld, fe_devptr_t y, int y_dtype, uint32_t rows,
                                  const fe_exl3_workspace *ws);
/* Several linears applied to the same input (the q, k, v or the gate, up projections of a layer), 1..64 rows: one GEMV
 * launch whose programs are those of the members' own launches, so y[i] has the bits of
 * fe_exl3_linear_forward(ls[i], ...). The launches' start-up and tails overlap and the members fill each other's gaps
 * on the CUs. Where forward() of every member rotates its own input the group does too (one launch); otherwise one
 * launch rotates the input for all members first (two launches). That needs 2..4 members of the same k and bits and a
 * workspace with room for all members' partial sums and rotated inputs (one created from these linears has it);
 * otherwise the members run one after the other (FE_EXL3_NO_GROUP=1 forces that). Which member's rotated input is left
 * in the workspace is unspecified. The reference loops over the linears (Proj::forward,
 * crates/fe-model/src/model.rs:365-403): this entry point has no counterpart there. */
int fe_exl3_linear_forward_group(const fe_exl3_linear *const *ls, size_t count, const fe_exl3_kernels *kern, fe_stream_t s,
                                 fe_devptr_t x, int x_dtype, const fe_devptr_t *ys, int y_dtype, uint32_t rows,
                                 const fe_exl3_workspace *ws);
/* Launches of that call: 1, 2, or 0 when the members run one after the other. */
int fe_exl3_linear_forward_group_launches(const fe_exl3_linear *const *ls, size_t count, uint32_t rows,
                                          const fe_exl3_workspace *ws);
/* The decode MLP block in one launch: yg = x @ W_gate, yu = x @ W_up (bf16 [rows][n]), y (+)= SwiGLU(yg, yu) @ W_down.
 * Whenever the one launch does not apply the call is fe_exl3_linear_forward_group on {gate, up} followed by
 * fe_exl3_linear_forward_swiglu on down (two launches), with the same bits: a row's result does not depend on the row
 * count of the call (1..64 rows), and every output has the bits of the linear's own forward. Option "chain_down_units"
 * (FE_EXL3_CHAIN_DOWN_UNITS; 2, 4 or 8; default 0 = off; set before the workspace is made) partitions down, in this call
 * only, into programs of that many units of 128 channels x 128 columns where that divides its column blocks, at every row
 * count the GEMV takes, so that rows still do not depend on the batch; down's bits are then its own forward's only where
 * the two partitions coincide. Short programs end the one launch sooner at one row (5120 x 17408 MLP, 4 units: 45.5
 * against 46.4 us at 4 bits, 53.2 against 55.7 at 5) and cost the two-launch form of the call from 8 rows on (4 bits, 8 /
 * 16 / 64 rows: 65 / 76 / 184 us a block against 60 / 69 / 161): for deployments that only ever decode single rows. This is the MLP block of a decode row
 * (crates/fe-model/src/model.rs:3184-3199), where the reference launches seven kernels; the entry point has no
 * counterpart there. In the one launch the programs of the down projection follow those of gate and up in the grid:
 * they request their first weights at once, wait until the column blocks of gate and up that hold their input channels
 * are published (every finished block of the front stage is written through to memory and then announced by a ready
 * word), and rotate SwiGLU(gate, up) from there; start-up, launch overhead and tail of the second launch disappear
 * under the first. The wait is bounded ("chain_spin" polls, about a microsecond each): when it runs out the program sets
 * the workspace's chain error word and goes on, the launch still ends normally, and its results are void;
 * fe_exl3_workspace_chain_status reports and clears that. It applies where every program rotates at most
 * "chain_rot_pairs" (32) pairs of (row, 128-channel block) of its own input (up to 4 rows on a 5120 x 17408 MLP), with the
 * same width, gate and up of one shape, and a workspace created from (at least) these three linears; "mlp_chain" 0
 * (FE_EXL3_NO_CHAIN=1) turns it off.
 * fe_exl3_mlp_forward_launches: 1 if the call is the one launch, else 0. */
int fe_exl3_mlp_forward(const fe_exl3_linear *gate, const fe_exl3_linear *up, const fe_exl3_linear *down,
                        const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype, fe_devptr_t yg, fe_devptr_t yu,
                        fe_devptr_t y, int y_dtype, uint32_t rows, const fe_exl3_workspace *ws);
int fe_exl3_mlp_forward_launches(const fe_exl3_linear *gate, const fe_exl3_linear *up, const fe_exl3_linear *down, uint32_t rows,
                                 int y_dtype, const fe_exl3_workspace *ws);
/* Synchronizes the device and returns the chain error word of the workspace (0: every bounded wait of the one-launch MLP
 * calls so far was met). When it is set, the results of the calls since the last check are void; the word and the launch
 * state behind it are cleared, and fe_exl3_mlp_forward on this workspace is its two-launch form from then on (the same
 * bits): an expired wait means that this system does not dispatch workgroups in grid order, which the one launch needs. */
int fe_exl3_workspace_chain_status(fe_exl3_workspace *ws, uint32_t *error);
/* forward() for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc). No counterpart in the reference, whose forward always takes a Workspace. The
 * rotated inputs, split partial sums and arrival counters live in one static device array of FE_EXL3_STATIC_BYTES that
 * every GPU the library runs on holds until the process ends; the call allocates and frees nothing. Same kernels and
 * the same bits as fe_exl3_linear_forward. Limits: 1..FE_EXL3_STATIC_ROWS rows, rows * k * 2 <= 1 MiB of rotated inputs,
 * (programs + n / 128) * rows * 512 bytes of partial sums <= FE_EXL3_STATIC_BYTES - 1 MiB - 16 KiB, n <= 524288; anything
 * larger is FE_ERR_WORKSPACE. `programs` follows the linear's plan (occ programs a CU, 1..5): the array is sized for the
 * widest tuned shape, 5120 x 17408, at 16 rows under occ 5 (1280 programs on 256 CUs: 11.06 MiB of partial sums). All
 * calls on one GPU share the array: calls that overlap on one GPU (two streams) race; order them. */
#define FE_EXL3_STATIC_BYTES (13u << 20)
#define FE_EXL3_STATIC_ROWS 16
int fe_exl3_linear_forward_static(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                  int x_dtype, fe_devptr_t y, int y_dtype, uint32_t rows);
/* Linear::rotate_input (linear.rs:289-298): xh = fp16(H(x * suh) / sqrt(128)) into the workspace. */
int fe_exl3_linear_rotate_input(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                int x_dtype, uint32_t rows, const fe_exl3_workspace *ws);
/* Linear::gemv_rotated (linear.rs:300-341): the trellis linear on already rotated fp16 inputs xh [rows][k]. */
int fe_exl3_linear_gemv_rotated(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype,
                                uint32_t rows, const fe_exl3_workspace *ws);

/* Kernels::reconstruct_hat_f16 (gpu/mod.rs:159-165): rotated-basis W_hat as fp16 [k][n]; stored layout only. */
int fe_exl3_reconstruct_hat_f16(const fe_exl3_kernels *kern, fe_stream_t s, const fe_exl3_view *w, fe_devptr_t out);
/* Kernels::reconstruct_bf16 (gpu/mod.rs:110-157): original-basis W as bf16, layout 0 = [k][n], 1 = [n][k];
 * scratch: f32 workspace of at least k * 128 * 4 bytes; stored layout only. */
int fe_exl3_reconstruct_bf16(const fe_exl3_kernels *kern, fe_stream_t s, const fe_exl3_view *w, fe_devptr_t out, int layout,
                             fe_devptr_t scratch, size_t scratch_bytes);

/* Probes (kernels/k-exl3/src/probe.rs): launch `launches` back-to-back runs and return the average milliseconds.
 * stream_read: 16-byte loads over `bytes` of `buf`; decode: ALU-only trellis decode of grid * 256 * 32 * iters weights. */
int fe_exl3_probe_stream_read(const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t buf, size_t bytes, uint32_t grid,
                              uint32_t launches, float *ms);
int fe_exl3_probe_decode(const fe_exl3_kernels *kern, fe_stream_t s, uint32_t bits, uint32_t grid, uint32_t iters,
                         uint32_t launches, float *ms);
/* Issue rate of one vector instruction of the decode (kernels/k-exl3/src/probe.rs:38-67, exl3_probe_{imad,idp,lop,...}):
 * grid x 256 lanes run 8 independent chains of `iters` dependent instructions each; op is one of "add", "and",
 * "mul_lo" (v_mul_lo_u32), "mad_u24", "bfe", "alignbit", "perm", "sad_u8", "sad_hi_u8", "pk_fma_f16", "fma_f32",
 * "dpp_mov". Lane-operations per second = grid * 256 * 8 * iters / (ms * 1e-3). */
int fe_exl3_probe_op(const fe_exl3_kernels *kern, fe_stream_t s, const char *op, uint32_t grid, uint32_t iters,
                     uint32_t launches, float *ms);

#ifdef __cplusplus
}
#endif
#endif
