/*
 * CPU oracle for the quantized-linear hot path (EXL3 trellis linear, NVFP4 linear).
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's own CPU algorithms. It is the
 * checker the GPU kernels are compared against and the CPU baseline that is timed beside them; nothing in the
 * product library links, loads or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference checkout).
 * All arrays are plain row-major buffers owned by the caller.
 */
#ifndef FE_ORACLE_H
#define FE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 / bf16 bit helpers (crates/fe-exl3/src/half.rs) ---------------------------------------------- */
double or_f16_to_f64(uint16_t h);                         /* half.rs:4-19 */
uint16_t or_f64_to_f16(double x);                         /* half.rs:26-65 */
uint16_t or_f16_fma(uint16_t a, uint16_t b, uint16_t c);  /* half.rs:68-72 */
uint16_t or_f32_to_bf16(float x);                         /* half.rs:75-81 */
float or_bf16_to_f32(uint16_t h);                         /* half.rs:83-85 */
uint16_t or_f64_to_bf16_torch(double x);                  /* half.rs:88-90 */
uint32_t or_bf16_ulp_diff(uint16_t a, uint16_t b);        /* half.rs:93-98 */

/* ---- EXL3 format (crates/fe-exl3/src/format.rs) -------------------------------------------------------- */
#define OR_MUL1 0x83DCD12Du /* format.rs:14 */

/* A borrowed EXL3 tensor: trellis words in the stored layout [k/16][n/16][8*bits]. format.rs:17-30 */
typedef struct {
    size_t k, n;
    uint32_t bits;
    const uint32_t *trellis;
    const uint16_t *suh; /* fp16 bits [k] */
    const uint16_t *svh; /* fp16 bits [n] */
} or_exl3;

size_t or_value_row(size_t lane, size_t j); /* format.rs:148-150 */
size_t or_value_col(size_t lane, size_t j); /* format.rs:154-156 */
/* stored -> strips layout [n/128][k/16][8][tw]; out has the same word count. format.rs:72-84 */
void or_strips(const or_exl3 *t, uint32_t *out);
/* Column slice: ranges = nr pairs (a, b), each 128-aligned. Writes trellis_out (k/16 * cols/16 * tw words) and
 * svh_out (cols). Returns cols, or 0 on an invalid range. format.rs:89-110 */
size_t or_slice_cols(const or_exl3 *t, const size_t *ranges, size_t nr, uint32_t *trellis_out, uint16_t *svh_out);
/* Row slice [k0, k1): writes trellis_out ((k1-k0)/16 * n/16 * tw words) and suh_out. Returns k1-k0 or 0.
 * format.rs:115-130 */
size_t or_slice_rows(const or_exl3 *t, size_t k0, size_t k1, uint32_t *trellis_out, uint16_t *suh_out);

/* ---- EXL3 CPU reference (crates/fe-exl3/src/cpu.rs) ----------------------------------------------------- */
/* 16-bit trellis state of position t, bit by bit. cpu.rs:14-23 */
uint32_t or_tile_state(const uint32_t *tile, uint32_t bits, size_t t);
/* The same state by the GPU recon formulation (two words + funnel shift). kernels/k-exl3/src/recon.rs:12-22 */
uint32_t or_tile_state_funnel(const uint32_t *tile, uint32_t bits, size_t t);
/* The same state by the GEMV formulation (per-lane word/offset, three-word window). kernels/k-exl3/src/gemv.rs:184-208,
 * 260-262 */
uint32_t or_tile_state_lane(const uint32_t *tile, uint32_t bits, size_t t);
uint16_t or_decode_mul1(uint32_t state);                                   /* cpu.rs:25-43 */
void or_decode_tile(const uint32_t *tile, uint32_t bits, uint16_t out[16][16]); /* cpu.rs:46-54 */
void or_w_hat_f16(const or_exl3 *t, size_t n0, size_t ns, uint16_t *w);    /* cpu.rs:57-69, w [k][ns] */
void or_fwht128(double *v);                                                /* cpu.rs:72-85 */
void or_weight_block_f64(const or_exl3 *t, size_t r0, size_t n0, size_t ns, double *w); /* cpu.rs:88-128, w [128][ns] */
/* layout 0 = KN ([k][ns]), 1 = NK ([ns][k]); threads <= 0 picks min(online cpus, 16). cpu.rs:140-176 */
void or_weight_bf16(const or_exl3 *t, size_t n0, size_t ns, int layout, int threads, uint16_t *out);
/* y [m][n] f64 = factored-form linear of x [m][k] f64. threads == 1 is the reference's loop order exactly;
 * threads > 1 splits the 128-column blocks over threads (each output is still summed in the same k order, so the
 * result is bit-identical). cpu.rs:180-215 */
void or_linear_f64(const or_exl3 *t, const double *x, size_t m, int threads, double *y);
void or_rotate_input_ref(const or_exl3 *t, const double *x, size_t m, uint16_t *xh); /* cpu.rs:218-234 */
/* y [m][nc] f64 from fp16 xh [m][k] and fp16 w_hat [k][nc]. cpu.rs:238-266 */
void or_gemv_ref(const or_exl3 *t, const uint16_t *w_hat, size_t nc, const uint16_t *xh, size_t m, double *y);

/* ---- NVFP4 / FP8 formats and CPU reference (crates/fe-fp4/src/format.rs) -------------------------------- */
extern const float OR_E2M1[16];                   /* format.rs:5 */
float or_e4m3_to_f32(uint8_t b);                  /* format.rs:19-27 */
uint8_t or_f32_to_e4m3(float x);                  /* format.rs:57-63 */
uint8_t or_f32_to_e2m1(float x);                  /* format.rs:66-69 */
/* x bf16 [k] -> codes [k/2], sf [k/16]. format.rs:72-90 */
void or_quant_fp4_row(const uint16_t *x, size_t k, float g, uint8_t *codes, uint8_t *sf);
void or_quant_fp8_row(const uint16_t *x, size_t k, float g, uint8_t *out); /* format.rs:93-95 */
size_t or_tiled_offset(size_t r, size_t b, size_t kb);                     /* format.rs:109-111 */
/* out has ceil(rows/128)*128*kb bytes, zero-filled first. format.rs:98-108 */
void or_tile_scales(const uint8_t *src, size_t rows, size_t kb, uint8_t *out);
void or_untile_scales(const uint8_t *t, size_t rows, size_t kb, uint8_t *out); /* format.rs:113-121 */
void or_dequant_fp4_row(const uint8_t *codes, const uint8_t *sf, float gs, float *out, size_t k); /* format.rs:136-142 */
void or_dequant_fp8_row(const uint8_t *codes, float gs, float *out, size_t k);                    /* format.rs:143-147 */
/* y [rows][n] f32 = a [rows][k] . w[n][k]^T, f64 accumulate, threaded over columns (threads <= 0: min(cpus, 20)).
 * format.rs:151-181 */
void or_ref_gemm(const float *a, size_t rows, const float *w, size_t n, size_t k, int threads, float *y);
/* Rows `keep` (nr ranges, concatenated) and bytes c0..c1 of a row-major byte matrix. crates/fe-fp4/src/lib.rs:254-262.
 * Returns bytes written. */
size_t or_select(const uint8_t *src, size_t row_len, const size_t *keep, size_t nr, size_t c0, size_t c1, uint8_t *out);
/* gate|up interleave permutation of into_swiglu: interleaved row r -> source row. crates/fe-fp4/src/lib.rs:393-397 */
size_t or_swiglu_perm(size_t r, size_t inter);

/* Host cores the threaded functions would use by default (reported by the CPU baseline). */
int or_default_threads(int cap);

#ifdef __cplusplus
}
#endif
#endif
