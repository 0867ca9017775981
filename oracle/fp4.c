/* NVFP4 / FP8 part of the CPU oracle (test infrastructure; see fe_oracle.h).
 * Follows crates/fe-fp4/src/format.rs, plus the two pure host helpers of crates/fe-fp4/src/lib.rs that shape the
 * weights (select, the gate|up interleave). */
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "fe_oracle.h"

/* format.rs:5 — code -> value, bit 3 is the sign */
const float OR_E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f, -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

static float f32_of_bits(uint32_t b) {
    float x;
    memcpy(&x, &b, 4);
    return x;
}

/* format.rs:19-27 */
float or_e4m3_to_f32(uint8_t b) {
    uint32_t e = (b >> 3) & 15, m = b & 7;
    if (e == 15 && m == 7) return NAN;
    float v = e == 0 ? (float)m / 512.0f : f32_of_bits(((e + 120) << 23) | (m << 20));
    return (b & 0x80) ? -v : v;
}

/* format.rs:30-42 — nearest entry of an ascending table of non-negative values; a tie goes to the even index;
 * anything above the last entry saturates to it. */
static size_t nearest(const float *t, size_t len, float a) {
    size_t i = 0;
    while (i < len && t[i] < a) i++; /* partition point of (v < a) */
    if (i == len) return len - 1;
    if (i > 0) {
        float lo = a - t[i - 1], hi = t[i] - a;
        if (lo < hi || (lo == hi && (i - 1) % 2 == 0)) i--;
    }
    return i;
}

/* format.rs:44-54 */
static float g_e4m3_pos[127];
static pthread_once_t g_e4m3_once = PTHREAD_ONCE_INIT;
static void e4m3_init(void) {
    for (int i = 0; i < 127; i++) g_e4m3_pos[i] = or_e4m3_to_f32((uint8_t)i);
}

/* format.rs:57-63 */
uint8_t or_f32_to_e4m3(float x) {
    if (x != x) return 0x7f;
    pthread_once(&g_e4m3_once, e4m3_init);
    uint8_t c = (uint8_t)nearest(g_e4m3_pos, 127, fabsf(x));
    if (signbit(x)) return c ? (uint8_t)(c | 0x80) : 0x80;
    return c;
}

/* format.rs:66-69 */
uint8_t or_f32_to_e2m1(float x) {
    uint8_t c = (uint8_t)nearest(OR_E2M1, 8, fabsf(x));
    return signbit(x) ? (uint8_t)(c | 8) : c;
}

/* format.rs:72-90 — all arithmetic in f32, in the reference's order: amax * (1/6) * g, then g / sv. */
void or_quant_fp4_row(const uint16_t *x, size_t k, float g, uint8_t *codes, uint8_t *sf) {
    for (size_t b = 0; b < k / 16; b++) {
        float f[16], amax = 0.0f;
        for (int i = 0; i < 16; i++) {
            f[i] = or_bf16_to_f32(x[b * 16 + i]);
            float a = fabsf(f[i]);
            amax = fmaxf(amax, a); /* f32::max ignores a NaN operand, like fmaxf */
        }
        volatile float sixth = 1.0f / 6.0f;
        volatile float t0 = amax * sixth;
        volatile float t1 = t0 * g;
        uint8_t s8 = or_f32_to_e4m3(t1);
        float sv = or_e4m3_to_f32(s8);
        volatile float mul = sv > 0.0f ? g / sv : 0.0f;
        for (int j = 0; j < 8; j++) {
            volatile float a = f[2 * j] * mul, c = f[2 * j + 1] * mul;
            uint8_t lo = or_f32_to_e2m1(a), hi = or_f32_to_e2m1(c);
            codes[b * 8 + j] = (uint8_t)(lo | (hi << 4));
        }
        sf[b] = s8;
    }
}

/* format.rs:93-95 */
void or_quant_fp8_row(const uint16_t *x, size_t k, float g, uint8_t *out) {
    for (size_t i = 0; i < k; i++) {
        volatile float v = or_bf16_to_f32(x[i]) * g;
        out[i] = or_f32_to_e4m3(v);
    }
}

/* format.rs:109-111 */
size_t or_tiled_offset(size_t r, size_t b, size_t kb) { return ((r / 128) * (kb / 8) + b / 8) * 1024 + (r % 128) * 8 + b % 8; }

/* format.rs:98-108 */
void or_tile_scales(const uint8_t *src, size_t rows, size_t kb, uint8_t *out) {
    size_t rp = (rows + 127) / 128 * 128;
    memset(out, 0, rp * kb);
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < kb; b++) out[or_tiled_offset(r, b, kb)] = src[r * kb + b];
}

/* format.rs:113-121 */
void or_untile_scales(const uint8_t *t, size_t rows, size_t kb, uint8_t *out) {
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < kb; b++) out[r * kb + b] = t[or_tiled_offset(r, b, kb)];
}

/* format.rs:136-142 — (E2M1 * scale) * gs in f32 */
void or_dequant_fp4_row(const uint8_t *codes, const uint8_t *sf, float gs, float *out, size_t k) {
    for (size_t i = 0; i < k; i++) {
        uint8_t c = codes[i / 2];
        uint8_t q = (i % 2 == 0) ? (c & 15) : (c >> 4);
        volatile float p = OR_E2M1[q] * or_e4m3_to_f32(sf[i / 16]);
        out[i] = p * gs;
    }
}

/* format.rs:143-147 */
void or_dequant_fp8_row(const uint8_t *codes, float gs, float *out, size_t k) {
    for (size_t i = 0; i < k; i++) out[i] = or_e4m3_to_f32(codes[i]) * gs;
}

/* format.rs:151-181 — each thread owns a contiguous run of columns; per output an f64 dot in k order, cast to f32. */
typedef struct {
    const float *a, *w;
    size_t rows, n, k, c0, c1;
    float *y;
} gemm_job;

static void *gemm_worker(void *arg) {
    gemm_job *j = (gemm_job *)arg;
    for (size_t r = 0; r < j->rows; r++) {
        const float *ar = j->a + r * j->k;
        for (size_t c = j->c0; c < j->c1; c++) {
            const float *wr = j->w + c * j->k;
            double s = 0.0;
            for (size_t i = 0; i < j->k; i++) s += (double)ar[i] * (double)wr[i];
            j->y[r * j->n + c] = (float)s;
        }
    }
    return NULL;
}

void or_ref_gemm(const float *a, size_t rows, const float *w, size_t n, size_t k, int threads, float *y) {
    if (threads <= 0) threads = or_default_threads(20);
    if (threads > 64) threads = 64;
    size_t chunk = (n + (size_t)threads - 1) / (size_t)threads;
    gemm_job jobs[64];
    pthread_t th[64];
    for (int t = 0; t < threads; t++) {
        size_t c0 = (size_t)t * chunk, c1 = (size_t)(t + 1) * chunk;
        if (c0 > n) c0 = n;
        if (c1 > n) c1 = n;
        jobs[t] = (gemm_job){a, w, rows, n, k, c0, c1, y};
        pthread_create(&th[t], NULL, gemm_worker, &jobs[t]);
    }
    for (int t = 0; t < threads; t++) pthread_join(th[t], NULL);
}

/* crates/fe-fp4/src/lib.rs:254-262 */
size_t or_select(const uint8_t *src, size_t row_len, const size_t *keep, size_t nr, size_t c0, size_t c1, uint8_t *out) {
    size_t w = 0;
    for (size_t i = 0; i < nr; i++)
        for (size_t r = keep[2 * i]; r < keep[2 * i + 1]; r++) {
            memcpy(out + w, src + r * row_len + c0, c1 - c0);
            w += c1 - c0;
        }
    return w;
}

/* crates/fe-fp4/src/lib.rs:393-397 */
size_t or_swiglu_perm(size_t r, size_t inter) {
    size_t blk = r / 16, w = r % 16;
    return w < 8 ? blk * 8 + w : inter + blk * 8 + w - 8;
}
