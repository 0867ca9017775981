/* EXL3 part of the CPU oracle (test infrastructure; see fe_oracle.h).
 * Follows crates/fe-exl3/src/format.rs and crates/fe-exl3/src/cpu.rs; the two extra tile_state formulations follow
 * the reference's GPU kernels so that all three can be checked against each other. */
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include "fe_oracle.h"

#define HAD_SCALE 0.08838834764831844 /* 1/sqrt(128), cpu.rs:10 */

int or_default_threads(int cap) {
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    if (n < 1) n = 4;
    if (cap > 0 && n > cap) n = cap;
    return (int)n;
}

/* ---- format.rs ------------------------------------------------------------------------------------------- */

/* format.rs:148-150: k inside the tile of value j of fragment lane `lane`. */
size_t or_value_row(size_t lane, size_t j) { return 2 * (lane & 3) + (j & 1) + 8 * ((j >> 1) & 1); }
/* format.rs:154-156: n inside the tile. */
size_t or_value_col(size_t lane, size_t j) { return (lane >> 2) + 8 * (j >> 2); }

static size_t tile_words(const or_exl3 *t) { return 8 * (size_t)t->bits; } /* format.rs:60-62 */

/* format.rs:64-68 */
static const uint32_t *tile_at(const or_exl3 *t, size_t kt, size_t nt) {
    return t->trellis + (kt * (t->n / 16) + nt) * tile_words(t);
}

/* format.rs:72-84: [n/128][k/16][8][tw] */
void or_strips(const or_exl3 *t, uint32_t *out) {
    size_t tw = tile_words(t), kts = t->k / 16, nts = t->n / 16;
    for (size_t b = 0; b < nts / 8; b++)
        for (size_t kt = 0; kt < kts; kt++)
            memcpy(out + (b * kts + kt) * 8 * tw, t->trellis + (kt * nts + b * 8) * tw, 8 * tw * sizeof(uint32_t));
}

/* format.rs:89-110 */
size_t or_slice_cols(const or_exl3 *t, const size_t *ranges, size_t nr, uint32_t *trellis_out, uint16_t *svh_out) {
    size_t tw = tile_words(t), nts = t->n / 16, cols = 0;
    for (size_t i = 0; i < nr; i++) {
        size_t a = ranges[2 * i], b = ranges[2 * i + 1];
        if (a % 128 || b % 128 || a >= b || b > t->n) return 0;
        cols += b - a;
    }
    uint32_t *dst = trellis_out;
    for (size_t kt = 0; kt < t->k / 16; kt++)
        for (size_t i = 0; i < nr; i++) {
            size_t a = ranges[2 * i], b = ranges[2 * i + 1];
            size_t words = (b - a) / 16 * tw;
            memcpy(dst, t->trellis + (kt * nts + a / 16) * tw, words * sizeof(uint32_t));
            dst += words;
        }
    uint16_t *sv = svh_out;
    for (size_t i = 0; i < nr; i++) {
        size_t a = ranges[2 * i], b = ranges[2 * i + 1];
        memcpy(sv, t->svh + a, (b - a) * sizeof(uint16_t));
        sv += b - a;
    }
    return cols;
}

/* format.rs:115-130 */
size_t or_slice_rows(const or_exl3 *t, size_t k0, size_t k1, uint32_t *trellis_out, uint16_t *suh_out) {
    if (k0 % 128 || k1 % 128 || k0 >= k1 || k1 > t->k) return 0;
    size_t row_words = t->n / 16 * tile_words(t);
    memcpy(trellis_out, t->trellis + k0 / 16 * row_words, (k1 - k0) / 16 * row_words * sizeof(uint32_t));
    memcpy(suh_out, t->suh + k0, (k1 - k0) * sizeof(uint16_t));
    return k1 - k0;
}

/* ---- cpu.rs ---------------------------------------------------------------------------------------------- */

/* cpu.rs:14-23: stream bits [(t+1)*bits - 16, (t+1)*bits), cyclic over 256*bits, MSB of each u32 first. */
uint32_t or_tile_state(const uint32_t *tile, uint32_t bits, size_t t) {
    size_t len = 256 * (size_t)bits;
    size_t start = ((t + 1) * bits + len - 16) % len;
    uint32_t s = 0;
    for (size_t b = 0; b < 16; b++) {
        size_t p = (start + b) % len;
        s = (s << 1) | ((tile[p / 32] >> (31 - (p % 32))) & 1u);
    }
    return s;
}

/* shf.r.clamp.b32: low 32 bits of hi:lo >> s (kernels/k-exl3/src/util.rs:60-66) */
static uint32_t funnel_r(uint32_t lo, uint32_t hi, uint32_t s) {
    if (s >= 32) return hi;
    return (uint32_t)(((((uint64_t)hi) << 32) | lo) >> s);
}
/* shf.l.clamp.b32: high 32 bits of hi:lo << s (util.rs:68-74) */
static uint32_t funnel_l(uint32_t lo, uint32_t hi, uint32_t s) {
    if (s >= 32) return lo;
    return (uint32_t)((((((uint64_t)hi) << 32) | lo) << s) >> 32);
}

/* kernels/k-exl3/src/recon.rs:12-22 */
uint32_t or_tile_state_funnel(const uint32_t *tile, uint32_t bits, size_t t) {
    uint32_t words = 8 * bits;
    uint32_t b1 = ((uint32_t)t + 1) * bits + 256 * bits;
    uint32_t b0 = b1 - 16;
    uint32_t i0 = b0 / 32, i1 = (b1 - 1) / 32;
    uint32_t s = (i1 + 1) * 32 - b1;
    return funnel_r(tile[i1 % words], tile[i0 % words], s) & 0xffff;
}

/* kernels/k-exl3/src/gemv.rs:184-194 */
static uint32_t window16(uint32_t hi, uint32_t mid, uint32_t lo, uint32_t d) {
    if (d <= 16) return (hi >> (16 - d)) & 0xffff;
    if (d < 32) return funnel_l(mid, hi, d) >> 16;
    if (d <= 48) return (mid >> (48 - d)) & 0xffff;
    return funnel_l(lo, mid, d - 32) >> 16;
}

/* The per-lane view of the GEMV kernels: lane = t / 8 reads LW consecutive words from `word`, aligns them by `off`
 * and cuts value j = t % 8 at j * bits. gemv.rs:198-208 (decode_lane), 212-224 (load_step), 260-262 (first/word/off). */
uint32_t or_tile_state_lane(const uint32_t *tile, uint32_t bits, size_t t) {
    uint32_t tw = 8 * bits, ln = (uint32_t)t / 8, j = (uint32_t)t % 8;
    uint32_t first = (8 * ln + 1) * bits + 256 * bits - 16;
    uint32_t word = (first >> 5) % tw, off = first & 31;
    /* LW = words a lane reads: 2 up to 4 bits, 3 above (gemv.rs:875-878 instantiate LW 2,2,2,3 for 2..5 bits) */
    uint32_t lw = bits <= 4 ? 2 : 3;
    uint32_t w[3] = {0, 0, 0};
    for (uint32_t q = 0; q < lw; q++) w[q] = tile[(word + q) % tw];
    uint32_t w2 = lw > 2 ? w[2] : 0;
    uint32_t hi = funnel_l(w[1], w[0], off), mid = funnel_l(w2, w[1], off), lo = off ? (w2 << off) : w2;
    return window16(hi, mid, lo, j * bits);
}

/* cpu.rs:25-35: the 1021 reachable values, fp16 fma(1024 + s, 0x1eee, 0xc931). */
static uint16_t g_mul1[1021];
static pthread_once_t g_mul1_once = PTHREAD_ONCE_INIT;
static void mul1_init(void) {
    for (int s = 0; s <= 1020; s++) g_mul1[s] = or_f16_fma((uint16_t)(0x6400 + s), 0x1eee, 0xc931);
}

/* cpu.rs:37-43 */
uint16_t or_decode_mul1(uint32_t state) {
    pthread_once(&g_mul1_once, mul1_init);
    uint32_t x = state * OR_MUL1;
    uint32_t s = (x & 0xff) + ((x >> 8) & 0xff) + ((x >> 16) & 0xff) + (x >> 24);
    return g_mul1[s];
}

/* cpu.rs:46-54 */
void or_decode_tile(const uint32_t *tile, uint32_t bits, uint16_t out[16][16]) {
    for (size_t lane = 0; lane < 32; lane++)
        for (size_t j = 0; j < 8; j++)
            out[or_value_row(lane, j)][or_value_col(lane, j)] = or_decode_mul1(or_tile_state(tile, bits, lane * 8 + j));
}

/* cpu.rs:57-69 */
void or_w_hat_f16(const or_exl3 *t, size_t n0, size_t ns, uint16_t *w) {
    uint16_t d[16][16];
    for (size_t kt = 0; kt < t->k / 16; kt++)
        for (size_t nt = 0; nt < ns / 16; nt++) {
            or_decode_tile(tile_at(t, kt, n0 / 16 + nt), t->bits, d);
            for (size_t r = 0; r < 16; r++) memcpy(w + (kt * 16 + r) * ns + nt * 16, d[r], 16 * sizeof(uint16_t));
        }
}

/* cpu.rs:72-85: unnormalised, natural (Sylvester) order. */
void or_fwht128(double *v) {
    for (size_t h = 1; h < 128; h *= 2)
        for (size_t i = 0; i < 128; i += 2 * h)
            for (size_t j = i; j < i + h; j++) {
                double a = v[j], b = v[j + h];
                v[j] = a + b;
                v[j + h] = a - b;
            }
}

/* cpu.rs:88-128 */
void or_weight_block_f64(const or_exl3 *t, size_t r0, size_t n0, size_t ns, double *w) {
    uint16_t d[16][16];
    for (size_t ktl = 0; ktl < 8; ktl++)
        for (size_t nt = 0; nt < ns / 16; nt++) {
            or_decode_tile(tile_at(t, r0 / 16 + ktl, n0 / 16 + nt), t->bits, d);
            for (size_t r = 0; r < 16; r++)
                for (size_t c = 0; c < 16; c++) w[(ktl * 16 + r) * ns + nt * 16 + c] = or_f16_to_f64(d[r][c]);
        }
    for (size_t r = 0; r < 128; r++)
        for (size_t b = 0; b < ns; b += 128) or_fwht128(w + r * ns + b);
    for (size_t h = 1; h < 128; h *= 2)
        for (size_t i = 0; i < 128; i += 2 * h)
            for (size_t j = i; j < i + h; j++)
                for (size_t c = 0; c < ns; c++) {
                    double a = w[j * ns + c], b = w[(j + h) * ns + c];
                    w[j * ns + c] = a + b;
                    w[(j + h) * ns + c] = a - b;
                }
    for (size_t r = 0; r < 128; r++) {
        double su = or_f16_to_f64(t->suh[r0 + r]) * HAD_SCALE * HAD_SCALE;
        for (size_t c = 0; c < ns; c++) w[r * ns + c] *= su * or_f16_to_f64(t->svh[n0 + c]);
    }
}

/* cpu.rs:140-176: 128-row blocks handed out to threads from a shared counter. */
typedef struct {
    const or_exl3 *t;
    size_t n0, ns;
    int layout;
    uint16_t *out;
    size_t next, blocks;
    pthread_mutex_t mu;
} wb_job;

static void *wb_worker(void *arg) {
    wb_job *j = (wb_job *)arg;
    double *w = (double *)malloc(128 * j->ns * sizeof(double));
    for (;;) {
        pthread_mutex_lock(&j->mu);
        size_t b = j->next++;
        pthread_mutex_unlock(&j->mu);
        if (b >= j->blocks) break;
        or_weight_block_f64(j->t, b * 128, j->n0, j->ns, w);
        for (size_t r = 0; r < 128; r++)
            for (size_t c = 0; c < j->ns; c++) {
                uint16_t v = or_f64_to_bf16_torch(w[r * j->ns + c]);
                if (j->layout == 0)
                    j->out[(b * 128 + r) * j->ns + c] = v;
                else
                    j->out[c * j->t->k + b * 128 + r] = v;
            }
    }
    free(w);
    return NULL;
}

void or_weight_bf16(const or_exl3 *t, size_t n0, size_t ns, int layout, int threads, uint16_t *out) {
    if (threads <= 0) threads = or_default_threads(16);
    wb_job j = {t, n0, ns, layout, out, 0, t->k / 128, PTHREAD_MUTEX_INITIALIZER};
    pthread_t th[64];
    if (threads > 64) threads = 64;
    for (int i = 0; i < threads; i++) pthread_create(&th[i], NULL, wb_worker, &j);
    for (int i = 0; i < threads; i++) pthread_join(th[i], NULL);
}

/* cpu.rs:180-215. One worker covers the 128-column blocks [b0, b1); with a single worker over all blocks this is
 * the reference's loop nest (kt outer, nt inner, then r, c, mi). */
typedef struct {
    const or_exl3 *t;
    const double *xh; /* H(x * suh), [m][k] */
    size_t m, b0, b1;
    double *z;
} lin_job;

static void *lin_worker(void *arg) {
    lin_job *j = (lin_job *)arg;
    const or_exl3 *t = j->t;
    size_t k = t->k, n = t->n, m = j->m;
    uint16_t d[16][16];
    for (size_t kt = 0; kt < k / 16; kt++)
        for (size_t nt = j->b0 * 8; nt < j->b1 * 8; nt++) {
            or_decode_tile(tile_at(t, kt, nt), t->bits, d);
            for (size_t r = 0; r < 16; r++)
                for (size_t c = 0; c < 16; c++) {
                    double wv = or_f16_to_f64(d[r][c]);
                    for (size_t mi = 0; mi < m; mi++) j->z[mi * n + nt * 16 + c] += j->xh[mi * k + kt * 16 + r] * wv;
                }
        }
    for (size_t mi = 0; mi < m; mi++)
        for (size_t b = j->b0; b < j->b1; b++) {
            double *blk = j->z + mi * n + b * 128;
            or_fwht128(blk);
            for (size_t i = 0; i < 128; i++) blk[i] *= or_f16_to_f64(t->svh[b * 128 + i]) * HAD_SCALE * HAD_SCALE;
        }
    return NULL;
}

void or_linear_f64(const or_exl3 *t, const double *x, size_t m, int threads, double *y) {
    size_t k = t->k, n = t->n;
    double *xh = (double *)malloc(m * k * sizeof(double));
    for (size_t mi = 0; mi < m; mi++) {
        for (size_t i = 0; i < k; i++) xh[mi * k + i] = x[mi * k + i] * or_f16_to_f64(t->suh[i]);
        for (size_t b = 0; b < k; b += 128) or_fwht128(xh + mi * k + b);
    }
    memset(y, 0, m * n * sizeof(double));
    size_t nb = n / 128;
    if (threads <= 0) threads = or_default_threads(64);
    if ((size_t)threads > nb) threads = (int)nb;
    if (threads > 64) threads = 64;
    lin_job jobs[64];
    pthread_t th[64];
    for (int i = 0; i < threads; i++) {
        jobs[i] = (lin_job){t, xh, m, nb * (size_t)i / (size_t)threads, nb * (size_t)(i + 1) / (size_t)threads, y};
        if (threads == 1)
            lin_worker(&jobs[i]);
        else
            pthread_create(&th[i], NULL, lin_worker, &jobs[i]);
    }
    if (threads > 1)
        for (int i = 0; i < threads; i++) pthread_join(th[i], NULL);
    free(xh);
}

/* cpu.rs:218-234 */
void or_rotate_input_ref(const or_exl3 *t, const double *x, size_t m, uint16_t *xh) {
    size_t k = t->k;
    double *row = (double *)malloc(k * sizeof(double));
    for (size_t mi = 0; mi < m; mi++) {
        for (size_t i = 0; i < k; i++) row[i] = x[mi * k + i] * or_f16_to_f64(t->suh[i]);
        for (size_t b = 0; b < k; b += 128) or_fwht128(row + b);
        for (size_t i = 0; i < k; i++) xh[mi * k + i] = or_f64_to_f16(row[i] * HAD_SCALE);
    }
    free(row);
}

/* cpu.rs:238-266 */
void or_gemv_ref(const or_exl3 *t, const uint16_t *w_hat, size_t nc, const uint16_t *xh, size_t m, double *y) {
    size_t k = t->k, n = nc;
    double *wf = (double *)malloc(k * n * sizeof(double));
    for (size_t i = 0; i < k * n; i++) wf[i] = or_f16_to_f64(w_hat[i]);
    memset(y, 0, m * n * sizeof(double));
    for (size_t mi = 0; mi < m; mi++) {
        double *zr = y + mi * n;
        for (size_t kk = 0; kk < k; kk++) {
            double xv = or_f16_to_f64(xh[mi * k + kk]);
            if (xv == 0.0) continue;
            const double *wr = wf + kk * n;
            for (size_t c = 0; c < n; c++) zr[c] += xv * wr[c];
        }
    }
    for (size_t mi = 0; mi < m; mi++)
        for (size_t b = 0; b < n; b += 128) {
            double *blk = y + mi * n + b;
            or_fwht128(blk);
            for (size_t i = 0; i < 128; i++) blk[i] *= or_f16_to_f64(t->svh[b + i]) * HAD_SCALE;
        }
    free(wf);
}
