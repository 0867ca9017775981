/* fp16 / bf16 bit helpers of the CPU oracle (test infrastructure; see fe_oracle.h).
 * Follows crates/fe-exl3/src/half.rs. */
#include <math.h>
#include <string.h>

#include "fe_oracle.h"

static uint64_t bits_of_f64(double x) {
    uint64_t b;
    memcpy(&b, &x, 8);
    return b;
}
static uint32_t bits_of_f32(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return b;
}
static float f32_of_bits(uint32_t b) {
    float x;
    memcpy(&x, &b, 4);
    return x;
}

/* half.rs:4-19 — exact widening. */
double or_f16_to_f64(uint16_t h) {
    int neg = (h >> 15) & 1;
    int e = (h >> 10) & 0x1f;
    int frac = h & 0x3ff;
    double v;
    if (e == 0) {
        v = ldexp((double)frac, -24);
    } else if (e == 31) {
        v = frac ? NAN : INFINITY;
    } else {
        v = ldexp(1024.0 + (double)frac, e - 25);
    }
    return neg ? -v : v;
}

/* half.rs:26-65 — one rounding, nearest-even, straight from the f64 significand.
 * Shift the 53-bit significand right by `drop` bits, look at what falls off. */
static uint64_t rne_shift(uint64_t sig, unsigned drop) {
    if (drop == 0) return sig;
    if (drop >= 64) return 0;
    uint64_t keep = sig >> drop;
    uint64_t lost = sig & ((1ull << drop) - 1);
    uint64_t mid = 1ull << (drop - 1);
    if (lost > mid || (lost == mid && (keep & 1))) keep++;
    return keep;
}

uint16_t or_f64_to_f16(double x) {
    uint64_t b = bits_of_f64(x);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000);
    if (x != x) return 0x7e00;
    if (x == 0.0) return sign;
    int e = (int)((b >> 52) & 0x7ff) - 1023;
    uint64_t sig = (b & ((1ull << 52) - 1)) | (1ull << 52);
    if (e < -14) {
        /* subnormal target: result counts units of 2^-24; value = sig * 2^(e-52) */
        int drop = 28 - e; /* (e - 52) - (-24) negated */
        uint64_t q = (drop >= 64) ? 0 : rne_shift(sig, (unsigned)drop);
        return (uint16_t)(sign | q); /* q == 1024 lands on the smallest normal by itself */
    }
    uint64_t q = rne_shift(sig, 42); /* 11 significant bits */
    if (q == 2048) {
        q = 1024;
        e++;
    }
    if (e > 15) return sign | 0x7c00;
    return (uint16_t)(sign | ((uint16_t)(e + 15) << 10) | (q & 0x3ff));
}

/* half.rs:68-72 — the product of two fp16 values has 22 significant bits, and for the magnitudes of the mul1
 * codebook the sum with c is exact in f64 too, so one f64 -> fp16 rounding equals a fused fp16 fma. */
uint16_t or_f16_fma(uint16_t a, uint16_t b, uint16_t c) {
    return or_f64_to_f16(or_f16_to_f64(a) * or_f16_to_f64(b) + or_f16_to_f64(c));
}

/* half.rs:75-81 */
uint16_t or_f32_to_bf16(float x) {
    uint32_t b = bits_of_f32(x);
    if (x != x) return (uint16_t)((b >> 16) | 0x40);
    return (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}

/* half.rs:83-85 */
float or_bf16_to_f32(uint16_t h) { return f32_of_bits((uint32_t)h << 16); }

/* half.rs:88-90 — f64 -> f32 (RNE) -> bf16 (RNE), the way torch converts a float64 tensor. */
uint16_t or_f64_to_bf16_torch(double x) { return or_f32_to_bf16((float)x); }

/* half.rs:93-98 */
uint32_t or_bf16_ulp_diff(uint16_t a, uint16_t b) {
    int oa = (a & 0x8000) ? -(int)(a & 0x7fff) : (int)a;
    int ob = (b & 0x8000) ? -(int)(b & 0x7fff) : (int)b;
    int d = oa - ob;
    return (uint32_t)(d < 0 ? -d : d);
}
