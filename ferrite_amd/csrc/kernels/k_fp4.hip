// NVFP4 linear for gfx950: e2m1 codes (element 2i in the low nibble of byte i), one e4m3 scale per 16 elements along
// K, an fp32 scale per output column. Activations are quantized to the same format first (the reference's prompt path
// is W4A4, crates/fe-fp4/src/lib.rs:512-530), then the GEMM runs over the quantized operands.
//
// gfx950's block-scaled MFMA takes e8m0 scales per 32 elements, which cannot express e4m3 per 16. A product
// e2m1 x e4m3 has at most 6 significant bits and lies in [2^-10, 2688], so twice that value is an exact, normal fp16
// number: both operands are expanded to fp16 (2 * code value * block scale) and multiplied on the f16 MFMA with fp32
// accumulation, which reproduces the block-scaled dot product up to summation order; the factor 4 comes off in the
// epilogue.
#include "gemm_core.h"

// ---- number formats ----------------------------------------------------------------------------------------------------

// Exact e4m3 (fn) -> f32 for non-NaN codes. (crates/fe-fp4/src/format.rs:19-27)
__device__ __forceinline__ float e4m3_to_f32(uint32_t b) {
    uint32_t e = (b >> 3) & 15, mn = b & 7;
    float v = e == 0 ? (float)mn * (1.0f / 512.0f) : __uint_as_float(((e + 120) << 23) | (mn << 20));
    return (b & 0x80) ? -v : v;
}

// a >= 0 -> e4m3 code, round to nearest even, saturating to 448 (0x7e); NaN -> 0x7f.
// (cvt.rn.satfinite.e4m3x2.f32; crates/fe-fp4/src/format.rs:57-63)
__device__ __forceinline__ uint32_t f32_to_e4m3_pos(float a) {
    if (a != a) return 0x7f;
    if (a >= 448.0f) return 0x7e;
    if (a < 0.015625f) return (uint32_t)__builtin_rintf(a * 512.0f);  // subnormals count 2^-9; 8 is the first normal
    uint32_t b = __float_as_uint(a);
    b += 0x7ffffu + ((b >> 20) & 1u);  // nearest even at 3 mantissa bits
    uint32_t c = (((b >> 23) - 120) << 3) | ((b >> 20) & 7u);
    return c > 0x7e ? 0x7e : c;
}

// f32 -> e2m1 code, round to nearest with ties to the even code, saturating to +-6.
// (cvt.rn.satfinite.e2m1x2.f32; crates/fe-fp4/src/format.rs:66-69)
__device__ __forceinline__ uint32_t f32_to_e2m1(float x) {
    float a = __builtin_fabsf(x);
    uint32_t c = (a > 0.25f) + (a >= 0.75f) + (a > 1.25f) + (a >= 1.75f) + (a > 2.5f) + (a >= 3.5f) + (a > 5.0f);
    return c | ((__float_as_uint(x) >> 28) & 8u);
}

// fp16 of twice the magnitude of the 8 e2m1 magnitudes: 0, 1, 2, 3, 4, 6, 8, 12; every low byte is zero, the high
// bytes are this table.
#define E2M1X2_HI_LO 0x42403c00u  // magnitudes 0..3 -> 0x00, 0x3c, 0x40, 0x42
#define E2M1X2_HI_HI 0x4a484644u  // magnitudes 4..7 -> 0x44, 0x46, 0x48, 0x4a

// 8 codes of one u32 -> 4 packed fp16 pairs (2 * value), elements in order.
__device__ __forceinline__ void e2m1x8_to_f16(uint32_t w, uint32_t (&out)[4]) {
    uint32_t sel_e = w & 0x07070707u;         // even elements (low nibbles) as byte selectors
    uint32_t sel_o = (w >> 4) & 0x07070707u;  // odd elements
    uint32_t hb_e = __builtin_amdgcn_perm(E2M1X2_HI_HI, E2M1X2_HI_LO, sel_e);
    uint32_t hb_o = __builtin_amdgcn_perm(E2M1X2_HI_HI, E2M1X2_HI_LO, sel_o);
    hb_e |= (w << 4) & 0x80808080u;  // sign: bit 3 of the nibble -> bit 7 of the fp16 high byte
    hb_o |= w & 0x80808080u;
    // pair i = (even element i, odd element i): bytes [0, hb_e.i, 0, hb_o.i]; selector 0x0c yields a zero byte
    out[0] = __builtin_amdgcn_perm(hb_o, hb_e, 0x040c000cu);
    out[1] = __builtin_amdgcn_perm(hb_o, hb_e, 0x050c010cu);
    out[2] = __builtin_amdgcn_perm(hb_o, hb_e, 0x060c020cu);
    out[3] = __builtin_amdgcn_perm(hb_o, hb_e, 0x070c030cu);
}

// Positive e4m3 scale -> the same value as packed fp16 (both halves). (b << 7) read as fp16 is value * 2^-8 for
// normal and subnormal codes alike; the multiply by 256 is exact and renormalises.
__device__ __forceinline__ f16x2 e4m3_to_f16x2(uint32_t b) {
    uint32_t h = (b & 0x7f) << 7;
    f16x2 v = __builtin_bit_cast(f16x2, h | (h << 16));
    const f16x2 c = {(_Float16)256.0f, (_Float16)256.0f};
    return v * c;
}

// ---- activation quantizer ------------------------------------------------------------------------------------------

// Ferrite's tiled scale layout [(rows / 128)][(kb / 8)][128][8] (crates/fe-fp4/src/format.rs:98-111).
__device__ __forceinline__ uint32_t sf_tiled(uint32_t row, uint32_t b, uint32_t kb) {
    return ((row >> 7) * (kb >> 3) + (b >> 3)) * 1024 + (row & 127) * 8 + (b & 7);
}

// bf16 x[M][ldx] -> codes [M][K/2], e4m3 block scales (tiled layout), and the dequantized operand the GEMM reads:
// aq[M][K] fp16 = 2 * code value * block scale. sf = e4m3(amax16 * (1/6) * g), q = e2m1(x * (g / sf)).
// One thread per 16-element block: grid ceil(M * K / 16 / 256), 256 threads.
// (kernels/k-fp4/src/lib.rs:162-197; CPU form crates/fe-fp4/src/format.rs:72-90)
extern "C" __global__ __launch_bounds__(256) void fe_fp4_quant(uint8_t* codes, uint8_t* sf, _Float16* aq, const uint16_t* x,
                                                               uint32_t m, uint32_t k, uint32_t ldx, float g) {
    uint32_t i = blockIdx.x * 256 + threadIdx.x;
    uint32_t kb = k >> 4;
    if (i >= m * kb) return;
    uint32_t row = i / kb, b = i - row * kb;
    const u32x4* p = (const u32x4*)(x + (size_t)row * ldx + b * 16);
    u32x4 r0 = p[0], r1 = p[1];
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f[2 * j] = __uint_as_float(r0[j] << 16), f[2 * j + 1] = __uint_as_float(r0[j] & 0xffff0000u);
        f[8 + 2 * j] = __uint_as_float(r1[j] << 16), f[9 + 2 * j] = __uint_as_float(r1[j] & 0xffff0000u);
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 16; j++) amax = __builtin_fmaxf(amax, __builtin_fabsf(f[j]));
    uint32_t s8 = f32_to_e4m3_pos(amax * (1.0f / 6.0f) * g);
    float sv = e4m3_to_f32(s8);
    float mul = sv > 0.f ? g / sv : 0.f;
    uint32_t q[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 16; j++) q[j >> 3] |= f32_to_e2m1(f[j] * mul) << (4 * (j & 7));
    u32x2 qv = {q[0], q[1]};
    *(u32x2*)(codes + (size_t)row * (k >> 1) + b * 8) = qv;
    sf[sf_tiled(row, b, kb)] = (uint8_t)s8;
    f16x2 sc = e4m3_to_f16x2(s8);
    uint32_t o[8];
    {
        uint32_t t[4];
        e2m1x8_to_f16(q[0], t);
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_bit_cast(f16x2, t[j]) * sc));
        e2m1x8_to_f16(q[1], t);
#pragma unroll
        for (int j = 0; j < 4; j++) o[4 + j] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_bit_cast(f16x2, t[j]) * sc));
    }
    u32x4* ap = (u32x4*)(aq + (size_t)row * k + b * 16);
    ap[0] = (u32x4){o[0], o[1], o[2], o[3]};
    ap[1] = (u32x4){o[4], o[5], o[6], o[7]};
}

// ---- GEMM --------------------------------------------------------------------------------------------------------------

// Weight tile producer: thread t expands 32 codes of row n0 + (t >> 1), k half t & 1 of the 64-wide k tile.
struct Fp4Producer {
    const uint8_t* w;   // codes of row n0 + (t >> 1), at byte (t & 1) * 16
    const uint8_t* sw;  // row-major scales of that row, at block (t & 1) * 2
    uint32_t row, half;
    u32x4 c;
    uint32_t s2;
    __device__ __forceinline__ void load(uint32_t kt) {
        c = __builtin_nontemporal_load((const u32x4*)(w + (size_t)kt * 32));
        s2 = *(const uint16_t*)(sw + kt * 4);
    }
    __device__ __forceinline__ void store(_Float16* Bs) const {
        uint32_t o[16];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t t[4];
            e2m1x8_to_f16(c[j], t);
            f16x2 sc = e4m3_to_f16x2((s2 >> (8 * (j >> 1))) & 0xff);
#pragma unroll
            for (int e = 0; e < 4; e++) o[4 * j + e] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_bit_cast(f16x2, t[e]) * sc));
        }
        u32x4* d = (u32x4*)(Bs + row * GM_PITCH + half * 32);
#pragma unroll
        for (int j = 0; j < 4; j++) d[j] = (u32x4){o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
    }
};

// C[M][ldc] = bf16((A_q . W_q^T) * alpha[n]) (+ res: bf16(bf16(.) + res)); A_q as the fp16 operand of fe_fp4_quant,
// W codes [N][K/2], scales row-major [N][K/16]. grid ceil(M / 128) * N / 128 (grouped raster), 256 threads, dynamic LDS
// GM_LDS_TILES. N % 128 == 0, K % 128 == 0. (kernels/k-fp4/src/lib.rs:285-470)
extern "C" __global__ __launch_bounds__(256, 2) void fe_gemm_nvfp4(uint16_t* c, const _Float16* aq, const uint8_t* w,
                                                                   const uint8_t* sw, const float* alpha, const uint16_t* res,
                                                                   uint32_t m, uint32_t n, uint32_t k, uint32_t ldc,
                                                                   uint32_t group_m) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    uint32_t tm, tn;
    gemm_raster(blockIdx.x, (m + GM_BM - 1) / GM_BM, n / GM_BN, group_m, tm, tn);
    const uint32_t m0 = tm * GM_BM, n0 = tn * GM_BN;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    Fp4Producer prod;
    prod.row = tid >> 1, prod.half = tid & 1;
    prod.w = w + (size_t)(n0 + prod.row) * (k >> 1) + prod.half * 16;
    prod.sw = sw + (size_t)(n0 + prod.row) * (k >> 4) + prod.half * 2;
    f32x16 acc[2][2];
    gemm_mainloop(aq, k, m, k, m0, prod, lds, acc);
#pragma unroll
    for (int j = 0; j < 2; j++) {
        uint32_t col = n0 + wn * 64 + 32 * j + (lane & 31);
        float al = alpha[col] * 0.25f;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                uint32_t row = m0 + wm * 64 + 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (row < m) {
                    size_t at = (size_t)row * ldc + col;
                    uint32_t v = f32_to_bf16_bits(acc[i][j][e] * al);
                    if (res) v = f32_to_bf16_bits(bf16_bits_to_f32(v) + bf16_bits_to_f32(res[at]));
                    c[at] = (uint16_t)v;
                }
            }
    }
}
