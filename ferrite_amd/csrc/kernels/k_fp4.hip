// NVFP4 linear for gfx950: e2m1 codes (element 2i in the low nibble of byte i), one e4m3 scale per 16 elements along
// K, an fp32 scale per output column. Activations are quantized to the same format first (the reference's prompt path
// is W4A4, crates/fe-fp4/src/lib.rs:512-530), then the GEMM runs over the quantized operands.
//
// gfx950's block-scaled MFMA takes e8m0 scales per 32 elements, which cannot express e4m3 per 16. A product
// e2m1 x e4m3 has at most 6 significant bits and lies in [2^-10, 2688], so a small power of two times that value is an
// exact, normal fp16 number: both operands are expanded to fp16 (activations as 2 * code value * block scale, weights
// as 8 * ...) and multiplied on the f16 MFMA with fp32 accumulation, which reproduces the block-scaled dot product up
// to summation order; the factor 16 comes off in the epilogue.
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

// The same conversion for two values at once in hardware: byte `BYTE` of `old` becomes e2m1(a) | e2m1(b) << 4
// (v_cvt_scalef32_pk_fp4_f32 with scale 1). Checked against f32_to_e2m1 on the GPU for every bf16 value, every f32 with
// an exponent of 2^-5 .. 2^4 (all code boundaries and ties), the smallest and the largest magnitudes, infinities, both
// signs: no difference. A NaN is the one input the instruction treats otherwise (largest magnitude, where the
// definition's compare chain and the reference's table search give magnitude 0), so a NaN goes in as a zero of its sign.
__device__ __forceinline__ float e2m1_nan_to_zero(float x) {
    return x == x ? x : __uint_as_float(__float_as_uint(x) & 0x80000000u);
}
template <int BYTE>
__device__ __forceinline__ uint32_t f32x2_to_e2m1_byte(uint32_t old, float a, float b) {
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, e2m1_nan_to_zero(a), e2m1_nan_to_zero(b), 1.0f, BYTE);
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

// Weights through the hardware conversion. v_cvt_scalef32_pk_f16_fp4 turns the two e2m1 codes of one byte into fp16 and
// multiplies by a power of two: it takes only the exponent of its f32 scale operand (measured: scale 1.5 gives x1, 448
// gives x256). An e4m3 block scale is 2^(max(e, 1) - 7) * t / 8 with t = m (+ 8 for a normal number), so a weight is
// cvt(code, 2^(max(e, 1) - 7)) * t / 8; code * t has at most 6 significant bits and is exact in fp16. The kernels keep
// the factor 8 (weights as code * 2^E * t, below 23040) and take it off with alpha in the epilogue.
struct Fp4Scale {
    float pow2;  // 2^(max(e, 1) - 7) as f32
    f16x2 t;     // (t, t) as fp16
};
__device__ __forceinline__ Fp4Scale fp4_scale(uint32_t b) {  // b: e4m3 code, sign bit clear
    uint32_t e = b >> 3, e1 = e < 1 ? e : 1;
    Fp4Scale s;
    s.pow2 = __uint_as_float(((e > 1 ? e : 1) + 120) << 23);
    _Float16 t = (_Float16)(uint16_t)((b & 7) | (e1 << 3));
    s.t = (f16x2){t, t};
    return s;
}
// Both forms of all 128 positive e4m3 codes as a 1 KB table in LDS (fp4_scale is about ten vector instructions per 16
// weights; a lookup is two and an LDS read). Filled by the first 128 threads; a barrier must follow before the first lookup.
__device__ __forceinline__ void fp4_scale_lut_fill(u32x2* lut) {
    if (threadIdx.x < 128) {
        Fp4Scale s = fp4_scale(threadIdx.x);
        lut[threadIdx.x] = (u32x2){__float_as_uint(s.pow2), __builtin_bit_cast(uint32_t, s.t)};
    }
}
// at = 8 x the scale's code (the table's byte offset)
__device__ __forceinline__ Fp4Scale fp4_scale_lut(const u32x2* lut, uint32_t at) {
    const u32x2 e = *(const u32x2*)((const char*)lut + at);
    const uint32_t t = e[1];  // (a bit cast straight from the vector's element reads the vector's first bytes)
    Fp4Scale s;
    s.pow2 = __uint_as_float(e[0]), s.t = __builtin_bit_cast(f16x2, t);
    return s;
}
// 8 codes of one u32 -> 8 fp16 (code * 2^E * t), elements in order
__device__ __forceinline__ u32x4 fp4x8_to_f16(uint32_t w, Fp4Scale s) {
    u32x4 o;
    o[0] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, s.pow2, 0) * s.t));
    o[1] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, s.pow2, 1) * s.t));
    o[2] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, s.pow2, 2) * s.t));
    o[3] = __builtin_bit_cast(uint32_t, (f16x2)(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, s.pow2, 3) * s.t));
    return o;
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
    for (int w = 0; w < 2; w++) {
        q[w] = f32x2_to_e2m1_byte<0>(q[w], f[8 * w + 0] * mul, f[8 * w + 1] * mul);
        q[w] = f32x2_to_e2m1_byte<1>(q[w], f[8 * w + 2] * mul, f[8 * w + 3] * mul);
        q[w] = f32x2_to_e2m1_byte<2>(q[w], f[8 * w + 4] * mul, f[8 * w + 5] * mul);
        q[w] = f32x2_to_e2m1_byte<3>(q[w], f[8 * w + 6] * mul, f[8 * w + 7] * mul);
    }
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

// Weight tile producer: thread t expands the 64 codes of row t of the 256-row weight tile. Codes and scales are
// addressed through strides, base + kt * skt for the thread's row, so both the row-major layout of the format and the
// k-tile-major layout of an uploaded linear ([n / 128][k / 64][128 rows][32 bytes of codes | 4 scales], one contiguous
// 4.5 KB read per 128 rows and k tile) are read by the same kernel.
struct Fp4Producer {
    const uint8_t* w;   // codes of this thread's row, k tile 0
    const uint8_t* sw;  // scales of this thread's row, k tile 0
    uint32_t w_skt, s_skt, row;
    struct Raw {
        u32x4 c[2];
        uint32_t s2[2];
    };
    static constexpr int kStoreValu = 96;  // about the VALU instructions of store()
    static constexpr bool kQuarters = false;
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
        r.c[half] = *(const u32x4*)(w + (size_t)kt * w_skt + 16 * half);
        r.s2[half] = *(const uint16_t*)(sw + (size_t)kt * s_skt + 2 * half);
    }
    // part 0: chunks 0..3 of the row, part 1: 4..7
    __device__ __forceinline__ void store(const Raw& r, unsigned char* Bs, int part) const {
#pragma unroll
        for (int d = 0; d < 8; d++) {
            if (d / 4 != part) continue;
            // (computed: looked up in an LDS table as the GEMV does, the reads queue behind the fragment reads of the
            // k tile in flight and the GEMM is 5 % slower)
            Fp4Scale sc = fp4_scale((r.s2[d >> 2] >> (8 * ((d >> 1) & 1))) & 0xff);
            *(u32x4*)(Bs + gm_swz(row, d)) = fp4x8_to_f16(r.c[d >> 2][d & 3], sc);
        }
    }
};

// The fp16 operands are 2 x the quantized activation and 8 x the quantized weight.
#define FP4_OPERAND_SCALE 0.0625f

// One row piece of the output: 4 columns from `col` of row `grow`, bf16((sum) * alpha) (+ res: bf16(bf16(.) + res)).
__device__ __forceinline__ void fp4_store4(uint16_t* c, const uint16_t* res, size_t at, const float (&v)[4], f32x4 al) {
    u32x2 o = {pack_bf16x2(v[0] * al[0], v[1] * al[1]), pack_bf16x2(v[2] * al[2], v[3] * al[3])};
    if (res) {
        u32x2 r = *(const u32x2*)(res + at);
#pragma unroll
        for (int e = 0; e < 2; e++)
            o[e] = pack_bf16x2(bf16_bits_to_f32(o[e] & 0xffff) + bf16_bits_to_f32(r[e] & 0xffff),
                               bf16_bits_to_f32(o[e] >> 16) + bf16_bits_to_f32(r[e] >> 16));
    }
    *(u32x2*)(c + at) = o;
}

// ---- FP8 (e4m3, one scale per tensor) -------------------------------------------------------------------------------------

// The two e4m3 codes of the low (HI = 0) or high half of w as packed fp16, exact (hardware conversion, scale 1).
__device__ __forceinline__ uint32_t e4m3x2_to_f16(uint32_t w, int hi) {
    f16x2 v = hi ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true) : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, v);
}

// f32 -> e4m3 code of either sign, round to nearest even, saturating; NaN -> 0x7f. (crates/fe-fp4/src/format.rs:57-63)
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
    if (x != x) return 0x7f;
    return f32_to_e4m3_pos(__builtin_fabsf(x)) | ((__float_as_uint(x) >> 24) & 0x80u);
}

// bf16 x[M][ldx] -> e4m3 codes [M][K], q = e4m3(x * g), and the fp16 operand the GEMM reads (an e4m3 value is an exact
// fp16 number). One thread per 8 elements: grid ceil(M * K / 8 / 256), 256 threads. K % 8 == 0.
// (kernels/k-fp4/src/lib.rs:199-214)
extern "C" __global__ __launch_bounds__(256) void fe_fp8_quant(uint8_t* codes, _Float16* aq, const uint16_t* x, uint32_t m,
                                                               uint32_t k, uint32_t ldx, float g) {
    uint32_t i = blockIdx.x * 256 + threadIdx.x, k8 = k >> 3;
    if (i >= m * k8) return;
    uint32_t row = i / k8, c = (i - row * k8) * 8;
    u32x4 r = *(const u32x4*)(x + (size_t)row * ldx + c);
    uint32_t q[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t lo = f32_to_e4m3(__uint_as_float(r[j] << 16) * g), hi = f32_to_e4m3(__uint_as_float(r[j] & 0xffff0000u) * g);
        q[j >> 1] |= (lo | (hi << 8)) << (16 * (j & 1));
    }
    *(u32x2*)(codes + (size_t)row * k + c) = (u32x2){q[0], q[1]};
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; j++)
        o[j] = e4m3x2_to_f16(q[j >> 1], j & 1);
    *(u32x4*)(aq + (size_t)row * k + c) = o;
}

// Weight tile producer for e4m3 weights: thread t expands the 64 codes (64 bytes) of row t of the 256-row weight tile
// with the hardware conversion (exact). Addressing as Fp4Producer, 64 bytes a row and k tile.
struct Fp8Producer {
    const uint8_t* w;
    uint32_t w_skt, row;
    struct Raw {
        u32x4 c[4];
    };
    static constexpr int kStoreValu = 40;
    static constexpr bool kQuarters = false;
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
        const uint8_t* p = w + (size_t)kt * w_skt + 32 * half;
        r.c[2 * half] = *(const u32x4*)p;
        r.c[2 * half + 1] = *(const u32x4*)(p + 16);
    }
    // part 0: chunks 0..3 of the row (bytes 0..31), part 1: 4..7
    __device__ __forceinline__ void store(const Raw& r, unsigned char* Bs, int part) const {
#pragma unroll
        for (int d = 0; d < 8; d++) {
            if (d / 4 != part) continue;
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; e++)
                o[e] = e4m3x2_to_f16(r.c[d >> 1][2 * (d & 1) + (e >> 1)], e & 1);
            *(u32x4*)(Bs + gm_swz(row, d)) = o;
        }
    }
};

// ---- fused gate|up epilogue: SwiGLU and NVFP4 re-quantization ---------------------------------------------------------------

// act = bf16(bf16(silu(g)) * u), g and u the bf16 GEMM outputs (kernels/k-fp4/src/lib.rs:669-673).
__device__ __forceinline__ float swiglu(float g, float u) {
    float s = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
    s = bf16_bits_to_f32(f32_to_bf16_bits(s));
    return bf16_bits_to_f32(f32_to_bf16_bits(s * u));
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, true);
}

// The weight rows of a fused gate|up linear are interleaved in blocks of 8 (gate f..f+7, up f..f+7, ...,
// crates/fe-fp4/src/lib.rs:386-417), so a group of 32 output columns holds 16 features: of the 8 lanes that hold it
// (4 columns each) lanes 0, 1 have gate f0..7, lanes 2, 3 up f0..7, lanes 4, 5 gate f8..15, lanes 6, 7 up f8..15. Takes
// the 4 sums of a lane (v, already times alpha's lane values `al`), forms act = SwiGLU(bf16 gate, bf16 up) on the gate
// lanes, quantizes each 16-feature block to NVFP4 with global scale qg exactly as fe_fp4_quant would quantize the bf16
// act (block scale from the block's amax, codes, tiled scale, fp16 operand), and stores for rows that exist. Every lane
// of the half wavefront must call it. col: the lane's first interleaved column; n: interleaved width (2 * inter).
// (kernels/k-fp4/src/lib.rs:675-745)
__device__ __forceinline__ void swiglu_quant_store(const float (&v)[4], f32x4 al, uint32_t l32, bool live, uint32_t row,
                                                   uint32_t col, uint32_t n, uint8_t* q_codes, uint8_t* q_sf, _Float16* q_aq,
                                                   float qg) {
    const uint32_t j = l32 & 7;
    const bool gate = (j & 2) == 0;
    float act[4], amax = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float y = bf16_bits_to_f32(f32_to_bf16_bits(v[e] * al[e]));
        float u = dpp_mov<DPP_QUAD_XOR2>(y);  // the up value of the same feature, two lanes on
        act[e] = swiglu(y, u);
        if (gate) amax = __builtin_fmaxf(amax, __builtin_fabsf(act[e]));
    }
    amax = __builtin_fmaxf(amax, dpp_mov<DPP_QUAD_XOR1>(amax));
    amax = __builtin_fmaxf(amax, dpp_mov<DPP_QUAD_XOR2>(amax));
    amax = __builtin_fmaxf(amax, dpp_mov<DPP_QUAD_XOR3>(dpp_mov<DPP_HALF_MIRROR>(amax)));  // lane ^ 4
    const uint32_t s8 = f32_to_e4m3_pos(amax * (1.0f / 6.0f) * qg);
    const float sv = e4m3_to_f32(s8);
    const float mul = sv > 0.f ? qg / sv : 0.f;
    uint32_t q = f32x2_to_e2m1_byte<0>(0u, act[0] * mul, act[1] * mul);
    q = f32x2_to_e2m1_byte<1>(q, act[2] * mul, act[3] * mul);
    const uint32_t word = q | (dpp_mov_u32<DPP_QUAD_XOR1>(q) << 16);  // 8 codes: this lane's 4 features and the next lane's
    if (!live || !gate) return;
    const uint32_t inter = n >> 1, kb = inter >> 4, blk = col >> 5;
    const uint32_t feat = blk * 16 + (j >> 2) * 8 + (j & 1) * 4;  // the lane's first feature
    uint32_t t[4];
    e2m1x8_to_f16(q, t);
    const f16x2 sc = e4m3_to_f16x2(s8);
    u32x2 o = {__builtin_bit_cast(uint32_t, (f16x2)(__builtin_bit_cast(f16x2, t[0]) * sc)),
               __builtin_bit_cast(uint32_t, (f16x2)(__builtin_bit_cast(f16x2, t[1]) * sc))};
    *(u32x2*)(q_aq + (size_t)row * inter + feat) = o;
    if ((j & 1) == 0) *(uint32_t*)(q_codes + (size_t)row * (inter >> 1) + (feat >> 1)) = word;
    if (j == 0) q_sf[sf_tiled(row, blk, kb)] = (uint8_t)s8;
}

// ---- GEMM kernels ------------------------------------------------------------------------------------------------------------

// Where the output of a GEMM goes: C (bf16, + residual) or, for a fused gate|up linear, the NVFP4-quantized SwiGLU.
struct FpOut {
    uint16_t* c;
    const uint16_t* res;
    uint32_t ldc;
    uint8_t* q_codes;
    uint8_t* q_sf;
    _Float16* q_aq;
    float qg;
};

// One row piece: 4 sums of columns col.. of row grow. SWIGLU: every lane of the half wavefront takes part.
template <bool SWIGLU>
__device__ __forceinline__ void fp_store_piece(const FpOut& o, const float (&v)[4], f32x4 al, uint32_t l32, uint32_t grow,
                                               uint32_t m, uint32_t col, uint32_t n) {
    if constexpr (SWIGLU) {
        swiglu_quant_store(v, al, l32, grow < m, grow < m ? grow : 0, col, n, o.q_codes, o.q_sf, o.q_aq, o.qg);
    } else {
        if (grow < m) fp4_store4(o.c, o.res, (size_t)grow * o.ldc + col, v, al);
    }
}

// C[M][ldc] = bf16((A_q . W_q^T) * alpha[n]) (+ res: bf16(bf16(.) + res)); A_q = the fp16 operand of the quantizer,
// W_q expanded by the producer make_prod(tn) of 256-column tile tn; `scale` = 1 / (the factors the two fp16 expansions
// carry). Tiles = ceil(M / 256) * ceil(N / 256) (grouped raster), spread over the grid as sc says (gemm_schedule): one
// piece a program, the cut tiles finished by the reduce kernel, or stream-K. 256 threads, dynamic LDS GM_LDS_TILES.
// N % 128 == 0, K % 128 == 0. (kernels/k-fp4/src/lib.rs:285-470)
template <bool SWIGLU, bool SK, class MakeProd>
__device__ __forceinline__ void fp_gemm_body(MakeProd make_prod, const FpOut& out, const _Float16* aq, const float* alpha,
                                             float scale, uint32_t m, uint32_t n, uint32_t k, uint32_t group_m,
                                             const GemmSched& sc) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    gemm_schedule<SK>(
        sc, (m + GM_BM - 1) / GM_BM, (n / 128 + 1) / 2, group_m, k / GM_BK, lds,
        [&](uint32_t tm, uint32_t tn, uint32_t kt0, uint32_t ktn, f32x16(&acc)[4][4]) {
            auto prod = make_prod(tn);
            gemm_mainloop(aq, k, m, kt0, ktn, tm * GM_BM, prod, lds, acc);
        },
        [&](uint32_t tm, uint32_t tn, f32x16(&acc)[4][4]) {
            const uint32_t m0 = tm * GM_BM, colb = tn * GM_BN + wn * 128;
            if (colb >= n) return;
            const uint32_t col = colb + 4 * (tid & 31);
            const f32x4 al = *(const f32x4*)(alpha + col) * scale;
            gemm_epilogue(
                acc, lds, [](float (&)[4][4], uint32_t) {},
                [&](uint32_t row, uint32_t l32, float (&v)[4]) {
                    fp_store_piece<SWIGLU>(out, v, al, l32, m0 + wm * 128 + row, m, col, n);
                });
        });
}

// Finishes the tiles that a GEMM kernel cut along K. grid (tiles - full_tiles) * 64, 256 threads.
template <bool SWIGLU>
__device__ __forceinline__ void fp_reduce_body(const FpOut& out, const float* part, const float* alpha, float scale,
                                               uint32_t m, uint32_t n, uint32_t group_m, uint32_t full_tiles,
                                               uint32_t splits) {
    const uint32_t nts = n / 128;
    gemm_reduce_rows(part, splits, [&](uint32_t t, uint32_t row, uint32_t cb, uint32_t l32, float (&v)[4]) {
        uint32_t tm, tn;
        gemm_raster(full_tiles + t, (m + GM_BM - 1) / GM_BM, (nts + 1) / 2, group_m, tm, tn);
        uint32_t grow = tm * GM_BM + row, col = tn * GM_BN + cb * 128 + 4 * l32;
        if (tn * GM_BN + cb * 128 >= n) return;  // the absent half of an odd last tile (uniform over the half wavefront)
        fp_store_piece<SWIGLU>(out, v, *(const f32x4*)(alpha + col) * scale, l32, grow, m, col, n);
    });
}

__device__ __forceinline__ Fp4Producer fp4_producer(const uint8_t* w, const uint8_t* sw, uint32_t tn, uint32_t nts,
                                                    uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt,
                                                    uint32_t s_skt, uint32_t s_sr) {
    const uint32_t tid = threadIdx.x;
    uint32_t nt = 2 * tn + (tid >> 7);
    nt = nt < nts ? nt : nts - 1;  // an odd count of 128-row tiles: the last program expands its first tile twice
    Fp4Producer prod;
    prod.row = tid;
    prod.w = w + (size_t)nt * w_snt + (size_t)(tid & 127) * w_sr;
    prod.sw = sw + (size_t)nt * s_snt + (size_t)(tid & 127) * s_sr;
    prod.w_skt = w_skt, prod.s_skt = s_skt;
    return prod;
}

// NVFP4: the codes of row r = 128 nt + i, k tile kt are 32 bytes at w + nt * w_snt + kt * w_skt + i * w_sr, its 4 scales
// at sw + nt * s_snt + kt * s_skt + i * s_sr.
// Every GEMM kernel comes in two forms, NAME (one piece a program) and NAME_sk (stream-K), with the same parameters.
#define FP4_GEMM_PARAMS                                                                                                    \
    uint16_t *c, const _Float16 *aq, const uint8_t *w, const uint8_t *sw, const float *alpha, const uint16_t *res, uint32_t m, \
        uint32_t n, uint32_t k, uint32_t ldc, uint32_t group_m, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt, \
        uint32_t s_skt, uint32_t s_sr, GemmSched sc
template <bool SK>
__device__ __forceinline__ void gemm_nvfp4_kernel(FP4_GEMM_PARAMS) {
    FpOut out = {c, res, ldc, nullptr, nullptr, nullptr, 0.f};
    fp_gemm_body<false, SK>(
        [&](uint32_t tn) { return fp4_producer(w, sw, tn, n / 128, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr); }, out, aq, alpha,
        FP4_OPERAND_SCALE, m, n, k, group_m, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_nvfp4(FP4_GEMM_PARAMS) {
    gemm_nvfp4_kernel<false>(c, aq, w, sw, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_nvfp4_sk(FP4_GEMM_PARAMS) {
    gemm_nvfp4_kernel<true>(c, aq, w, sw, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr, sc);
}

extern "C" __global__ __launch_bounds__(256) void fe_gemm_nvfp4_reduce(uint16_t* c, const float* part, const float* alpha,
                                                                       const uint16_t* res, uint32_t m, uint32_t n,
                                                                       uint32_t ldc, uint32_t group_m, uint32_t full_tiles,
                                                                       uint32_t splits, float scale) {
    FpOut out = {c, res, ldc, nullptr, nullptr, nullptr, 0.f};
    fp_reduce_body<false>(out, part, alpha, scale, m, n, group_m, full_tiles, splits);
}

// Fused MLP front: act = SwiGLU(x . [gate|up]^T), NVFP4-quantized with global scale qg (1 / input_scale of the down
// projection) into q_codes [M][inter/2], q_sf (tiled, kb = inter/16) and the fp16 operand q_aq [M][inter]; w, sw, alpha =
// gate and up interleaved in blocks of 8 rows, N = 2 inter, N % 256 == 0. (kernels/k-fp4/src/lib.rs:747-752)
#define FP4_SWIGLU_PARAMS                                                                                                \
    const _Float16 *aq, const uint8_t *w, const uint8_t *sw, const float *alpha, uint32_t m, uint32_t n, uint32_t k,           \
        uint32_t group_m, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt, uint32_t s_skt, uint32_t s_sr,        \
        GemmSched sc, uint8_t *q_codes, uint8_t *q_sf, _Float16 *q_aq, float qg
template <bool SK>
__device__ __forceinline__ void gemm_nvfp4_swiglu_kernel(FP4_SWIGLU_PARAMS) {
    FpOut out = {nullptr, nullptr, 0, q_codes, q_sf, q_aq, qg};
    fp_gemm_body<true, SK>(
        [&](uint32_t tn) { return fp4_producer(w, sw, tn, n / 128, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr); }, out, aq, alpha,
        FP4_OPERAND_SCALE, m, n, k, group_m, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_nvfp4_swiglu(FP4_SWIGLU_PARAMS) {
    gemm_nvfp4_swiglu_kernel<false>(aq, w, sw, alpha, m, n, k, group_m, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr, sc, q_codes, q_sf,
                                    q_aq, qg);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_nvfp4_swiglu_sk(FP4_SWIGLU_PARAMS) {
    gemm_nvfp4_swiglu_kernel<true>(aq, w, sw, alpha, m, n, k, group_m, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr, sc, q_codes, q_sf,
                                   q_aq, qg);
}

extern "C" __global__ __launch_bounds__(256) void fe_gemm_nvfp4_swiglu_reduce(const float* part, const float* alpha, uint32_t m,
                                                                              uint32_t n, uint32_t group_m, uint32_t full_tiles,
                                                                              uint32_t splits, uint8_t* q_codes, uint8_t* q_sf,
                                                                              _Float16* q_aq, float qg) {
    FpOut out = {nullptr, nullptr, 0, q_codes, q_sf, q_aq, qg};
    fp_reduce_body<true>(out, part, alpha, FP4_OPERAND_SCALE, m, n, group_m, full_tiles, splits);
}

// FP8: the 64 codes of row r = 128 nt + i, k tile kt are at w + nt * w_snt + kt * w_skt + i * w_sr; both fp16 expansions
// are the values themselves. Finished by fe_gemm_nvfp4_reduce with scale 1. (kernels/k-fp4/src/lib.rs:472-484)
#define FP8_GEMM_PARAMS                                                                                                     \
    uint16_t *c, const _Float16 *aq, const uint8_t *w, const float *alpha, const uint16_t *res, uint32_t m, uint32_t n, uint32_t k, \
        uint32_t ldc, uint32_t group_m, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, GemmSched sc
template <bool SK>
__device__ __forceinline__ void gemm_fp8_kernel(FP8_GEMM_PARAMS) {
    const uint32_t nts = n / 128, tid = threadIdx.x;
    FpOut out = {c, res, ldc, nullptr, nullptr, nullptr, 0.f};
    fp_gemm_body<false, SK>(
        [&](uint32_t tn) {
            uint32_t nt = 2 * tn + (tid >> 7);
            nt = nt < nts ? nt : nts - 1;
            Fp8Producer prod;
            prod.row = tid;
            prod.w = w + (size_t)nt * w_snt + (size_t)(tid & 127) * w_sr;
            prod.w_skt = w_skt;
            return prod;
        },
        out, aq, alpha, 1.0f, m, n, k, group_m, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_fp8(FP8_GEMM_PARAMS) {
    gemm_fp8_kernel<false>(c, aq, w, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_fp8_sk(FP8_GEMM_PARAMS) {
    gemm_fp8_kernel<true>(c, aq, w, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, sc);
}

// The same linear on the 8-bit matrix instruction: activations are the quantizer's e4m3 codes [M][K], weights stay codes
// in LDS, a k tile is 128 wide (two of the 64-wide weight tiles of the layout above). Same products (an e4m3 x e4m3
// product is exact in f32) and f32 sums as fe_gemm_fp8, at twice the MFMA rate and half the LDS bytes per flop.
struct Fp8CodeProducer {
    const uint8_t* w[2];  // the two 128-row weight tiles + this thread's (row, chunk) offset
    uint32_t w_skt, w_sr, st;
    struct Raw {
        u32x4 c[2][4];
    };
    static constexpr int kStoreValu = 0;
    static constexpr bool kQuarters = false;
    // thread t: 16-byte chunk t & 7 of rows (t >> 3) + 32 j of each 128-row half; chunks 0..3 come from 64-wide weight
    // tile 2 kt, chunks 4..7 from 2 kt + 1
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != half) continue;
            const uint8_t* p = w[b] + (size_t)(2 * kt) * w_skt;
#pragma unroll
            for (int j = 0; j < 4; j++) r.c[b][j] = *(const u32x4*)(p + (size_t)(32 * j) * w_sr);
        }
    }
    __device__ __forceinline__ void store(const Raw& r, unsigned char* Bs, int part) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != part) continue;
#pragma unroll
            for (int j = 0; j < 4; j++) *(u32x4*)(Bs + 16384 * b + st + 4096 * j) = r.c[b][j];
        }
    }
};

#define FP8C_GEMM_PARAMS                                                                                                   \
    uint16_t *c, const uint8_t *aq, const uint8_t *w, const float *alpha, const uint16_t *res, uint32_t m, uint32_t n, uint32_t k, \
        uint32_t ldc, uint32_t group_m, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, GemmSched sc
template <bool SK>
__device__ __forceinline__ void gemm_fp8_codes_kernel(FP8C_GEMM_PARAMS) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t nts = n / 128, tid = threadIdx.x, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    FpOut out = {c, res, ldc, nullptr, nullptr, nullptr, 0.f};
    gemm_schedule<SK>(
        sc, (m + GM_BM - 1) / GM_BM, (nts + 1) / 2, group_m, k / 128, lds,
        [&](uint32_t tm, uint32_t tn, uint32_t kt0, uint32_t ktn, f32x16(&acc)[4][4]) {
            Fp8CodeProducer prod;
            const uint32_t chunk = tid & 7, row = tid >> 3;
#pragma unroll
            for (int b = 0; b < 2; b++) {
                uint32_t nt = 2 * tn + b;
                nt = nt < nts ? nt : nts - 1;  // an odd count of 128-row tiles: the last program copies its first tile twice
                prod.w[b] = w + (size_t)nt * w_snt + (size_t)(chunk >> 2) * w_skt + (size_t)row * w_sr + (chunk & 3) * 16;
            }
            prod.w_skt = w_skt, prod.w_sr = w_sr, prod.st = gm_swz(row, chunk);
            gemm_mainloop_f8(aq, k, m, kt0, ktn, tm * GM_BM, prod, lds, acc);
        },
        [&](uint32_t tm, uint32_t tn, f32x16(&acc)[4][4]) {
            const uint32_t m0 = tm * GM_BM, colb = tn * GM_BN + wn * 128;
            if (colb >= n) return;
            const uint32_t col = colb + 4 * (tid & 31);
            const f32x4 al = *(const f32x4*)(alpha + col);
            gemm_epilogue(
                acc, lds, [](float (&)[4][4], uint32_t) {},
                [&](uint32_t r, uint32_t l32, float (&v)[4]) {
                    fp_store_piece<false>(out, v, al, l32, m0 + wm * 128 + r, m, col, n);
                });
        });
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_fp8_codes(FP8C_GEMM_PARAMS) {
    gemm_fp8_codes_kernel<false>(c, aq, w, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, sc);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_fp8_codes_sk(FP8C_GEMM_PARAMS) {
    gemm_fp8_codes_kernel<true>(c, aq, w, alpha, res, m, n, k, ldc, group_m, w_snt, w_skt, w_sr, sc);
}

// ---- GEMV (1..48 rows) -------------------------------------------------------------------------------------------------

#define FP4_GEMV_RG 8  // 16-row groups of a 128-row weight tile

// One k tile of one 128-row weight tile as a wavefront reads it: lane L = 16 g + r takes, of row 16 rg + r, the 16 codes
// k = 16 g .. 16 g + 15 (8 bytes) and the row's four scale bytes (it uses byte g), and of activation rows r, 16 + r, ...
// (XR groups of 16) the same 16 values. The k index inside an MFMA is only a summation index, so the A operand (weights)
// and the B operand (activations) merely have to agree: MFMA j of a row group multiplies k = 16 g + 8 j .. + 7 of lane
// group g.
template <int XR>
struct Fp4GemvStage {
    u32x2 cw[FP4_GEMV_RG];
    uint32_t sc[FP4_GEMV_RG];
    f16x8 x[XR][2];
};

// c[m][ldc] = bf16((A_q . W_q^T) * alpha[n]) (+ res) for m <= 16 XR rows: the decode-sized form of fe_gemm_nvfp4, bound
// by the read of the weights, which every row count reads once. grid (n / 128) * sk, 256 threads: a program takes one
// 128-row weight tile and one of sk runs of k tiles, its four wavefronts alternate k tiles. Each wavefront expands its
// codes in registers straight into the A operand of v_mfma_f32_16x16x32_f16 (rows = weight rows, columns = activation
// rows; one expansion serves all XR groups of activation rows); the wavefronts' sums meet in LDS. With sk > 1 the
// splits leave f32 partials in z (per weight tile and split, 8 KB per group of 16 activation rows, in the order the
// lanes hold them); the last to arrive (counters[tile]) adds them in split order, finishes the tile and re-arms the
// counter, so the result does not depend on timing. A row's sums do not depend on XR. Weight
// addressing as in fe_gemm_nvfp4.
template <int XR>
__device__ __forceinline__ void gemv_nvfp4_body(uint16_t* c, const _Float16* aq, const uint8_t* w, const uint8_t* sw,
                                                const float* alpha, const uint16_t* res, float* z, uint32_t* counters,
                                                uint32_t m, uint32_t n, uint32_t k, uint32_t ldc, uint32_t sk,
                                                uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt,
                                                uint32_t s_skt, uint32_t s_sr) {
    __shared__ f32x4 red[4][FP4_GEMV_RG][64];
    __shared__ uint32_t last_flag;
    __shared__ u32x2 scale_lut[128];  // the loop is bound by vector instruction issue and the LDS pipe is idle in it
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    fp4_scale_lut_fill(scale_lut);
    const uint32_t scale_rot = (8 * g + 29) & 31;  // rotating right by this leaves the lane's scale byte times 8 in bits 3..10
    const uint32_t nts = n / 128, nt = blockIdx.x % nts, split = blockIdx.x / nts;
    const uint32_t ktiles = k / 64, kt_begin = split * ktiles / sk, kt_end = (split + 1) * ktiles / sk;
    const uint8_t* wp = w + (size_t)nt * w_snt + (size_t)r * w_sr + 8 * g;
    const uint8_t* sp = sw + (size_t)nt * s_snt + (size_t)r * s_sr;
    const _Float16* xp[XR];
#pragma unroll
    for (int xr = 0; xr < XR; xr++) xp[xr] = aq + (size_t)(16 * xr + r < m ? 16 * xr + r : m - 1) * k + 16 * g;

    auto load = [&](Fp4GemvStage<XR>& st, uint32_t kt) {
        const uint8_t* wk = wp + (size_t)kt * w_skt;
        const uint8_t* sk_ = sp + (size_t)kt * s_skt;
#pragma unroll
        for (int rg = 0; rg < FP4_GEMV_RG; rg++) {
            st.cw[rg] = __builtin_nontemporal_load((const u32x2*)(wk + (size_t)(16 * rg) * w_sr));
            st.sc[rg] = __builtin_nontemporal_load((const uint32_t*)(sk_ + (size_t)(16 * rg) * s_sr));
        }
#pragma unroll
        for (int xr = 0; xr < XR; xr++) {
            st.x[xr][0] = *(const f16x8*)(xp[xr] + kt * 64);
            st.x[xr][1] = *(const f16x8*)(xp[xr] + kt * 64 + 8);
        }
    };
    f32x4 acc[XR][FP4_GEMV_RG];
#pragma unroll
    for (int xr = 0; xr < XR; xr++)
#pragma unroll
        for (int rg = 0; rg < FP4_GEMV_RG; rg++) acc[xr][rg] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const Fp4GemvStage<XR>& st) {
#pragma unroll
        for (int rg = 0; rg < FP4_GEMV_RG; rg++) {
            const uint32_t at = __builtin_amdgcn_alignbit(st.sc[rg], st.sc[rg], scale_rot) & 0x3f8;
            const Fp4Scale s = fp4_scale_lut(scale_lut, at);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                u32x4 a = fp4x8_to_f16(st.cw[rg][j], s);
#pragma unroll
                for (int xr = 0; xr < XR; xr++)
                    acc[xr][rg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), st.x[xr][j], acc[xr][rg], 0, 0, 0);
            }
        }
    };
    // NS k tiles in flight per wavefront (a ring of stages indexed by constants; three, four and six were measured and
    // are no faster). Loads past the end of the run are skipped (a wavefront-uniform branch).
    constexpr int NS = 2;
    Fp4GemvStage<XR> st[NS];
    uint32_t kt = kt_begin + wave;
#pragma unroll
    for (int i = 0; i < NS; i++)
        if (kt + 4 * i < kt_end) load(st[i], kt + 4 * i);
    __syncthreads();  // scale_lut
    // (the scheduling barriers keep each refill where it is written: the compiler otherwise sinks the loads to just
    // before their use, a whole stage later)
    for (; kt < kt_end; kt += 4 * NS) {
#pragma unroll
        for (int i = 0; i < NS; i++) {
            if (kt + 4 * i < kt_end) compute(st[i]);
            __builtin_amdgcn_sched_barrier(0);
            if (kt + 4 * (i + NS) < kt_end) load(st[i], kt + 4 * (i + NS));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // The four wavefronts' sums meet in LDS, one group of activation rows at a time; wavefront v finishes weight row
    // groups 2 v and 2 v + 1. Lane (r, g) then holds, for weight row group rg, output row 16 xr + r, columns
    // n0 + 16 rg + 4 g .. + 3.
    const uint32_t col = nt * 128 + 32 * wave + 4 * g;  // + 16 h
    f32x4 sum[XR][2];
#pragma unroll
    for (int xr = 0; xr < XR; xr++) {
        if (xr) __syncthreads();
#pragma unroll
        for (int rg = 0; rg < FP4_GEMV_RG; rg++) red[wave][rg][lane] = acc[xr][rg];
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; h++) {
            sum[xr][h] = red[0][2 * wave + h][lane];
#pragma unroll
            for (int v = 1; v < 4; v++) sum[xr][h] += red[v][2 * wave + h][lane];
        }
    }
    auto finish = [&](uint32_t row, const f32x4 (&v)[2]) {
        if (row >= m) return;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t cc = col + 16 * h;
            float o[4] = {v[h][0], v[h][1], v[h][2], v[h][3]};
            fp4_store4(c, res, (size_t)row * ldc + cc, o, *(const f32x4*)(alpha + cc) * FP4_OPERAND_SCALE);
        }
    };
    if (sk == 1) {
#pragma unroll
        for (int xr = 0; xr < XR; xr++) finish(16 * xr + r, sum[xr]);
        return;
    }
    // Partials cross to another program, possibly on another XCD with its own L2: agent-scope accesses, ordered by the
    // barriers around the arrival counter. A program's partial lies in z as its lanes hold it (a wavefront's store is 1 KB
    // in one piece), and the finisher's lanes hold the same elements: zp(split, xr, h) is this lane's f32x4.
    auto zp = [&](uint32_t sp, int xr, int h) {
        return z + ((((size_t)nt * sk + sp) * XR + xr) * 8 + 2 * wave + h) * 256 + 4 * lane;
    };
#pragma unroll
    for (int xr = 0; xr < XR; xr++) {
        if (16 * xr + r < m) {
#pragma unroll
            for (int h = 0; h < 2; h++) store_agent_f32x4(zp(split, xr, h), sum[xr][h]);
        }
    }
    agent_stores_wait();  // this lane's stores are acknowledged at agent scope
    __syncthreads();
    if (tid == 0) {
        uint32_t old = __hip_atomic_fetch_add(&counters[nt], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (old == sk - 1);
    }
    __syncthreads();
    if (!last_flag) return;
    if (tid == 0) __hip_atomic_store(&counters[nt], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the loads of up to 8 splits are in flight together (an agent-scope load takes a trip to memory); sums in split order
    const __amdgpu_buffer_rsrc_t zrs = __builtin_amdgcn_make_buffer_rsrc((void*)z, 0, nts * sk * XR * 8192u, 0x00020000);
#pragma unroll
    for (int xr = 0; xr < XR; xr++) {
        const uint32_t row = 16 * xr + r;
        if (row >= m) continue;
        f32x4 tot[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        for (uint32_t s0 = 0; s0 < sk; s0 += 8) {
            f32x4 t[16];
#pragma unroll
            for (int b = 0; b < 8; b++) {
                if (s0 + b < sk) {
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        t[2 * b + h] = load_agent_f32x4(zrs, (uint32_t)((const char*)zp(s0 + b, xr, h) - (const char*)z), 0);
                } else {
                    t[2 * b] = t[2 * b + 1] = (f32x4){0.f, 0.f, 0.f, 0.f};
                }
            }
            agent_loads_wait(t);
#pragma unroll
            for (int b = 0; b < 8; b++)
                if (s0 + b < sk) {
#pragma unroll
                    for (int h = 0; h < 2; h++) tot[h] += t[2 * b + h];
                }
        }
        finish(row, tot);
    }
}

#define FP4_GEMV_KERNEL(XR)                                                                                            \
    extern "C" __global__ __launch_bounds__(256, 2) void fe_gemv_nvfp4_x##XR(                                          \
        uint16_t* c, const _Float16* aq, const uint8_t* w, const uint8_t* sw, const float* alpha, const uint16_t* res, \
        float* z, uint32_t* counters, uint32_t m, uint32_t n, uint32_t k, uint32_t ldc, uint32_t sk, uint32_t w_snt,   \
        uint32_t w_skt, uint32_t w_sr, uint32_t s_snt, uint32_t s_skt, uint32_t s_sr) {                                \
        gemv_nvfp4_body<XR>(c, aq, w, sw, alpha, res, z, counters, m, n, k, ldc, sk, w_snt, w_skt, w_sr, s_snt, s_skt, \
                            s_sr);                                                                                     \
    }
FP4_GEMV_KERNEL(1)
FP4_GEMV_KERNEL(2)
FP4_GEMV_KERNEL(3)  // (four groups of rows would not fit the registers of two programs a CU)

// ---- GEMV over strips of 16 weight rows (1..16 rows): no hand-off between programs ------------------------------------------
//
// A program takes one strip of 16 weight rows over all of K; its W wavefronts (blockDim.x / 64: 4, 8 or 16, the host's
// choice, so that a launch has four or more wavefronts a SIMD) take groups of four k tiles in turn and their sums meet
// in LDS. Nothing crosses between programs: no partial sums in memory, no arrival counters, no finisher.
//
// What bounds a kernel that reads 9/16 byte a weight is the address unit: a vector memory instruction occupies it for
// 16 clocks whatever it fetches. So a load step of a wavefront is four k tiles at once: lane L = 16 g + r takes row r
// of k tile kt0 + g whole, 32 bytes of codes as two 16-byte loads and its four scale bytes as one dword (three
// instructions per 2 KB of codes, where a lane that takes 16 codes of one k tile needs two per 512 bytes); the MFMA's k
// index is only a summation index, so step s of the group multiplies, in lane group g, the 16 codes of scale block s of
// k tile kt0 + g with the same 16 activations. The activations (m rows of k fp16: the host takes this kernel only where
// they fit in 48 KB) are staged in LDS once per program and read from there. A row's bits depend on (k, W) only.
struct Fp4StripStage {
    u32x4 c[2];   // the lane's row of k tile kt0 + g: 64 codes
    uint32_t sc;  // its four scale bytes
};
#define FP4_STRIP_WAVES_MAX 16

__device__ __forceinline__ void gemv_nvfp4_strip_body(uint16_t* c, const _Float16* aq, const uint8_t* w, const uint8_t* sw,
                                                      const float* alpha, const uint16_t* res, uint32_t m, uint32_t n, uint32_t k,
                                                      uint32_t ldc, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt,
                                                      uint32_t s_skt, uint32_t s_sr) {
    constexpr int XR = 1;  // up to 16 activation rows
    __shared__ f32x4 red[FP4_STRIP_WAVES_MAX][64];
    __shared__ u32x2 scale_lut[128];
    extern __shared__ __attribute__((aligned(16))) unsigned char xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6, r = lane & 15, g = lane >> 4;
    fp4_scale_lut_fill(scale_lut);
    for (uint32_t i = tid; i < m * (k / 8); i += blockDim.x) ((u32x4*)xs)[i] = ((const u32x4*)aq)[i];
    const uint32_t strip = blockIdx.x, nt = strip >> 3, rg = strip & 7;  // the strip: 16-row group rg of weight tile nt
    const uint32_t groups = k / 256;                                      // groups of four k tiles
    const uint8_t* wp = w + (size_t)nt * w_snt + (size_t)(16 * rg + r) * w_sr + (size_t)g * w_skt;
    const uint8_t* sp = sw + (size_t)nt * s_snt + (size_t)(16 * rg + r) * s_sr + (size_t)g * s_skt;
    uint32_t xo[XR];  // byte offset in xs of the lane's activation row at k tile g
#pragma unroll
    for (int xr = 0; xr < XR; xr++) xo[xr] = ((16 * xr + r < m ? 16 * xr + r : m - 1) * k + 64 * g) * 2;

    auto load = [&](Fp4StripStage& st, uint32_t gi) {
        const uint8_t* p = wp + (size_t)gi * 4 * w_skt;
        st.c[0] = __builtin_nontemporal_load((const u32x4*)p);
        st.c[1] = __builtin_nontemporal_load((const u32x4*)(p + 16));
        st.sc = __builtin_nontemporal_load((const uint32_t*)(sp + (size_t)gi * 4 * s_skt));
    };
    f32x4 acc[XR];
#pragma unroll
    for (int xr = 0; xr < XR; xr++) acc[xr] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const Fp4StripStage& st, uint32_t gi) {
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {  // scale block blk of the lane's k tile: codes 16 blk .. 16 blk + 15
            const Fp4Scale s = fp4_scale_lut(scale_lut, __builtin_amdgcn_ubfe(st.sc, 8 * blk, 8) << 3);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                u32x4 a = fp4x8_to_f16(st.c[blk >> 1][2 * (blk & 1) + j], s);
#pragma unroll
                for (int xr = 0; xr < XR; xr++) {
                    const f16x8 x = *(const f16x8*)(xs + xo[xr] + gi * 512 + 32 * blk + 16 * j);
                    acc[xr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), x, acc[xr], 0, 0, 0);
                }
            }
        }
    };
    constexpr int NS = 4;  // groups in flight a wavefront (16 k tiles)
    Fp4StripStage st[NS];
    uint32_t gi = wave;
#pragma unroll
    for (int i = 0; i < NS; i++)
        if (gi + waves * i < groups) load(st[i], gi + waves * i);
    __syncthreads();  // scale_lut, xs
    for (; gi < groups; gi += waves * NS) {
#pragma unroll
        for (int i = 0; i < NS; i++) {
            if (gi + waves * i < groups) compute(st[i], gi + waves * i);
            __builtin_amdgcn_sched_barrier(0);
            if (gi + waves * (i + NS) < groups) load(st[i], gi + waves * (i + NS));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // The wavefronts' sums meet in LDS, one group of activation rows at a time; wavefront 0 adds them in wavefront order.
    // Lane (r, g) holds output row 16 xr + r, columns 16 strip + 4 g .. + 3.
    const uint32_t col = 16 * strip + 4 * g;
#pragma unroll
    for (int xr = 0; xr < XR; xr++) {
        if (xr) __syncthreads();
        red[wave][lane] = acc[xr];
        __syncthreads();
        const uint32_t row = 16 * xr + r;
        if (wave == 0 && row < m) {
            f32x4 sum = red[0][lane];
            for (uint32_t v = 1; v < waves; v++) sum += red[v][lane];
            float o[4] = {sum[0], sum[1], sum[2], sum[3]};
            fp4_store4(c, res, (size_t)row * ldc + col, o, *(const f32x4*)(alpha + col) * FP4_OPERAND_SCALE);
        }
    }
}

extern "C" __global__ __launch_bounds__(1024) void fe_gemv_nvfp4_strips(uint16_t* c, const _Float16* aq, const uint8_t* w,
                                                                        const uint8_t* sw, const float* alpha, const uint16_t* res,
                                                                        uint32_t m, uint32_t n, uint32_t k, uint32_t ldc, uint32_t w_snt,
                                                                        uint32_t w_skt, uint32_t w_sr, uint32_t s_snt, uint32_t s_skt,
                                                                        uint32_t s_sr) {
    gemv_nvfp4_strip_body(c, aq, w, sw, alpha, res, m, n, k, ldc, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr);
}

// The same strips when a wavefront's share of K is GPW <= 5 groups and the activations are at most four 16-byte pieces a
// thread: every load of the workgroup goes out before anything waits. The activations' loads first (they
// are few and mostly hit L2; loads return in order), then the wavefront's whole share of the strip, then the activations
// go to LDS while the weights are on their way, and the groups are taken in the order they arrive. No load sits under a
// condition (a wavefront with fewer groups than the others requests its last group again and does not use it; a thread
// past the end of the activations requests the last piece again), so the compiler counts its waits exactly instead of
// waiting for everything at the head of a loop. A vector memory instruction costs the address unit the same whether
// its data is wanted or not, so the kernel exists per GPW and the host picks a number of wavefronts that divides the
// groups where it can (any number up to 16, not only powers of two).
template <int GPW>
__device__ __forceinline__ void gemv_nvfp4_strip_once_body(uint16_t* c, const _Float16* aq, const uint8_t* w, const uint8_t* sw,
                                                           const float* alpha, const uint16_t* res, uint32_t m, uint32_t k,
                                                           uint32_t ldc, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr,
                                                           uint32_t s_snt, uint32_t s_skt, uint32_t s_sr) {
    __shared__ f32x4 red[FP4_STRIP_WAVES_MAX][64];
    __shared__ u32x2 scale_lut[128];
    extern __shared__ __attribute__((aligned(16))) unsigned char xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6, r = lane & 15, g = lane >> 4;
    constexpr int XV = 4;
    const uint32_t xn = m * (k / 8);  // 16-byte pieces of the activations
    u32x4 xv[XV];
    uint32_t xi[XV];
#pragma unroll
    for (int i = 0; i < XV; i++) {
        xi[i] = tid + i * blockDim.x;
        xi[i] = xi[i] < xn ? xi[i] : xn - 1;
        xv[i] = ((const u32x4*)aq)[xi[i]];
    }
    const uint32_t strip = blockIdx.x, nt = strip >> 3, rg = strip & 7;  // the strip: 16-row group rg of weight tile nt
    const uint32_t groups = k / 256;                                      // groups of four k tiles
    const uint8_t* wp = w + (size_t)nt * w_snt + (size_t)(16 * rg + r) * w_sr + (size_t)g * w_skt;
    const uint8_t* sp = sw + (size_t)nt * s_snt + (size_t)(16 * rg + r) * s_sr + (size_t)g * s_skt;
    Fp4StripStage st[GPW];
#pragma unroll
    for (int i = 0; i < GPW; i++) {
        uint32_t gi = wave + waves * i;
        gi = gi < groups ? gi : groups - 1;
        const uint8_t* p = wp + (size_t)gi * 4 * w_skt;
        st[i].c[0] = __builtin_nontemporal_load((const u32x4*)p);
        st[i].c[1] = __builtin_nontemporal_load((const u32x4*)(p + 16));
        st[i].sc = __builtin_nontemporal_load((const uint32_t*)(sp + (size_t)gi * 4 * s_skt));
    }
    fp4_scale_lut_fill(scale_lut);
#pragma unroll
    for (int i = 0; i < XV; i++) ((u32x4*)xs)[xi[i]] = xv[i];
    __syncthreads();  // scale_lut, xs
    const uint32_t xo = ((r < m ? r : m - 1) * k + 64 * g) * 2;  // byte offset in xs of the lane's activation row at k tile g
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < GPW; i++) {
        const uint32_t gi = wave + waves * i;
        if (gi < groups) {
#pragma unroll
            for (int blk = 0; blk < 4; blk++) {  // scale block blk of the lane's k tile: codes 16 blk .. 16 blk + 15
                const Fp4Scale sc = fp4_scale_lut(scale_lut, __builtin_amdgcn_ubfe(st[i].sc, 8 * blk, 8) << 3);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    u32x4 a = fp4x8_to_f16(st[i].c[blk >> 1][2 * (blk & 1) + j], sc);
                    const f16x8 x = *(const f16x8*)(xs + xo + gi * 512 + 32 * blk + 16 * j);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), x, acc, 0, 0, 0);
                }
            }
        }
    }
    // The wavefronts' sums meet in LDS; wavefront 0 adds them in wavefront order. Lane (r, g) holds output row r, columns
    // 16 strip + 4 g .. + 3. (The groups of a wavefront are added in the order of the kernel above: the same bits.)
    const uint32_t col = 16 * strip + 4 * g;
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && r < m) {
        f32x4 sum = red[0][lane];
        for (uint32_t v = 1; v < waves; v++) sum += red[v][lane];
        float o[4] = {sum[0], sum[1], sum[2], sum[3]};
        fp4_store4(c, res, (size_t)r * ldc + col, o, *(const f32x4*)(alpha + col) * FP4_OPERAND_SCALE);
    }
}

#define FP4_STRIPS_ONCE_KERNEL(GPW)                                                                                       \
    extern "C" __global__ __launch_bounds__(1024) void fe_gemv_nvfp4_strips_once_g##GPW(                                  \
        uint16_t* c, const _Float16* aq, const uint8_t* w, const uint8_t* sw, const float* alpha, const uint16_t* res,   \
        uint32_t m, uint32_t n, uint32_t k, uint32_t ldc, uint32_t w_snt, uint32_t w_skt, uint32_t w_sr, uint32_t s_snt, \
        uint32_t s_skt, uint32_t s_sr) {                                                                                  \
        (void)n;                                                                                                          \
        gemv_nvfp4_strip_once_body<GPW>(c, aq, w, sw, alpha, res, m, k, ldc, w_snt, w_skt, w_sr, s_snt, s_skt, s_sr);     \
    }
FP4_STRIPS_ONCE_KERNEL(1)
FP4_STRIPS_ONCE_KERNEL(2)
FP4_STRIPS_ONCE_KERNEL(3)
FP4_STRIPS_ONCE_KERNEL(4)
FP4_STRIPS_ONCE_KERNEL(5)

// ---- matrix-unit peak probe ---------------------------------------------------------------------------------------------
//
// Every wavefront issues iters x 16 independent matrix instructions (the GEMM core's 4 x 4 accumulator pieces, 256
// accumulator registers) on operands that stay in registers: no memory traffic, no LDS (kernels/k-fp4/src/lib.rs:866-916,
// fe_fp4_peak). KIND 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_32x32x16_bf16, 2: v_mfma_f32_32x32x64_f8f6f4 on e4m3
// codes (the unscaled form). seed == 0: every operand element is 0.5 or 1 (few bits toggle from one instruction to the
// next, the reference's kind of pattern); otherwise signs and mantissas are random bits of the seed (an even seed:
// only the top five mantissa bits of the 16-bit kinds), magnitudes in [0.5, 2), as the operands of a GEMM on real data toggle: the clock the board holds under its power limit depends on
// it. One float a lane is written so that nothing is dead code. Flops of a launch: wavefronts x iters x 16 x 2 x 32 x 32 x
// (16 or 64).
template <int KIND>
__device__ __forceinline__ void mfma_peak_body(float* out, uint32_t iters, uint32_t seed) {
    const uint32_t lane = threadIdx.x & 63;
    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;
    uint32_t rs = seed * 0x9e3779b9u + (blockIdx.x * 256 + threadIdx.x) * 0x85ebca6bu;
    auto rnd = [&]() {
        rs ^= rs << 13, rs ^= rs >> 17, rs ^= rs << 5;
        return seed ? rs : 0u;
    };
    // 16-bit pairs: sign and mantissa from the random word, exponent of 0.5 or 1; e4m3 quadruples likewise
    // (an even seed keeps only the top five mantissa bits of the 16-bit kinds: the six significant bits of an NVFP4 operand)
    const uint32_t keep16 = seed & 1 ? (KIND == 1 ? 0x80ff80ffu : 0x87ff87ffu) : (KIND == 1 ? 0x80fc80fcu : 0x87e087e0u);
    const uint32_t base16 = KIND == 1 ? 0x3f003f00u : 0x38003800u;
    auto h = [&](uint32_t flip) { return ((rnd() & keep16) | base16) ^ flip; };
    auto c = [&](uint32_t flip) { return (int)(((rnd() & 0x8f8f8f8fu) | 0x30303030u) ^ flip); };
    u32x4 a16[4], b16[4];
    gm_i32x8 a8[4], b8[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a16[i] = (u32x4){h(0), h((lane & 1) << 15), h(0), h((uint32_t)i << 31)};
        b16[i] = (u32x4){h((lane & 2) << 14), h(0), h((uint32_t)i << 15), h(0)};
        a8[i] = (gm_i32x8){c(0), c((lane & 1) << 7), c((uint32_t)i << 31), c(0), c(0), c(0), c(0), c(0)};
        b8[i] = (gm_i32x8){c(0), c((lane & 2) << 6), c(0), c(0), c(0), c((uint32_t)i << 15), c(0), c(0)};
    }
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (KIND == 0)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a16[i]), __builtin_bit_cast(f16x8, b16[j]),
                                                                      acc[i][j], 0, 0, 0);
                else if constexpr (KIND == 1)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a16[i]), __builtin_bit_cast(bf16x8, b16[j]),
                                                                       acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8[i], b8[j], acc[i][j], 0, 0, 0, 0, 0, 0);
            }
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) sum += acc[i][j][e];
    out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_mfma_peak_f16(float* out, uint32_t iters, uint32_t seed) {
    mfma_peak_body<0>(out, iters, seed);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_mfma_peak_bf16(float* out, uint32_t iters, uint32_t seed) {
    mfma_peak_body<1>(out, iters, seed);
}
extern "C" __global__ __launch_bounds__(256, 1) void fe_mfma_peak_f8(float* out, uint32_t iters, uint32_t seed) {
    mfma_peak_body<2>(out, iters, seed);
}
