// Device helpers shared by the gfx950 kernels: 16-bit float conversions, wavefront exchanges, the 128-point
// Walsh-Hadamard transform over half a wavefront, and the vector types the MFMA builtins take.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// dword-aligned forms: a lane's run of trellis words starts at any word
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t u32x3_a4 __attribute__((ext_vector_type(3), aligned(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

#define FE_HAD_SCALE 0.08838834764831844f  // 1 / sqrt(128); as f32 bits 0x3db504f3

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// f32 -> bf16 bits, round to nearest even, NaN stays a quiet NaN: the hardware conversion (v_cvt_pk_bf16_f32).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// (lo, hi) f32 -> packed fp16x2, round to nearest even.
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// Value of lane (lane ^ MASK) for MASK < 32, through the LDS crossbar (no memory is touched).
template <int MASK>
__device__ __forceinline__ float swz_xor(float v) {
    // BitMode pattern: offset[15] = 0, and_mask = 0x1f, or_mask = 0, xor_mask = MASK
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (MASK << 10) | 0x1f));
}

template <int MASK>
__device__ __forceinline__ float dpp_quad_xor(float v) {
    static_assert(MASK == 1 || MASK == 2, "quad permutes cover lane ^ 1 and lane ^ 2");
    // quad_perm selectors: [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E
    constexpr int ctrl = MASK == 1 ? 0xB1 : 0x4E;
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xf, 0xf, false));
}

// Unscaled natural-order (Sylvester) Walsh-Hadamard transform of 128 f32 held by 32 consecutive lanes, 4 a lane
// (element 4 * (lane & 31) + q). Both halves of a wavefront transform their own 128 values at once.
__device__ __forceinline__ void fwht128_half_wave(float (&v)[4], uint32_t lane) {
    float a = v[0] + v[1], b = v[0] - v[1], c = v[2] + v[3], d = v[2] - v[3];
    v[0] = a + c;
    v[1] = b + d;
    v[2] = a - c;
    v[3] = b - d;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        float x = v[q], o;
        o = dpp_quad_xor<1>(x);
        x = (lane & 1) ? o - x : x + o;
        o = dpp_quad_xor<2>(x);
        x = (lane & 2) ? o - x : x + o;
        o = swz_xor<4>(x);
        x = (lane & 4) ? o - x : x + o;
        o = swz_xor<8>(x);
        x = (lane & 8) ? o - x : x + o;
        o = swz_xor<16>(x);
        x = (lane & 16) ? o - x : x + o;
        v[q] = x;
    }
}

// 16 bytes at agent scope: partial sums that one program leaves for another, possibly on another XCD with its own L2.
// The store goes through to memory, the load reads past this XCD's L2 (the sc1 forms that clang emits for 4-byte
// agent-scope atomics; it has no 16-byte ones). The compiler does not count these loads: agent_loads_wait must come
// between the last load and the first use of any loaded value.
__device__ __forceinline__ void store_agent_f32x4(float* p, f32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ f32x4 load_agent_f32x4(const float* p) {
    f32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int N>
__device__ __forceinline__ void agent_loads_wait(f32x4 (&t)[N]) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < N; i++) asm volatile("" : "+v"(t[i]));
}
