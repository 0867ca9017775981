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
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
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

// A DPP move: every lane reads a lane of its own row of 16, so no lane is out of bounds and bound_ctrl costs nothing; it
// lets the compiler fold the move into the add that consumes it.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, true));
}
#define DPP_QUAD_XOR1 0xB1     // quad_perm [1,0,3,2]: lane ^ 1
#define DPP_QUAD_XOR2 0x4E     // quad_perm [2,3,0,1]: lane ^ 2
#define DPP_QUAD_XOR3 0x1B     // quad_perm [3,2,1,0]: lane ^ 3
#define DPP_HALF_MIRROR 0x141  // lane ^ 7 inside 8 lanes
#define DPP_ROW_MIRROR 0x140   // lane ^ 15 inside 16 lanes

template <int MASK>
__device__ __forceinline__ float dpp_quad_xor(float v) {
    static_assert(MASK == 1 || MASK == 2, "quad permutes cover lane ^ 1 and lane ^ 2");
    return dpp_mov<MASK == 1 ? DPP_QUAD_XOR1 : DPP_QUAD_XOR2>(v);
}

// One butterfly stage across lanes for N values at once: partner + sign * own, sign -1 on the lane whose bit is set.
// Written stage by stage over all the values so that the independent chains interleave.
template <int N>
__device__ __forceinline__ void fwht_lane_stages(float (&x)[N], uint32_t lane) {
    const float s1 = (lane & 1) ? -1.f : 1.f, s2 = (lane & 2) ? -1.f : 1.f, s4 = (lane & 4) ? -1.f : 1.f;
    const float s8 = (lane & 8) ? -1.f : 1.f, s16 = (lane & 16) ? -1.f : 1.f;
    float t[N];
#pragma unroll
    for (int i = 0; i < N; i++) t[i] = x[i] * s1;
#pragma unroll
    for (int i = 0; i < N; i++) x[i] = dpp_mov<DPP_QUAD_XOR1>(x[i]) + t[i];
#pragma unroll
    for (int i = 0; i < N; i++) t[i] = x[i] * s2;
#pragma unroll
    for (int i = 0; i < N; i++) x[i] = dpp_mov<DPP_QUAD_XOR2>(x[i]) + t[i];
    // lane ^ 4 = mirror of 8 (lane ^ 7), then mirror of 4 (lane ^ 3); lane ^ 8 = mirror of 16, then mirror of 8
    float u[N];
#pragma unroll
    for (int i = 0; i < N; i++) t[i] = x[i] * s4, u[i] = dpp_mov<DPP_HALF_MIRROR>(x[i]);
#pragma unroll
    for (int i = 0; i < N; i++) x[i] = dpp_mov<DPP_QUAD_XOR3>(u[i]) + t[i];
#pragma unroll
    for (int i = 0; i < N; i++) t[i] = x[i] * s8, u[i] = dpp_mov<DPP_ROW_MIRROR>(x[i]);
#pragma unroll
    for (int i = 0; i < N; i++) x[i] = dpp_mov<DPP_HALF_MIRROR>(u[i]) + t[i];
    // lane ^ 16 crosses rows of 16: through the LDS crossbar
#pragma unroll
    for (int i = 0; i < N; i++) u[i] = swz_xor<16>(x[i]);
#pragma unroll
    for (int i = 0; i < N; i++) x[i] = __builtin_fmaf(x[i], s16, u[i]);
}

// Unscaled natural-order (Sylvester) Walsh-Hadamard transform of 128 f32 held by 32 consecutive lanes, 4 a lane
// (element 4 * (lane & 31) + q). Both halves of a wavefront transform their own 128 values at once.
__device__ __forceinline__ void fwht128_half_wave(float (&v)[4], uint32_t lane) {
    float a = v[0] + v[1], b = v[0] - v[1], c = v[2] + v[3], d = v[2] - v[3];
    v[0] = a + c;
    v[1] = b + d;
    v[2] = a - c;
    v[3] = b - d;
    fwht_lane_stages(v, lane);
}

// The same for R rows at once (v[r] as above), the rows' chains interleaved.
template <int R>
__device__ __forceinline__ void fwht128_half_wave_rows(float (&v)[R][4], uint32_t lane) {
    float x[4 * R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float a = v[r][0] + v[r][1], b = v[r][0] - v[r][1], c = v[r][2] + v[r][3], d = v[r][2] - v[r][3];
        x[4 * r] = a + c, x[4 * r + 1] = b + d, x[4 * r + 2] = a - c, x[4 * r + 3] = b - d;
    }
    fwht_lane_stages(x, lane);
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int q = 0; q < 4; q++) v[r][q] = x[4 * r + q];
}

// Two elements of SwiGLU on bf16 pairs: bf16(bf16(silu(g)) * u), silu(g) = g / (1 + exp(-g)) in f32
// (kernels/k-core/src/misc.rs:58-71). One definition, so that every kernel that applies it rounds alike.
__device__ __forceinline__ uint32_t silu_mul_bf16x2(uint32_t g, uint32_t u) {
    float v[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        float gv = bf16_bits_to_f32((g >> (16 * i)) & 0xffff), uv = bf16_bits_to_f32((u >> (16 * i)) & 0xffff);
        float s = gv * __builtin_amdgcn_rcpf(1.0f + __expf(-gv));
        v[i] = bf16_bits_to_f32(f32_to_bf16_bits(s)) * uv;
    }
    return pack_bf16x2(v[0], v[1]);
}

// Data that one program leaves for another, possibly on another XCD with its own L2, crosses at agent scope: stores go
// through to memory (the sc1 form that clang emits for agent-scope atomic stores; it has no 16-byte ones), loads read past
// this XCD's L2. agent_stores_wait() returns when the lane's stores are acknowledged. The loads are 8-byte relaxed
// agent-scope atomic loads, which the compiler counts in its own s_waitcnt.
__device__ __forceinline__ void store_agent_f32x4(float* p, f32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_agent_u32x2(void* p, u32x2 v) {
    asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void agent_stores_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ f32x4 load_agent_f32x4(const float* p) {
    const uint64_t a = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t b = __hip_atomic_load((const uint64_t*)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return (f32x4){__uint_as_float((uint32_t)a), __uint_as_float((uint32_t)(a >> 32)), __uint_as_float((uint32_t)b),
                   __uint_as_float((uint32_t)(b >> 32))};
}
// The same 16-byte agent-scope load through a buffer resource (cache policy bit 4 = sc1): an ordinary load to the
// compiler, which schedules many of them together and counts them in its waits. Byte offsets: voff per lane, soff uniform;
// out of the resource's range the load returns zero.
__device__ __forceinline__ f32x4 load_agent_f32x4(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 16));
}
// For code written around explicit waits: nothing to do, the compiler waits for the loads above itself.
template <int N>
__device__ __forceinline__ void agent_loads_wait(f32x4 (&)[N]) {}
