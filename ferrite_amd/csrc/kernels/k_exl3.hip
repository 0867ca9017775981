// EXL3 (trellis-coded, Hadamard-rotated) linear for gfx950: input rotation, the decode GEMV for 1..64 rows,
// whole-tensor reconstruct, and probes.
//
// The trellis of a 16x16 tile is a cyclic stream of 256 * BITS bits, most significant bit of each u32 first; position t
// owns the 16-bit state ending at stream bit (t + 1) * BITS (crates/fe-exl3/src/cpu.rs:12-23). Position
// t = 8 * f + i sits at row k = 2 (f & 3) + (i & 1) + 8 ((i >> 1) & 1), column n = (f >> 2) + 8 (i >> 2) of the tile
// (crates/fe-exl3/src/format.rs:146-156). A state decodes to fp16 by the mul1 codebook
// (crates/fe-exl3/src/cpu.rs:25-43, kernels/k-exl3/src/util.rs:76-85).
#include <type_traits>

#include "gemm_core.h"

// ---- the mul1 codebook ------------------------------------------------------------------------------------------

// x = state * 0x83DCD12D mod 2^32 for the 16-bit state in the low (HI = 0) or high (HI = 1) half of r; the other half
// of r may hold anything. On gfx950 v_mul_lo_u32 issues at the same rate as the other 3-operand integer instructions,
// while the shift or mask that isolates the state is one of the double-rate simple instructions.
template <int HI>
__device__ __forceinline__ uint32_t mul1_x(uint32_t r) {
    uint32_t s = HI ? (r >> 16) : (r & 0xffffu);
    return s * 0x83DCD12Du;
}

// Two codebook values as packed fp16 (x0's in the low half): 0x6400 + byte sum is fp16(1024 + sum); one fused
// fp16 multiply-add by 0x1eee with 0xc931 added, a single rounding per value.
__device__ __forceinline__ uint32_t mul1_finish2(uint32_t x0, uint32_t x1) {
    uint32_t h = __builtin_amdgcn_sad_u8(x0, 0u, 0x64006400u);
    h = __builtin_amdgcn_sad_hi_u8(x1, 0u, h);
    f16x2 v = __builtin_bit_cast(f16x2, h);
    const f16x2 c1 = __builtin_bit_cast(f16x2, 0x1eee1eeeu);
    const f16x2 c2 = __builtin_bit_cast(f16x2, 0xc931c931u);
    f16x2 o = __builtin_elementwise_fma(v, c1, c2);
    return __builtin_bit_cast(uint32_t, o);
}

__device__ __forceinline__ uint32_t decode2_mul1(uint32_t s0, uint32_t s1) {
    return mul1_finish2(mul1_x<0>(s0), mul1_x<0>(s1));
}

// ---- whole-tensor reconstruct (bits at run time: load-time code) ---------------------------------------------------

// 16-bit state of position p of a tile: two words and a funnel shift (kernels/k-exl3/src/recon.rs:12-22).
__device__ __forceinline__ uint32_t tile_state_rt(const uint32_t* tile, uint32_t bits, uint32_t p) {
    uint32_t words = 8 * bits;
    uint32_t b1 = (p + 1) * bits + 256 * bits;
    uint32_t b0 = b1 - 16;
    uint32_t i0 = b0 / 32, i1 = (b1 - 1) / 32;
    uint32_t s = (i1 + 1) * 32 - b1;
    uint32_t a = tile[i0 % words], b = tile[i1 % words];
    return (uint32_t)((((uint64_t)a << 32) | b) >> s) & 0xffff;
}

// W_hat (rotated basis) of columns nt0 * 16 .. + ns: grid (ns / 128, k / 16), 256 threads; half-wavefront w of the
// block decodes tile (blockIdx.y, nt0 + 8 blockIdx.x + w), lane f of it the 8 values of fragment lane f.
// OUT_F32 = 0: fp16 bits [k][ns]; 1: f32 [k][ns]. (kernels/k-exl3/src/recon.rs:24-51, 131-157)
template <int OUT_F32>
__device__ __forceinline__ void recon_hat_body(void* out, const uint32_t* trellis, uint32_t n_tiles, uint32_t nt0,
                                               uint32_t ns, uint32_t bits) {
    uint32_t hw = threadIdx.x / 32, f = threadIdx.x % 32;
    uint32_t kt = blockIdx.y, ntl = blockIdx.x * 8 + hw;
    const uint32_t* tile = trellis + (size_t)(kt * n_tiles + nt0 + ntl) * 8 * bits;
#pragma unroll
    for (uint32_t j = 0; j < 8; j += 2) {
        uint32_t h = decode2_mul1(tile_state_rt(tile, bits, f * 8 + j), tile_state_rt(tile, bits, f * 8 + j + 1));
#pragma unroll
        for (uint32_t e = 0; e < 2; e++) {
            uint32_t jj = j + e, v = e ? (h >> 16) : (h & 0xffff);
            uint32_t row = 2 * (f & 3) + (jj & 1) + 8 * ((jj >> 1) & 1);
            uint32_t col = (f >> 2) + 8 * (jj >> 2);
            size_t at = (size_t)(kt * 16 + row) * ns + ntl * 16 + col;
            if (OUT_F32)
                ((float*)out)[at] = f16_bits_to_f32(v);
            else
                ((uint16_t*)out)[at] = (uint16_t)v;
        }
    }
}

extern "C" __global__ __launch_bounds__(256) void exl3_recon_hat_f16(uint16_t* out, const uint32_t* trellis,
                                                                     uint32_t n_tiles, uint32_t nt0, uint32_t ns,
                                                                     uint32_t bits) {
    recon_hat_body<0>(out, trellis, n_tiles, nt0, ns, bits);
}

extern "C" __global__ __launch_bounds__(256) void exl3_recon_hat_f32(float* out, const uint32_t* trellis,
                                                                     uint32_t n_tiles, uint32_t nt0, uint32_t ns,
                                                                     uint32_t bits) {
    recon_hat_body<1>(out, trellis, n_tiles, nt0, ns, bits);
}

// In place: H over each row's 128-column blocks, * svh[n0 + col] / sqrt(128). grid (ns / 256, k), 64 threads: each
// half of the wavefront owns one 128-column block (ns / 128 odd: the last block's upper half idles).
// (kernels/k-exl3/src/recon.rs:54-64)
extern "C" __global__ __launch_bounds__(64) void exl3_had_rows(float* buf, uint32_t ns, const uint16_t* svh, uint32_t n0) {
    uint32_t lane = threadIdx.x, l32 = lane & 31;
    uint32_t c = (blockIdx.x * 2 + (lane >> 5)) * 128 + 4 * l32;
    bool live = c < ns;
    float* p = buf + (size_t)blockIdx.y * ns + (live ? c : 0);
    float v[4] = {p[0], p[1], p[2], p[3]};
    fwht128_half_wave(v, l32);
    if (live) {
#pragma unroll
        for (int q = 0; q < 4; q++) p[q] = v[q] * FE_HAD_SCALE * f16_bits_to_f32(svh[n0 + c + q]);
    }
}

// H over k (128-row blocks) * suh / sqrt(128) -> bf16, [k][n] (nk = 0, ld = n) or [n][k] (nk = 1, ld = k).
// grid (ns / 32, k / 128), 128 threads, a 128 x 32 f32 tile in LDS. (kernels/k-exl3/src/recon.rs:66-128)
extern "C" __global__ __launch_bounds__(128) void exl3_had_cols_bf16(const float* buf, uint16_t* out, uint32_t ns,
                                                                      const uint16_t* suh, uint32_t n0, uint32_t ld,
                                                                      uint32_t nk) {
    constexpr uint32_t PITCH = 33;
    __shared__ float sm[128 * PITCH];
    uint32_t hw = threadIdx.x / 32, l32 = threadIdx.x % 32;
    uint32_t r0 = blockIdx.y * 128, c0 = blockIdx.x * 32;
    for (uint32_t i = 0; i < 32; i++) {
        uint32_t r = hw * 32 + i;
        sm[r * PITCH + l32] = buf[(size_t)(r0 + r) * ns + c0 + l32];
    }
    __syncthreads();
    for (uint32_t cc = 0; cc < 8; cc++) {
        uint32_t c = hw * 8 + cc;
        float v[4];
#pragma unroll
        for (uint32_t q = 0; q < 4; q++) v[q] = sm[(4 * l32 + q) * PITCH + c];
        fwht128_half_wave(v, l32);
#pragma unroll
        for (uint32_t q = 0; q < 4; q++) {
            uint32_t r = 4 * l32 + q;
            sm[r * PITCH + c] = v[q] * FE_HAD_SCALE * f16_bits_to_f32(suh[r0 + r]);
        }
    }
    __syncthreads();
    if (nk) {
        for (uint32_t cc = 0; cc < 8; cc++) {
            uint32_t c = hw * 8 + cc;
            float v[4];
#pragma unroll
            for (uint32_t q = 0; q < 4; q++) v[q] = sm[(4 * l32 + q) * PITCH + c];
            uint32_t* p = (uint32_t*)(out + (size_t)(n0 + c0 + c) * ld + r0 + 4 * l32);
            p[0] = pack_bf16x2(v[0], v[1]);
            p[1] = pack_bf16x2(v[2], v[3]);
        }
    } else {
        for (uint32_t i = 0; i < 32; i++) {
            uint32_t r = hw * 32 + i;
            out[(size_t)(r0 + r) * ld + n0 + c0 + l32] = (uint16_t)f32_to_bf16_bits(sm[r * PITCH + l32]);
        }
    }
}

// ---- input rotation ------------------------------------------------------------------------------------------------

// One 128-element block of a row: fp16(H(x * suh) / sqrt(128)), 4 elements a lane of a half wavefront. The input is
// bf16 (mode 0) or f32 (mode 1) rows, or (mode 2) SwiGLU of two bf16 arrays, x = gate and x2 = up, taken on the way in:
// bf16(bf16(silu(gate)) * up), the bits fe_silu_mul would have left in memory. `xat` indexes the input (row * ld + c),
// `c` is the block's channel of this lane. Split in two so that a caller can issue the loads early; all 32 lanes of the
// half wavefront take part in rot_finish.
struct RotSrc {
    const void *x, *x2;
    uint32_t mode, ld;  // ld: elements between input rows
};
struct RotRaw {
    f32x4 xf;
    u32x2 xb, ub, s;
};
__device__ __forceinline__ RotRaw rot_load(const RotSrc& src, const uint16_t* suh, size_t xat, uint32_t c) {
    RotRaw r;
    if (src.mode == 1) {
        r.xf = *(const f32x4*)((const float*)src.x + xat);
    } else {
        r.xb = *(const u32x2*)((const uint16_t*)src.x + xat);
        if (src.mode == 2) r.ub = *(const u32x2*)((const uint16_t*)src.x2 + xat);
    }
    r.s = *(const u32x2*)(suh + c);
    return r;
}
// The same for mode 2 when gate and up were written by other programs of this launch, possibly on another XCD: the
// loads are agent-scope buffer loads (gs, us: resources over the two arrays), which miss this XCD's L2.
__device__ __forceinline__ RotRaw rot_load_agent(__amdgpu_buffer_rsrc_t gs, __amdgpu_buffer_rsrc_t us, const uint16_t* suh,
                                                 uint32_t xat, uint32_t c) {
    RotRaw r;
    r.xb = __builtin_amdgcn_raw_buffer_load_b64(gs, 2 * xat, 0, 16);
    r.ub = __builtin_amdgcn_raw_buffer_load_b64(us, 2 * xat, 0, 16);
    r.s = *(const u32x2*)(suh + c);
    return r;
}
__device__ __forceinline__ u32x2 rot_finish(const RotRaw& r, uint32_t mode, uint32_t l32) {
    float v[4];
    if (mode == 1) {
        v[0] = r.xf[0], v[1] = r.xf[1], v[2] = r.xf[2], v[3] = r.xf[3];
    } else {
        u32x2 xb = r.xb;
        if (mode == 2) xb = (u32x2){silu_mul_bf16x2(r.xb[0], r.ub[0]), silu_mul_bf16x2(r.xb[1], r.ub[1])};
        v[0] = __uint_as_float(xb[0] << 16), v[1] = __uint_as_float(xb[0] & 0xffff0000u);
        v[2] = __uint_as_float(xb[1] << 16), v[3] = __uint_as_float(xb[1] & 0xffff0000u);
    }
    v[0] *= f16_bits_to_f32(r.s[0] & 0xffff), v[1] *= f16_bits_to_f32(r.s[0] >> 16);
    v[2] *= f16_bits_to_f32(r.s[1] & 0xffff), v[3] *= f16_bits_to_f32(r.s[1] >> 16);
    fwht128_half_wave(v, l32);
    return (u32x2){pack_f16x2(v[0] * FE_HAD_SCALE, v[1] * FE_HAD_SCALE), pack_f16x2(v[2] * FE_HAD_SCALE, v[3] * FE_HAD_SCALE)};
}

// xh[row][k] = fp16(H(x * suh) / sqrt(128)). grid (ceil(k / 512), rows), 128 threads: each half wavefront one
// 128-element block, 4 elements a lane. (kernels/k-exl3/src/gemv.rs:147-170)
__device__ __forceinline__ void rot_in_body(const RotSrc& src, const uint16_t* suh, uint16_t* xh, uint32_t k) {
    uint32_t l32 = threadIdx.x & 31;
    uint32_t blk = blockIdx.x * 4 + threadIdx.x / 32;
    bool live = blk * 128 < k;
    uint32_t c = (live ? blk : 0) * 128 + 4 * l32;
    u32x2 o = rot_finish(rot_load(src, suh, (size_t)blockIdx.y * src.ld + c, c), src.mode, l32);
    if (live) *(u32x2*)(xh + (size_t)blockIdx.y * k + c) = o;
}
extern "C" __global__ __launch_bounds__(128) void exl3_rot_in(const void* x, uint32_t x_mode, const uint16_t* suh,
                                                               uint16_t* xh, uint32_t k, const void* x2, uint32_t ldx) {
    rot_in_body(RotSrc{x, x2, x_mode, ldx}, suh, xh, k);
}

#define FE_EXL3_GROUP_MAX 4  // linears of one launch

// The same input rotated for several linears (each by its own suh into its own xh): grid (ceil(k / 512), rows, members).
struct RotGroup {
    const uint16_t* suh[FE_EXL3_GROUP_MAX];
    uint16_t* xh[FE_EXL3_GROUP_MAX];
};
extern "C" __global__ __launch_bounds__(128) void exl3_rot_in_group(RotGroup g, const void* x, uint32_t x_mode, uint32_t k) {
    rot_in_body(RotSrc{x, nullptr, x_mode, k}, g.suh[blockIdx.z], g.xh[blockIdx.z], k);
}

// ---- decode GEMV: the lane mapping and the decode ----------------------------------------------------------------------
//
// A program works on one 128-column block at a time; 256 threads = 4 wavefronts, wavefront w owning tiles 2w, 2w + 1 of
// the block's 8. A wavefront's load step covers 4 consecutive k steps of its two tiles: lane L = 16 g + r reads k step g,
// tile r >> 3, the BITS words of fragment lanes 4q .. 4q + 3 (q = r & 7) plus the word before them, which is all its 32
// states need. Those states are rows n = q and n = q + 8 of the tile over all 16 k, so after decoding the lane holds, for
// each of the two, the 16 values as two 8-value MFMA operands (k 0..7 and k 8..15) in k order. v_mfma_f32_16x16x32_f16
// then sums over the 4 k steps: A = decoded weights (row r), B = 16 rotated input rows (column = input row), and the
// accumulator of lane L holds output column 4 (L >> 4) + i of the 16 rows-of-A, input row L & 15.

template <int BITS>
struct LaneWords {
    uint32_t w[BITS + 1];  // w[0] = the word before the lane's run
};

template <int BITS>
__device__ __forceinline__ LaneWords<BITS> load_lane_words(const uint32_t* run, const uint32_t* prev) {
    LaneWords<BITS> r;
    r.w[0] = __builtin_nontemporal_load(prev);
    if constexpr (BITS == 1) {
        r.w[1] = __builtin_nontemporal_load(run);
    } else if constexpr (BITS == 2) {
        u32x2_a4 t = __builtin_nontemporal_load((const u32x2_a4*)run);
        r.w[1] = t[0], r.w[2] = t[1];
    } else if constexpr (BITS == 3) {
        u32x3_a4 t = __builtin_nontemporal_load((const u32x3_a4*)run);
        r.w[1] = t[0], r.w[2] = t[1], r.w[3] = t[2];
    } else {
        u32x4_a4 t = __builtin_nontemporal_load((const u32x4_a4*)run);
        r.w[1] = t[0], r.w[2] = t[1], r.w[3] = t[2], r.w[4] = t[3];
        if constexpr (BITS == 5) {
            r.w[5] = __builtin_nontemporal_load(run + 4);
        } else if constexpr (BITS == 6) {
            u32x2_a4 u = __builtin_nontemporal_load((const u32x2_a4*)(run + 4));
            r.w[5] = u[0], r.w[6] = u[1];
        } else if constexpr (BITS == 7) {
            u32x3_a4 u = __builtin_nontemporal_load((const u32x3_a4*)(run + 4));
            r.w[5] = u[0], r.w[6] = u[1], r.w[7] = u[2];
        } else if constexpr (BITS == 8) {
            u32x4_a4 u = __builtin_nontemporal_load((const u32x4_a4*)(run + 4));
            r.w[5] = u[0], r.w[6] = u[1], r.w[7] = u[2], r.w[8] = u[3];
        }
    }
    return r;
}

// The lane's local stream: bit 0 = most significant bit of w[0]; local position U (0..31) owns the 16 bits ending at local
// bit (U + 1) * BITS + 32. A state either lies inside one word (one extract), or straddles the boundary between w[i - 1]
// and w[i]: all states that straddle one boundary are cut out of one 32-bit window over it (low half of w[i - 1], high
// half of w[i]): BITS funnel shifts a load step instead of one per state or per pair of states.
template <int BITS>
struct LaneWindows {
    uint32_t b[BITS + 1];  // b[i], i >= 1: the window over the boundary in front of w[i]
};
template <int BITS>
__device__ __forceinline__ LaneWindows<BITS> lane_windows(const LaneWords<BITS>& lw) {
    LaneWindows<BITS> win;
    win.b[0] = 0;
#pragma unroll
    for (int i = 1; i <= BITS; i++) {
        uint32_t r = __builtin_amdgcn_alignbit(lw.w[i - 1], lw.w[i], 16);
        // opaque to the optimizer, which would otherwise fold window and extract into a funnel shift and a mask per state
        asm("" : "+v"(r));
        win.b[i] = r;
    }
    return win;
}

// x = state * MUL1 of local position U.
template <int BITS, int U>
__device__ __forceinline__ uint32_t lane_x(const LaneWords<BITS>& lw, const LaneWindows<BITS>& win) {
    constexpr int end = (U + 1) * BITS + 32, wi = end / 32, r = end % 32;
    uint32_t state;
    if constexpr (r == 0)
        state = lw.w[wi - 1] & 0xffffu;
    else if constexpr (r == 16)
        state = lw.w[wi] >> 16;
    else if constexpr (r > 16)
        state = __builtin_amdgcn_ubfe(lw.w[wi], 32 - r, 16);
    else
        state = __builtin_amdgcn_ubfe(win.b[wi], 16 - r, 16);
    return state * 0x83DCD12Du;
}

// The lane's 32 values as MFMA operands op[h][kh]: rows n = q + 8 h of the tile, k = 8 kh .. 8 kh + 7 in order.
// Local position u = 8 c + i (fragment lane 4q + c, value i) is k = 2c + (i & 1) + 8 ((i >> 1) & 1), n half i >> 2.
template <int BITS>
__device__ __forceinline__ void decode_lane(const LaneWords<BITS>& lw, f16x8 (&op)[2][2]) {
    const LaneWindows<BITS> win = lane_windows<BITS>(lw);
#define FE_PAIR(H, KH, C) mul1_finish2(lane_x<BITS, 8 * (C) + 2 * (KH) + 4 * (H)>(lw, win), lane_x<BITS, 8 * (C) + 2 * (KH) + 4 * (H) + 1>(lw, win))
#define FE_OP(H, KH)                                                                             \
    {                                                                                            \
        u32x4 t = {FE_PAIR(H, KH, 0), FE_PAIR(H, KH, 1), FE_PAIR(H, KH, 2), FE_PAIR(H, KH, 3)};  \
        op[H][KH] = __builtin_bit_cast(f16x8, t);                                                \
    }
    FE_OP(0, 0) FE_OP(0, 1) FE_OP(1, 0) FE_OP(1, 1)
#undef FE_OP
#undef FE_PAIR
}

// Row half H of the same: op[kh] = decode_lane's op[H][kh], with only the windows and extracts those 16 values need.
template <int BITS>
__device__ __forceinline__ void decode_lane_half(const LaneWords<BITS>& lw, int h, f16x8 (&op)[2]) {
    const LaneWindows<BITS> win = lane_windows<BITS>(lw);
#define FE_PAIR(H, KH, C) mul1_finish2(lane_x<BITS, 8 * (C) + 2 * (KH) + 4 * (H)>(lw, win), lane_x<BITS, 8 * (C) + 2 * (KH) + 4 * (H) + 1>(lw, win))
#define FE_OP(H, KH)                                                                             \
    {                                                                                            \
        u32x4 t = {FE_PAIR(H, KH, 0), FE_PAIR(H, KH, 1), FE_PAIR(H, KH, 2), FE_PAIR(H, KH, 3)};  \
        op[KH] = __builtin_bit_cast(f16x8, t);                                                   \
    }
    if (h == 0) {
        FE_OP(0, 0) FE_OP(0, 1)
    } else {
        FE_OP(1, 0) FE_OP(1, 1)
    }
#undef FE_OP
#undef FE_PAIR
}

// Store 4 consecutive outputs. mode: 0 bf16, 1 f32, 2 bf16 y += v (f32 add, one rounding), 3 f32 y += v.
// (kernels/k-exl3/src/gemv.rs:122-145)
__device__ __forceinline__ void store4(void* y, uint32_t mode, size_t i, float (&v)[4]) {
    if (mode & 1) {
        float* p = (float*)y + i;
        f32x4 o = {v[0], v[1], v[2], v[3]};
        if (mode & 2) o += *(const f32x4*)p;
        *(f32x4*)p = o;
    } else {
        uint32_t* p = (uint32_t*)((uint16_t*)y + i);
        if (mode & 2) {
            uint32_t a = p[0], b = p[1];
            v[0] += __uint_as_float(a << 16), v[1] += __uint_as_float(a & 0xffff0000u);
            v[2] += __uint_as_float(b << 16), v[3] += __uint_as_float(b & 0xffff0000u);
        }
        u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *(u32x2*)p = o;
    }
}

// H over the 128 sums of a row (4 a lane of a half wavefront), * svh / sqrt(128), stored. (gemv.rs:172-180)
__device__ __forceinline__ void finish_row(float (&v)[4], uint32_t l32, const uint16_t* svh, uint32_t col, void* y,
                                           uint32_t mode, size_t at) {
    fwht128_half_wave(v, l32);
    u32x2 s = *(const u32x2*)(svh + col);
    v[0] = v[0] * FE_HAD_SCALE * f16_bits_to_f32(s[0] & 0xffff);
    v[1] = v[1] * FE_HAD_SCALE * f16_bits_to_f32(s[0] >> 16);
    v[2] = v[2] * FE_HAD_SCALE * f16_bits_to_f32(s[1] & 0xffff);
    v[3] = v[3] * FE_HAD_SCALE * f16_bits_to_f32(s[1] >> 16);
    store4(y, mode, at, v);
}

// The lane's four output scales as finish_row applies them, for callers that finish many rows of the same columns.
__device__ __forceinline__ f32x4 row_scales(const uint16_t* svh, uint32_t col) {
    u32x2 s = *(const u32x2*)(svh + col);
    return (f32x4){f16_bits_to_f32(s[0] & 0xffff), f16_bits_to_f32(s[0] >> 16), f16_bits_to_f32(s[1] & 0xffff),
                   f16_bits_to_f32(s[1] >> 16)};
}
#ifndef FE_STAGE_NB1
#define FE_STAGE_NB1 4
#endif
#define GEMV_RED_PITCH 132  // floats a row of the 128-column partial sums (16-byte aligned, banks spread)

// ---- decode GEMV, balanced over the CUs (1..64 rows) ------------------------------------------------------------------
//
// Work unit = one 128-channel block of K of one 128-column block of N (two load steps); units are ordered column block
// by column block and the member's `programs` programs each take one contiguous run of them, base + 1 units for the first
// rem programs and base for the rest, whatever the shape: with a multiple of the CU count of programs, which the CUs take
// round by round, the CUs' shares differ by at most one unit. (Spreading the longer runs evenly over the program numbers
// is worse: their period can divide the CU count, and then a CU gets only long runs or only short ones.) A run may start and end inside a column block, so a block's sum is assembled from segments: each program
// leaves the partial sums of its segment of block nb in z[program + nb] and bumps the block's arrival counter; the
// program that arrives last adds the segments in program order (the order does not depend on who is last: deterministic),
// applies the output rotation and re-arms the counter. The partition depends on (k, n, programs) only, never on the
// row count: row r of a batch has the bits of the single-row call. Inside a program: 4 wavefronts owning 2 of the
// block's 8 tiles each, the rotated inputs of the run staged in LDS (rotated here when src.x is set), four load steps in
// flight per lane. Several linears of one input share a launch: each member's programs are exactly those of its own
// launch (same runs, same sums, same bits). (kernels/k-exl3/src/gemv.rs:412-587 is the reference's split-K form.)
struct GemvMember {
    const uint32_t* trellis;
    const uint16_t *svh, *suh;
    uint16_t* xh;        // rotated inputs [m][k]: read, or (rotating here) left there by the programs of column block 0
    void* y;
    float* z;            // segment partial sums [programs + n / 128][m][128]
    uint32_t* counters;  // arrivals per column block, zero at rest
    uint32_t n, programs, stride_k, stride_nb;
    uint32_t base, rem;            // units / programs, units % programs, units = (n / 128) * (k / 128)
    uint32_t inv_base, inv_base1;  // floor((2^32 - 1) / base), floor((2^32 - 1) / (base + 1))
};
struct GemvJob {
    uint32_t count, first[FE_EXL3_GROUP_MAX + 1];  // member i owns workgroups first[i] .. first[i + 1] - 1 of the grid
    GemvMember m[FE_EXL3_GROUP_MAX];
};

// x / d for x < 2^31 with inv = floor((2^32 - 1) / d): a multiply-high and one correction (uniform operands: scalar code).
__device__ __forceinline__ uint32_t udiv_inv(uint32_t x, uint32_t d, uint32_t inv) {
    uint32_t q = __umulhi(x, inv);
    return q + ((q + 1) * d <= x ? 1u : 0u);
}

// The ring of load steps turned left by `phase` slots (phase < DEPTH), so that the oldest step in flight sits in slot 0
// again: one pass of moves whatever the phase.
template <int BITS, int DEPTH>
__device__ __forceinline__ void ring_turn(LaneWords<BITS> (&ring)[DEPTH], uint32_t phase) {
    static_assert(DEPTH == 4, "the turns below are written out for four slots");
    if (phase == 1) {
        LaneWords<BITS> t = ring[0];
        ring[0] = ring[1], ring[1] = ring[2], ring[2] = ring[3], ring[3] = t;
    } else if (phase == 2) {
        LaneWords<BITS> t0 = ring[0], t1 = ring[1];
        ring[0] = ring[2], ring[1] = ring[3], ring[2] = t0, ring[3] = t1;
    } else if (phase == 3) {
        LaneWords<BITS> t = ring[3];
        ring[3] = ring[2], ring[2] = ring[1], ring[1] = ring[0], ring[0] = t;
    }
}

// The word before a lane's run is the last word of the run of lane q - 1 of the same tile (q = lane & 7; for q = 0 the
// tile's last word, lane q = 7): a move across lanes instead of a second load per step. The 16 lanes of a DPP row are the
// two tiles of one k step, so lane i takes lane i - 1 (row_shr:1) or, at q = 0, lane i + 7 (row_ror:9).
__device__ __forceinline__ uint32_t lane_prev_word(uint32_t last) {
    const uint32_t shr = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)last, 0x111, 0xf, 0xf, false);
    const uint32_t ror = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)last, 0x129, 0xf, 0xf, false);
    return (threadIdx.x & 7) ? shr : ror;
}

// A lane's words of one load step through a buffer resource over the whole trellis: the lane's byte offsets (run, word
// before the run) are loop constants in vector registers and the step's position is a scalar offset, so walking the run
// costs no vector instructions; reads past the end of the trellis return zero instead of faulting. Streaming (nt) loads.
template <int BITS>
__device__ __forceinline__ LaneWords<BITS> load_lane_words_buf(__amdgpu_buffer_rsrc_t rs, uint32_t run_b, uint32_t prev_b,
                                                               uint32_t soff) {
    constexpr int NT = 2;
    LaneWords<BITS> r;
    (void)prev_b;
    r.w[0] = 0;  // the word before the run comes from the neighbouring lane when the step is decoded (lane_prev_word)
    if constexpr (BITS == 1) {
        r.w[1] = __builtin_amdgcn_raw_buffer_load_b32(rs, run_b, soff, NT);
    } else if constexpr (BITS == 2) {
        u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(rs, run_b, soff, NT);
        r.w[1] = t[0], r.w[2] = t[1];
    } else if constexpr (BITS == 3) {
        u32x3 t = __builtin_amdgcn_raw_buffer_load_b96(rs, run_b, soff, NT);
        r.w[1] = t[0], r.w[2] = t[1], r.w[3] = t[2];
    } else {
        u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(rs, run_b, soff, NT);
        r.w[1] = t[0], r.w[2] = t[1], r.w[3] = t[2], r.w[4] = t[3];
        if constexpr (BITS == 5) {
            r.w[5] = __builtin_amdgcn_raw_buffer_load_b32(rs, run_b + 16, soff, NT);
        } else if constexpr (BITS == 6) {
            u32x2 u = __builtin_amdgcn_raw_buffer_load_b64(rs, run_b + 16, soff, NT);
            r.w[5] = u[0], r.w[6] = u[1];
        } else if constexpr (BITS == 7) {
            u32x3 u = __builtin_amdgcn_raw_buffer_load_b96(rs, run_b + 16, soff, NT);
            r.w[5] = u[0], r.w[6] = u[1], r.w[7] = u[2];
        } else if constexpr (BITS == 8) {
            u32x4 u = __builtin_amdgcn_raw_buffer_load_b128(rs, run_b + 16, soff, NT);
            r.w[5] = u[0], r.w[6] = u[1], r.w[7] = u[2], r.w[8] = u[3];
        }
    }
    return r;
}


// Timeline of the decode GEMV (a build with -DFE_GEMV_STAMPS, never the shipped one): wavefront w of workgroup g leaves
// the 100 MHz wall clock at up to twelve points of its life at stamps[(4 g + w) * 12 + slot], u64, where stamps lies
// 128 KB into the rotated-input area of the launch's first member (single-row launches on a workspace of 64 rows).
#ifdef FE_GEMV_STAMPS
#define FE_STAMP(slot)                                                                                  \
    do {                                                                                                \
        if (stamp_at && (threadIdx.x & 63) == 0) stamp_at[slot] = __builtin_amdgcn_s_memrealtime();     \
    } while (0)
#else
#define FE_STAMP(slot) \
    do {               \
    } while (0)
#endif

// The decode MLP in one launch (exl3_mlp_b*): the front stage's programs (gate and up, CHAIN = 1) write their outputs
// through to memory and publish every finished column block; the programs of the down stage (CHAIN = 2), which follow
// them in the grid, request their first weights, wait for the blocks their channels need and rotate SwiGLU(gate, up)
// straight from the front stage's outputs. Workgroups are dispatched in grid order, so a waiting program only ever waits
// for programs that are already resident or done; the wait is bounded all the same (spin_limit polls, then the error
// word is set and the program goes on with what it finds, so every launch ends). state: [0] sequence number of the
// last completed launch, [1] error word, [2] finished column blocks of the down stage,
// [(1 + i * nbf + b) * FE_CHAIN_STRIDE] the ready word of front member i's block b = the sequence number of the launch
// that finished it. The down stage's last finisher advances [0]; nothing is cleared between launches, so a captured
// launch replays. Polls are trips to memory: with the ready words packed into a few cache lines the watchers crowd
// one memory channel and slow the front stage's own hand-offs down (56.5 us for the 27B-shaped MLP at 4 bits against
// 46.5 us with a word per 256 bytes and 50.9 us for the two launches), and polling more often than every half
// microsecond costs more than it finds out.
#ifndef FE_CHAIN_STRIDE
#define FE_CHAIN_STRIDE 64  // u32 words from one ready word to the next
#endif
#ifndef FE_CHAIN_SLEEP
#define FE_CHAIN_SLEEP 16  // s_sleep units (64 cycles each) between two polls of a waiting program
#endif
struct ChainCtx {
    uint32_t* state;
    uint32_t* ready;  // front stage: this member's ready words; down stage: those of front members 0 (gate) and 1 (up)
    uint32_t nbf;     // column blocks of a front member = 128-channel blocks of the down stage's input
    uint32_t nb_down, spin_limit;
};
__device__ __forceinline__ uint32_t load_agent_u32(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// FENCED: the hand-off written with the memory model's own means (plain stores, a release fence at agent scope, the
// arrival, an acquire fence, plain loads) instead of write-through stores and loads that pass the L2: the slow form
// (the release writes the whole L2 back), kept as a cross-check of the fast one (option "handoff_fenced").
template <int BITS, int RG, int CHAIN = 0, bool FENCED = false>
__device__ __forceinline__ void gemvb_body(const GemvMember& mb, uint32_t p0, uint32_t np, uint32_t k, uint32_t m, uint32_t y_mode,
                                           uint32_t chunk, uint32_t inv_spb, const RotSrc src, uint16_t* stamp_base,
                                           const ChainCtx ch = ChainCtx{}) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ uint32_t last_flag;
    uint32_t chain_target = 0;  // this launch's sequence number
    if constexpr (CHAIN != 0) chain_target = load_agent_u32(ch.state) + 1;
#ifdef FE_GEMV_STAMPS
    unsigned long long* stamp_at =
        stamp_base && m == 1 ? (unsigned long long*)(stamp_base + 65536) + (size_t)(blockIdx.x * 4 + (threadIdx.x >> 6)) * 12 : nullptr;
    FE_STAMP(0);
#else
    (void)stamp_base;
#endif
    constexpr uint32_t tw = 8 * BITS;
    constexpr int DEPTH = 4;  // load steps in flight per lane (5 and 6 measured 2..5 % slower, 8 10 %: 22.9 against 20.7 us)
    constexpr int GROUP = 8;  // steps of straight-line code per loop iteration (a multiple of DEPTH)
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t r = lane & 15, g = lane >> 4, q = r & 7, tau = r >> 3;
    const uint32_t n = mb.n, spb = k / 64, upb = spb / 2;  // load steps, units a column block
    const uint32_t base = mb.base, rem = mb.rem;
    // This workgroup runs the programs p0 .. p0 + np - 1 of the partition one after the other. Their runs are contiguous, so
    // to the loads and the staging they are one run; where one program's run ends its sums are flushed as that program's
    // (its own slot in z, its own arrival), exactly as if it had been launched on its own: the same sums in the same
    // order, without a second start-up.
    auto run_start = [&](uint32_t q) { return q * base + (q < rem ? q : rem); };
    const uint32_t u0 = run_start(p0);
    const uint32_t S = 2 * (run_start(p0 + np) - u0);  // load steps of this workgroup's run
    if (S == 0) return;
    uint32_t pl = p0, lend = 2 * (run_start(p0 + 1) - u0);  // the program at work and the load step at which its run ends
    uint32_t nb = udiv_inv(2 * u0, spb, inv_spb), st = 2 * u0 - nb * spb;  // where the run stands: column block, load step
    const uint32_t nb_run0 = nb, st_run0 = st;

    // [min(m, 32)][GEMV_RED_PITCH] sums of a finished segment: more than 32 rows pass through it in two halves, so that the
    // programs of 33..64 rows still fit three to a CU
    float* red = (float*)lds;
    const uint32_t red_rows = RG > 2 ? 32 : m;
    unsigned char* xs = (unsigned char*)(red + red_rows * GEMV_RED_PITCH);  // [m][xpitch] rotated inputs of a chunk of the run
    const uint32_t xpitch = chunk * 128 + 16;

    const uint32_t lane_word = g * mb.stride_k + (2 * wave + tau) * tw;
    const uint32_t run_b = 4 * (lane_word + q * BITS), prev_b = 4 * (lane_word + (q * BITS + tw - 1) % tw);
    const uint32_t step_bytes = 16 * mb.stride_k;                     // 4 k steps
    const uint32_t wrap_bytes = 4 * mb.stride_nb - spb * step_bytes;  // from the end of a column block to the next (mod 2^32)
    const __amdgpu_buffer_rsrc_t trs =
        __builtin_amdgcn_make_buffer_rsrc((void*)mb.trellis, 0, (k / 16) * (n / 16) * tw * 4, 0x00020000);
    uint32_t snext = nb * mb.stride_nb * 4 + st * step_bytes;  // byte offset of the next load step to request

    uint32_t xrow[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        uint32_t row = 16 * rg + r;
        xrow[rg] = (row < m ? row : m - 1) * xpitch + g * 32;
    }
    f32x4 acc[RG][2];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) acc[rg][0] = acc[rg][1] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const uint32_t hw = tid >> 5, l32 = tid & 31;
    // Rotating here: (row, 128-channel block) pairs of a chunk go to the half wavefronts: half wavefront hw takes blocks hw,
    // hw + 8, ... of every row. The first pair's loads go out ahead of the trellis loads (loads return in order), so
    // that the rotation runs while the first trellis words are still on their way.
    const bool rotating = src.x != nullptr;
    struct RotAt {
        size_t at, xat;
        uint32_t c, off;
        bool keep;
    };
    auto rot_at = [&](uint32_t c0, uint32_t row, uint32_t b) {
        RotAt a;
        uint32_t gst = st_run0 + c0 + 2 * b, blk = 0;  // load step counted from the start of the run's first column block
        if (gst >= spb) gst -= spb, blk = 1;
        if (gst >= spb) blk += gst / spb, gst %= spb;
        a.c = gst * 64 + 4 * l32;
        a.at = (size_t)row * k + a.c;
        a.xat = (size_t)row * src.ld + a.c;
        a.off = row * xpitch + b * 256 + 8 * l32;
        a.keep = nb_run0 + blk == 0;  // column block 0 sees every channel: its programs leave xh behind
        return a;
    };
    RotRaw rot_raw = {};
    // (resources over gate and up for the down stage's agent-scope loads; unused otherwise)
    const __amdgpu_buffer_rsrc_t chain_gs = __builtin_amdgcn_make_buffer_rsrc((void*)src.x, 0, m * src.ld * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t chain_us = __builtin_amdgcn_make_buffer_rsrc((void*)src.x2, 0, m * src.ld * 2, 0x00020000);
    auto load_pair = [&](const RotAt& a) {
        if constexpr (CHAIN == 2)
            return rot_load_agent(chain_gs, chain_us, mb.suh, (uint32_t)a.xat, a.c);
        else
            return rot_load(src, mb.suh, a.xat, a.c);
    };
    const uint32_t rot_mode = CHAIN == 2 ? 2u : src.mode;
    if (rotating && CHAIN != 2) {
        const uint32_t nblk = (S < chunk ? S : chunk) / 2;
        if (hw < nblk) {
            RotAt a = rot_at(0, 0, hw);
            rot_raw = load_pair(a);
        }
    }
    // the output scales of this lane's four columns of the block the run stands in (for the program that finishes it)
    u32x2 sv = *(const u32x2*)(mb.svh + nb * 128 + 4 * l32);

    // refill cursor: the next load step to request
    uint32_t rj = 0, rst = st;
    auto issue = [&](LaneWords<BITS>& slot) {
        slot = load_lane_words_buf<BITS>(trs, run_b, prev_b, snext);
        if (rj + 1 < S) {  // past the end of the run the last step is requested again (and never used)
            rj++;
            snext += step_bytes;
            if (++rst == spb) rst = 0, snext += wrap_bytes;
        }
    };
    LaneWords<BITS> ring[DEPTH];  // indexed by constants only, so it stays in registers
#pragma unroll
    for (int j = 0; j < DEPTH; j++) issue(ring[j]);
    FE_STAMP(1);
    if constexpr (CHAIN == 2) {
        // Unit j of the run reads channels block (st_run0 / 2 + j) % upb of the input: lanes 0..31 of the workgroup's first
        // wavefront watch gate's ready words of the run's units, lanes 32..63 up's (the host keeps a run within 32 units);
        // the other wavefronts wait at the barrier, which costs no issue slots. A poll is a trip to memory; between polls
        // the wavefront sleeps, so that the watchers do not crowd the memory channel that holds the words.
        uint32_t chain_spins = 0;
        if (wave == 0) {
            const uint32_t units = S / 2, j = lane & 31;
            uint32_t kb = st_run0 / 2 + j;
            kb -= kb >= upb ? upb : 0;
            kb = kb >= upb ? kb % upb : kb;
            const uint32_t* rw = ch.ready + ((lane >> 5) * ch.nbf + kb) * FE_CHAIN_STRIDE;
            bool pending = true;
            for (uint32_t spins = 0; spins < ch.spin_limit; spins++, chain_spins++) {
                const uint32_t v = j < units ? load_agent_u32(rw) : chain_target;
                pending = __builtin_amdgcn_ballot_w64(v != chain_target) != 0;
                if (!pending) break;
                __builtin_amdgcn_s_sleep(FE_CHAIN_SLEEP);
            }
            if (pending && lane == 0) __hip_atomic_fetch_or(ch.state + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        FE_STAMP(9);
#ifdef FE_GEMV_STAMPS
        if (stamp_at && lane == 0) stamp_at[10] = chain_spins;
#endif
    }

    auto one = [&](LaneWords<BITS>& slot, uint32_t t) {  // t: load step within the staged chunk
        f16x8 op[2][2];
        slot.w[0] = lane_prev_word(slot.w[BITS]);
        decode_lane<BITS>(slot, op);
        issue(slot);
        // keep the refill where it is issued: left alone, the scheduler sinks the loads to the end of the group, right in
        // front of the wait for them
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const unsigned char* xp = xs + xrow[rg] + t * 128;
            f16x8 x0 = *(const f16x8*)xp, x1 = *(const f16x8*)(xp + 16);
            acc[rg][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[0][0], x0, acc[rg][0], 0, 0, 0);
            acc[rg][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[1][0], x0, acc[rg][1], 0, 0, 0);
            acc[rg][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[0][1], x1, acc[rg][0], 0, 0, 0);
            acc[rg][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[1][1], x1, acc[rg][1], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // H over the 128 sums of a row (4 a lane of a half wavefront), * svh / sqrt(128) with the prefetched scales, stored.
    auto finish = [&](float (&v)[4], uint32_t col0, uint32_t row) {
        fwht128_half_wave(v, l32);
        v[0] = v[0] * FE_HAD_SCALE * f16_bits_to_f32(sv[0] & 0xffff);
        v[1] = v[1] * FE_HAD_SCALE * f16_bits_to_f32(sv[0] >> 16);
        v[2] = v[2] * FE_HAD_SCALE * f16_bits_to_f32(sv[1] & 0xffff);
        v[3] = v[3] * FE_HAD_SCALE * f16_bits_to_f32(sv[1] >> 16);
        if constexpr (CHAIN == 1)  // bf16, written through: the down stage's programs read it in this launch
            store_agent_u32x2((uint16_t*)mb.y + (size_t)row * n + col0 + 4 * l32,
                              (u32x2){pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])});
        else
            store4(mb.y, y_mode, (size_t)row * n + col0 + 4 * l32, v);
    };
    // A column block is finished (all of the workgroup's threads come here). Front stage: once every lane's stores are
    // acknowledged, its ready word takes this launch's number. Down stage: the block is counted, and the last one
    // completes the launch.
    auto block_done = [&](uint32_t fnb) {
        if constexpr (CHAIN == 1) {
            agent_stores_wait();
            __syncthreads();
            if (tid == 0) __hip_atomic_store(ch.ready + fnb * FE_CHAIN_STRIDE, chain_target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#ifdef FE_GEMV_STAMPS
            if (tid == 0 && stamp_at)
                ((unsigned long long*)(stamp_base + 65536))[16384 * 12 + (ch.ready - (ch.state + FE_CHAIN_STRIDE)) / FE_CHAIN_STRIDE + fnb] = __builtin_amdgcn_s_memrealtime();
#endif
        } else if constexpr (CHAIN == 2) {
            if (tid == 0) {
                const uint32_t old = __hip_atomic_fetch_add(ch.state + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (old + 1 == ch.nb_down) {
                    __hip_atomic_store(ch.state + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(ch.state, chain_target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        (void)fnb;
    };

    // The segment of column block fnb that ends here: its sums meet in LDS, and then either are the block's sums (the
    // block lies in this run alone) or go to z for the program that arrives last at the block.
    // More than 32 rows (RG > 2): the sums of rows 0..31, then of rows 32.., meet in `red`; use(row, its sums) is called for
    // each row by the half wavefront that takes it.
    auto through_red_halves = [&](auto use) {
        float* rp = red + 32 * wave + 16 * (g >> 1) + 4 * (g & 1);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            __syncthreads();  // the readers before are done with `red`
#pragma unroll
            for (int rg = 2 * h; rg < (2 * h + 2 < RG ? 2 * h + 2 : RG); rg++) {
                const uint32_t row = 16 * rg + r;  // accumulator column = input row
                if (row < m) {
                    *(f32x4*)(rp + (row - 32 * h) * GEMV_RED_PITCH) = acc[rg][0];
                    *(f32x4*)(rp + (row - 32 * h) * GEMV_RED_PITCH + 8) = acc[rg][1];
                }
                acc[rg][0] = acc[rg][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
            __syncthreads();
            const uint32_t end = m < 32u * h + 32 ? m : 32u * h + 32;
            for (uint32_t row = 32 * h + hw; row < end; row += 8)
                use(row, *(const f32x4*)(red + (row - 32 * h) * GEMV_RED_PITCH + 4 * l32));
        }
    };

    auto flush = [&](uint32_t fnb, uint32_t p) {
        if constexpr (RG <= 2) __syncthreads();  // the previous segment's readers are done with `red`
        // rows 4 g .. 4 g + 3 of A are columns 16 (g >> 1) + 4 (g & 1) + 8 h .. + 3 of the wavefront's 32 (tile g >> 1 of
        // its pair, n = 4 (g & 1) + i + 8 h): a lane's four sums of either half are four neighbouring columns
        if constexpr (RG <= 2) {
            float* rp = red + 32 * wave + 16 * (g >> 1) + 4 * (g & 1);
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                uint32_t row = 16 * rg + r;  // accumulator column = input row
                if (row < m) {
                    *(f32x4*)(rp + row * GEMV_RED_PITCH) = acc[rg][0];
                    *(f32x4*)(rp + row * GEMV_RED_PITCH + 8) = acc[rg][1];
                }
                acc[rg][0] = acc[rg][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
            __syncthreads();
        }
        FE_STAMP(4);
        const uint32_t col0 = fnb * 128;
        // programs of the block's first and last unit
        const uint32_t cut = rem * (base + 1), ua = fnb * upb, ub = ua + upb - 1;
        const uint32_t first_prog = ua < cut ? udiv_inv(ua, base + 1, mb.inv_base1) : rem + udiv_inv(ua - cut, base, mb.inv_base);
        const uint32_t last_prog = ub < cut ? udiv_inv(ub, base + 1, mb.inv_base1) : rem + udiv_inv(ub - cut, base, mb.inv_base);
        if (first_prog == last_prog) {
            if constexpr (RG > 2) {
                through_red_halves([&](uint32_t row, f32x4 t) {
                    float v[4] = {t[0], t[1], t[2], t[3]};
                    finish(v, col0, row);
                });
            } else {
                for (uint32_t row = hw; row < m; row += 8) {
                    f32x4 t = *(const f32x4*)(red + row * GEMV_RED_PITCH + 4 * l32);
                    float v[4] = {t[0], t[1], t[2], t[3]};
                    finish(v, col0, row);
                }
            }
            block_done(fnb);
            return;
        }
        // Hand-off of the segment's sums to another program, possibly on another XCD with its own L2:
        //  1. every lane stores its piece with agent-scope (write-through) stores and waits until they are acknowledged;
        //  2. the workgroup barrier orders all lanes' acknowledged stores before lane 0's arrival at the counter
        //     (an agent-scope atomic, performed at the shared level);
        //  3. the program whose arrival completes the count reads the segments with agent-scope loads (past its own L2)
        //     after the barrier that publishes last_flag.
        // Every byte that crosses is written through and read through, so no cache write-back or invalidate is needed.
        float* zseg = mb.z + (size_t)(p + fnb) * m * 128;
        if constexpr (RG > 2) {
            through_red_halves([&](uint32_t row, f32x4 t) { store_agent_f32x4(zseg + row * 128 + 4 * l32, t); });
            agent_stores_wait();
        } else if constexpr (FENCED) {
            for (uint32_t row = hw; row < m; row += 8)
                *(f32x4*)(zseg + row * 128 + 4 * l32) = *(const f32x4*)(red + row * GEMV_RED_PITCH + 4 * l32);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        } else {
            for (uint32_t row = hw; row < m; row += 8)
                store_agent_f32x4(zseg + row * 128 + 4 * l32, *(const f32x4*)(red + row * GEMV_RED_PITCH + 4 * l32));
            agent_stores_wait();
        }
        FE_STAMP(5);
        __syncthreads();
        if (tid == 0) {
            uint32_t old = __hip_atomic_fetch_add(&mb.counters[fnb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_flag = (old == last_prog - first_prog);
        }
        __syncthreads();
        FE_STAMP(6);
        if (last_flag) {
            if constexpr (FENCED) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            // A half wavefront finishes rows hw, hw + 8, ...: RB of them at a time with SB segments each, 8 or 12 agent-scope
            // loads in flight (each takes a trip to memory: the trips overlap); every row's segments are added in program
            // order (as many in flight as the registers hold without costing the kernel a resident wavefront). Up to 8 rows
            // every half wavefront has at most one row and takes all of the batch from it.
            const uint32_t nseg = last_prog - first_prog + 1;
            const __amdgpu_buffer_rsrc_t zrs = __builtin_amdgcn_make_buffer_rsrc(
                (void*)(mb.z + (size_t)(first_prog + fnb) * m * 128), 0, nseg * m * 512, 0x00020000);
            auto rows_of = [&](auto rb_tag) {
                constexpr int RB = decltype(rb_tag)::value, SB = (BITS <= 4 && RG == 1 ? 12 : 8) / RB;
                for (uint32_t row0 = hw; row0 < m; row0 += 8 * RB) {
                    float v[RB][4];
#pragma unroll
                    for (int j = 0; j < RB; j++) v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.f;
                    for (uint32_t sp0 = 0; sp0 < nseg; sp0 += SB) {
                        f32x4 t[RB * SB];
#pragma unroll
                        for (int j = 0; j < RB; j++) {
                            const uint32_t row = row0 + 8 * j < m ? row0 + 8 * j : row0;
#pragma unroll
                            for (int b = 0; b < SB; b++)  // (past the last segment: out of the buffer's range, reads zero)
                                t[j * SB + b] = FENCED ? __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                             zrs, row * 512 + 16 * l32, (sp0 + b) * m * 512, 0))
                                                       : load_agent_f32x4(zrs, row * 512 + 16 * l32, (sp0 + b) * m * 512);
                        }
#pragma unroll
                        for (int j = 0; j < RB; j++)
#pragma unroll
                            for (int b = 0; b < SB; b++)
                                if (sp0 + b < nseg) {
#pragma unroll
                                    for (int e = 0; e < 4; e++) v[j][e] += t[j * SB + b][e];
                                }
                    }
#pragma unroll
                    for (int j = 0; j < RB; j++) {
                        const uint32_t row = row0 + 8 * j;
                        if (row < m) finish(v[j], col0, row);
                    }
                }
            };
            if (m <= 8)
                rows_of(std::integral_constant<int, 1>{});
            else
                rows_of(std::integral_constant<int, 2>{});
            if (tid == 0) __hip_atomic_store(&mb.counters[fnb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            block_done(fnb);
            FE_STAMP(7);
        }
    };

    for (uint32_t c0 = 0; c0 < S; c0 += chunk) {
        const uint32_t cs = S - c0 < chunk ? S - c0 : chunk;
        if (c0) __syncthreads();  // the previous chunk's readers are done with xs
        if (rotating) {
            const uint32_t nblk = cs / 2;
            uint32_t row = 0, b = hw;
            RotAt a = {};
            const bool any = b < nblk;
            if (any) {
                a = rot_at(c0, row, b);
                if (c0 || CHAIN == 2) rot_raw = load_pair(a);
            }
            while (any && row < m) {
                u32x2 o = rot_finish(rot_raw, rot_mode, l32);
                *(u32x2*)(xs + a.off) = o;
                if (a.keep && mb.xh) *(u32x2*)(mb.xh + a.at) = o;
                b += 8;
                if (b >= nblk) b = hw, row++;
                if (row < m) {
                    a = rot_at(c0, row, b);
                    rot_raw = load_pair(a);
                }
            }
        } else {  // rotated inputs of the chunk's load steps -> xs [row][cs * 64 fp16], NB 16-byte pieces in flight a thread
            constexpr int NB = RG == 1 ? FE_STAGE_NB1 : 8;
            const uint32_t chunks16 = cs * 8, total = m * chunks16, inv16 = 0xffffffffu / chunks16;
            for (uint32_t i0 = tid; i0 < total; i0 += 256 * NB) {
                u32x4 v[NB];
                uint32_t off[NB];
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const uint32_t i = i0 + 256 * j < total ? i0 + 256 * j : i0;  // past the end: a piece again, not stored
                    const uint32_t row = udiv_inv(i, chunks16, inv16), c = i - row * chunks16;
                    uint32_t gst = st_run0 + c0 + (c >> 3);
                    if (gst >= spb) gst -= spb;
                    if (gst >= spb) gst %= spb;
                    v[j] = *(const u32x4*)(mb.xh + (size_t)row * k + gst * 64 + (c & 7) * 8);
                    off[j] = row * xpitch + c * 16;
                }
#pragma unroll
                for (int j = 0; j < NB; j++)
                    if (i0 + 256 * j < total) *(u32x4*)(xs + off[j]) = v[j];
            }
        }
        __syncthreads();
        FE_STAMP(2);
        // the chunk's load steps, segment by segment (a segment ends with its column block, with the chunk ...
        uint32_t i = 0;
        while (i < cs) {
            uint32_t seg = cs - i < spb - st ? cs - i : spb - st;
            seg = seg < lend - (c0 + i) ? seg : lend - (c0 + i);  // ... or with the program's run
            // Whole groups of GROUP steps run as straight-line code: no branches inside, and the refill of a ring slot is
            // unconditional, so each load lands straight in the slot its words were just decoded from and only that
            // slot's next use waits for it. The wait at the top of a group has to cover every load in flight (the
            // compiler cannot count across the back edge).
            const uint32_t full = seg / GROUP * GROUP;
            for (uint32_t s0 = 0; s0 < full; s0 += GROUP) {
#pragma unroll
                for (int j = 0; j < GROUP; j++) one(ring[j % DEPTH], i + s0 + j);
            }
            for (uint32_t s0 = full; s0 < seg; s0 += DEPTH) {  // the remainder, slot by slot
#pragma unroll
                for (int j = 0; j < DEPTH; j++)
                    if (s0 + j < seg) one(ring[j], i + s0 + j);
            }
            ring_turn<BITS, DEPTH>(ring, seg % DEPTH);
            FE_STAMP(3);
            i += seg, st += seg;
            const bool block_end = st == spb, run_end = c0 + i == lend;
            if (block_end || run_end) {
                flush(nb, pl);
                if (block_end) {
                    nb++, st = 0;
                    if (c0 + i < S) sv = *(const u32x2*)(mb.svh + nb * 128 + 4 * l32);  // the next block's output scales
                }
                if (run_end) pl++, lend = 2 * (run_start(pl + 1) - u0);
            }
        }
    }
    FE_STAMP(8);
}

// (second launch bound: wavefronts per SIMD the registers must allow. Four programs a CU for up to 16 rows.)
#define GEMVB_KERNEL(BITS, RG)                                                                                        \
    extern "C" __global__ __launch_bounds__(256, RG == 1 ? 4 : 2) void exl3_gemvb_b##BITS##_r##RG(                    \
        GemvJob job, const void* x, const void* x2, uint32_t x_mode, uint32_t ldx, uint32_t k, uint32_t m,             \
        uint32_t y_mode, uint32_t chunk, uint32_t inv_spb, uint32_t fuse) {                                            \
        uint32_t i = 0;                                                                                               \
        while (i + 1 < job.count && blockIdx.x >= job.first[i + 1]) i++;                                              \
        const uint32_t p0 = (blockIdx.x - job.first[i]) * fuse, left = job.m[i].programs - p0;                        \
        gemvb_body<BITS, RG>(job.m[i], p0, left < fuse ? left : fuse, k, m, y_mode, chunk, inv_spb,                   \
                             RotSrc{x, x2, x_mode, ldx}, job.m[0].xh);                                                \
    }
#define GEMVB_FENCED_KERNEL(BITS)                                                                                     \
    extern "C" __global__ __launch_bounds__(256, 4) void exl3_gemvb_b##BITS##_r1_fenced(                              \
        GemvJob job, const void* x, const void* x2, uint32_t x_mode, uint32_t ldx, uint32_t k, uint32_t m,             \
        uint32_t y_mode, uint32_t chunk, uint32_t inv_spb, uint32_t fuse) {                                            \
        uint32_t i = 0;                                                                                               \
        while (i + 1 < job.count && blockIdx.x >= job.first[i + 1]) i++;                                              \
        const uint32_t p0 = (blockIdx.x - job.first[i]) * fuse, left = job.m[i].programs - p0;                        \
        gemvb_body<BITS, 1, 0, true>(job.m[i], p0, left < fuse ? left : fuse, k, m, y_mode, chunk, inv_spb,           \
                                     RotSrc{x, x2, x_mode, ldx}, job.m[0].xh);                                        \
    }
#define GEMVB_FAMILY(BITS) GEMVB_KERNEL(BITS, 1) GEMVB_KERNEL(BITS, 2) GEMVB_KERNEL(BITS, 3) GEMVB_KERNEL(BITS, 4) GEMVB_FENCED_KERNEL(BITS)

// The decode MLP in one launch, 1..16 rows: grid = the front stage's workgroups (gate and up, alternating when their
// counts are equal, so that block b of both is finished at about the same time), then the down stage's. Down workgroup
// w runs program perm[w] (the host's table: the programs sorted by the last channel block their run reads, so that they
// come in the order in which the front stage finishes their inputs; null: program w).
struct MlpChain {
    GemvJob front;
    GemvMember down;
    uint32_t* state;
    const uint32_t* perm;
    uint32_t front_wgs, interleave;
    uint32_t k1, chunk1, inv_spb1, fuse1;
    uint32_t k2, chunk2, inv_spb2, fuse2;
    uint32_t spin_limit, pad;
};
#define MLP_KERNEL(BITS)                                                                                              \
    extern "C" __global__ __launch_bounds__(256, 4) void exl3_mlp_b##BITS(MlpChain c, const void* x, uint32_t x_mode,  \
                                                                          uint32_t ldx, uint32_t m, uint32_t y_mode) { \
        const uint32_t w = blockIdx.x, nbf = c.front.m[0].n / 128, nbd = c.down.n / 128;                              \
        if (w < c.front_wgs) {                                                                                        \
            uint32_t i = 0, lw = w;                                                                                   \
            if (c.interleave) {                                                                                       \
                i = w & 1, lw = w >> 1;                                                                               \
            } else {                                                                                                  \
                while (i + 1 < c.front.count && w >= c.front.first[i + 1]) i++;                                       \
                lw = w - c.front.first[i];                                                                            \
            }                                                                                                         \
            const uint32_t p0 = lw * c.fuse1, left = c.front.m[i].programs - p0;                                      \
            gemvb_body<BITS, 1, 1>(c.front.m[i], p0, left < c.fuse1 ? left : c.fuse1, c.k1, m, 0, c.chunk1, c.inv_spb1, \
                                   RotSrc{x, nullptr, x_mode, ldx}, c.front.m[0].xh,                                  \
                                   ChainCtx{c.state, c.state + (1 + i * nbf) * FE_CHAIN_STRIDE, nbf, nbd, c.spin_limit}); \
        } else {                                                                                                      \
            uint32_t lw = w - c.front_wgs;                                                                            \
            if (c.perm) lw = c.perm[lw];                                                                              \
            const uint32_t p0 = lw * c.fuse2, left = c.down.programs - p0;                                            \
            gemvb_body<BITS, 1, 2>(c.down, p0, left < c.fuse2 ? left : c.fuse2, c.k2, m, y_mode, c.chunk2, c.inv_spb2, \
                                   RotSrc{c.front.m[0].y, c.front.m[1].y, 2, c.front.m[0].n}, c.front.m[0].xh,        \
                                   ChainCtx{c.state, c.state + FE_CHAIN_STRIDE, nbf, nbd, c.spin_limit});             \
        }                                                                                                             \
    }
MLP_KERNEL(2)
MLP_KERNEL(3)
MLP_KERNEL(4)
MLP_KERNEL(5)
MLP_KERNEL(6)
MLP_KERNEL(8)
GEMVB_FAMILY(2)
GEMVB_FAMILY(3)
GEMVB_FAMILY(4)
GEMVB_FAMILY(5)
GEMVB_FAMILY(6)
GEMVB_FAMILY(8)

// ---- prefill GEMM ----------------------------------------------------------------------------------------------------

// Weight tile producer of the prefill GEMM: a 64-wide k tile of a 128-column block is 4 k steps x 8 tiles; wavefront w
// takes k step w, lane L tile L >> 3, rows n = (L & 7) and (L & 7) + 8 of it (the same run of words as in the GEMV),
// in both 128-column blocks of the 256-column output tile.
template <int BITS>
struct Exl3Producer {
    const uint32_t* base[2];  // the two blocks' trellis + this lane's tile
    uint32_t stride_k, run_off, prev_off, brow, ks;
    struct Raw {
        LaneWords<BITS> w[2];
    };
    static constexpr int kStoreValu = 240;  // about the VALU instructions of the four quarters together
    static constexpr bool kQuarters = true;  // the main loop spreads the decode over its four slices
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != half) continue;
            const uint32_t* p = base[b] + (size_t)(kt * 4 + ks) * stride_k;
            r.w[b] = load_lane_words<BITS>(p + run_off, p + prev_off);
        }
    }
    // quarter q: row half q & 1 (rows n = brow + 8 (q & 1) of the lane's tile) of column block q >> 1
    __device__ __forceinline__ void store_quarter(const Raw& r, unsigned char* Bs, int q) const {
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (2 * b + h != q) continue;
                f16x8 op[2];
                decode_lane_half<BITS>(r.w[b], h, op);
#pragma unroll
                for (int kh = 0; kh < 2; kh++) *(f16x8*)(Bs + gm_swz(128 * b + brow + 8 * h, 2 * ks + kh)) = op[kh];
            }
    }
};

// y[m][n] (+)= H(xh @ W_hat) * svh / sqrt(128) for prefill-sized m: xh fp16 [m][k] (rotated inputs), 256 x 256 output
// tiles; a wavefront's 128 columns are exactly one Hadamard block, so the output rotation is local to the wavefront.
// Tiles = ceil(m / 256) * ceil(n / 256) (grouped raster), spread over the grid as sc says (gemm_schedule): one piece a
// program, the cut tiles finished by exl3_gemm_reduce, or stream-K. 256 threads, dynamic LDS GM_LDS_TILES (the epilogue
// reuses it). make_producer(tn) builds the weight producer of 256-column tile tn.
template <bool SK, class MakeProducer>
__device__ __forceinline__ void exl3_gemm_tile(const _Float16* __restrict__ xh, const uint16_t* __restrict__ svh, void* y,
                                               uint32_t n, uint32_t k, uint32_t m, uint32_t y_mode, uint32_t group_m,
                                               const GemmSched& sched, MakeProducer make_producer) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t nbs = n / 128;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    gemm_schedule<SK>(
        sched, (m + GM_BM - 1) / GM_BM, (nbs + 1) / 2, group_m, k / GM_BK, lds,
        [&](uint32_t tm, uint32_t tn, uint32_t kt0, uint32_t ktn, f32x16(&acc)[4][4]) {
            auto prod = make_producer(tn);
            gemm_mainloop(xh, k, m, kt0, ktn, tm * GM_BM, prod, lds, acc);
        },
        [&](uint32_t tm, uint32_t tn, f32x16(&acc)[4][4]) {
            const uint32_t m0 = tm * GM_BM, nb = 2 * tn + wn;
            if (nb >= nbs) return;
            const uint32_t col = nb * 128 + 4 * (lane & 31);
            const f32x4 sc = row_scales(svh, col);
            // one copy of the epilogue per output mode, so that the row loop has no mode branches
            auto run = [&](auto mode_tag) {
                constexpr uint32_t MODE = decltype(mode_tag)::value;
                gemm_epilogue(
                    acc, lds,
                    [&](float (&v)[4][4], uint32_t l32) {
                        fwht128_half_wave_rows(v, l32);
#pragma unroll
                        for (int u = 0; u < 4; u++)
#pragma unroll
                            for (int e = 0; e < 4; e++) v[u][e] = v[u][e] * FE_HAD_SCALE * sc[e];  // finish_row's products
                    },
                    [&](uint32_t row, uint32_t, float (&v)[4]) {
                        uint32_t grow = m0 + wm * 128 + row;
                        if (grow < m) store4(y, MODE, (size_t)grow * n + col, v);
                    });
            };
            if (y_mode == 0)
                run(std::integral_constant<uint32_t, 0>{});
            else if (y_mode == 1)
                run(std::integral_constant<uint32_t, 1>{});
            else if (y_mode == 2)
                run(std::integral_constant<uint32_t, 2>{});
            else
                run(std::integral_constant<uint32_t, 3>{});
        });
}

// The GEMM decoding the trellis itself: every 256-row tile of the output decodes its weights again.
template <int BITS, bool SK>
__device__ __forceinline__ void exl3_gemm_body(const _Float16* __restrict__ xh, const uint32_t* __restrict__ trellis,
                                               const uint16_t* __restrict__ svh, void* y, uint32_t n, uint32_t k, uint32_t m,
                                               uint32_t y_mode, uint32_t stride_k, uint32_t stride_nb, uint32_t group_m,
                                               const GemmSched& sched) {
    exl3_gemm_tile<SK>(xh, svh, y, n, k, m, y_mode, group_m, sched, [&](uint32_t tn) {
        constexpr uint32_t tw = 8 * BITS;
        const uint32_t lane = threadIdx.x & 63, nbs = n / 128;
        Exl3Producer<BITS> prod;
        uint32_t tj = lane >> 3, q = lane & 7;
        uint32_t nb1 = 2 * tn + 1 < nbs ? 2 * tn + 1 : 2 * tn;  // an odd block count: the last tile decodes block 2 tn twice
        prod.base[0] = trellis + (size_t)(2 * tn) * stride_nb + tj * tw;
        prod.base[1] = trellis + (size_t)nb1 * stride_nb + tj * tw;
        prod.stride_k = stride_k;
        prod.run_off = q * BITS;
        prod.prev_off = (q * BITS + tw - 1) % tw;
        prod.brow = tj * 16 + q;
        prod.ks = threadIdx.x >> 6;
        return prod;
    });
}

// ---- prefill over decoded weights -----------------------------------------------------------------------------------
//
// For many rows the trellis is decoded once per call into `hat`, fp16, as the very images the GEMM keeps in LDS: block
// (tn, kt) of 32 KB = rows n = 256 tn .. + 255 of k tile kt, 128 bytes a row, 16-byte chunk c of row r at the position gm_swz
// gives it. The GEMM over it then copies blocks instead of decoding, with the same fragments, the same MFMA order and
// so the same bits as exl3_gemm_b*.

// grid (n / 128, gy), 256 threads; program (nb, j) decodes k tiles j, j + gy, ... of column block nb with the lane
// mapping of Exl3Producer. The 16 KB of a k tile pass through LDS (two buffers, one barrier a tile) so that they leave
// as whole 1 KB runs per wavefront instead of scattered 16-byte pieces.
template <int BITS>
__device__ __forceinline__ void exl3_hat_tiles_body(const uint32_t* __restrict__ trellis, unsigned char* __restrict__ hat,
                                                    uint32_t k, uint32_t stride_k, uint32_t stride_nb) {
    __shared__ __attribute__((aligned(16))) unsigned char img[2][GM_B_BYTES / 2];
    constexpr uint32_t tw = 8 * BITS;
    const uint32_t lane = threadIdx.x & 63, ks = threadIdx.x >> 6, tj = lane >> 3, q = lane & 7;
    const uint32_t nb = blockIdx.x, ktiles = k / GM_BK;
    const uint32_t* base = trellis + (size_t)nb * stride_nb + tj * tw;
    const uint32_t run_off = q * BITS, prev_off = (q * BITS + tw - 1) % tw;
    const uint32_t row = tj * 16 + q;
    unsigned char* out = hat + (size_t)(nb >> 1) * ktiles * GM_B_BYTES + (nb & 1) * (GM_B_BYTES / 2) + 16 * threadIdx.x;
    uint32_t kt = blockIdx.y;
    if (kt >= ktiles) return;
    const uint32_t* p = base + (size_t)(kt * 4 + ks) * stride_k;
    LaneWords<BITS> cur = load_lane_words<BITS>(p + run_off, p + prev_off);
    for (uint32_t it = 0; kt < ktiles; kt += gridDim.y, it++) {
        uint32_t nk = kt + gridDim.y < ktiles ? kt + gridDim.y : kt;
        const uint32_t* pn = base + (size_t)(nk * 4 + ks) * stride_k;
        LaneWords<BITS> nxt = load_lane_words<BITS>(pn + run_off, pn + prev_off);
        f16x8 op[2][2];
        decode_lane<BITS>(cur, op);
        unsigned char* buf = img[it & 1];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int kh = 0; kh < 2; kh++) *(f16x8*)(buf + gm_swz(row + 8 * h, 2 * ks + kh)) = op[h][kh];
        __syncthreads();
        unsigned char* blk = out + (size_t)kt * GM_B_BYTES;
#pragma unroll
        for (int j = 0; j < 4; j++) *(u32x4*)(blk + 4096 * j) = *(const u32x4*)(buf + 16 * threadIdx.x + 4096 * j);
        cur = nxt;
    }
}

// Weight producer over `hat`: a k tile of the 256-column tile is one 32 KB block, copied as it is; thread t moves chunks
// t + 256 j (j < 4) of each 16 KB half.
struct HatProducer {
    const unsigned char* base;  // the tile's blocks + 16 * thread
    struct Raw {
        u32x4 c[2][4];
    };
    static constexpr int kStoreValu = 0;
    static constexpr bool kQuarters = false;
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != half) continue;
            const unsigned char* p = base + (size_t)kt * GM_B_BYTES + b * (GM_B_BYTES / 2);
#pragma unroll
            for (int j = 0; j < 4; j++) r.c[b][j] = *(const u32x4*)(p + 4096 * j);
        }
    }
    __device__ __forceinline__ void store(const Raw& r, unsigned char* Bs, int part) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != part) continue;
#pragma unroll
            for (int j = 0; j < 4; j++) *(u32x4*)(Bs + b * (GM_B_BYTES / 2) + 16 * threadIdx.x + 4096 * j) = r.c[b][j];
        }
    }
};

// (every GEMM kernel comes as NAME, one piece a program, and NAME_sk, stream-K, with the same parameters)
#define HAT_GEMM_PARAMS                                                                                                  \
    const _Float16 *xh, const unsigned char *hat, const uint16_t *svh, void *y, uint32_t n, uint32_t k, uint32_t m, uint32_t y_mode, \
        uint32_t group_m, GemmSched sched
template <bool SK>
__device__ __forceinline__ void exl3_gemm_hat_kernel(HAT_GEMM_PARAMS) {
    exl3_gemm_tile<SK>(xh, svh, y, n, k, m, y_mode, group_m, sched, [&](uint32_t tn) {
        HatProducer prod;
        prod.base = hat + (size_t)tn * (k / GM_BK) * GM_B_BYTES + 16 * threadIdx.x;
        return prod;
    });
}
extern "C" __global__ __launch_bounds__(256, 1) void exl3_gemm_hat(HAT_GEMM_PARAMS) {
    exl3_gemm_hat_kernel<false>(xh, hat, svh, y, n, k, m, y_mode, group_m, sched);
}
extern "C" __global__ __launch_bounds__(256, 1) void exl3_gemm_hat_sk(HAT_GEMM_PARAMS) {
    exl3_gemm_hat_kernel<true>(xh, hat, svh, y, n, k, m, y_mode, group_m, sched);
}

// Finishes the tiles that exl3_gemm_b* cut along K: sums their partial slots and applies the output rotation and scale.
// grid (tiles - full_tiles) * 64, 256 threads.
extern "C" __global__ __launch_bounds__(256) void exl3_gemm_reduce(const float* part, const uint16_t* svh, void* y, uint32_t n,
                                                                   uint32_t m, uint32_t y_mode, uint32_t group_m,
                                                                   uint32_t full_tiles, uint32_t splits) {
    const uint32_t nbs = n / 128;
    gemm_reduce_rows(part, splits, [&](uint32_t t, uint32_t row, uint32_t cb, uint32_t l32, float (&v)[4]) {
        uint32_t tm, tn;
        gemm_raster(full_tiles + t, (m + GM_BM - 1) / GM_BM, (nbs + 1) / 2, group_m, tm, tn);
        uint32_t grow = tm * GM_BM + row, nb = 2 * tn + cb;
        if (grow < m && nb < nbs) finish_row(v, l32, svh, nb * 128 + 4 * l32, y, y_mode, (size_t)grow * n + nb * 128 + 4 * l32);
    });
}

#define GEMM_KERNEL_(NAME, BITS, SK)                                                                                   \
    extern "C" __global__ __launch_bounds__(256, 1) void NAME(                                                         \
        const _Float16* xh, const uint32_t* trellis, const uint16_t* svh, void* y, uint32_t n, uint32_t k, uint32_t m,  \
        uint32_t y_mode, uint32_t stride_k, uint32_t stride_nb, uint32_t group_m, GemmSched sched) {                    \
        exl3_gemm_body<BITS, SK>(xh, trellis, svh, y, n, k, m, y_mode, stride_k, stride_nb, group_m, sched);           \
    }
#define GEMM_KERNEL(BITS)                       \
    GEMM_KERNEL_(exl3_gemm_b##BITS, BITS, false) \
    GEMM_KERNEL_(exl3_gemm_b##BITS##_sk, BITS, true)
#define HAT_KERNEL(BITS)                                                                                      \
    extern "C" __global__ __launch_bounds__(256) void exl3_hat_tiles_b##BITS(                                 \
        const uint32_t* trellis, unsigned char* hat, uint32_t k, uint32_t stride_k, uint32_t stride_nb) {     \
        exl3_hat_tiles_body<BITS>(trellis, hat, k, stride_k, stride_nb);                                      \
    }
HAT_KERNEL(2)
HAT_KERNEL(3)
HAT_KERNEL(4)
HAT_KERNEL(5)
HAT_KERNEL(6)
HAT_KERNEL(8)
GEMM_KERNEL(2)
GEMM_KERNEL(3)
GEMM_KERNEL(4)
GEMM_KERNEL(5)
GEMM_KERNEL(6)
GEMM_KERNEL(8)

// ---- probes ----------------------------------------------------------------------------------------------------------

// Streaming read of `bytes` (a multiple of 16 * 256 * gridDim.x * unroll) with 16-byte loads; each thread xors what it
// read into one word of out so the loads stay. (kernels/k-exl3/src/probe.rs:7-36)
extern "C" __global__ __launch_bounds__(256) void exl3_probe_v4(const u32x4* in, uint32_t* out, uint64_t vec_count) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x, stride = (uint64_t)gridDim.x * 256;
    u32x4 a = {0, 0, 0, 0};
    for (; i + 3 * stride < vec_count; i += 4 * stride) {
        u32x4 v0 = __builtin_nontemporal_load(in + i), v1 = __builtin_nontemporal_load(in + i + stride);
        u32x4 v2 = __builtin_nontemporal_load(in + i + 2 * stride), v3 = __builtin_nontemporal_load(in + i + 3 * stride);
        a ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < vec_count; i += stride) a ^= __builtin_nontemporal_load(in + i);
    uint32_t x = a[0] ^ a[1] ^ a[2] ^ a[3];
    if (x == 0x9e3779b9u) out[0] = x;  // practically never: keeps the loads alive without a store stream
}

// Decode-only probe: every lane decodes `iters` load steps of synthetic words and feeds them to the matrix instruction as
// the GEMV does (no memory traffic, no LDS): the ALU ceiling of the trellis decode in weights per second at the GEMV's
// occupancy (launch 4 programs a CU). The words change from step to step by additions that do not depend on the results,
// as words from memory would not. out receives a checksum.
template <int BITS>
__device__ __forceinline__ void probe_decode_body(uint32_t* out, uint32_t iters, uint32_t seed) {
    LaneWords<BITS> lw;
#pragma unroll
    for (int i = 0; i <= BITS; i++) lw.w[i] = (seed + i) * 0x9e3779b9u * (threadIdx.x + 1 + blockIdx.x * 256);
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    const f16x8 xb = {1, 1, 1, 1, 1, 1, 1, 1};
    for (uint32_t it = 0; it < iters; it++) {
        f16x8 op[2][2];
        decode_lane<BITS>(lw, op);
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[0][0], xb, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[1][0], xb, acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[0][1], xb, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[1][1], xb, acc1, 0, 0, 0);
#pragma unroll
        for (int i = 0; i <= BITS; i++) lw.w[i] += 0x9e3779b9u + i;
    }
    const float sum = acc0[0] + acc0[1] + acc0[2] + acc0[3] + acc1[0] + acc1[1] + acc1[2] + acc1[3];
    out[blockIdx.x * blockDim.x + threadIdx.x] = __float_as_uint(sum);
}
extern "C" __global__ __launch_bounds__(256, 4) void exl3_probe_decode_b3(uint32_t* out, uint32_t iters, uint32_t seed) {
    probe_decode_body<3>(out, iters, seed);
}
extern "C" __global__ __launch_bounds__(256, 4) void exl3_probe_decode_b4(uint32_t* out, uint32_t iters, uint32_t seed) {
    probe_decode_body<4>(out, iters, seed);
}
extern "C" __global__ __launch_bounds__(256, 4) void exl3_probe_decode_b5(uint32_t* out, uint32_t iters, uint32_t seed) {
    probe_decode_body<5>(out, iters, seed);
}

// Instruction throughput probes: 8 independent chains of `iters` dependent instructions a lane, no memory traffic
// (kernels/k-exl3/src/probe.rs:38-67 measures its decode's instructions the same way). The instructions are the ones the
// trellis decode is made of, plus an add and an and as the plain 32-bit yardsticks; the issue rate of an instruction is
// lanes x 8 x iters over the launch time.
#define OP_PROBE(NAME, ASM)                                                                                            \
    extern "C" __global__ __launch_bounds__(256) void exl3_probe_op_##NAME(uint32_t* out, uint32_t iters, uint32_t seed) { \
        uint32_t x[8];                                                                                                 \
        _Pragma("unroll") for (int j = 0; j < 8; j++) x[j] = (seed + j) ^ (threadIdx.x * 0x9e3779b9u);                 \
        const uint32_t c = 0x83DCD12Du;                                                                                \
        for (uint32_t i = 0; i < iters; i++) {                                                                         \
            _Pragma("unroll") for (int j = 0; j < 8; j++) asm volatile(ASM : "+v"(x[j]) : "v"(c));                     \
        }                                                                                                              \
        const uint32_t r = x[0] ^ x[1] ^ x[2] ^ x[3] ^ x[4] ^ x[5] ^ x[6] ^ x[7];                                      \
        if (r == 0x12345678u) *out = r;                                                                                \
    }
OP_PROBE(add, "v_add_u32 %0, %0, %1")
OP_PROBE(and, "v_and_b32 %0, %0, %1")
OP_PROBE(mul_lo, "v_mul_lo_u32 %0, %0, %1")
OP_PROBE(mad_u24, "v_mad_u32_u24 %0, %0, %1, %1")
OP_PROBE(bfe, "v_bfe_u32 %0, %0, 5, 16")
OP_PROBE(alignbit, "v_alignbit_b32 %0, %0, %1, 16")
OP_PROBE(perm, "v_perm_b32 %0, %0, %1, %1")
OP_PROBE(sad_u8, "v_sad_u8 %0, %0, 0, %1")
OP_PROBE(sad_hi_u8, "v_sad_hi_u8 %0, %0, 0, %1")
OP_PROBE(pk_fma_f16, "v_pk_fma_f16 %0, %0, %1, %1")
OP_PROBE(fma_f32, "v_fma_f32 %0, %0, %1, %1")
OP_PROBE(dpp_mov, "v_mov_b32_dpp %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf")
