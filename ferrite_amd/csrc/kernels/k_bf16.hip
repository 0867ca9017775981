// The plain bf16 weight form of the caller's linear: y[M][N] = x[M][K] . W[N][K]^T (+ residual), W row-major bf16, f32
// sums, bf16 out. A GEMM on the shared 256 x 256 MFMA tile loop and two decode-sized GEMVs (kernels/k-core/src/gemm.rs).
#include "gemm_core.h"

// 4 sums of columns at.. of one row -> bf16; with res: bf16(bf16(sum) + res) (gemm.rs:152-158).
__device__ __forceinline__ void bf16_store4(uint16_t* c, const uint16_t* res, size_t at, const float (&v)[4]) {
    u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
    if (res) {
        u32x2 r = *(const u32x2*)(res + at);
#pragma unroll
        for (int e = 0; e < 2; e++)
            o[e] = pack_bf16x2(bf16_bits_to_f32(o[e] & 0xffff) + bf16_bits_to_f32(r[e] & 0xffff),
                               bf16_bits_to_f32(o[e] >> 16) + bf16_bits_to_f32(r[e] >> 16));
    }
    *(u32x2*)(c + at) = o;
}

// ---- GEMM ------------------------------------------------------------------------------------------------------------

// A weight k tile is already what the LDS tile holds: thread t copies 16-byte chunk t & 7 of rows (t >> 3) + 32 j of each
// 128-row half. Rows past n re-read row n - 1 (their columns are never stored).
struct Bf16Producer {
    const unsigned char* w;
    uint32_t off[2][4];  // byte offset of row (t >> 3) + 32 j of half b, chunk t & 7, k tile 0
    uint32_t st;
    struct Raw {
        u32x4 c[2][4];
    };
    static constexpr int kStoreValu = 0;
    static constexpr bool kQuarters = false;
    __device__ __forceinline__ void load(uint32_t kt, Raw& r, int half) const {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            if (b != half) continue;
            const unsigned char* p = w + (size_t)kt * (GM_BK * 2);
#pragma unroll
            for (int j = 0; j < 4; j++) r.c[b][j] = *(const u32x4*)(p + off[b][j]);
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

// C[M][ldc] = bf16(A . W^T) (+ res); A bf16 [M][lda], W bf16 [N][K]. grid full_tiles + (tiles - full_tiles) * splits with
// tiles = ceil(M / 256) * ceil(N / 256), 256 threads, dynamic LDS GM_LDS_TILES; tiles past full_tiles leave partials in
// `part` for fe_gemm_bf16_reduce. K % 64 == 0, N % 8 == 0, lda % 8 == 0, ldc % 4 == 0, operands under 4 GB.
// (kernels/k-core/src/gemm.rs:128-167: fe_gemm_bf16, tile 128 x 128 x 32 on mma.m16n8k16 there)
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_bf16(uint16_t* c, const uint16_t* a, const uint16_t* w,
                                                                  const uint16_t* res, uint32_t m, uint32_t n, uint32_t k,
                                                                  uint32_t lda, uint32_t ldc, uint32_t group_m,
                                                                  uint32_t full_tiles, uint32_t splits, float* part) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const GemmWork wk = gemm_work(blockIdx.x, (m + GM_BM - 1) / GM_BM, (n + GM_BN - 1) / GM_BN, group_m, k / GM_BK, full_tiles, splits);
    const uint32_t m0 = wk.tm * GM_BM, n0 = wk.tn * GM_BN;
    Bf16Producer prod;
    const uint32_t chunk = tid & 7, row = tid >> 3;
    prod.w = (const unsigned char*)w;
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t r = n0 + 128 * b + row + 32 * j;
            r = r < n ? r : n - 1;
            prod.off[b][j] = (r * k + chunk * 8) * 2;
        }
    prod.st = gm_swz(row, chunk);
    f32x16 acc[4][4];
    gemm_mainloop<Bf16Producer, true>((const _Float16*)a, lda, m, wk.kt0, wk.ktn, m0, prod, lds, acc);
    if (wk.partial) {
        gemm_store_partial(acc, lds, part + (size_t)wk.slot * GM_PART_FLOATS);
        return;
    }
    const uint32_t col = n0 + wn * 128 + 4 * (tid & 31);
    gemm_epilogue(
        acc, lds, [](float (&)[4][4], uint32_t) {},
        [&](uint32_t r, uint32_t, float (&v)[4]) {
            const uint32_t grow = m0 + wm * 128 + r;
            if (grow < m && col < n) bf16_store4(c, res, (size_t)grow * ldc + col, v);
        });
}

// Finishes the tiles fe_gemm_bf16 cut along K. grid (tiles - full_tiles) * 64, 256 threads.
extern "C" __global__ __launch_bounds__(256) void fe_gemm_bf16_reduce(uint16_t* c, const float* part, const uint16_t* res,
                                                                      uint32_t m, uint32_t n, uint32_t ldc, uint32_t group_m,
                                                                      uint32_t full_tiles, uint32_t splits) {
    gemm_reduce_rows(part, splits, [&](uint32_t t, uint32_t row, uint32_t cb, uint32_t l32, float (&v)[4]) {
        uint32_t tm, tn;
        gemm_raster(full_tiles + t, (m + GM_BM - 1) / GM_BM, (n + GM_BN - 1) / GM_BN, group_m, tm, tn);
        const uint32_t grow = tm * GM_BM + row, col = tn * GM_BN + cb * 128 + 4 * l32;
        if (grow < m && col < n) bf16_store4(c, res, (size_t)grow * ldc + col, v);
    });
}

// SwiGLU over a gate|up linear whose weight rows are interleaved in blocks of 8 ([gate 0..8, up 0..8, gate 8..16, ...],
// fe_interleave_gu): of the 4 lanes that hold one 16-column block of a row, lanes 0, 1 have the 8 gate sums and lanes 2, 3
// the matching up sums. Every lane takes part (a quad exchange); lanes 0, 1 store
// act[row][8 blk + 4 (lane & 1) ..] = bf16(bf16(silu(bf16(gate))) * bf16(up)), act row stride inter = n / 2.
// (kernels/k-core/src/gemm.rs:264-279)
__device__ __forceinline__ void bf16_swiglu_store4(uint16_t* act, const float (&v)[4], uint32_t l32, bool live, uint32_t grow,
                                                   uint32_t col, uint32_t n) {
    float u[4];
#pragma unroll
    for (int e = 0; e < 4; e++) u[e] = dpp_quad_xor<2>(v[e]);
    if (!live || (l32 & 2) || col >= n) return;
    const u32x2 o = {silu_mul_bf16x2(pack_bf16x2(v[0], v[1]), pack_bf16x2(u[0], u[1])),
                     silu_mul_bf16x2(pack_bf16x2(v[2], v[3]), pack_bf16x2(u[2], u[3]))};
    *(u32x2*)(act + (size_t)grow * (n >> 1) + (col >> 4) * 8 + 4 * (l32 & 1)) = o;
}

// act[M][N / 2] = SwiGLU(A . W^T) for interleaved gate|up weights W [N][K], N % 16 == 0: fe_gemm_bf16 with the epilogue
// above (and fe_gemm_bf16_swiglu_reduce for the tiles cut along K). (kernels/k-core/src/gemm.rs:264-279: fe_gemm_swiglu)
extern "C" __global__ __launch_bounds__(256, 1) void fe_gemm_bf16_swiglu(uint16_t* act, const uint16_t* a, const uint16_t* w,
                                                                         uint32_t m, uint32_t n, uint32_t k, uint32_t lda,
                                                                         uint32_t group_m, uint32_t full_tiles,
                                                                         uint32_t splits, float* part) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const GemmWork wk = gemm_work(blockIdx.x, (m + GM_BM - 1) / GM_BM, (n + GM_BN - 1) / GM_BN, group_m, k / GM_BK, full_tiles, splits);
    const uint32_t m0 = wk.tm * GM_BM, n0 = wk.tn * GM_BN;
    Bf16Producer prod;
    const uint32_t chunk = tid & 7, row = tid >> 3;
    prod.w = (const unsigned char*)w;
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t r = n0 + 128 * b + row + 32 * j;
            r = r < n ? r : n - 1;
            prod.off[b][j] = (r * k + chunk * 8) * 2;
        }
    prod.st = gm_swz(row, chunk);
    f32x16 acc[4][4];
    gemm_mainloop<Bf16Producer, true>((const _Float16*)a, lda, m, wk.kt0, wk.ktn, m0, prod, lds, acc);
    if (wk.partial) {
        gemm_store_partial(acc, lds, part + (size_t)wk.slot * GM_PART_FLOATS);
        return;
    }
    const uint32_t col = n0 + wn * 128 + 4 * (tid & 31);
    gemm_epilogue(
        acc, lds, [](float (&)[4][4], uint32_t) {},
        [&](uint32_t r, uint32_t l32, float (&v)[4]) {
            const uint32_t grow = m0 + wm * 128 + r;
            bf16_swiglu_store4(act, v, l32, grow < m, grow, col, n);
        });
}

extern "C" __global__ __launch_bounds__(256) void fe_gemm_bf16_swiglu_reduce(uint16_t* act, const float* part, uint32_t m,
                                                                             uint32_t n, uint32_t group_m,
                                                                             uint32_t full_tiles, uint32_t splits) {
    gemm_reduce_rows(part, splits, [&](uint32_t t, uint32_t row, uint32_t cb, uint32_t l32, float (&v)[4]) {
        uint32_t tm, tn;
        gemm_raster(full_tiles + t, (m + GM_BM - 1) / GM_BM, (n + GM_BN - 1) / GM_BN, group_m, tm, tn);
        const uint32_t grow = tm * GM_BM + row, col = tn * GM_BN + cb * 128 + 4 * l32;
        bf16_swiglu_store4(act, v, l32, grow < m, grow, col, n);
    });
}

// dst row 16 b + i = gate row 8 b + i for i < 8, up row 8 b + i - 8 otherwise: the weight layout of fe_gemm_bf16_swiglu.
// grid 2 inter, 256 threads; k % 8 == 0. (kernels/k-core/src/gemm.rs:281-296: fe_interleave_gu)
extern "C" __global__ __launch_bounds__(256) void fe_interleave_gu(uint16_t* dst, const uint16_t* gate, const uint16_t* up,
                                                                   uint32_t k) {
    const uint32_t r = blockIdx.x, b = r / 16, i = r % 16;
    const uint16_t* src = i < 8 ? gate + (size_t)(b * 8 + i) * k : up + (size_t)(b * 8 + i - 8) * k;
    uint16_t* d = dst + (size_t)r * k;
    for (uint32_t j = threadIdx.x; j < k / 8; j += 256) *((u32x4*)d + j) = *((const u32x4*)src + j);
}

// ---- GEMV (1..8 rows) ------------------------------------------------------------------------------------------------

__device__ __forceinline__ float dot8_bf16(u32x4 w, u32x4 x, float acc) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
        // the elements are copied out first: __builtin_bit_cast applied to a vector element reads element 0
        const uint32_t wp = w[p], xp = x[p];
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, wp), __builtin_bit_cast(bf16x2, xp), acc, false);
    }
    return acc;
}

// Sum over each row of 16 lanes, left in all 16 (four DPP adds: no LDS traffic, unlike a butterfly of ds_bpermute).
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<DPP_QUAD_XOR1>(v);
    v += dpp_mov<DPP_QUAD_XOR2>(v);
    v += dpp_mov<DPP_HALF_MIRROR>(v);
    v += dpp_mov<DPP_ROW_MIRROR>(v);
    return v;
}

// One wavefront: the sums of x rows 0..MR-1 (rows >= m repeat row m - 1) with NC weight rows over the 16-byte chunks
// [c0, c1) of K, lane L taking chunks c0 + L, c0 + L + 64, ... in ascending order, one v_dot2 per element pair; then
// every 16 lanes add up (the sum of lanes 16 q .. 16 q + 15 is left in all of them).
template <int MR, int NC>
__device__ __forceinline__ void gemv_bf16_sums(const uint16_t* a, const uint16_t* const (&wr)[NC], uint32_t m, uint32_t lda,
                                               uint32_t c0, uint32_t c1, float (&acc)[MR][NC]) {
    const uint32_t lane = threadIdx.x & 63;
    const uint16_t* xr[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) {
        xr[r] = a + (size_t)((uint32_t)r < m ? r : m - 1) * lda;
#pragma unroll
        for (int j = 0; j < NC; j++) acc[r][j] = 0.f;
    }
#pragma unroll 2
    for (uint32_t i = c0 + lane; i < c1; i += 64) {
        u32x4 wv[NC], xv[MR];
#pragma unroll
        for (int j = 0; j < NC; j++) wv[j] = __builtin_nontemporal_load((const u32x4*)wr[j] + i);
#pragma unroll
        for (int r = 0; r < MR; r++) xv[r] = *((const u32x4*)xr[r] + i);
#pragma unroll
        for (int r = 0; r < MR; r++)
#pragma unroll
            for (int j = 0; j < NC; j++) acc[r][j] = dot8_bf16(wv[j], xv[r], acc[r][j]);
    }
#pragma unroll
    for (int r = 0; r < MR; r++)
#pragma unroll
        for (int j = 0; j < NC; j++) acc[r][j] = row16_sum(acc[r][j]);
}

// y[r][n] = bf16(x[r][:] . W[n][:]) (+ res) for r < m <= MR. grid N / NC, 256 threads: a program takes NC consecutive
// columns; K is walked in steps of 64 chunks of 16 bytes (a 1 KB run of every weight row a step), wavefront w takes
// steps [w S / 4, (w + 1) S / 4) of the S steps, and the sixteen sums (4 wavefronts x 4 rows of 16 lanes) are added in order. So a row's bits depend
// on K only, neither on the other rows nor on NC: the host picks NC by the shape and the row count (more columns a program
// read x less often, fewer columns give more programs), where the reference picks between two kernels by the shape.
// K % 8 == 0, N % NC == 0, lda % 8 == 0. (kernels/k-core/src/gemm.rs:172-262: fe_gemv_bf16 and fe_gemv_bf16_kw)
template <int MR, int NC>
__device__ __forceinline__ void gemv_bf16_body(uint16_t* c, const uint16_t* a, const uint16_t* w, const uint16_t* res,
                                               uint32_t m, uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc) {
    __shared__ float red[16][MR][NC];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = blockIdx.x * NC;
    const uint16_t* wr[NC];
#pragma unroll
    for (int j = 0; j < NC; j++) wr[j] = w + (size_t)(col + j) * k;
    const uint32_t chunks = k / 8, steps = (chunks + 63) / 64;
    const uint32_t c0 = (wave * steps / 4) * 64, c1 = ((wave + 1) * steps / 4) * 64;
    float acc[MR][NC];
    gemv_bf16_sums<MR, NC>(a, wr, m, lda, c0, c1 < chunks ? c1 : chunks, acc);
    if ((lane & 15) == 0) {
#pragma unroll
        for (int r = 0; r < MR; r++)
#pragma unroll
            for (int j = 0; j < NC; j++) red[threadIdx.x >> 4][r][j] = acc[r][j];
    }
    __syncthreads();
    const uint32_t r = threadIdx.x / NC, j = threadIdx.x % NC;
    if (r < m) {
        float y = red[0][r][j];
        for (int q = 1; q < 16; q++) y += red[q][r][j];
        const size_t at = (size_t)r * ldc + col + j;
        if (res) y = bf16_bits_to_f32(f32_to_bf16_bits(y)) + bf16_bits_to_f32(res[at]);
        c[at] = (uint16_t)f32_to_bf16_bits(y);
    }
}

#define BF16_GEMV_KERNEL(MR, NC)                                                                                           \
    extern "C" __global__ __launch_bounds__(256) void fe_gemv_bf16_r##MR##_c##NC(uint16_t* c, const uint16_t* a,           \
                                                                                 const uint16_t* w, const uint16_t* res,  \
                                                                                 uint32_t m, uint32_t n, uint32_t k,      \
                                                                                 uint32_t lda, uint32_t ldc) {            \
        gemv_bf16_body<MR, NC>(c, a, w, res, m, n, k, lda, ldc);                                                           \
    }
#define BF16_GEMV_ROWS(MR) BF16_GEMV_KERNEL(MR, 1) BF16_GEMV_KERNEL(MR, 2) BF16_GEMV_KERNEL(MR, 4) BF16_GEMV_KERNEL(MR, 8)
BF16_GEMV_ROWS(1)
BF16_GEMV_ROWS(2)
BF16_GEMV_ROWS(4)
BF16_GEMV_ROWS(8)
