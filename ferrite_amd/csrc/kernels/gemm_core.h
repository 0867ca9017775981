// LDS-staged f16 MFMA GEMM core for prefill-sized M: C[128 x 128 tile] = A[M][K] (f16, row-major, from global) times a
// weight tile that a producer decodes into LDS as f16 [n][k]. 256 threads = 4 wavefronts in a 2 x 2 grid, each owning a
// 64 x 64 piece as 2 x 2 v_mfma_f32_32x32x16_f16 accumulators. The next k tile's global loads are issued before the
// current tile's MFMAs, so memory latency overlaps the matrix work.
#pragma once
#include "kcommon.h"

#define GM_BM 128
#define GM_BN 128
#define GM_BK 64
#define GM_PITCH 72  // f16 elements a row of an LDS tile: 64 + 8 pad (16-byte aligned rows, bank spread)
#define GM_LDS_TILES (2 * GM_BM * GM_PITCH * 2)  // bytes of the A and B tiles

// Grouped raster: `group` row tiles (fastest) sweep all column tiles before the next group, so programs that run
// together share weight panels in L2 (kernels/k-fp4/src/lib.rs:298-308).
__device__ __forceinline__ void gemm_raster(uint32_t pid, uint32_t tiles_m, uint32_t tiles_n, uint32_t group, uint32_t& tm,
                                            uint32_t& tn) {
    uint32_t per_group = group * tiles_n;
    uint32_t first_m = (pid / per_group) * group;
    uint32_t gsize = tiles_m - first_m < group ? tiles_m - first_m : group;
    uint32_t r = pid % per_group;
    tm = first_m + r % gsize;
    tn = r / gsize;
}

// acc[i][j]: rows m0 + 64 wm + 32 i .., columns n0 + 64 wn + 32 j ..; lane L holds column L & 31, rows
// 8 (e >> 2) + 4 (L >> 5) + (e & 3) for element e of the 16.
template <class Producer>
__device__ __forceinline__ void gemm_mainloop(const _Float16* __restrict__ a, uint32_t lda, uint32_t m, uint32_t k,
                                              uint32_t m0, Producer& prod, unsigned char* lds, f32x16 (&acc)[2][2]) {
    _Float16* As = (_Float16*)lds;
    _Float16* Bs = As + GM_BM * GM_PITCH;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // A: 128 rows x 8 chunks of 16 bytes; thread t takes chunk t & 7 of rows (t >> 3) + 32 j
    const uint32_t a_chunk = tid & 7, a_row = tid >> 3;
    u32x4 areg[4];
    auto load_a = [&](uint32_t kt) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t row = m0 + a_row + 32 * j;
            if (row < m)
                areg[j] = *(const u32x4*)(a + (size_t)row * lda + kt * GM_BK + a_chunk * 8);
            else
                areg[j] = (u32x4){0, 0, 0, 0};
        }
    };
    auto store_a = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) *(u32x4*)(As + (a_row + 32 * j) * GM_PITCH + a_chunk * 8) = areg[j];
    };

    const uint32_t ktiles = k / GM_BK;
    load_a(0);
    prod.load(0);
    for (uint32_t kt = 0; kt < ktiles; kt++) {
        store_a();
        prod.store(Bs);
        __syncthreads();
        if (kt + 1 < ktiles) {
            load_a(kt + 1);
            prod.load(kt + 1);
        }
#pragma unroll
        for (int kk = 0; kk < GM_BK / 16; kk++) {
            f16x8 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                af[i] = *(const f16x8*)(As + (wm * 64 + 32 * i + (lane & 31)) * GM_PITCH + kk * 16 + 8 * (lane >> 5));
#pragma unroll
            for (int j = 0; j < 2; j++)
                bf[j] = *(const f16x8*)(Bs + (wn * 64 + 32 * j + (lane & 31)) * GM_PITCH + kk * 16 + 8 * (lane >> 5));
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
}
