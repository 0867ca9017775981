// LDS-staged f16 MFMA GEMM core for prefill-sized M: C[256 x 256 tile] = A[M][K] (f16, row-major, from global) times a
// weight tile that a producer decodes into LDS as f16 [n][k]. 256 threads = 4 wavefronts in a 2 x 2 grid, each owning a
// 128 x 128 piece as 4 x 4 v_mfma_f32_32x32x16_f16 accumulators (256 accumulator registers a lane, one wavefront a
// SIMD). The large tile is what keeps the kernel off the memory system: a k tile of 64 brings 32 KB of activations and
// the packed weights of 256 columns from L2 for 64 MFMAs a wavefront (half the bytes per flop of a 256 x 128 tile), and
// moves 64 KB into and 128 KB out of LDS in the time of 2048 MFMA cycles. LDS holds two k tiles (one barrier per
// k tile). Rows of an LDS tile are 64 f16 = 8 chunks of 16 bytes, chunk c of row r stored at position
// c ^ (r & 7) ^ ((r >> 3) & 1) (gm_swz below), which leaves neither the tile writes nor the fragment reads a bank
// conflict (SQ_LDS_BANK_CONFLICT reads 0 for every GEMM kernel).
#pragma once
#include "kcommon.h"

#define GM_BM 256
#define GM_BN 256
#define GM_BK 64
#define GM_A_BYTES (GM_BM * GM_BK * 2)
#define GM_B_BYTES (GM_BN * GM_BK * 2)
#define GM_STAGE_BYTES (GM_A_BYTES + GM_B_BYTES)
#define GM_LDS_TILES (2 * GM_STAGE_BYTES)  // 128 KB
#define GM_EPI_PITCH 132                   // floats a row of a wavefront's 32 x 128 epilogue slab
#define GM_EPI_SLAB (32 * GM_EPI_PITCH * 4)

// Byte offset of 16-byte chunk c (0..7) of row r inside a [rows][64 f16] tile. The chunk is XORed with
// (r & 7) ^ ((r >> 3) & 1). A 16-byte write serves 8 consecutive lanes a cycle over 32 banks: lanes that hold 8
// consecutive rows at one chunk (the weight producers) need 8 different XOR values, which r & 7 gives. A 16-byte read
// serves 16 lanes a cycle over 64 banks, the lanes {0-3, 12-15, 20-27} or {4-11, 16-19, 28-31} of a half-wavefront
// (measured with two-lane probes): a fragment read has row = lane & 31 at one chunk, so those 16 rows need 16
// different (r & 1, XOR value) pairs. With r & 7 alone rows 0-3 and 24-27 (and 12-15, 20-23) collide, every fragment
// read takes 8 bank cycles instead of 4; flipping bit 0 for odd (r >> 3) separates them and keeps the writes clean.
__device__ __forceinline__ uint32_t gm_swz(uint32_t r, uint32_t c) {
    return r * 128 + ((c ^ (r & 7) ^ ((r >> 3) & 1)) << 4);
}

// Grouped raster: `group` row tiles (fastest) sweep all column tiles before the next group, so programs that run
// together share weight panels in L2 (kernels/k-fp4/src/lib.rs:298-308). Workgroups go to the 8 XCDs round-robin, so
// with a group of 8 row tiles each XCD's L2 keeps one 256-row panel of activations.
//
// group == 0 is the raster for weights that are large in memory (decoded fp16 tiles): column tiles are dealt to the XCDs
// instead, tile tn of a band of 8 to XCD tn % 8, all row tiles of it in turn, so that each weight panel is fetched into
// one L2 only and the (smaller) activations into all of them. A last band of fewer than 8 column tiles is swept column
// tile fastest.
__device__ __forceinline__ void gemm_raster(uint32_t pid, uint32_t tiles_m, uint32_t tiles_n, uint32_t group, uint32_t& tm,
                                            uint32_t& tn) {
    if (group == 0) {
        uint32_t bands = tiles_n / 8, in_bands = bands * 8 * tiles_m;
        if (pid < in_bands) {
            uint32_t q = pid / 8;
            tn = (q / tiles_m) * 8 + pid % 8;
            tm = q % tiles_m;
        } else {
            uint32_t r = tiles_n - bands * 8, idx = pid - in_bands;
            tn = bands * 8 + idx % r;
            tm = idx / r;
        }
        return;
    }
    uint32_t per_group = group * tiles_n;
    uint32_t first_m = (pid / per_group) * group;
    uint32_t gsize = tiles_m - first_m < group ? tiles_m - first_m : group;
    uint32_t r = pid % per_group;
    tm = first_m + r % gsize;
    tn = r / gsize;
}

// What a program computes on the one-piece schedule (the stream-K schedule is further down). Programs 0 .. full_tiles - 1
// take one output tile each over all of K. The remaining tiles
// (a last round that would leave most CUs idle) are cut `splits` ways along K: program full_tiles + i takes k tiles
// [kt0, kt0 + ktn) of tile full_tiles + i / splits and leaves its 256 x 256 f32 partial in slot i of the workspace; a
// reduce kernel adds the slots of a tile in split order and finishes it, so results do not depend on timing.
struct GemmWork {
    uint32_t tm, tn, kt0, ktn, slot;
    bool partial;
};

__device__ __forceinline__ GemmWork gemm_work(uint32_t pid, uint32_t tiles_m, uint32_t tiles_n, uint32_t group,
                                              uint32_t ktiles, uint32_t full_tiles, uint32_t splits) {
    GemmWork w;
    uint32_t tile = pid, split = 0, ns = 1;
    w.partial = pid >= full_tiles;
    w.slot = 0;
    if (w.partial) {
        w.slot = pid - full_tiles;
        tile = full_tiles + w.slot / splits;
        split = w.slot % splits;
        ns = splits;
    }
    gemm_raster(tile, tiles_m, tiles_n, group, w.tm, w.tn);
    w.kt0 = split * ktiles / ns;
    w.ktn = (split + 1) * ktiles / ns - w.kt0;
    return w;
}

// acc[i][j]: rows m0 + 128 wm + 32 i .., columns n0 + 128 wn + 32 j ..; lane L holds column L & 31, rows
// 8 (e >> 2) + 4 (L >> 5) + (e & 3) for element e of the 16. The producer supplies a register image Raw of its share of
// a weight k tile, load(kt, raw, half) (global -> the registers of half 0 or 1) and store(raw, Bs, part) for part 0, 1
// (decode that half of
// the share -> LDS tile of GM_BN rows, chunks placed with gm_swz), kQuarters (false; true: store_quarter(raw, Bs, q)
// for q = 0..3 instead of store, see below) and kStoreValu, about the number of VALU
// instructions of the two parts together.
//
// Schedule of one k tile (a wavefront runs alone on its SIMD, so the overlap is arranged inside the instruction stream):
// the registers that carry a tile from memory to LDS are reloaded with tile kt + 2 right after they are written out; the LDS writes of tile kt + 1 are issued between the MFMAs of tile kt; MFMA fragments are read from LDS one 16-wide k slice ahead. The barrier sits before the last slice, whose
// fragments are already in registers, so the first fragments of tile kt + 1 load under the last 16 MFMAs of tile kt.
// Loads past the end re-read the last tile / row and are never used: the loop body has no branches.
// BF16: the operands are bf16 (v_mfma_f32_32x32x16_bf16) instead of fp16; everything else is bytes and the same.
template <class Producer, bool BF16 = false>
__device__ __forceinline__ void gemm_mainloop(const _Float16* __restrict__ a, uint32_t lda, uint32_t m, uint32_t kt0,
                                              uint32_t ktiles, uint32_t m0, Producer& prod, unsigned char* lds,
                                              f32x16 (&acc)[4][4]) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // A: 256 rows x 8 chunks; thread t takes chunk t & 7 of rows (t >> 3) + 32 j. Byte offsets from `a` (< 4 GB, checked
    // by the host), so the address of a load is a uniform base plus a 32-bit lane offset.
    const uint32_t a_chunk = tid & 7, a_row = tid >> 3;
    uint32_t aoff[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        uint32_t row = m0 + a_row + 32 * j;
        row = row < m ? row : m - 1;
        aoff[j] = (row * lda + a_chunk * 8) * 2;
    }
    const unsigned char* abytes = (const unsigned char*)a + kt0 * (GM_BK * 2);  // k tiles kt0 .. kt0 + ktiles - 1
    u32x4 areg[8];
    auto load_a = [&](uint32_t kt, int j0, int j1) {
        kt = kt < ktiles ? kt : ktiles - 1;
        const unsigned char* ak = abytes + kt * (GM_BK * 2);
#pragma unroll
        for (int j = j0; j < j1; j++) areg[j] = *(const u32x4*)(ak + aoff[j]);
    };
    auto load_b = [&](typename Producer::Raw& r, uint32_t kt, int half) {
        prod.load(kt0 + (kt < ktiles ? kt : ktiles - 1), r, half);
    };
    const uint32_t a_st = gm_swz(a_row, a_chunk);  // + 32 j rows = + 4096 j bytes (the swizzle depends on row & 15 only)
    auto store_a = [&](unsigned char* st, int j0, int j1) {
#pragma unroll
        for (int j = j0; j < j1; j++) *(u32x4*)(st + a_st + 4096 * j) = areg[j];
    };
    // fragment addresses: row (lane & 31) of each 32-row piece, chunk 2 kk + (lane >> 5)
    const uint32_t fr = lane & 31, fc = lane >> 5;
    uint32_t foff[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) foff[kk] = gm_swz(fr, 2 * kk + fc);
    const uint32_t fa_base = wm * 128 * 128, fb_base = GM_A_BYTES + wn * 128 * 128;
    f16x8 fa[2][4], fb[2][4];
    auto read_frags = [&](int set, const unsigned char* st, int kk) {
#pragma unroll
        for (int i = 0; i < 4; i++) fa[set][i] = *(const f16x8*)(st + fa_base + 4096 * i + foff[kk]);
#pragma unroll
        for (int j = 0; j < 4; j++) fb[set][j] = *(const f16x8*)(st + fb_base + 4096 * j + foff[kk]);
    };
    auto mfmas = [&](int set) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                if constexpr (BF16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][i]),
                                                                         __builtin_bit_cast(bf16x8, fb[set][j]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
    };

    if constexpr (Producer::kQuarters) {
        // A producer whose decode is many vector ALU instructions (the trellis: about 240 a k tile and lane) spreads it
        // over all four slices, a quarter each (store_quarter(raw, Bs, q), q = 0..3), so that no slice has more of them
        // between two MFMAs than the matrix pipe covers. Quarter 0 of tile kt + 2 is decoded in slice 3 of tile kt, after
        // the barrier, into the stage that tile kt has just left; quarters 1..3 in slices 0..2 of tile kt + 1. Two
        // register images: `braw` of the tile whose quarters 1..3 are due, `bnext` of the one after it.
        constexpr int kValu = Producer::kStoreValu / 4 / 16 + 1;
        typename Producer::Raw braw, bnext;
        // (the scheduling barriers keep the loads of tile 1 in the order of the loop's own: weights, then activations.
        // The waits the compiler places in the loop are the stricter of those this order and the loop's need; with the
        // loads of the prologue interleaved, every k tile began by waiting for activation loads it had just issued.)
        load_b(braw, 0, 0);
        load_b(braw, 0, 1);
        load_a(0, 0, 8);
        load_b(bnext, 1, 0);
        load_b(bnext, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < 4; q++) prod.store_quarter(braw, lds + GM_A_BYTES, q);
        store_a(lds, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
        load_a(1, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
        prod.store_quarter(bnext, lds + GM_STAGE_BYTES + GM_A_BYTES, 0);
        braw = bnext;
        __syncthreads();
        read_frags(0, lds, 0);
        for (uint32_t kt = 0; kt < ktiles; kt++) {
            const unsigned char* cur = lds + (kt & 1) * GM_STAGE_BYTES;
            unsigned char* nxt = lds + ((kt + 1) & 1) * GM_STAGE_BYTES;
            // slice 0
            read_frags(1, cur, 1);
            prod.store_quarter(braw, nxt + GM_A_BYTES, 1);
            mfmas(0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // slice 1
            read_frags(0, cur, 2);
            prod.store_quarter(braw, nxt + GM_A_BYTES, 2);
            store_a(nxt, 0, 2);
            load_b(bnext, kt + 2, 0);
            load_b(bnext, kt + 2, 1);
            mfmas(1);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // slice 2
            read_frags(1, cur, 3);
            prod.store_quarter(braw, nxt + GM_A_BYTES, 3);
            store_a(nxt, 2, 8);
            mfmas(0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            // slice 3, with the first fragments of tile kt + 1 and the first quarter of tile kt + 2
            read_frags(0, nxt, 0);
            load_a(kt + 2, 0, 8);
            prod.store_quarter(bnext, lds + (kt & 1) * GM_STAGE_BYTES + GM_A_BYTES, 0);
            mfmas(1);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            braw = bnext;
        }
    } else {
        typename Producer::Raw braw;
        // (scheduling barriers: the loads of tile 1 in the loop's own order, weights then activations, see above)
        load_b(braw, 0, 0);
        load_b(braw, 0, 1);
        load_a(0, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < 2; p++) prod.store(braw, lds + GM_A_BYTES, p);
        store_a(lds, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
        load_b(braw, 1, 0);
        load_b(braw, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        load_a(1, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        read_frags(0, lds, 0);

        // One k tile: writes tile kt + 1 into the other LDS stage (weights from braw, half in each of the first two slices,
        // activations from areg, a quarter in the second and the rest in the third) and reloads the registers with tile kt + 2 in the slice after they are
        // written out, so that every slice carries a similar share of the memory instructions. The
        // sched_group_barrier sequences ask for one MFMA, then a few of the other instructions, and so on, so that memory
        // instructions are issued while the matrix pipe works instead of in bursts that hold back the next MFMA.
        for (uint32_t kt = 0; kt < ktiles; kt++) {
            const unsigned char* cur = lds + (kt & 1) * GM_STAGE_BYTES;
            unsigned char* nxt = lds + ((kt + 1) & 1) * GM_STAGE_BYTES;
            constexpr int kValu = Producer::kStoreValu / 2 / 16 + 1;  // vector ALU instructions between two MFMAs
            // slice 0
            read_frags(1, cur, 1);
            prod.store(braw, nxt + GM_A_BYTES, 0);
            mfmas(0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // slice 1
            read_frags(0, cur, 2);
            prod.store(braw, nxt + GM_A_BYTES, 1);
            store_a(nxt, 0, 2);  // a quarter of the activations' LDS writes here: slice 2 is the one bound by the LDS
            load_b(braw, kt + 2, 0);
            load_b(braw, kt + 2, 1);
            mfmas(1);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // slice 2
            read_frags(1, cur, 3);
            store_a(nxt, 2, 8);
            mfmas(0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            // slice 3, with the first fragments of tile kt + 1
            read_frags(0, nxt, 0);
            load_a(kt + 2, 0, 8);
            mfmas(1);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();  // the LDS tiles are free for the epilogue
}

// The same loop for 8-bit operands (e4m3 codes on both sides) on v_mfma_f32_32x32x64_f8f6f4: a k tile is 128 codes
// wide, so rows are again 128 bytes and tiles, swizzle, loads and LDS writes are those of gemm_mainloop; a lane's
// operand of one MFMA is 32 consecutive codes of its row (two 16-byte chunks), the k tile is two MFMA steps of 64.
// The k index inside an MFMA is a summation index only, and both operands are read with the same lane mapping.
// a: codes [m][lda] (bytes). The producer's store writes 128 code bytes a row (no expansion).
typedef int gm_i32x8 __attribute__((ext_vector_type(8)));
template <class Producer>
__device__ __forceinline__ void gemm_mainloop_f8(const uint8_t* __restrict__ a, uint32_t lda, uint32_t m, uint32_t kt0,
                                                 uint32_t ktiles, uint32_t m0, Producer& prod, unsigned char* lds,
                                                 f32x16 (&acc)[4][4]) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    const uint32_t a_chunk = tid & 7, a_row = tid >> 3;
    uint32_t aoff[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        uint32_t row = m0 + a_row + 32 * j;
        row = row < m ? row : m - 1;
        aoff[j] = row * lda + a_chunk * 16;
    }
    const unsigned char* abytes = (const unsigned char*)a + kt0 * 128;
    u32x4 areg[8];
    auto load_a = [&](uint32_t kt, int j0, int j1) {
        kt = kt < ktiles ? kt : ktiles - 1;
        const unsigned char* ak = abytes + kt * 128;
#pragma unroll
        for (int j = j0; j < j1; j++) areg[j] = *(const u32x4*)(ak + aoff[j]);
    };
    auto load_b = [&](typename Producer::Raw& r, uint32_t kt, int half) {
        prod.load(kt0 + (kt < ktiles ? kt : ktiles - 1), r, half);
    };
    const uint32_t a_st = gm_swz(a_row, a_chunk);
    auto store_a = [&](unsigned char* st, int j0, int j1) {
#pragma unroll
        for (int j = j0; j < j1; j++) *(u32x4*)(st + a_st + 4096 * j) = areg[j];
    };
    // fragment addresses: row (lane & 31) of each 32-row piece, chunks 4 kk + 2 (lane >> 5) and the next one
    const uint32_t fr = lane & 31, fc = lane >> 5;
    uint32_t foff[2][2];
#pragma unroll
    for (int kk = 0; kk < 2; kk++)
#pragma unroll
        for (int h = 0; h < 2; h++) foff[kk][h] = gm_swz(fr, 4 * kk + 2 * fc + h);
    const uint32_t fa_base = wm * 128 * 128, fb_base = GM_A_BYTES + wn * 128 * 128;
    gm_i32x8 fa[2][4], fb[2][4];
    auto read_one = [&](const unsigned char* p, int kk) {
        u32x4 lo = *(const u32x4*)(p + foff[kk][0]), hi = *(const u32x4*)(p + foff[kk][1]);
        return (gm_i32x8){(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };
    auto read_a = [&](int set, const unsigned char* st, int i0, int i1) {  // step kk = set
#pragma unroll
        for (int i = i0; i < i1; i++) fa[set][i] = read_one(st + fa_base + 4096 * i, set);
    };
    auto read_b = [&](int set, const unsigned char* st, int j0, int j1) {
#pragma unroll
        for (int j = j0; j < j1; j++) fb[set][j] = read_one(st + fb_base + 4096 * j, set);
    };
    // 8 MFMAs: rows i0, i0 + 1 of the wavefront's 4 x 4 pieces, first against columns 0, 1, then 2, 3
    auto mfmas = [&](int set, int i0) {
#pragma unroll
        for (int jh = 0; jh < 2; jh++)
#pragma unroll
            for (int i = i0; i < i0 + 2; i++)
#pragma unroll
                for (int j = 2 * jh; j < 2 * jh + 2; j++)  // formats 0, 0: e4m3 x e4m3; zero scale operands select the unscaled instruction
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0, 0, 0, 0);
    };

    typename Producer::Raw braw;
    // (scheduling barriers: the loads of tile 1 in the loop's own order, weights then activations, as in gemm_mainloop)
    load_b(braw, 0, 0);
    load_b(braw, 0, 1);
    load_a(0, 0, 8);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 2; p++) prod.store(braw, lds + GM_A_BYTES, p);
    store_a(lds, 0, 8);
    __builtin_amdgcn_sched_barrier(0);
    load_b(braw, 1, 0);
    load_b(braw, 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    load_a(1, 0, 8);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_a(0, lds, 0, 2);
    read_b(0, lds, 0, 4);

    // One k tile = two MFMA steps of 64, four slices of 8 MFMAs (64 cycles each). Every fragment is read a whole slice
    // before its first use (with four wavefronts queueing reads and writes the LDS answers hundreds of cycles late):
    // the slices that work on rows 0, 1 of a step read rows 2, 3 of it (4 reads) and carry the LDS writes of tile
    // kt + 1 (weights in the first, activations in the third); the slices on rows 2, 3 read the next step's rows 0, 1
    // and all its weight fragments (12 reads) and reload the registers just written out (issuing those loads right after
    // the writes, a slice earlier, made the writing slices longer by more than the loads' earlier arrival saved). The
    // barrier sits before the last slice, which starts on the fragments of tile kt + 1. Cycle stamps per k tile (2048
    // cycles of MFMAs): 705 / 508 / 555 / 494 and 137 at the barrier; the two slices that write LDS are bound by it
    // (8 writes and 4 reads a wavefront are 618 cycles of the LDS pipe for the four of them).
    for (uint32_t kt = 0; kt < ktiles; kt++) {
        const unsigned char* cur = lds + (kt & 1) * GM_STAGE_BYTES;
        unsigned char* nxt = lds + ((kt + 1) & 1) * GM_STAGE_BYTES;
        // slice 0: step 0, rows 0, 1
        read_a(0, cur, 2, 4);
        prod.store(braw, nxt + GM_A_BYTES, 0);
        prod.store(braw, nxt + GM_A_BYTES, 1);
        mfmas(0, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // slice 1: step 0, rows 2, 3
        read_a(1, cur, 0, 2);
        read_b(1, cur, 0, 4);
        load_b(braw, kt + 2, 0);
        load_b(braw, kt + 2, 1);
        mfmas(0, 2);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // slice 2: step 1, rows 0, 1
        read_a(1, cur, 2, 4);
        store_a(nxt, 0, 8);
        mfmas(1, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        // slice 3: step 1, rows 2, 3, with the first fragments of tile kt + 1
        read_a(0, nxt, 0, 2);
        read_b(0, nxt, 0, 4);
        load_a(kt + 2, 0, 8);
        mfmas(1, 2);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();  // the LDS tiles are free for the epilogue
}

// Hands the wavefront's 128 x 128 accumulators out row by row: 32 rows at a time pass through the wavefront's own LDS
// slab (GM_EPI_SLAB bytes at lds + wave * GM_EPI_SLAB) so that 32 consecutive lanes hold 128 consecutive columns of one
// row, 4 a lane. Both halves of the wavefront work on a row of their own. Four row pairs are in flight together:
// transform(v[4][4], l32) works on all four at once (it must not branch, so that its cross-lane exchanges overlap),
// after that store(row in 0..127, l32, v[4]) is called for each. No workgroup barrier: only this
// wavefront touches its slab.
// Orders the wavefront's own LDS writes before its own LDS reads (and the other way round): the lanes of a wavefront
// issue their LDS instructions together and the LDS executes them in order, so only the compiler has to be kept from
// moving accesses across this point. (A workgroup-scope fence would also wait for the global stores in flight, once
// per 32 rows.)
__device__ __forceinline__ void gm_slab_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

template <class Transform, class Store>
__device__ __forceinline__ void gemm_epilogue(f32x16 (&acc)[4][4], unsigned char* lds, Transform transform, Store store) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, hw = lane >> 5;
    float* slab = (float*)(lds + wave * GM_EPI_SLAB);
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                slab[(8 * (e >> 2) + 4 * hw + (e & 3)) * GM_EPI_PITCH + 32 * j + l32] = acc[i][j][e];
        gm_slab_sync();
        for (int rr = 0; rr < 16; rr += 4) {
            float v[4][4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                f32x4 t = *(const f32x4*)(slab + (2 * (rr + u) + hw) * GM_EPI_PITCH + 4 * l32);
                v[u][0] = t[0], v[u][1] = t[1], v[u][2] = t[2], v[u][3] = t[3];
            }
            transform(v, l32);
#pragma unroll
            for (int u = 0; u < 4; u++) store(32 * i + 2 * (rr + u) + hw, l32, v[u]);
        }
        gm_slab_sync();
    }
}

#define GM_PART_FLOATS (GM_BM * GM_BN)  // floats of one partial slot

// Leaves the program's accumulators in its partial slot, row-major [256][256] f32.
__device__ __forceinline__ void gemm_store_partial(f32x16 (&acc)[4][4], unsigned char* lds, float* slot) {
    const uint32_t wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
    gemm_epilogue(
        acc, lds, [](float (&)[4][4], uint32_t) {},
        [&](uint32_t row, uint32_t l32, float (&v)[4]) {
            *(f32x4*)(slot + (wm * 128 + row) * GM_BN + wn * 128 + 4 * l32) = (f32x4){v[0], v[1], v[2], v[3]};
        });
}

// Body of a reduce kernel: grid (tiles cut along K) * 64, 256 threads. Each half wavefront sums the `splits` slots of one
// row of one 128-column half of a tile, 4 columns a lane, in split order, and hands them to fn(t, row in 0..255,
// column half, l32, v[4]) with t the tile's index among the cut tiles.
template <class RowFn>
__device__ __forceinline__ void gemm_reduce_rows(const float* __restrict__ part, uint32_t splits, RowFn fn) {
    const uint32_t t = blockIdx.x >> 6, hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
    const uint32_t row = 4 * (blockIdx.x & 63) + (hw >> 1), cb = hw & 1;
    const float* p = part + (size_t)t * splits * GM_PART_FLOATS + row * GM_BN + cb * 128 + 4 * l32;
    f32x4 sum = *(const f32x4*)p;
    for (uint32_t sp = 1; sp < splits; sp++) sum += *(const f32x4*)(p + (size_t)sp * GM_PART_FLOATS);
    float v[4] = {sum[0], sum[1], sum[2], sum[3]};
    fn(t, row, cb, l32, v);
}

// ---- Stream-K schedule -------------------------------------------------------------------------------------------------
// The tiles' k tiles, laid end to end in raster order (tile-major, K ascending), are one sequence of units; program p of P
// takes the contiguous run of base = units / P of them (+ 1 for the first units % P programs), so every program does the
// same work to within one k tile whatever the tile count, and there is no mostly empty last round and no reduce launch.
// A run crosses tile boundaries: each piece of a tile (segment) is one pass of the main loop. A tile that lies in one
// run is finished there. Otherwise its pieces meet through the workspace: a piece that is not the last to arrive leaves
// its accumulators in a slot (two slots a program: one for a run's first segment, one for its last) and bumps the tile's
// arrival counter; the piece whose arrival completes the count adds the pieces in piece order, starting from zero, with
// its own accumulators in their place, and finishes the tile: the sums do not depend on which piece came last. The
// hand-off is the decode GEMV's: write-through stores, acknowledged, then a relaxed agent-scope atomic; the reader's loads
// bypass its L2; counters return to zero.
#define GM_PART_BYTES (GM_PART_FLOATS * 4)

__device__ __forceinline__ uint32_t sk_start(uint32_t p, uint32_t base, uint32_t rem) { return p * base + (p < rem ? p : rem); }
// the program whose run holds unit u
__device__ __forceinline__ uint32_t sk_owner(uint32_t u, uint32_t base, uint32_t rem) {
    const uint32_t big = rem * (base + 1);
    return u < big ? u / (base + 1) : rem + (u - big) / base;
}

// Program p has worked through k tiles of tile `tile` (units t0 .. t0 + ktiles - 1) that other programs share. Returns
// true if this program finishes the tile, with the sum of all pieces in acc; false if it has left its piece in the
// workspace. Every branch is uniform over the workgroup. lds: free (the main loop ended with a barrier).
__device__ __forceinline__ bool gemm_sk_meet(f32x16 (&acc)[4][4], uint32_t p, uint32_t tile, uint32_t t0, uint32_t ktiles,
                                             uint32_t base, uint32_t rem, float* part, uint32_t part_bytes, uint32_t* counters,
                                             unsigned char* lds) {
    const uint32_t tid = threadIdx.x;
    const uint32_t first = sk_owner(t0, base, rem), last = sk_owner(t0 + ktiles - 1, base, rem);
    const uint32_t n = last - first + 1, me = p - first;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)part, 0, part_bytes, 0x00020000);
    volatile uint32_t* flag = (volatile uint32_t*)lds;
    uint32_t* cnt = counters + tile;
    // a run's piece of a tile in which the run does not begin is the run's last segment
    auto slot_of = [&](uint32_t q) { return 2 * q + (sk_start(q, base, rem) < t0 ? 1u : 0u); };
    // (a read-modify-write, which is performed where all XCDs meet: no stale copy of the counter can answer it)
    if (tid == 0) *flag = __hip_atomic_fetch_add(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    uint32_t seen = *flag;
    __syncthreads();
    if (seen != n - 1) {  // someone is still at work: leave the piece
        const uint32_t so = slot_of(p) * GM_PART_BYTES;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const f32x4 v = {acc[i][j][4 * e], acc[i][j][4 * e + 1], acc[i][j][4 * e + 2], acc[i][j][4 * e + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rs, tid * 16,
                                                           so + ((i * 4 + j) * 4 + e) * 4096, 16);
                }
        agent_stores_wait();
        __syncthreads();
        if (tid == 0) *flag = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        seen = *flag;
        __syncthreads();
        if (seen != n - 1) return false;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f32x4 t[16];
#pragma unroll
        for (int c = 0; c < 16; c++) t[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        for (uint32_t q = 0; q < n; q++) {
            if (q == me) {
#pragma unroll
                for (int c = 0; c < 16; c++)
                    t[c] += (f32x4){acc[i][c >> 2][4 * (c & 3)], acc[i][c >> 2][4 * (c & 3) + 1], acc[i][c >> 2][4 * (c & 3) + 2],
                                    acc[i][c >> 2][4 * (c & 3) + 3]};
            } else {
                const uint32_t so = slot_of(first + q) * GM_PART_BYTES + i * 16 * 4096;
                f32x4 ld[16];
#pragma unroll
                for (int c = 0; c < 16; c++) ld[c] = load_agent_f32x4(rs, tid * 16, so + c * 4096);
#pragma unroll
                for (int c = 0; c < 16; c++) t[c] += ld[c];
            }
        }
#pragma unroll
        for (int c = 0; c < 16; c++)
#pragma unroll
            for (int x = 0; x < 4; x++) acc[i][c >> 2][4 * (c & 3) + x] = t[c][x];
    }
    if (tid == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// How a GEMM launch is spread over its programs. sk_base == 0: one piece a program (gemm_work: whole tiles, then the
// cut tiles, whose partials a reduce kernel adds). Otherwise stream-K: grid = the programs; the first full_tiles tiles (a
// multiple of the grid) are computed whole, round-robin, and the tiles after them are shared as runs of sk_base (+ 1 for
// the first sk_rem) k tiles; part holds two slots a program, counters one word a tile, zero at rest.
struct GemmSched {
    uint32_t full_tiles, splits, sk_base, sk_rem;
    float* part;
    uint32_t part_bytes;
    uint32_t* counters;
};

// Runs the program's share of the schedule: main(tm, tn, kt0, ktn, acc) is one pass of the main loop over k tiles
// kt0 .. kt0 + ktn - 1 of tile (tm, tn), finish(tm, tn, acc) the tile's epilogue. One call site of each, whatever the
// schedule. SK picks the schedule at compile time (a kernel that holds both spills around its 256 accumulators):
// sc.sk_base must be nonzero exactly when SK.
template <bool SK, class Main, class Finish>
__device__ __forceinline__ void gemm_schedule(const GemmSched& sc, uint32_t tiles_m, uint32_t tiles_n, uint32_t group,
                                              uint32_t ktiles, unsigned char* lds, Main main, Finish finish) {
    const uint32_t p = blockIdx.x;
    f32x16 acc[4][4];
    if constexpr (!SK) {
        const GemmWork wk = gemm_work(p, tiles_m, tiles_n, group, ktiles, sc.full_tiles, sc.splits);
        main(wk.tm, wk.tn, wk.kt0, wk.ktn, acc);
        if (wk.partial)
            gemm_store_partial(acc, lds, sc.part + (size_t)wk.slot * GM_PART_FLOATS);
        else
            finish(wk.tm, wk.tn, acc);
    } else {
        // the first sc.full_tiles tiles (a multiple of the grid) are taken whole, program p those p, p + grid, ...; the
        // runs are laid over the tiles after them
        const uint32_t whole = sc.full_tiles;
        uint32_t next_whole = p;
        uint32_t u = sk_start(p, sc.sk_base, sc.sk_rem);
        const uint32_t uend = sk_start(p + 1, sc.sk_base, sc.sk_rem);
        while (next_whole < whole || u < uend) {
            uint32_t tile, t0 = 0, kt0 = 0, ktn = ktiles;
            if (next_whole < whole) {
                tile = next_whole;
                next_whole += gridDim.x;
            } else {
                const uint32_t rel = u / ktiles;
                t0 = rel * ktiles, kt0 = u - t0;
                ktn = ktiles - kt0 < uend - u ? ktiles - kt0 : uend - u;
                tile = whole + rel;
                u += ktn;
            }
            uint32_t tm, tn;
            gemm_raster(tile, tiles_m, tiles_n, group, tm, tn);
            __syncthreads();  // the epilogue of the segment before is done with the LDS
            main(tm, tn, kt0, ktn, acc);
            bool fin = true;
            if (ktn != ktiles)
                fin = gemm_sk_meet(acc, p, tile, t0, ktiles, sc.sk_base, sc.sk_rem, sc.part, sc.part_bytes, sc.counters, lds);
            if (fin) finish(tm, tn, acc);
        }
    }
}
