// Shared by the host-side sources of libferrite_amd: error plumbing, device buffers, embedded code objects.
#pragma once
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <cstdlib>

#include "fe_hip.h"

int fe_set_error(int code, const char *call, const char *detail);
int fe_check_hip(int code, const char *call);

#define FE_TRY(x)            \
    do {                     \
        int _c = (x);        \
        if (_c) return _c;   \
    } while (0)

// gfx950 code objects linked into the library (fe_embed.S)
extern "C" const unsigned char fe_k_exl3_hsaco[];
extern "C" const unsigned char fe_k_exl3_hsaco_end[];
extern "C" const unsigned char fe_k_fp4_hsaco[];
extern "C" const unsigned char fe_k_fp4_hsaco_end[];
extern "C" const unsigned char fe_k_route_hsaco[];
extern "C" const unsigned char fe_k_route_hsaco_end[];
extern "C" const unsigned char fe_k_bf16_hsaco[];
extern "C" const unsigned char fe_k_bf16_hsaco_end[];

// The embedded image, or the file the environment variable names.
int fe_load_module(fe_module_t *out, const char *env, const unsigned char *begin, const unsigned char *end);

// Device memory owned until destruction, or a borrowed view (DeviceBuffer / DeviceBuffer::view,
// crates/fe-cuda/src/lib.rs:201-297).
struct FeBuf {
    fe_devptr_t p = 0;
    size_t bytes = 0;
    bool owned = false;
    FeBuf() = default;
    FeBuf(const FeBuf &) = delete;
    FeBuf &operator=(const FeBuf &) = delete;
    ~FeBuf() { release(); }
    int alloc(size_t n) {
        release();
        FE_TRY(fe_hip_malloc(&p, n));
        bytes = n;
        owned = true;
        return 0;
    }
    int zeroed(size_t n) {
        FE_TRY(alloc(n));
        if (fe_hip_zero_alloc_on()) return 0;  // fe_hip_malloc has cleared the block and synchronized
        FE_TRY(fe_hip_memset_d8(p, 0, n, nullptr));
        return fe_hip_synchronize();
    }
    int from_host(const void *src, size_t n) {
        FE_TRY(alloc(n));
        return fe_hip_memcpy_htod(p, src, n);
    }
    void view(fe_devptr_t q, size_t n) {
        release();
        p = q;
        bytes = n;
        owned = false;
    }
    void release() {
        if (owned && p) fe_hip_free(p);
        p = 0;
        bytes = 0;
        owned = false;
    }
};

// forward() of an EXL3 linear for at most max_rows rows over caller-provided device memory instead of a workspace object:
// arrival counters (zero at rest), rotated inputs, split partial sums. Sizes that do not fit are FE_ERR_WORKSPACE.
// Allocates nothing. (fe_exl3.cpp; used by fe_exl3_linear_forward_static.)
struct fe_exl3_linear;
struct fe_exl3_kernels;
int fe_exl3_forward_over(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype,
                         fe_devptr_t y, int y_dtype, uint32_t rows, uint32_t max_rows, fe_devptr_t counters,
                         size_t counters_bytes, fe_devptr_t xh, size_t xh_bytes, fe_devptr_t z, size_t z_bytes, const char *fn);
// Looks up the static scratch array of fe_exl3_linear_forward_static on the current device and clears its counters
// (fe_exl3_static.hip); fe_hip_init calls it for the device it binds.
int fe_exl3_static_setup_current_device();

// How the prefill GEMM's output tiles (256 x 256) are spread over the CUs: `full` tiles are computed whole, one per
// program; the `tiles - full` tiles of a last, mostly empty round are each cut `splits` ways along K (partials in a
// workspace, then a reduce kernel). splits == 1 means nothing is cut (full == tiles).
struct FeGemmSplit {
    uint32_t tiles = 0, full = 0, splits = 1;
    uint32_t programs() const { return full + (tiles - full) * splits; }
    uint32_t cut() const { return tiles - full; }
};
constexpr size_t kFeGemmPartBytes = 256 * 256 * 4;  // one partial slot
constexpr uint32_t kFeGemmSlotsPerCu = 2;           // slots a workspace holds per CU
// The cut that finishes the last round soonest: s pieces a tile take ceil(rem s / cus) rounds of 1 / s of a tile's time;
// every piece also writes its 256 KB partial and the reduce kernel reads it back (about 2 % of a tile's time a piece).
// At most `slots` pieces in all and `cap` a tile (1: never cut).
inline FeGemmSplit fe_gemm_split(uint32_t tiles, uint32_t ktiles, uint32_t cus, uint32_t slots, uint32_t cap = 8) {
    FeGemmSplit g;
    g.tiles = g.full = tiles;
    if (!cus || !slots) return g;
    const uint32_t rem = tiles % cus;
    if (rem == 0) return g;
    cap = std::min(cap, ktiles / 4);                                        // at least 4 k tiles a program
    cap = std::min(cap, slots / rem);
    uint32_t best = 1;
    float best_cost = 1.0f;
    for (uint32_t sp = 2; sp <= cap; sp++) {
        const float cost = (float)((rem * sp + cus - 1) / cus) / (float)sp + 0.02f * (float)sp;
        if (cost < best_cost - 1e-6f) best = sp, best_cost = cost;
    }
    if (best < 2) return g;
    g.full = tiles - rem;
    g.splits = best;
    return g;
}

// The schedule argument of the GEMM kernels (GemmSched of kernels/gemm_core.h) and what to launch with it.
struct FeGemmSchedArgs {
    uint32_t full_tiles, splits, sk_base, sk_rem;
    fe_devptr_t part;
    uint32_t part_bytes, pad_;
    fe_devptr_t counters;
};
struct FeGemmSchedule {
    FeGemmSplit split;     // the one-piece schedule (when !stream_k): its cut tiles need the reduce launch
    FeGemmSchedArgs args;
    uint32_t programs = 0;
    bool stream_k = false;
};
// mode 0: always one piece a program. mode 2: runs over all tiles wherever the workspace allows, mode 3: as many whole
// rounds as leave runs that are in step (both for tests). mode 1: stream-K where it is the faster schedule, as measured
// (MI355X, NVFP4, FP8 and EXL3, 20..1088 tiles). It pays where the one-piece schedule cannot fill its last round: the
// tiles of that round (all tiles when there are fewer than CUs) then run as runs over all CUs, behind the whole rounds.
// Taken when the one-piece schedule cuts those tiles (tiles that run whole in one partly filled round are left alone:
// 192 or 224 tiles on as many CUs clock higher under the power limit, stream-K loses 1..12 % there), a tile has at most
// three pieces (runs of at least half a tile: the piece that arrives last adds the others alone, about 5 us a piece; 32
// tiles of 8 pieces: 74 against 39 us), and either
//  (a) the cut leaves a partly filled round and the runs are equal and in step, programs 8 apart (the same XCD) at the same
//      depth of K at the same time, so that they share panels in their L2 (160 tiles on 256 CUs, 2048 rows x 5120
//      columns: NVFP4 300 -> 284 us, FP8 166 -> 154, EXL3 over kept tiles 358 -> 352, decoding 393 -> 363), or
//  (b) small weight operand only (small_b: packed weights of a few KB a k tile; NVFP4, the decoding EXL3 GEMM): the cut
//      loses 12 % or more to its rounds, whether or not the runs are in step (129..160 tiles: three pieces a tile, a
//      second round half empty; NVFP4 +14..27 %, EXL3 +11..15 %; 1536 rows x 17408 columns = 256 whole + 152: 241 -> 227
//      us). Where it loses 7 % (120 or 240 tiles) stream-K loses 9..20 %: programs that are not in step stream their
//      operands past the L2.
// With a whole number of rounds stream-K and the one-piece schedule are within 1 % of each other: one piece a program.
// Whole rounds and runs that are in step over more than the last round (576 tiles as 256 + runs of 100 k tiles) spare the
// reduce launch and are 1..3 % faster: taken for a small weight operand, (c) below; (d) and (e) below are two more cases
// of a small weight operand, runs over all tiles behind no whole round.
// With decoded fp16 tiles or FP8 codes as the weight operand (32 KB a k tile) runs behind whole rounds lose 4..9 %.
// Needs two partial slots a program and a zeroed counter a tile.
constexpr uint32_t kFeXcds = 8;
inline FeGemmSchedule fe_gemm_schedule(uint32_t tiles, uint32_t ktiles, uint32_t cus, fe_devptr_t part, size_t part_bytes,
                                       fe_devptr_t counters, size_t counters_len, uint32_t cap, int mode, bool small_b) {
    FeGemmSchedule r;
    const uint32_t slots = (uint32_t)(part_bytes / kFeGemmPartBytes);
    r.split = fe_gemm_split(tiles, ktiles, cus, slots, cap);
    r.programs = r.split.programs();
    r.args = {r.split.full, r.split.splits, 0, 0, part, (uint32_t)std::min<size_t>(part_bytes, 0xffffffffu), 0, counters};
    const uint32_t programs = std::min<uint32_t>({cus, tiles * ktiles, slots / 2});
    if (!mode || !programs || !counters || tiles > counters_len || (uint64_t)tiles * ktiles >= (1ull << 31) ||
        (size_t)programs * 2 * kFeGemmPartBytes > 0xffffffffu)
        return r;
    // whole rounds first (mode 3, and mode 1 where it pays), the runs over the tiles after them
    uint32_t whole = 0, base = 0, rem = 0;
    auto runs = [&](uint32_t rounds) {
        whole = rounds * programs;
        const uint32_t units = (tiles - whole) * ktiles;
        base = units / programs, rem = units % programs;
    };
    auto good = [&]() { return rem == 0 && 2 * base >= ktiles && (kFeXcds * base) % ktiles == 0; };
    auto most_whole_rounds = [&](uint32_t at_least) {
        for (uint32_t rounds = tiles / programs + 1; rounds-- > at_least;) {
            runs(rounds);
            if (base > 0 && good()) return true;
        }
        return false;
    };
    runs(0);
    if (mode == 1) {
        // the tiles of the last, partly filled round (all tiles when there are fewer than CUs): are runs over them worth it?
        const uint32_t last = tiles % cus;
        bool take = false;
        // (e) small weight operand, short K (up to 128 k tiles), between one and 2 1/8 rounds with a cut last round of at
        // most 5/8 of the CUs: equal runs over all tiles, in step, instead of whole rounds with runs behind them or a cut
        // (every tile then has two pieces, but the programs reach their tile ends at different times; behind a whole round
        // all of them meet at once). 5120-wide K, NVFP4 / decoding EXL3, us: 320 tiles 184.5 -> 181 / 235.5 -> 230; 384:
        // 213 -> 204.5 / 265.5 -> 263; 416: 238 -> 232 / 302 -> 292.5; 544: 286 -> 284.7 / 364 -> 356.5. With a fuller last
        // round (448 tiles: 248 -> 250 / 315 -> 320), from 2 1/4 rounds on (576, 640, 1088 tiles) and with 272 k tiles a tile
        // (320 tiles: 675 -> 728) it loses 1..8 %: not taken.
        if (small_b && last && 8 * last <= 5 * cus && tiles > cus && 8 * tiles <= 17 * cus && ktiles <= 128 &&
            r.split.splits > 1 && programs == cus) {
            runs(0);
            take = good() && base >= 64;
        }
        if (!take && last && (tiles < cus || small_b)) {
            runs(tiles / cus);
            // what the one-piece schedule loses to its partly filled rounds, as a fraction of the balanced time
            const uint32_t sp = r.split.splits;
            const float one_piece = (float)((last * sp + cus - 1) / cus) / (float)sp, balanced = (float)last / (float)cus;
            const float gain = one_piece / balanced - 1.0f;
            take = programs == cus && 2 * base >= ktiles && sp > 1 && ((good() && gain > 0.0f) || (small_b && gain >= 0.12f));
        }
        // (c) small weight operand, a cut last round of too many pieces a tile: one whole round fewer, so that the runs are
        // longer, if they are then in step (576 tiles = 256 whole + runs of 100 k tiles over 320: no reduce launch, NVFP4
        // 312 -> 309 us, EXL3 404 -> 392). A last round that runs whole (480 tiles: 224 on as many CUs) is left alone: runs
        // of 70 behind a whole round are 2..4.5 % slower there.
        if (!take && small_b && last && tiles > cus && r.split.splits > 1) take = most_whole_rounds(1);
        // (d) small weight operand, one whole round and a last round of few tiles (an eighth of the CUs or fewer), which (c)
        // cannot turn into runs in step: runs over all tiles, if they are equal, at least a tile long (two pieces a tile)
        // and keep the programs of an XCD at no more than two depths of K at a time. 272 tiles of 80 k tiles (1024 rows x
        // 17408 columns; the one-piece schedule cuts the 16 tiles 7 ways and adds a reduce launch), runs of 85: EXL3
        // 199.5 -> 190.8 us, NVFP4 155.0 -> 154.3; 288 tiles, runs of 90: EXL3 211 -> 201, NVFP4 165 -> 162. Behind a
        // second whole round (528 tiles as 256 + runs of 85) nothing is gained: not taken.
        if (!take && small_b && last && tiles > cus && tiles < 2 * cus && 8 * last <= cus && r.split.splits > 1 &&
            programs == cus) {
            runs(0);
            const uint32_t step = (kFeXcds * base) % ktiles;
            take = rem == 0 && base >= ktiles && base >= 64 && (step == 0 || 2 * step == ktiles);
        }
        if (!take) return r;
    } else if (mode >= 3 && !most_whole_rounds(0)) {
        return r;
    }
    if (base == 0 || (base >= ktiles && rem == 0 && base % ktiles == 0 && whole == 0)) return r;  // whole tiles only: nothing to gain
    r.stream_k = true;
    r.programs = programs;
    r.args.full_tiles = whole;
    r.args.sk_base = base, r.args.sk_rem = rem;
    return r;
}
