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
