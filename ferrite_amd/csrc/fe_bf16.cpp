// fe_bf16: host side of the plain bf16 linear (see include/fe_bf16.h). Follows crates/fe-model/src/model.rs:310-345;
// the kernels are ferrite_amd/csrc/kernels/k_bf16.hip.
#include "fe_bf16.h"

#include <cstdio>
#include <cstdlib>

#include "fe_exl3.h"  // error codes
#include <string>

#include "fe_internal.h"

namespace {
constexpr uint32_t kGemmLds = 2 * (256 + 256) * 64 * 2;  // GM_LDS_TILES
constexpr uint32_t kTileM = 256, kTileN = 256;           // GM_BM, GM_BN
constexpr uint32_t kGemvRows = 8;                        // rows of one GEMV pass (model.rs:326)
constexpr uint32_t kSmallBatch = 16;                     // X3_ROWS: batches up to here are decode rows (model.rs:172)
}  // namespace

struct fe_bf16_kernels {
    fe_module_t module = nullptr;
    fe_function_t gemm = nullptr, reduce = nullptr, swiglu = nullptr, swiglu_reduce = nullptr, interleave = nullptr;
    fe_function_t gemv[4][4] = {};  // [rows 1, 2, 4, 8][columns of a program 1, 2, 4, 8]
    uint32_t cus = 0;
    FeBuf part;
    // Switches, read from the environment once at load (fe_bf16_kernels_set_option changes them afterwards)
    int32_t nc = -1;           // columns a GEMV program takes (1, 2, 4, 8); -1 = by the shape (FE_BF16_NC)
    int32_t raster_group = -1; // raster group of the GEMM; -1 = by the shape (FE_BF16_GROUP)
    uint32_t gemm_splits = 8;  // most pieces a cut output tile takes (FE_GEMM_SPLITS; 1: never cut)
};

// log2 of the columns a GEMV program takes. Measured on 5120 x 17408, 17408 x 5120 and 5120 x 5120: 4 columns are best
// for 1 and 2 rows (5120 x 17408: 29 us at 1 row), 8 for 3..8 rows of a wide linear (31.7 against 33.8 us at 4 rows,
// 42.6 against 43.8 at 8; one column: 83 us at 8 rows); narrow linears take fewer so that the grid still has a few
// programs a CU.
static int gemv_cols(uint32_t n, int form) { return n >= 8192 && form >= 2 ? 3 : n >= 4096 ? 2 : n >= 1024 ? 1 : 0; }

// Raster of the GEMM's output tiles (gemm_raster). Weights at least as large as the activations: column tiles are dealt
// to the XCDs (group 0), each weight panel through one L2, the smaller activations through all of them; else row tiles
// in groups of 8. Measured at M = 2048 in alternation with groups of 8: 5120 x 17408 323 against 344 us,
// 17408 x 5120 342 against 365 us, 5120 x 34816 618 against 648 us.
static uint32_t bf16_raster_group(uint32_t m, uint32_t n, uint32_t k, uint32_t tiles_m) {
    (void)k;
    return n >= m ? 0 : tiles_m < 8 ? tiles_m : 8;
}

static int check(const char *fn, fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda, fe_devptr_t w, fe_devptr_t res,
                 uint32_t n, uint32_t k) {
    if (!y || !x || !w) return fe_set_error(FE_ERR_ARG, fn, "null pointer");
    if (!n || !k || n % 8 || k % 64) {
        char msg[120];
        snprintf(msg, sizeof msg, "bf16 linear n %u k %u (n %% 8 == 0, k %% 64 == 0)", n, k);
        return fe_set_error(FE_ERR_SHAPE, fn, msg);
    }
    if (lda % 8 || lda < k || x % 16 || w % 16) return fe_set_error(FE_ERR_ARG, fn, "x / w rows must be 16-byte aligned, lda >= k");
    if (ldy % 4 || ldy < n || y % 8 || (res && res % 8)) return fe_set_error(FE_ERR_ARG, fn, "y / res rows must be 8-byte aligned, ldy >= n");
    return 0;
}

extern "C" {

int fe_bf16_kernels_load(fe_bf16_kernels **out) {
    if (!out) return fe_set_error(FE_ERR_ARG, "fe_bf16_kernels_load", "null out");
    auto *k = new fe_bf16_kernels;
    int c = fe_load_module(&k->module, "FE_BF16_HSACO", fe_k_bf16_hsaco, fe_k_bf16_hsaco_end);
    if (!c) c = fe_hip_module_get_function(&k->gemm, k->module, "fe_gemm_bf16");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm, kGemmLds);
    if (!c) c = fe_hip_module_get_function(&k->reduce, k->module, "fe_gemm_bf16_reduce");
    if (!c) c = fe_hip_module_get_function(&k->swiglu, k->module, "fe_gemm_bf16_swiglu");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->swiglu, kGemmLds);
    if (!c) c = fe_hip_module_get_function(&k->swiglu_reduce, k->module, "fe_gemm_bf16_swiglu_reduce");
    if (!c) c = fe_hip_module_get_function(&k->interleave, k->module, "fe_interleave_gu");
    for (int i = 0; i < 4 && !c; i++)
        for (int j = 0; j < 4 && !c; j++) {
            char nm[32];
            snprintf(nm, sizeof nm, "fe_gemv_bf16_r%d_c%d", 1 << i, 1 << j);
            c = fe_hip_module_get_function(&k->gemv[i][j], k->module, nm);
        }
    int cus = 0;
    if (!c) c = fe_hip_cu_count(&cus);
    k->cus = (uint32_t)cus;
    if (const char *e = getenv("FE_BF16_NC")) k->nc = atoi(e);
    if (const char *e = getenv("FE_BF16_GROUP")) k->raster_group = atoi(e);
    if (const char *e = getenv("FE_GEMM_SPLITS")) k->gemm_splits = (uint32_t)atoi(e);
    if (!c) c = k->part.alloc((size_t)kFeGemmSlotsPerCu * k->cus * kFeGemmPartBytes);
    if (c) {
        fe_bf16_kernels_destroy(k);
        return c;
    }
    *out = k;
    return 0;
}

int fe_bf16_kernels_destroy(fe_bf16_kernels *k) {
    if (!k) return 0;
    k->part.release();
    if (k->module) fe_hip_module_unload(k->module);
    delete k;
    return 0;
}

int fe_bf16_kernels_set_option(fe_bf16_kernels *k, const char *name, int32_t value) {
    if (!k || !name) return fe_set_error(FE_ERR_ARG, "fe_bf16_kernels_set_option", "null argument");
    const std::string nm = name;
    if (nm == "nc") k->nc = value;
    else if (nm == "raster_group") k->raster_group = value;
    else if (nm == "gemm_splits") k->gemm_splits = (uint32_t)value;
    else return fe_set_error(FE_ERR_ARG, "fe_bf16_kernels_set_option", name);
    return 0;
}

int fe_bf16_gemv(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda,
                 fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k) {
    const char *fn = "fe_bf16_gemv";
    if (!kern) return fe_set_error(FE_ERR_ARG, fn, "null kernels");
    if (m == 0) return 0;
    if (m > kGemvRows) return fe_set_error(FE_ERR_ARG, fn, "at most 8 rows a call");
    FE_TRY(check(fn, y, ldy, x, lda, w, res, n, k));
    const int form = m <= 1 ? 0 : m <= 2 ? 1 : m <= 4 ? 2 : 3;
    // columns of a program: the results do not depend on it. More columns read x less often (x is read once per program
    // and step, the weights once in all), fewer give more programs
    int cols = gemv_cols(n, form);
    if (kern->nc > 0) cols = kern->nc >= 8 ? 3 : kern->nc >= 4 ? 2 : kern->nc >= 2 ? 1 : 0;
    void *args[] = {&y, &x, &w, &res, &m, &n, &k, &lda, &ldy};
    return fe_hip_launch(kern->gemv[form][cols], n >> cols, 1, 1, 256, 1, 1, 0, s, args);
}

int fe_bf16_gemm(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda,
                 fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k) {
    const char *fn = "fe_bf16_gemm";
    if (!kern) return fe_set_error(FE_ERR_ARG, fn, "null kernels");
    if (m == 0) return 0;
    FE_TRY(check(fn, y, ldy, x, lda, w, res, n, k));
    if ((uint64_t)m * lda * 2 >= (1ull << 32) || (uint64_t)n * k * 2 >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, fn, "operand of 4 GB or more");
    const uint32_t tiles_m = (m + kTileM - 1) / kTileM, tiles_n = (n + kTileN - 1) / kTileN;
    uint32_t group = bf16_raster_group(m, n, k, tiles_m);
    if (kern->raster_group >= 0) group = (uint32_t)kern->raster_group;
    if (group > tiles_m) group = tiles_m;
    FeGemmSplit gs = fe_gemm_split(tiles_m * tiles_n, k / 64, kern->cus, (uint32_t)(kern->part.bytes / kFeGemmPartBytes), kern->gemm_splits);
    uint32_t full = gs.full, splits = gs.splits;
    fe_devptr_t part = kern->part.p;
    void *args[] = {&y, &x, &w, &res, &m, &n, &k, &lda, &ldy, &group, &full, &splits, &part};
    FE_TRY(fe_hip_launch(kern->gemm, gs.programs(), 1, 1, 256, 1, 1, kGemmLds, s, args));
    if (!gs.cut()) return 0;
    void *rargs[] = {&y, &part, &res, &m, &n, &ldy, &group, &full, &splits};
    return fe_hip_launch(kern->reduce, gs.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

int fe_bf16_interleave_gu(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t dst, fe_devptr_t gate, fe_devptr_t up,
                          uint32_t inter, uint32_t k) {
    const char *fn = "fe_bf16_interleave_gu";
    if (!kern || !dst || !gate || !up) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (!inter || !k || inter % 8 || k % 8 || dst % 16 || gate % 16 || up % 16)
        return fe_set_error(FE_ERR_SHAPE, fn, "inter % 8 == 0, k % 8 == 0, 16-byte aligned rows");
    void *args[] = {&dst, &gate, &up, &k};
    return fe_hip_launch(kern->interleave, 2 * inter, 1, 1, 256, 1, 1, 0, s, args);
}

int fe_bf16_gemm_swiglu(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t act, fe_devptr_t x, uint32_t lda,
                        fe_devptr_t w, uint32_t m, uint32_t inter, uint32_t k) {
    const char *fn = "fe_bf16_gemm_swiglu";
    if (!kern) return fe_set_error(FE_ERR_ARG, fn, "null kernels");
    if (m == 0) return 0;
    uint32_t n = 2 * inter;
    FE_TRY(check(fn, act, n, x, lda, w, 0, n, k));  // act rows have stride inter = n / 2, a multiple of 8
    if (n % 16) return fe_set_error(FE_ERR_SHAPE, fn, "inter % 8 == 0");
    if ((uint64_t)m * lda * 2 >= (1ull << 32) || (uint64_t)n * k * 2 >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, fn, "operand of 4 GB or more");
    const uint32_t tiles_m = (m + kTileM - 1) / kTileM, tiles_n = (n + kTileN - 1) / kTileN;
    uint32_t group = bf16_raster_group(m, n, k, tiles_m);
    if (kern->raster_group >= 0) group = (uint32_t)kern->raster_group;
    if (group > tiles_m) group = tiles_m;
    FeGemmSplit gs = fe_gemm_split(tiles_m * tiles_n, k / 64, kern->cus, (uint32_t)(kern->part.bytes / kFeGemmPartBytes), kern->gemm_splits);
    uint32_t full = gs.full, splits = gs.splits;
    fe_devptr_t part = kern->part.p;
    void *args[] = {&act, &x, &w, &m, &n, &k, &lda, &group, &full, &splits, &part};
    FE_TRY(fe_hip_launch(kern->swiglu, gs.programs(), 1, 1, 256, 1, 1, kGemmLds, s, args));
    if (!gs.cut()) return 0;
    void *rargs[] = {&act, &part, &m, &n, &group, &full, &splits};
    return fe_hip_launch(kern->swiglu_reduce, gs.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

int fe_bf16_linear_forward(const fe_bf16_kernels *kern, fe_stream_t s, fe_devptr_t y, uint32_t ldy, fe_devptr_t x,
                           uint32_t lda, fe_devptr_t w, fe_devptr_t res, uint32_t m, uint32_t n, uint32_t k, uint32_t dec) {
    const char *fn = "fe_bf16_linear_forward";
    if (!kern) return fe_set_error(FE_ERR_ARG, fn, "null kernels");
    if (m == 0) return 0;
    FE_TRY(check(fn, y, ldy, x, lda, w, res, n, k));
    // decode / verify rows: the GEMV in passes of up to 8 rows, so that a row's bits do not depend on the batch
    uint32_t d = m <= kSmallBatch ? m : (dec < m ? dec : m);
    if (k % 256) d = 0;
    for (uint32_t r = 0; r < d; r += kGemvRows) {
        const uint32_t mr = d - r < kGemvRows ? d - r : kGemvRows;
        FE_TRY(fe_bf16_gemv(kern, s, y + (size_t)r * ldy * 2, ldy, x + (size_t)r * lda * 2, lda, w,
                            res ? res + (size_t)r * ldy * 2 : 0, mr, n, k));
    }
    if (d == m) return 0;
    return fe_bf16_gemm(kern, s, y + (size_t)d * ldy * 2, ldy, x + (size_t)d * lda * 2, lda, w,
                        res ? res + (size_t)d * ldy * 2 : 0, m - d, n, k);
}

}  // extern "C"
