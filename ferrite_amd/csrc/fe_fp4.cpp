// fe_fp4: host side of the NVFP4 prompt linear (see include/fe_fp4.h). Follows crates/fe-fp4/src/lib.rs; the kernels
// are ferrite_amd/csrc/kernels/k_fp4.hip.
#include "fe_fp4.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "fe_exl3.h"  // error codes
#include "fe_internal.h"

namespace {
constexpr uint32_t kTile = 128;                 // crates/fe-fp4/src/lib.rs:28
constexpr uint32_t kGemmLds = 2 * (256 + 256) * 64 * 2;  // GM_LDS_TILES: two k tiles of A and W, 256 rows each
constexpr uint32_t kTileM = 256;                        // GM_BM
constexpr uint32_t kTileN = 256;                        // GM_BN
}  // namespace

struct fe_fp4_kernels {
    fe_module_t module = nullptr;
    fe_function_t quant4 = nullptr, gemm4 = nullptr, reduce4 = nullptr, gemv4[3] = {nullptr, nullptr, nullptr};
    fe_function_t strip4 = nullptr;  // the GEMV over strips of 16 weight rows, up to 16 activation rows (no hand-off)
    fe_function_t strip_once[5] = {};  // ... with every load of a workgroup issued before anything waits: 1..5 groups of K a wavefront
    fe_function_t quant8 = nullptr, gemm8 = nullptr, swiglu4 = nullptr, swiglu_reduce4 = nullptr;
    fe_function_t gemm8c = nullptr;  // FP8 on the 8-bit matrix instruction, operands as codes
    fe_function_t gemm4_sk = nullptr, gemm8_sk = nullptr, gemm8c_sk = nullptr, swiglu4_sk = nullptr;  // the same on the stream-K schedule
    uint32_t cus = 0;
    // Switches of the launch paths: read from the environment once, at load; fe_fp4_kernels_set_option changes them
    // afterwards. No forward call reads the environment.
    uint32_t group_m = 8;      // raster group height in row tiles; 0 = all (FE_FP4_GROUP, lib.rs:31-32, 68)
    uint32_t gemv = 1;         // up to 64 rows run the GEMV (FE_FP4_NO_GEMV=1: the GEMM's single tile row)
    uint32_t gemv_sk = 0;      // K splits of the GEMV over weight tiles; 0 = two programs a CU (FE_FP4_GEMV_SK)
    uint32_t gemv_strips = 1;  // the GEMV runs over strips of 16 weight rows, K split inside the workgroup (FE_FP4_NO_STRIPS=1: over weight tiles and K splits)
    uint32_t gemv_once = 1;    // strips whose loads all go out at once, where a wavefront's share of K allows (FE_FP4_NO_ONCE=1: never)
    uint32_t gemv_waves = 0;   // wavefronts of a strip's workgroup: 4, 8 or 16; 0 = four or more wavefronts a SIMD (FE_FP4_GEMV_WAVES)
    int32_t xcd = -1;          // column tiles dealt to the XCDs: -1 = where the weights are the larger operand (FE_FP4_XCD)
    uint32_t fp8_f16 = 0;      // FP8 linears as fp16 expansion on the 16-bit matrix instruction (FE_FP8_F16=1)
    uint32_t gemm_splits = 8;  // most pieces a cut output tile takes (FE_GEMM_SPLITS; 1: never cut)
    int32_t gemm_sk = 1;       // stream-K schedule of the GEMMs: 0 never, 1 where measured faster, 2 always (FE_GEMM_SK)
};

struct fe_fp4_linear {
    std::string name;
    uint32_t n = 0, k = 0;
    float g = 1.0f;
    bool fp8 = false;  // Kind::Fp8 (e4m3 codes [n][k], no block scales), else Kind::Nvfp4 (lib.rs:229-233)
    FeBuf w, sw, alpha;
    // byte strides of the codes / scales of (128-row tile, 64-wide k tile, row in tile); see fe_gemm_nvfp4
    uint32_t w_snt = 0, w_skt = 0, w_sr = 0, s_snt = 0, s_skt = 0, s_sr = 0;
};

struct fe_fp4_workspace {
    uint32_t max_rows = 0, max_k = 0;
    FeBuf codes, sf, aq, part, counters;  // part: partial sums of the GEMM (one slot a CU) or of the GEMV's splits
};
constexpr uint32_t kGemvRows = 48;      // rows of one fe_gemv_nvfp4 pass (three groups of 16)
constexpr uint32_t kGemvMaxRows = 64;   // up to here the GEMV runs (two passes above 48 rows); above, the GEMM
constexpr uint32_t kGemvCounters = 8192;  // arrival counters: weight tiles of 128 rows (n <= 1 M)

extern "C" {

int fe_fp4_kernels_load(fe_fp4_kernels **out) {
    if (!out) return fe_set_error(FE_ERR_ARG, "fe_fp4_kernels_load", "null out");
    auto *k = new fe_fp4_kernels;
    int c = fe_load_module(&k->module, "FE_FP4_HSACO", fe_k_fp4_hsaco, fe_k_fp4_hsaco_end);
    if (!c) c = fe_hip_module_get_function(&k->quant4, k->module, "fe_fp4_quant");
    if (!c) c = fe_hip_module_get_function(&k->gemm4, k->module, "fe_gemm_nvfp4");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm4, kGemmLds);
    if (!c) c = fe_hip_module_get_function(&k->reduce4, k->module, "fe_gemm_nvfp4_reduce");
    for (int xr = 1; xr <= 3 && !c; xr++) {
        char nm[32];
        snprintf(nm, sizeof nm, "fe_gemv_nvfp4_x%d", xr);
        c = fe_hip_module_get_function(&k->gemv4[xr - 1], k->module, nm);
    }
    if (!c) c = fe_hip_module_get_function(&k->strip4, k->module, "fe_gemv_nvfp4_strips");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->strip4, 48 * 1024);
    for (int g = 1; g <= 5 && !c; g++) {
        const std::string nm = "fe_gemv_nvfp4_strips_once_g" + std::to_string(g);
        c = fe_hip_module_get_function(&k->strip_once[g - 1], k->module, nm.c_str());
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->strip_once[g - 1], 48 * 1024);
    }
    if (!c) c = fe_hip_module_get_function(&k->quant8, k->module, "fe_fp8_quant");
    if (!c) c = fe_hip_module_get_function(&k->gemm8, k->module, "fe_gemm_fp8");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm8, kGemmLds);
    if (!c) c = fe_hip_module_get_function(&k->gemm8c, k->module, "fe_gemm_fp8_codes");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm8c, kGemmLds);
    struct { fe_function_t *f; const char *nm; } sks[] = {
        {&k->gemm4_sk, "fe_gemm_nvfp4_sk"}, {&k->gemm8_sk, "fe_gemm_fp8_sk"}, {&k->gemm8c_sk, "fe_gemm_fp8_codes_sk"},
        {&k->swiglu4_sk, "fe_gemm_nvfp4_swiglu_sk"}};
    for (auto &e : sks) {
        if (!c) c = fe_hip_module_get_function(e.f, k->module, e.nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(*e.f, kGemmLds);
    }
    if (!c) c = fe_hip_module_get_function(&k->swiglu4, k->module, "fe_gemm_nvfp4_swiglu");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->swiglu4, kGemmLds);
    if (!c) c = fe_hip_module_get_function(&k->swiglu_reduce4, k->module, "fe_gemm_nvfp4_swiglu_reduce");
    int cus = 0;
    if (!c) c = fe_hip_cu_count(&cus);
    k->cus = (uint32_t)cus;
    if (const char *g = getenv("FE_FP4_GROUP")) k->group_m = (uint32_t)atoi(g);
    if (const char *e = getenv("FE_FP4_NO_GEMV")) k->gemv = atoi(e) ? 0 : 1;
    if (const char *e = getenv("FE_FP4_GEMV_SK")) k->gemv_sk = (uint32_t)atoi(e);
    if (const char *e = getenv("FE_FP4_NO_STRIPS")) k->gemv_strips = atoi(e) ? 0 : 1;
    if (const char *e = getenv("FE_FP4_NO_ONCE")) k->gemv_once = atoi(e) ? 0 : 1;
    if (const char *e = getenv("FE_FP4_GEMV_WAVES")) k->gemv_waves = (uint32_t)atoi(e);
    if (const char *e = getenv("FE_FP4_XCD")) k->xcd = atoi(e) ? 1 : 0;
    if (const char *e = getenv("FE_FP8_F16")) k->fp8_f16 = atoi(e) ? 1 : 0;
    if (const char *e = getenv("FE_GEMM_SPLITS")) k->gemm_splits = (uint32_t)atoi(e);
    if (const char *e = getenv("FE_GEMM_SK")) k->gemm_sk = atoi(e);
    if (c) {
        fe_fp4_kernels_destroy(k);
        return c;
    }
    *out = k;
    return 0;
}

int fe_fp4_kernels_destroy(fe_fp4_kernels *k) {
    if (!k) return 0;
    if (k->module) fe_hip_module_unload(k->module);
    delete k;
    return 0;
}

int fe_fp4_kernels_set_option(fe_fp4_kernels *k, const char *name, int32_t value) {
    if (!k || !name) return fe_set_error(FE_ERR_ARG, "fe_fp4_kernels_set_option", "null argument");
    const std::string nm = name;
    if (nm == "group_m") k->group_m = (uint32_t)value;
    else if (nm == "gemv") k->gemv = value ? 1 : 0;
    else if (nm == "gemv_sk") k->gemv_sk = (uint32_t)value;
    else if (nm == "gemv_strips") k->gemv_strips = (uint32_t)value;
    else if (nm == "gemv_once") k->gemv_once = (uint32_t)value;
    else if (nm == "gemv_waves") k->gemv_waves = (uint32_t)value;
    else if (nm == "xcd") k->xcd = value;
    else if (nm == "fp8_f16") k->fp8_f16 = value ? 1 : 0;
    else if (nm == "gemm_splits") k->gemm_splits = (uint32_t)value;
    else if (nm == "gemm_sk") k->gemm_sk = value;
    else return fe_set_error(FE_ERR_ARG, "fe_fp4_kernels_set_option", name);
    return 0;
}

int fe_gemm_schedule_query(uint32_t tiles, uint32_t ktiles, uint32_t cus, int32_t mode, int32_t small_b, uint32_t *stream_k,
                           uint32_t *programs, uint32_t *whole, uint32_t *splits, uint32_t *run, uint32_t *run_rem) {
    if (!tiles || !ktiles || !cus || !stream_k || !programs || !whole || !splits || !run || !run_rem)
        return fe_set_error(FE_ERR_ARG, "fe_gemm_schedule_query", "null or zero argument");
    // a stand-in workspace: nonzero addresses that are never dereferenced here
    const FeGemmSchedule s = fe_gemm_schedule(tiles, ktiles, cus, 1, (size_t)cus * kFeGemmSlotsPerCu * kFeGemmPartBytes, 1,
                                              (size_t)tiles, 8, mode, small_b != 0);
    *stream_k = s.stream_k ? 1 : 0, *programs = s.programs, *whole = s.args.full_tiles;
    *splits = s.stream_k ? 1 : s.split.splits, *run = s.args.sk_base, *run_rem = s.args.sk_rem;
    return 0;
}

static int check_shape(const char *name, uint32_t n, uint32_t k) {
    if (!n || !k || n % kTile || k % 128) {
        char msg[160];
        snprintf(msg, sizeof msg, "%s: nvfp4 linear n %u k %u (multiples of 128)", name ? name : "?", n, k);
        return fe_set_error(FE_ERR_SHAPE, "fe_fp4_linear", msg);
    }
    return 0;
}

int fe_fp4_linear_upload(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, const uint8_t *codes,
                         const uint8_t *scales, const float *alpha, float g) {
    if (!out || !codes || !scales || !alpha) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_upload", "null argument");
    FE_TRY(check_shape(name, n, k));
    if (!(g > 0.0f)) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_upload", "input_scale 0");  // lib.rs:345
    auto *l = new fe_fp4_linear;
    l->name = name ? name : "";
    l->n = n, l->k = k, l->g = g;
    // k-tile-major device layout: the 128 rows of a tile contribute 32 bytes of codes (4 scales) each to one k tile,
    // stored contiguously, so a program's weight read for a k tile is one 4 KB (512 byte) run
    const uint32_t kts = k / 64, nts = n / kTile;
    std::vector<uint8_t> wt((size_t)n * k / 2), st((size_t)n * k / 16);
    for (uint32_t nt = 0; nt < nts; nt++)
        for (uint32_t r = 0; r < kTile; r++) {
            const uint8_t *wrow = codes + (size_t)(nt * kTile + r) * (k / 2), *srow = scales + (size_t)(nt * kTile + r) * (k / 16);
            for (uint32_t kt = 0; kt < kts; kt++) {
                memcpy(&wt[(((size_t)nt * kts + kt) * kTile + r) * 32], wrow + kt * 32, 32);
                memcpy(&st[(((size_t)nt * kts + kt) * kTile + r) * 4], srow + kt * 4, 4);
            }
        }
    l->w_snt = kts * kTile * 32, l->w_skt = kTile * 32, l->w_sr = 32;
    l->s_snt = kts * kTile * 4, l->s_skt = kTile * 4, l->s_sr = 4;
    int c = l->w.from_host(wt.data(), wt.size());
    if (!c) c = l->sw.from_host(st.data(), st.size());
    if (!c) c = l->alpha.from_host(alpha, (size_t)n * 4);
    if (c) {
        delete l;
        return c;
    }
    *out = l;
    return 0;
}

int fe_fp4_linear_from_view(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, fe_devptr_t codes,
                            fe_devptr_t scales, fe_devptr_t alpha, float g) {
    if (!out || !codes || !scales || !alpha) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_from_view", "null argument");
    FE_TRY(check_shape(name, n, k));
    auto *l = new fe_fp4_linear;
    l->name = name ? name : "";
    l->n = n, l->k = k, l->g = g;
    l->w.view(codes, (size_t)n * k / 2);
    l->sw.view(scales, (size_t)n * k / 16);
    l->alpha.view(alpha, (size_t)n * 4);
    // the format's row-major layout, read in place
    l->w_snt = kTile * (k / 2), l->w_skt = 32, l->w_sr = k / 2;
    l->s_snt = kTile * (k / 16), l->s_skt = 4, l->s_sr = k / 16;
    *out = l;
    return 0;
}

int fe_fp8_linear_upload(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, const uint8_t *codes,
                         const float *alpha, float g) {
    if (!out || !codes || !alpha) return fe_set_error(FE_ERR_ARG, "fe_fp8_linear_upload", "null argument");
    FE_TRY(check_shape(name, n, k));
    if (!(g > 0.0f)) return fe_set_error(FE_ERR_ARG, "fe_fp8_linear_upload", "input_scale 0");
    auto *l = new fe_fp4_linear;
    l->name = name ? name : "";
    l->n = n, l->k = k, l->g = g, l->fp8 = true;
    // k-tile-major like the NVFP4 codes: [n / 128][k / 64][128 rows][64 bytes]
    const uint32_t kts = k / 64, nts = n / kTile;
    std::vector<uint8_t> wt((size_t)n * k);
    for (uint32_t nt = 0; nt < nts; nt++)
        for (uint32_t r = 0; r < kTile; r++) {
            const uint8_t *wrow = codes + (size_t)(nt * kTile + r) * k;
            for (uint32_t kt = 0; kt < kts; kt++) memcpy(&wt[(((size_t)nt * kts + kt) * kTile + r) * 64], wrow + kt * 64, 64);
        }
    l->w_snt = kts * kTile * 64, l->w_skt = kTile * 64, l->w_sr = 64;
    int c = l->w.from_host(wt.data(), wt.size());
    if (!c) c = l->alpha.from_host(alpha, (size_t)n * 4);
    if (c) {
        delete l;
        return c;
    }
    *out = l;
    return 0;
}

int fe_fp8_linear_from_view(fe_fp4_linear **out, const char *name, uint32_t n, uint32_t k, fe_devptr_t codes,
                            fe_devptr_t alpha, float g) {
    if (!out || !codes || !alpha) return fe_set_error(FE_ERR_ARG, "fe_fp8_linear_from_view", "null argument");
    FE_TRY(check_shape(name, n, k));
    auto *l = new fe_fp4_linear;
    l->name = name ? name : "";
    l->n = n, l->k = k, l->g = g, l->fp8 = true;
    l->w.view(codes, (size_t)n * k);
    l->alpha.view(alpha, (size_t)n * 4);
    l->w_snt = kTile * k, l->w_skt = 64, l->w_sr = k;
    *out = l;
    return 0;
}

int fe_fp4_linear_destroy(fe_fp4_linear *l) {
    delete l;
    return 0;
}

int fe_fp4_linear_shape(const fe_fp4_linear *l, uint32_t *n, uint32_t *k, float *g) {
    if (!l) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_shape", "null linear");
    if (n) *n = l->n;
    if (k) *k = l->k;
    if (g) *g = l->g;
    return 0;
}

int fe_fp4_workspace_create(fe_fp4_workspace **out, uint32_t max_rows, uint32_t max_k) {
    if (!out || !max_rows || !max_k || max_k % 128) return fe_set_error(FE_ERR_ARG, "fe_fp4_workspace_create", "bad size");
    auto *ws = new fe_fp4_workspace;
    ws->max_rows = max_rows, ws->max_k = max_k;
    const size_t rp = (size_t)(max_rows + kTile - 1) / kTile * kTile;
    // codes sized for one byte an element like the reference's (lib.rs:213-225: enough for FP8, NVFP4 uses half)
    int c = ws->codes.alloc(rp * max_k);
    if (!c) c = ws->sf.zeroed(rp * max_k / 16);
    if (!c) c = ws->aq.alloc(rp * max_k * 2);
    int cus = 0;
    if (!c) c = fe_hip_cu_count(&cus);
    if (!c && cus > 0) c = ws->part.alloc((size_t)cus * kFeGemmSlotsPerCu * kFeGemmPartBytes);
    if (!c) c = ws->counters.zeroed(kGemvCounters * 4);
    if (c) {
        delete ws;
        return c;
    }
    *out = ws;
    return 0;
}

int fe_fp4_workspace_destroy(fe_fp4_workspace *ws) {
    delete ws;
    return 0;
}

int fe_fp4_workspace_buffers(const fe_fp4_workspace *ws, fe_devptr_t *codes, fe_devptr_t *sf, uint32_t *max_rows,
                             uint32_t *max_k) {
    if (!ws) return fe_set_error(FE_ERR_ARG, "fe_fp4_workspace_buffers", "null workspace");
    if (codes) *codes = ws->codes.p;
    if (sf) *sf = ws->sf.p;
    if (max_rows) *max_rows = ws->max_rows;
    if (max_k) *max_k = ws->max_k;
    return 0;
}

int fe_fp4_workspace_operand(const fe_fp4_workspace *ws, fe_devptr_t *aq) {
    if (!ws || !aq) return fe_set_error(FE_ERR_ARG, "fe_fp4_workspace_operand", "null argument");
    *aq = ws->aq.p;
    return 0;
}

int fe_fp4_linear_quantize(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                           fe_devptr_t x, uint32_t lda, uint32_t m) {
    if (!l || !kern || !ws) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_quantize", "null argument");
    if (m > ws->max_rows || l->k > ws->max_k) {  // lib.rs:521-522
        char msg[200];
        snprintf(msg, sizeof msg, "%s: workspace %ux%u < %ux%u", l->name.c_str(), ws->max_rows, ws->max_k, m, l->k);
        return fe_set_error(FE_ERR_WORKSPACE, "fe_fp4_linear_quantize", msg);
    }
    if (m == 0) return 0;
    if (!x || lda < l->k || lda % 8 || x % 16) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_quantize", "x must be 16-byte aligned rows of >= k");
    uint32_t k = l->k;
    float g = l->g;
    fe_devptr_t codes = ws->codes.p, sf = ws->sf.p, aq = ws->aq.p;
    if (l->fp8) {
        void *args8[] = {&codes, &aq, &x, &m, &k, &lda, &g};
        return fe_hip_launch(kern->quant8, (m * (k / 8) + 255) / 256, 1, 1, 256, 1, 1, 0, s, args8);
    }
    void *args[] = {&codes, &sf, &aq, &x, &m, &k, &lda, &g};
    const uint32_t blocks16 = m * (k / 16);
    return fe_hip_launch(kern->quant4, (blocks16 + 255) / 256, 1, 1, 256, 1, 1, 0, s, args);
}

int fe_fp4_linear_gemm(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                       fe_devptr_t y, uint32_t ldy, uint32_t m, fe_devptr_t res) {
    if (!l || !kern || !ws) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_gemm", "null argument");
    if (m == 0) return 0;  // lib.rs:535-537
    if (m > ws->max_rows || l->k > ws->max_k) return fe_set_error(FE_ERR_WORKSPACE, "fe_fp4_linear_gemm", "rows or k exceed the workspace");
    // lib.rs:156-157
    if (!y || ldy % 8 || y % 16 || (res && res % 16) || ldy < l->n)
        return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_gemm", "gemm: y/res must be 16-byte aligned rows");
    uint32_t n = l->n, k = l->k;
    if (!l->fp8 && m <= kGemvMaxRows && n / kTile <= kGemvCounters && kern->gemv) {
        // decode-sized: the weight-read-bound GEMV, up to 48 rows a pass. Two programs fit a CU: as many programs as run
        // at once, not more (a second round of short programs costs more than idle CUs in the first).
        const uint32_t nts = n / kTile, kts = k / 64;
        // Strips of 16 weight rows over all of K, one a workgroup, the activations staged in LDS: no hand-off between
        // programs. Every program stages all m rows of activations, so it pays where that is small beside the weights:
        // one or two rows, or up to four on narrow linears (measured, cold weights: 5120 x 17408 at 1 row 14.3 against 15.4 us for
        // the weight tiles with K splits, 5120 x 5120 at 1..4 rows 7.2-7.8 against 9.7-10.0; at k = 17408 the staging
        // costs more than the hand-off it saves: 17.0 against 15.8). gemv_strips 2 forces it wherever it fits.
        const bool strips_fit = k % 256 == 0 && (size_t)m * k * 2 <= 48 * 1024 && m <= 16;
        const bool strips_pay = k <= 8192 && (m <= 2 || (n <= 8192 && m <= 4));  // (5120 x 17408 at 2 rows: 14.3 against 15.3 us; at 4: 16.5)
        if (kern->gemv_strips && strips_fit && (strips_pay || kern->gemv_strips == 2)) {
            const uint32_t strips = n / 16;
            uint32_t waves = 4;  // wavefronts of a workgroup: two or more a SIMD in all
            while (waves < 16 && strips * waves < 8 * kern->cus) waves *= 2;
            if (kern->gemv_waves && kern->gemv_waves <= 16 && !(kern->gemv_waves & (kern->gemv_waves - 1))) waves = kern->gemv_waves;
            while (waves > 1 && waves > kts / 4) waves /= 2;
            // Where a wavefront's share of K can be at most five groups of four k tiles and the activations at most four
            // 16-byte pieces a thread, the kernel that issues every load at once, with the number of wavefronts (any, up to
            // 16) that wastes the fewest loads: a wavefront with fewer groups than the others requests one again, and a
            // load instruction costs the address unit the same either way (5120 x 5120: 8 wavefronts of 3 groups for 20
            // groups 9.3 us, 10 of 2 groups measured faster).
            fe_function_t strip_fn = kern->strip4;
            if (kern->gemv_once) {
                const uint32_t groups = k / 256, want = kern->gemv_waves ? waves : std::max(4u, (8 * kern->cus + strips - 1) / strips);
                uint32_t best_w = 0, best_waste = ~0u;
                for (uint32_t w1 = std::min(want, 16u); w1 <= (kern->gemv_waves ? want : 16u); w1++) {
                    const uint32_t gpw = (groups + w1 - 1) / w1;
                    if (gpw > 5 || w1 > groups || ((size_t)m * (k / 8) + 64 * w1 - 1) / (64 * w1) > 4) continue;
                    if (w1 * gpw - groups < best_waste) best_waste = w1 * gpw - groups, best_w = w1;
                }
                if (best_w) waves = best_w, strip_fn = kern->strip_once[(groups + best_w - 1) / best_w - 1];
            }
            fe_devptr_t w = l->w.p, sw = l->sw.p, alpha = l->alpha.p;
            uint32_t w_snt = l->w_snt, w_skt = l->w_skt, w_sr = l->w_sr, s_snt = l->s_snt, s_skt = l->s_skt, s_sr = l->s_sr;
            for (uint32_t r0 = 0; r0 < m; r0 += kGemvRows) {
                uint32_t rows = m - r0 < kGemvRows ? m - r0 : kGemvRows;
                fe_devptr_t yy = y + (size_t)r0 * ldy * 2, aq = ws->aq.p + (size_t)r0 * k * 2, rr = res ? res + (size_t)r0 * ldy * 2 : 0;
                void *args[] = {&yy, &aq, &w, &sw, &alpha, &rr, &rows, &n, &k, &ldy, &w_snt, &w_skt, &w_sr, &s_snt, &s_skt, &s_sr};
                FE_TRY(fe_hip_launch(strip_fn, strips, 1, 1, 64 * waves, 1, 1, rows * k * 2, s, args));
            }
            return 0;
        }
        uint32_t sk = 2 * kern->cus / nts;
        if (kern->gemv_sk) sk = kern->gemv_sk;
        if (sk > 16) sk = 16;
        if (sk > kts / 4) sk = kts / 4;
        while (sk > 1 && (size_t)sk * kGemvRows * n * 4 > ws->part.bytes) sk--;
        if (sk < 1) sk = 1;
        fe_devptr_t w = l->w.p, sw = l->sw.p, alpha = l->alpha.p, z = ws->part.p, cnt = ws->counters.p;
        uint32_t w_snt = l->w_snt, w_skt = l->w_skt, w_sr = l->w_sr, s_snt = l->s_snt, s_skt = l->s_skt, s_sr = l->s_sr;
        for (uint32_t r0 = 0; r0 < m; r0 += kGemvRows) {
            uint32_t rows = m - r0 < kGemvRows ? m - r0 : kGemvRows;
            fe_devptr_t yy = y + (size_t)r0 * ldy * 2, aq = ws->aq.p + (size_t)r0 * k * 2, rr = res ? res + (size_t)r0 * ldy * 2 : 0;
            void *args[] = {&yy, &aq, &w, &sw, &alpha, &rr, &z, &cnt, &rows, &n, &k, &ldy, &sk, &w_snt, &w_skt, &w_sr, &s_snt, &s_skt, &s_sr};
            FE_TRY(fe_hip_launch(kern->gemv4[(rows + 15) / 16 - 1], nts * sk, 1, 1, 256, 1, 1, 0, s, args));
        }
        return 0;
    }
    if ((uint64_t)m * k * 2 >= (1ull << 32) || (uint64_t)n * k >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_fp4_linear_gemm", "operand of 4 GB or more");
    const uint32_t tiles_m = (m + kTileM - 1) / kTileM, tiles_n = (n + kTileN - 1) / kTileN;
    uint32_t group = kern->group_m == 0 || kern->group_m > tiles_m ? tiles_m : kern->group_m;  // lib.rs:148-151
    // FP8 codes: the weights are the larger operand from n >= m on, and at the 8-bit instruction's rate their traffic
    // shows: column tiles are dealt to the XCDs (gemm_raster with group 0), each weight panel through one L2
    if (l->fp8 && n >= m) group = 0;
    if (kern->xcd >= 0) group = kern->xcd ? 0 : group ? group : tiles_m;
    fe_devptr_t aq = ws->aq.p, w = l->w.p, sw = l->sw.p, alpha = l->alpha.p;
    uint32_t w_snt = l->w_snt, w_skt = l->w_skt, w_sr = l->w_sr, s_snt = l->s_snt, s_skt = l->s_skt, s_sr = l->s_sr;
    // FP8 runs on the 8-bit matrix instruction over the codes of both operands, k tiles of 128 (FE_FP8_F16=1: the fp16
    // expansion on the 16-bit instruction, k tiles of 64; same products, another order of the f32 sums)
    const bool codes8 = l->fp8 && !kern->fp8_f16;
    FeGemmSchedule sch = fe_gemm_schedule(tiles_m * tiles_n, codes8 ? k / 128 : k / 64, kern->cus, ws->part.p, ws->part.bytes,
                                          ws->counters.p, kGemvCounters, kern->gemm_splits, kern->gemm_sk, /*small_b=*/!l->fp8);
    // stream-K programs sit at different depths of K: one row tile at a time (column tiles fastest) keeps those that are
    // in step on one panel of activations
    if (sch.stream_k && kern->xcd < 0) group = 1;
    float scale = l->fp8 ? 1.0f : 0.0625f;  // what the fp16 expansions of the two operands carry (FP4_OPERAND_SCALE)
    if (codes8) {
        fe_devptr_t codes = ws->codes.p;
        void *args8[] = {&y, &codes, &w, &alpha, &res, &m, &n, &k, &ldy, &group, &w_snt, &w_skt, &w_sr, &sch.args};
        FE_TRY(fe_hip_launch(sch.stream_k ? kern->gemm8c_sk : kern->gemm8c, sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args8));
    } else if (l->fp8) {
        void *args8[] = {&y, &aq, &w, &alpha, &res, &m, &n, &k, &ldy, &group, &w_snt, &w_skt, &w_sr, &sch.args};
        FE_TRY(fe_hip_launch(sch.stream_k ? kern->gemm8_sk : kern->gemm8, sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args8));
    } else {
        void *args[] = {&y,     &aq,    &w,     &sw,   &alpha, &res,   &m,    &n,       &k,
                        &ldy,   &group, &w_snt, &w_skt, &w_sr, &s_snt, &s_skt, &s_sr, &sch.args};
        FE_TRY(fe_hip_launch(sch.stream_k ? kern->gemm4_sk : kern->gemm4, sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args));
    }
    if (sch.stream_k || !sch.split.cut()) return 0;
    uint32_t full = sch.split.full, splits = sch.split.splits;
    fe_devptr_t part = ws->part.p;
    void *rargs[] = {&y, &part, &alpha, &res, &m, &n, &ldy, &group, &full, &splits, &scale};
    return fe_hip_launch(kern->reduce4, sch.split.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

int fe_fp4_linear_forward(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                          fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda, uint32_t m, fe_devptr_t res) {
    FE_TRY(fe_fp4_linear_quantize(l, kern, s, ws, x, lda, m));
    return fe_fp4_linear_gemm(l, kern, s, ws, y, ldy, m, res);
}

int fe_fp4_linear_forward_swiglu(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s,
                                 const fe_fp4_workspace *ws, const fe_fp4_workspace *act, fe_devptr_t x, uint32_t lda,
                                 uint32_t m, float down_g) {
    if (!l || !kern || !ws || !act) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_forward_swiglu", "null argument");
    if (l->fp8 || l->n % 256) {  // lib.rs:388-392, 500
        char msg[200];
        snprintf(msg, sizeof msg, "%s: not an NVFP4 gate|up pair (n %u)", l->name.c_str(), l->n);
        return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_forward_swiglu", msg);
    }
    if (m == 0) return 0;
    uint32_t n = l->n, k = l->k, inter = n / 2;
    if (m > act->max_rows || inter > act->max_k)
        return fe_set_error(FE_ERR_WORKSPACE, "fe_fp4_linear_forward_swiglu", "rows or n / 2 exceed the act workspace");
    if (!(down_g > 0.0f)) return fe_set_error(FE_ERR_ARG, "fe_fp4_linear_forward_swiglu", "down_g");
    FE_TRY(fe_fp4_linear_quantize(l, kern, s, ws, x, lda, m));
    if ((uint64_t)m * k * 2 >= (1ull << 32) || (uint64_t)n * k / 2 >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_fp4_linear_forward_swiglu", "operand of 4 GB or more");
    const uint32_t tiles_m = (m + kTileM - 1) / kTileM, tiles_n = (n + kTileN - 1) / kTileN;
    uint32_t group = kern->group_m == 0 || kern->group_m > tiles_m ? tiles_m : kern->group_m;
    fe_devptr_t aq = ws->aq.p, w = l->w.p, sw = l->sw.p, alpha = l->alpha.p, part = ws->part.p;
    fe_devptr_t q_codes = act->codes.p, q_sf = act->sf.p, q_aq = act->aq.p;
    uint32_t w_snt = l->w_snt, w_skt = l->w_skt, w_sr = l->w_sr, s_snt = l->s_snt, s_skt = l->s_skt, s_sr = l->s_sr;
    FeGemmSchedule sch = fe_gemm_schedule(tiles_m * tiles_n, k / 64, kern->cus, ws->part.p, ws->part.bytes, ws->counters.p,
                                          kGemvCounters, kern->gemm_splits, kern->gemm_sk >= 2 ? kern->gemm_sk : 0, true);
    // (stream-K only when forced: this kernel's stream-K form was slower wherever measured, 688 -> 714 us on 5120 x 34816)
    if (sch.stream_k && kern->xcd < 0) group = 1;
    void *args[] = {&aq,    &w,     &sw,    &alpha, &m,       &n,       &k,    &group, &w_snt, &w_skt,
                    &w_sr,  &s_snt, &s_skt, &s_sr,  &sch.args, &q_codes, &q_sf, &q_aq,  &down_g};
    FE_TRY(fe_hip_launch(sch.stream_k ? kern->swiglu4_sk : kern->swiglu4, sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args));
    if (sch.stream_k || !sch.split.cut()) return 0;
    const FeGemmSplit &gs = sch.split;
    uint32_t full = gs.full, splits = gs.splits;
    void *rargs[] = {&part, &alpha, &m, &n, &group, &full, &splits, &q_codes, &q_sf, &q_aq, &down_g};
    return fe_hip_launch(kern->swiglu_reduce4, gs.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

}  // extern "C"

// Matrix-unit peak (fe_mfma_peak_*): `launches` launches of grid x 256 threads between two events, after one warm-up.
extern "C" int fe_fp4_mfma_peak(const fe_fp4_kernels *kern, fe_stream_t s, int kind, uint32_t seed, uint32_t grid, uint32_t iters,
                                uint32_t launches, float *ms) {
    const char *fn = "fe_fp4_mfma_peak";
    if (!kern || kind < 0 || kind > 2 || !grid || !launches) return fe_set_error(FE_ERR_ARG, fn, "kind 0 (f16), 1 (bf16), 2 (f8)");
    static const char *names[] = {"fe_mfma_peak_f16", "fe_mfma_peak_bf16", "fe_mfma_peak_f8"};
    fe_function_t f = nullptr;
    FE_TRY(fe_hip_module_get_function(&f, kern->module, names[kind]));
    FeBuf out;
    FE_TRY(out.alloc((size_t)grid * 256 * 4));
    fe_devptr_t o = out.p;
    void *args[] = {&o, &iters, &seed};
    fe_event_t a = nullptr, b = nullptr;
    FE_TRY(fe_hip_event_create(&a));
    int c = fe_hip_event_create(&b);
    if (!c) c = fe_hip_launch(f, grid, 1, 1, 256, 1, 1, 0, s, args);
    if (!c) c = fe_hip_event_record(a, s);
    for (uint32_t i = 0; !c && i < launches; i++) c = fe_hip_launch(f, grid, 1, 1, 256, 1, 1, 0, s, args);
    if (!c) c = fe_hip_event_record(b, s);
    if (!c) c = fe_hip_event_sync(b);
    float t = 0;
    if (!c) c = fe_hip_event_elapsed_ms(&t, a, b);
    fe_hip_event_destroy(a);
    fe_hip_event_destroy(b);
    if (!c && ms) *ms = t / (float)launches;
    return c;
}
