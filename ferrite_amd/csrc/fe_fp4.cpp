// fe_fp4: host side of the NVFP4 prompt linear (see include/fe_fp4.h). Follows crates/fe-fp4/src/lib.rs; the kernels
// are ferrite_amd/csrc/kernels/k_fp4.hip.
#include "fe_fp4.h"

#include <cstdio>
#include <cstdlib>
#include <string>

#include "fe_exl3.h"  // error codes
#include "fe_internal.h"

namespace {
constexpr uint32_t kTile = 128;                 // crates/fe-fp4/src/lib.rs:28
constexpr uint32_t kGemmLds = 2 * 128 * 72 * 2;  // GM_LDS_TILES
}  // namespace

struct fe_fp4_kernels {
    fe_module_t module = nullptr;
    fe_function_t quant4 = nullptr, gemm4 = nullptr;
    uint32_t group_m = 8;  // raster group height in row tiles; 0 = all (FE_FP4_GROUP, lib.rs:31-32, 68)
};

struct fe_fp4_linear {
    std::string name;
    uint32_t n = 0, k = 0;
    float g = 1.0f;
    FeBuf w, sw, alpha;
};

struct fe_fp4_workspace {
    uint32_t max_rows = 0, max_k = 0;
    FeBuf codes, sf, aq;
};

extern "C" {

int fe_fp4_kernels_load(fe_fp4_kernels **out) {
    if (!out) return fe_set_error(FE_ERR_ARG, "fe_fp4_kernels_load", "null out");
    auto *k = new fe_fp4_kernels;
    int c = fe_load_module(&k->module, "FE_FP4_HSACO", fe_k_fp4_hsaco, fe_k_fp4_hsaco_end);
    if (!c) c = fe_hip_module_get_function(&k->quant4, k->module, "fe_fp4_quant");
    if (!c) c = fe_hip_module_get_function(&k->gemm4, k->module, "fe_gemm_nvfp4");
    if (const char *g = getenv("FE_FP4_GROUP")) k->group_m = (uint32_t)atoi(g);
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
    int c = l->w.from_host(codes, (size_t)n * k / 2);
    if (!c) c = l->sw.from_host(scales, (size_t)n * k / 16);
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
    const uint32_t tiles_m = (m + kTile - 1) / kTile;
    uint32_t group = kern->group_m == 0 || kern->group_m > tiles_m ? tiles_m : kern->group_m;  // lib.rs:148-151
    fe_devptr_t aq = ws->aq.p, w = l->w.p, sw = l->sw.p, alpha = l->alpha.p;
    void *args[] = {&y, &aq, &w, &sw, &alpha, &res, &m, &n, &k, &ldy, &group};
    return fe_hip_launch(kern->gemm4, tiles_m * (n / kTile), 1, 1, 256, 1, 1, kGemmLds, s, args);
}

int fe_fp4_linear_forward(const fe_fp4_linear *l, const fe_fp4_kernels *kern, fe_stream_t s, const fe_fp4_workspace *ws,
                          fe_devptr_t y, uint32_t ldy, fe_devptr_t x, uint32_t lda, uint32_t m, fe_devptr_t res) {
    FE_TRY(fe_fp4_linear_quantize(l, kern, s, ws, x, lda, m));
    return fe_fp4_linear_gemm(l, kern, s, ws, y, ldy, m, res);
}

}  // extern "C"
