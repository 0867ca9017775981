// fe_exl3: host side of the EXL3 linear (see include/fe_exl3.h). Launch geometry, workspaces and argument checks
// follow crates/fe-exl3/src/linear.rs and crates/fe-exl3/src/gpu/mod.rs; the kernels are ferrite_amd/csrc/kernels/k_exl3.hip.
#include "fe_exl3.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "fe_internal.h"

namespace {

constexpr uint32_t kMaxRowsPerPass = 64;    // 4 row groups of 16
constexpr uint32_t kHatRows = 513;          // rows from which the prefill decodes once into fp16 tiles (3 output tile rows)
constexpr uint32_t kStreamRows = 16;        // the streamed GEMV takes one row group
constexpr uint32_t kGroupMax = 4;           // FE_EXL3_GROUP_MAX: linears of one grouped launch
constexpr uint32_t kGroupRows = 64;         // rows of a grouped launch (one GEMV pass)
constexpr uint32_t kLdsBudget = 60 * 1024;  // staged inputs of one GEMV program
constexpr uint32_t kJobLdsBudget = 76 * 1024;  // LDS of one program of the balanced GEMV
constexpr uint32_t kRedPitch = 132;         // GEMV_RED_PITCH
constexpr uint32_t kGemmLds = 2 * (256 + 256) * 64 * 2;  // two k tiles of A and W, 256 rows each; the epilogue reuses it

bool env_is(const char *name, const char *v) {
    const char *e = getenv(name);
    return e && strcmp(e, v) == 0;
}

const int kBits[] = {2, 3, 4, 5, 6, 8};

int bits_slot(uint32_t bits) {
    for (int i = 0; i < 6; i++)
        if ((uint32_t)kBits[i] == bits) return i;
    return -1;
}

}  // namespace

struct fe_exl3_kernels {
    fe_module_t module = nullptr;
    fe_function_t recon_hat_f32 = nullptr, recon_hat_f16 = nullptr, had_rows = nullptr, had_cols_bf16 = nullptr;
    fe_function_t rot_in = nullptr, rot_in_group = nullptr, probe_v4 = nullptr;
    fe_function_t probe_decode[3] = {nullptr, nullptr, nullptr};  // 3, 4, 5 bits
    fe_function_t gemv[6][4] = {};                                // [bits slot][row groups - 1]
    fe_function_t gemv_stream[6] = {};                            // 1..16 rows, streamed over the whole tensor
    fe_function_t gemv_group[6][4] = {};                          // several linears of one input, [bits slot][row groups - 1]
    fe_function_t gemvb[6][4] = {};                               // balanced over the CUs (plan ver 3), 1..4 linears a launch
    uint32_t cus = 0;
    fe_function_t gemm[6] = {};
    fe_function_t gemm_reduce = nullptr;
    fe_function_t hat_tiles[6] = {};  // trellis -> fp16 weights as the GEMM's LDS images
    fe_function_t gemm_hat = nullptr; // the GEMM over them
    uint32_t group_m = 8;
};

struct fe_exl3_linear {
    std::string name;
    uint32_t k = 0, n = 0, bits = 0;
    fe_exl3_plan plan{};
    uint32_t programs = 0;  // grid of the streamed GEMV (plan.ver == 2)
    fe_exl3_view view{};
    FeBuf trellis, suh, svh;  // owned copies (upload), empty for from_view
    FeBuf hat;                // decoded fp16 tiles kept with the linear (fe_exl3_linear_keep_decoded), else empty
    const fe_exl3_kernels *kern = nullptr;
};

struct fe_exl3_workspace {
    uint32_t max_rows = 0, max_k = 0;
    FeBuf xh, z, counters, part;  // part: partial tiles of the prefill GEMM (rows > 64 only)
    FeBuf hat;                    // decoded fp16 weights of one linear (workspaces of kHatRows rows or more)
    size_t z_len = 0, counters_len = 0;
};

int fe_load_module(fe_module_t *out, const char *env, const unsigned char *begin, const unsigned char *end) {
    const char *path = getenv(env);
    if (path && *path) return fe_hip_module_load_file(out, path);
    return fe_hip_module_load(out, begin, (size_t)(end - begin));
}

// (words between k steps, words between 128-column blocks), crates/fe-exl3/src/gpu/mod.rs:28-33
static void view_strides(const fe_exl3_view &v, uint32_t *stride_k, uint32_t *stride_nb) {
    uint32_t tw = 8 * v.bits;
    if (v.strips) {
        *stride_k = 8 * tw;
        *stride_nb = v.k / 16 * 8 * tw;
    } else {
        *stride_k = v.n / 16 * tw;
        *stride_nb = 8 * tw;
    }
}

extern "C" {

int fe_exl3_kernels_load(fe_exl3_kernels **out) {
    if (!out) return fe_set_error(FE_ERR_ARG, "fe_exl3_kernels_load", "null out");
    auto *k = new fe_exl3_kernels;
    int c = fe_load_module(&k->module, "FE_EXL3_HSACO", fe_k_exl3_hsaco, fe_k_exl3_hsaco_end);
    auto get = [&](fe_function_t *f, const char *name) {
        if (!c) c = fe_hip_module_get_function(f, k->module, name);
    };
    get(&k->recon_hat_f32, "exl3_recon_hat_f32");
    get(&k->recon_hat_f16, "exl3_recon_hat_f16");
    get(&k->had_rows, "exl3_had_rows");
    get(&k->had_cols_bf16, "exl3_had_cols_bf16");
    get(&k->rot_in, "exl3_rot_in");
    get(&k->rot_in_group, "exl3_rot_in_group");
    get(&k->probe_v4, "exl3_probe_v4");
    for (int b = 3; b <= 5; b++) {
        char nm[64];
        snprintf(nm, sizeof nm, "exl3_probe_decode_b%d", b);
        get(&k->probe_decode[b - 3], nm);
    }
    for (int i = 0; i < 6; i++) {
        char nm[64];
        for (int rg = 1; rg <= 4; rg++) {
            snprintf(nm, sizeof nm, "exl3_gemv_b%d_r%d", kBits[i], rg);
            get(&k->gemv[i][rg - 1], nm);
            if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemv[i][rg - 1], 64 * 1024);
        }
        snprintf(nm, sizeof nm, "exl3_gemv_stream_b%d", kBits[i]);
        get(&k->gemv_stream[i], nm);
        for (int rg = 1; rg <= 4; rg++) {
            snprintf(nm, sizeof nm, "exl3_gemvb_b%d_r%d", kBits[i], rg);
            get(&k->gemvb[i][rg - 1], nm);
            if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemvb[i][rg - 1], 84 * 1024);
        }
        for (int rg = 1; rg <= 4; rg++) {
            if (rg == 1)
                snprintf(nm, sizeof nm, "exl3_gemv_group_b%d", kBits[i]);
            else
                snprintf(nm, sizeof nm, "exl3_gemv_group_b%d_r%d", kBits[i], rg);
            get(&k->gemv_group[i][rg - 1], nm);
            if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemv_group[i][rg - 1], 64 * 1024);
        }
        snprintf(nm, sizeof nm, "exl3_gemm_b%d", kBits[i]);
        get(&k->gemm[i], nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm[i], kGemmLds);
        snprintf(nm, sizeof nm, "exl3_hat_tiles_b%d", kBits[i]);
        get(&k->hat_tiles[i], nm);
        if (i == 0) get(&k->gemm_reduce, "exl3_gemm_reduce");
    }
    get(&k->gemm_hat, "exl3_gemm_hat");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm_hat, kGemmLds);
    if (const char *g = getenv("FE_EXL3_GROUP")) k->group_m = (uint32_t)atoi(g);
    if (!c) {
        int cus = 0;
        c = fe_hip_cu_count(&cus);
        k->cus = (uint32_t)cus;
    }
    if (c) {
        fe_exl3_kernels_destroy(k);
        return c;
    }
    *out = k;
    return 0;
}

int fe_exl3_kernels_destroy(fe_exl3_kernels *k) {
    if (!k) return 0;
    if (k->module) fe_hip_module_unload(k->module);
    delete k;
    return 0;
}

// K splits for `blocks` programs: the divisor of the load-step count whose program count comes closest to the target
// while a program keeps at least min_steps load steps (the role of tf_plan, crates/fe-exl3/src/linear.rs:100-129; one
// load step = 4 k steps = 64 input channels). Programs of fewer than 8 steps cost more in start-up, partial sums and
// hand-off than their spread over the CUs gains: 5120 x 5120 at 1 row takes 11.9 us cut 10 ways and 13.3 us cut 16
// ways, 5120 x 1024 9.5 us cut 10 ways and 13.8 us cut 40 ways.
int fe_exl3_plan_for(uint32_t k, uint32_t n, uint32_t bits, uint32_t blocks, fe_exl3_plan *out) {
    (void)bits;
    if (!out || !k || !n || k % 128 || n % 128) return fe_set_error(FE_ERR_SHAPE, "fe_exl3_plan_for", "k, n must be multiples of 128");
    const uint32_t steps = k / 64, nb = n / 128, min_steps = std::min(8u, std::max(2u, steps / 2));
    // the divisor of the step count whose program count nb * d comes closest (as a ratio) to `blocks`
    uint32_t sk = 1;
    double best = 1e30;
    for (uint32_t d = 1; d <= steps; d++) {
        if (steps % d) continue;
        if (steps / d < min_steps) break;
        double ratio = (double)nb * d / (blocks ? blocks : 1);
        double miss = ratio < 1.0 ? 1.0 / ratio : ratio;
        if (miss < best) best = miss, sk = d;
    }
    if (env_is("FE_EXL3_NOSPLIT", "1") || env_is("FE_EXL3_SPLIT", "0")) sk = 1;
    // ver 3 (the default): the GEMV balanced over the CUs, occ programs per CU, for 1..64 rows, one summation order for all
    // of them. ver 1 (FE_EXL3_VER=1): the split-K GEMV, sk splits. ver 2 (FE_EXL3_STREAM=1): rows 1..16 run the streamed
    // GEMV with occ programs per CU.
    uint32_t ver = env_is("FE_EXL3_STREAM", "1") ? 2 : 3, occ = 0;
    if (const char *v = getenv("FE_EXL3_VER")) ver = (uint32_t)atoi(v);
    if (ver == 2) occ = 2;
    if (ver == 3) occ = 4;
    if (const char *o = getenv("FE_EXL3_OCC")) occ = (uint32_t)atoi(o);
    *out = fe_exl3_plan{sk, 4, ver, ver == 1 ? 0 : occ};
    return 0;
}

int fe_exl3_plan_parse(const char *s, fe_exl3_plan *out) {
    if (!s || !out) return fe_set_error(FE_ERR_ARG, "fe_exl3_plan_parse", "null");
    unsigned v[4] = {0, 0, 1, 0};
    int got = sscanf(s, " %u , %u , %u , %u", &v[0], &v[1], &v[2], &v[3]);
    if (got < 2) return fe_set_error(FE_ERR_ARG, "fe_exl3_plan_parse", s);
    *out = fe_exl3_plan{v[0], v[1], v[2], v[3]};
    return 0;
}

// Programs of the streamed GEMV: occ per CU, at most one per eight work units (FE_EXL3_PROGRAMS overrides the count).
static uint32_t stream_programs(const fe_exl3_kernels *kern, const fe_exl3_plan &p, uint32_t k, uint32_t n) {
    if (p.ver == 3) {
        // balanced GEMV: occ programs per CU, each a run of at least min_units 128-channel blocks of one column block
        const uint32_t units = (k / 128) * (n / 128), occ = p.occ ? p.occ : 4;
        uint32_t min_units = 4;
        if (const char *e = getenv("FE_EXL3_MIN_UNITS")) min_units = std::max(1, atoi(e));  // tuning
        return std::max(1u, std::min(occ * std::max(kern->cus, 1u), units / min_units));
    }
    if (p.ver != 2) return 0;
    const uint32_t units = (k / 64) * (n / 128), occ = p.occ ? p.occ : 2;
    uint32_t progs = std::min(occ * kern->cus, units / 8);
    if (const char *e = getenv("FE_EXL3_PROGRAMS")) progs = std::min((uint32_t)atoi(e), units);  // tuning and tests
    return std::max(1u, progs);
}

static int check_fit(const char *name, uint32_t k, uint32_t n, uint32_t bits, const fe_exl3_plan &p) {
    char msg[160];
    if (bits_slot(bits) < 0) {
        snprintf(msg, sizeof msg, "%s: %u bits (kernels exist for 2, 3, 4, 5, 6, 8)", name, bits);
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_linear", msg);
    }
    // linear.rs:244: k, n multiples of 128 and the K range divides into the plan's pieces (here: load steps of 64)
    if (!k || !n || k % 128 || n % 128 || p.sk == 0 || (k / 64) % p.sk) {
        snprintf(msg, sizeof msg, "%s: %ux%u does not fit plan sk %u", name, k, n, p.sk);
        return fe_set_error(FE_ERR_SHAPE, "fe_exl3_linear", msg);
    }
    return 0;
}

int fe_exl3_linear_from_view(fe_exl3_linear **out, const fe_exl3_kernels *kern, const char *name, const fe_exl3_view *view,
                             const fe_exl3_plan *plan) {
    if (!out || !kern || !view || !plan) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_from_view", "null argument");
    FE_TRY(check_fit(name ? name : "?", view->k, view->n, view->bits, *plan));
    auto *l = new fe_exl3_linear;
    l->name = name ? name : "";
    l->k = view->k, l->n = view->n, l->bits = view->bits;
    l->plan = *plan;
    l->view = *view;
    l->kern = kern;
    l->programs = stream_programs(kern, *plan, view->k, view->n);
    *out = l;
    return 0;
}

int fe_exl3_linear_upload(fe_exl3_linear **out, const fe_exl3_kernels *kern, const char *name, uint32_t k, uint32_t n,
                          uint32_t bits, const uint32_t *trellis, const uint16_t *suh, const uint16_t *svh, int strips,
                          const fe_exl3_plan *plan, uint32_t blocks) {
    if (!out || !kern || !trellis || !suh || !svh) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_upload", "null argument");
    fe_exl3_plan p;
    if (plan)
        p = *plan;
    else
        FE_TRY(fe_exl3_plan_for(k, n, bits, blocks, &p));
    FE_TRY(check_fit(name ? name : "?", k, n, bits, p));
    auto *l = new fe_exl3_linear;
    l->name = name ? name : "";
    l->k = k, l->n = n, l->bits = bits, l->plan = p, l->kern = kern;
    l->programs = stream_programs(kern, p, k, n);
    const size_t tw = 8 * (size_t)bits, kt = k / 16, nt = n / 16, words = kt * nt * tw;
    int c = 0;
    if (strips) {
        // [n/128][k/16][8][tw] (Exl3Tensor::strips, crates/fe-exl3/src/format.rs:70-84)
        std::vector<uint32_t> st(words);
        for (size_t b = 0; b < nt / 8; b++)
            for (size_t t = 0; t < kt; t++)
                memcpy(&st[(b * kt + t) * 8 * tw], &trellis[(t * nt + b * 8) * tw], 8 * tw * sizeof(uint32_t));
        c = l->trellis.from_host(st.data(), words * 4);
    } else {
        c = l->trellis.from_host(trellis, words * 4);
    }
    if (!c) c = l->suh.from_host(suh, (size_t)k * 2);
    if (!c) c = l->svh.from_host(svh, (size_t)n * 2);
    if (c) {
        delete l;
        return c;
    }
    l->view = fe_exl3_view{k, n, bits, l->trellis.p, l->suh.p, l->svh.p, strips ? 1u : 0u};
    *out = l;
    return 0;
}

int fe_exl3_linear_destroy(fe_exl3_linear *l) {
    delete l;
    return 0;
}

int fe_exl3_linear_view(const fe_exl3_linear *l, fe_exl3_view *view, fe_exl3_plan *plan) {
    if (!l) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_view", "null linear");
    if (view) *view = l->view;
    if (plan) *plan = l->plan;
    return 0;
}

size_t fe_exl3_linear_weight_bytes(const fe_exl3_linear *l) { return l ? (size_t)l->k * l->n * l->bits / 8 : 0; }

// Many rows: decoding the trellis once into fp16 tiles and running the GEMM over them beats decoding inside the GEMM,
// where each 256-row tile of the output decodes its weights again. From kHatRows rows on (FE_EXL3_HAT_ROWS overrides; 0
// turns the form off) and only with a workspace created for that many rows, which then holds the largest linear's
// decoded weights (2 bytes a weight).
static uint32_t hat_rows() {
    const char *e = getenv("FE_EXL3_HAT_ROWS");  // read per call: tests compare both forms in one process
    if (!e) return kHatRows;
    int v = atoi(e);
    return v <= 0 ? 0xffffffffu : std::max<uint32_t>((uint32_t)v, kMaxRowsPerPass + 1);
}
static size_t hat_bytes(const fe_exl3_linear *l) { return (size_t)((l->n / 128 + 1) / 2) * 256 * l->k * 2; }

int fe_exl3_workspace_create(fe_exl3_workspace **out, fe_exl3_linear *const *linears, size_t count, uint32_t max_rows) {
    if (!out || (count && !linears) || !max_rows) return fe_set_error(FE_ERR_ARG, "fe_exl3_workspace_create", "bad argument");
    size_t max_k = 128, max_z = 0, max_zs = 0, max_nb = 1, max_hat = 0;
    std::vector<size_t> zs, nbs;  // per linear, for the grouped launch: room for the kGroupMax largest together
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = linears[i];
        zs.push_back(l->plan.ver == 3 ? (size_t)(l->programs + l->n / 128) * 128 : l->plan.ver == 2 ? 0 : (size_t)l->plan.sk * l->n);
        nbs.push_back(l->n / 128);
        max_hat = std::max(max_hat, hat_bytes(l));
        max_k = std::max<size_t>(max_k, l->k);
        if (l->plan.ver != 3 && l->plan.sk > 1) max_z = std::max<size_t>(max_z, (size_t)l->plan.sk * l->n);
        if (l->plan.ver == 3) max_z = std::max<size_t>(max_z, (size_t)(l->programs + l->n / 128) * 128);
        if (l->plan.ver == 2) max_zs = std::max<size_t>(max_zs, (size_t)(l->programs + l->n / 128) * 128);
        max_nb = std::max<size_t>(max_nb, l->n / 128);
    }
    auto *ws = new fe_exl3_workspace;
    ws->max_rows = max_rows, ws->max_k = (uint32_t)max_k;
    auto top = [](std::vector<size_t> &v) {
        std::sort(v.begin(), v.end(), std::greater<size_t>());
        size_t t = 0;
        for (size_t i = 0; i < v.size() && i < kGroupMax; i++) t += v[i];
        return t;
    };
    const size_t group_z = top(zs), group_nb = top(nbs);
    ws->z_len = std::max<size_t>(std::max(max_z * std::min(max_rows, kMaxRowsPerPass), max_zs * std::min(max_rows, kStreamRows)), 4);
    ws->z_len = std::max(ws->z_len, group_z * std::min(max_rows, kGroupRows));
    ws->counters_len = std::max((size_t)((max_rows + 7) / 8) * max_nb, group_nb);
    // (rotated inputs: one linear's at max_rows, or a group's at up to kGroupRows rows each)
    int c = ws->xh.alloc((size_t)std::max(max_rows, kGroupMax * std::min(max_rows, kGroupRows)) * max_k * 2);
    if (!c) c = ws->z.alloc(ws->z_len * 4);
    if (!c) c = ws->counters.zeroed(ws->counters_len * 4);
    int cus = 0;
    if (!c && max_rows > kMaxRowsPerPass) c = fe_hip_cu_count(&cus);
    if (!c && cus > 0) c = ws->part.alloc((size_t)cus * kFeGemmSlotsPerCu * kFeGemmPartBytes);
    // zeroed once: the unused half of the last tile of an odd count of column blocks is read (and its sums discarded)
    if (!c && max_rows >= hat_rows() && max_hat) c = ws->hat.zeroed(max_hat);
    if (c) {
        delete ws;
        return c;
    }
    *out = ws;
    return 0;
}

int fe_exl3_workspace_destroy(fe_exl3_workspace *ws) {
    delete ws;
    return 0;
}

int fe_exl3_workspace_xh(const fe_exl3_workspace *ws, fe_devptr_t *xh, uint32_t *max_rows, uint32_t *max_k) {
    if (!ws) return fe_set_error(FE_ERR_ARG, "fe_exl3_workspace_xh", "null workspace");
    if (xh) *xh = ws->xh.p;
    if (max_rows) *max_rows = ws->max_rows;
    if (max_k) *max_k = ws->max_k;
    return 0;
}

// The input of a rotation: bf16 (mode 0) or f32 (mode 1) rows of stride ld, or (mode 2) SwiGLU of two bf16 arrays,
// x = gate and x2 = up, taken on the way in (RotSrc of k_exl3.hip).
struct RotInput {
    fe_devptr_t x = 0, x2 = 0;
    uint32_t mode = 0, ld = 0;
};

static int launch_rot(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, const RotInput &in, uint32_t rows,
                      const fe_exl3_workspace *ws, const char *fn) {
    if (rows == 0 || rows > ws->max_rows || l->k > ws->max_k) {
        char msg[160];
        snprintf(msg, sizeof msg, "%s: rows %u (workspace %u x %u)", l->name.c_str(), rows, ws->max_rows, ws->max_k);
        return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
    }
    uint32_t mode = in.mode, k = l->k, ld = in.ld;
    fe_devptr_t x = in.x, x2 = in.x2, suh = l->view.suh, xh = ws->xh.p;
    void *args[] = {&x, &mode, &suh, &xh, &k, &x2, &ld};
    return fe_hip_launch(kern->rot_in, (k + 511) / 512, rows, 1, 128, 1, 1, 0, s, args);
}

int fe_exl3_linear_rotate_input(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                int x_dtype, uint32_t rows, const fe_exl3_workspace *ws) {
    if (!l || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_rotate_input", "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32)
        return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_rotate_input", "x is bf16 or f32");
    RotInput in;
    in.x = x, in.mode = (uint32_t)x_dtype & 1, in.ld = l->k;
    return launch_rot(l, kern, s, in, rows, ws, "fe_exl3_linear_rotate_input");
}

// trellis -> fp16 tiles (exl3_hat_tiles_b*) into `hat`, hat_bytes(l) bytes
static int launch_decode(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t hat) {
    const fe_exl3_kernels *kern = l->kern;
    uint32_t k = l->k, stride_k, stride_nb;
    view_strides(l->view, &stride_k, &stride_nb);
    const uint32_t ktiles = k / 64, nbs = l->n / 128;
    const uint32_t gy = std::min(ktiles, std::max(1u, (8 * std::max(kern->cus, 1u) + nbs - 1) / nbs));
    fe_devptr_t tr = l->view.trellis;
    void *dargs[] = {&tr, &hat, &k, &stride_k, &stride_nb};
    return fe_hip_launch(kern->hat_tiles[bits_slot(l->bits)], nbs, gy, 1, 256, 1, 1, 0, s, dargs);
}

static int launch_gemm(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype, uint32_t rows,
                       const fe_exl3_workspace *ws) {
    const fe_exl3_kernels *kern = l->kern;
    uint32_t n = l->n, k = l->k, mode = (uint32_t)y_dtype, stride_k, stride_nb, group = kern->group_m;
    view_strides(l->view, &stride_k, &stride_nb);
    if ((uint64_t)rows * k * 2 >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_linear_gemv_rotated", "rotated input of 4 GB or more");
    const uint32_t tiles_m = (rows + 255) / 256, tiles_n = (n / 128 + 1) / 2;
    if (group == 0 || group > tiles_m) group = tiles_m;
    FeGemmSplit g = fe_gemm_split(tiles_m * tiles_n, k / 64, kern->cus, (uint32_t)(ws->part.bytes / kFeGemmPartBytes));
    uint32_t full = g.full, splits = g.splits;
    fe_devptr_t tr = l->view.trellis, svh = l->view.svh, part = ws->part.p;
    const bool kept = l->hat.bytes != 0;  // decoded once and kept: any row count above the GEMV's runs over it
    if (kept || (rows >= hat_rows() && ws->hat.bytes >= hat_bytes(l))) {
        fe_devptr_t hat = kept ? l->hat.p : ws->hat.p;
        if (!kept) FE_TRY(launch_decode(l, s, hat));
        group = 0;  // the raster that deals column tiles to the XCDs: each decoded weight panel goes through one L2
        void *args[] = {&xh, &hat, &svh, &y, &n, &k, &rows, &mode, &group, &full, &splits, &part};
        FE_TRY(fe_hip_launch(kern->gemm_hat, g.programs(), 1, 1, 256, 1, 1, kGemmLds, s, args));
    } else {
        void *args[] = {&xh, &tr, &svh, &y, &n, &k, &rows, &mode, &stride_k, &stride_nb, &group, &full, &splits, &part};
        FE_TRY(fe_hip_launch(kern->gemm[bits_slot(l->bits)], g.programs(), 1, 1, 256, 1, 1, kGemmLds, s, args));
    }
    if (!g.cut()) return 0;
    void *rargs[] = {&part, &svh, &y, &n, &rows, &mode, &group, &full, &splits};
    return fe_hip_launch(kern->gemm_reduce, g.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

// Decode-sized rows. With in.x != 0 the split-K kernel rotates that input itself and leaves the rotated rows in xh
// (callers check fused_rotation_fits first); otherwise it reads xh.
static int launch_rows(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype, uint32_t rows,
                       const fe_exl3_workspace *ws, const RotInput &in);
static uint32_t gemv_chunk(uint32_t rows, uint32_t steps);

// The split-K kernel can rotate its own input when every program's K range is whole 128-element blocks.
static bool fused_rotation_fits(const fe_exl3_linear *l, uint32_t rows) {
    const char *e = getenv("FE_EXL3_NO_FUSED_ROT");  // read per call: tests compare both paths in one process
    const bool off = e && atoi(e) != 0;
    const fe_exl3_plan &p = l->plan;
    if (p.ver == 3) {
        // every program rotates the channels of its own run: (row, 128-channel block) pairs, 8 at a time
        if (off || rows < 1 || rows > kMaxRowsPerPass) return false;
        uint32_t pairs = 16;
        if (const char *t = getenv("FE_EXL3_FUSED_ROT_PAIRS")) pairs = (uint32_t)atoi(t);
        const uint32_t units = (l->k / 128) * (l->n / 128);
        return rows * ((units + l->programs - 1) / l->programs) <= pairs;
    }
    if (off || rows < 1 || rows > kMaxRowsPerPass || p.ver == 2 || (l->k / 64 / p.sk) % 2) return false;
    // every column block repeats the rotation of its K range: (row, 128-block) pairs a program, 8 at a time. Measured on
    // 5120 x 17408 (8 blocks a program): one launch wins up to 4 rows (19.9 against 22.3 us at 1 row), the separate
    // rotation from 8 rows on (25.2 against 23.7 us).
    uint32_t pairs = 32;
    if (const char *t = getenv("FE_EXL3_FUSED_ROT_PAIRS")) pairs = (uint32_t)atoi(t);
    return rows * (l->k / 128 / p.sk) <= pairs;
}

int fe_exl3_linear_gemv_rotated(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype,
                                uint32_t rows, const fe_exl3_workspace *ws) {
    return launch_rows(l, s, xh, y, y_dtype, rows, ws, RotInput{});
}

// mirrors GemvJob of k_exl3.hip
struct GemvJobArgs {
    uint32_t count, first[kGroupMax + 1];
    struct Member {
        fe_devptr_t trellis, svh, suh, xh, y, z, counters;
        uint32_t n, programs, stride_k, stride_nb, base, rem, inv_base, inv_base1;
    } m[kGroupMax];
};
static_assert(sizeof(GemvJobArgs) == 24 + kGroupMax * 88, "GemvJob layout");

// Room a balanced launch takes in the workspace: partial sums (floats) and counters of one member at `rows` rows.
static size_t job_z(const fe_exl3_linear *l, uint32_t rows) { return (size_t)(l->programs + l->n / 128) * 128 * rows; }

// The balanced GEMV (plan ver 3) for 1..4 linears of one input in one launch: member i reads its rotated input at xhs[i]
// (in.x == 0) or rotates in.x itself and leaves the result at xhs[i]. The caller has checked rows, k and bits.
static int launch_job(const fe_exl3_linear *const *ls, size_t count, fe_stream_t s, const fe_devptr_t *xhs, const fe_devptr_t *ys,
                      int y_dtype, uint32_t rows, const fe_exl3_workspace *ws, const RotInput &in, const char *fn) {
    GemvJobArgs g{};
    g.count = (uint32_t)count;
    uint32_t programs = 0, run_steps = 0;
    size_t z_at = 0, cnt_at = 0;
    char msg[200];
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = ls[i];
        GemvJobArgs::Member &m = g.m[i];
        if (z_at + job_z(l, rows) > ws->z_len || cnt_at + l->n / 128 > ws->counters_len) {
            snprintf(msg, sizeof msg, "%s: %u rows do not fit the workspace (partial sums %zu of %zu floats, counters %zu of %zu)",
                     l->name.c_str(), rows, z_at + job_z(l, rows), ws->z_len, cnt_at + l->n / 128, ws->counters_len);
            return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
        }
        m.trellis = l->view.trellis, m.svh = l->view.svh, m.suh = l->view.suh, m.xh = xhs[i], m.y = ys[i];
        m.z = ws->z.p + z_at * 4, m.counters = ws->counters.p + cnt_at * 4;
        m.n = l->n, m.programs = l->programs;
        view_strides(l->view, &m.stride_k, &m.stride_nb);
        g.first[i] = programs;
        programs += l->programs;
        z_at += job_z(l, rows), cnt_at += l->n / 128;
        const uint32_t units = (l->k / 128) * (l->n / 128);
        m.base = units / l->programs, m.rem = units % l->programs;
        m.inv_base = 0xffffffffu / m.base, m.inv_base1 = 0xffffffffu / (m.base + 1);
        run_steps = std::max(run_steps, 2 * ((units + l->programs - 1) / l->programs));
    }
    for (size_t i = count; i <= kGroupMax; i++) g.first[i] = programs;
    // staged inputs: the whole run where the LDS budget holds it for `rows` rows, else chunks of a multiple of 4 load steps
    const uint32_t red = rows * kRedPitch * 4;
    uint32_t chunk = std::max(4u, ((kJobLdsBudget - red) / rows - 16) / 128 / 4 * 4);
    chunk = std::min(chunk, (run_steps + 3) / 4 * 4);
    uint32_t lds = red + rows * (chunk * 128 + 16);
    // Exactly occ programs a CU: the dispatcher fills a CU as far as registers and LDS allow (5 programs) before it moves
    // on, which would leave CUs empty while others hold 5; an LDS request that fits occ times into the CU's 160 KB, and
    // not occ + 1 times, makes the CUs take occ each.
    if (const uint32_t occ = ls[0]->plan.occ; occ && !env_is("FE_EXL3_NO_LDS_PAD", "1")) lds = std::max(lds, 163840u / (occ + 1) + 512);
    uint32_t k = ls[0]->k, mode = (uint32_t)y_dtype, x_mode = in.mode, ldx = in.ld;
    fe_devptr_t x = in.x, x2 = in.x2;
    // (the last argument exists only in timeline-probe builds of the code object; the shipped kernels take ten)
    static const fe_devptr_t stamps = getenv("FE_EXL3_STAMPS") ? (fe_devptr_t)strtoull(getenv("FE_EXL3_STAMPS"), nullptr, 0) : 0;
    fe_devptr_t st = stamps;
    uint32_t inv_spb = 0xffffffffu / (k / 64);
    void *args[] = {&g, &x, &x2, &x_mode, &ldx, &k, &rows, &mode, &chunk, &inv_spb, &st};
    return fe_hip_launch(ls[0]->kern->gemvb[bits_slot(ls[0]->bits)][(rows + 15) / 16 - 1], programs, 1, 1, 256, 1, 1, lds, s, args);
}

static int launch_rows(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype, uint32_t rows,
                       const fe_exl3_workspace *ws, const RotInput &in) {
    if (!l || !ws || !xh || !y) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_gemv_rotated", "null argument");
    if (y_dtype < 0 || y_dtype > 3) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_gemv_rotated", "bad y dtype");
    const fe_exl3_plan &p = l->plan;
    char msg[200];
    if (rows > kMaxRowsPerPass) {
        if (rows > ws->max_rows) {
            snprintf(msg, sizeof msg, "%s: rows %u do not fit the workspace (max %u)", l->name.c_str(), rows, ws->max_rows);
            return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_linear_gemv_rotated", msg);
        }
        return launch_gemm(l, s, xh, y, y_dtype, rows, ws);
    }
    if (p.ver == 3) {
        if (rows == 0 || rows > ws->max_rows) {
            snprintf(msg, sizeof msg, "%s: rows %u do not fit the workspace (max %u)", l->name.c_str(), rows, ws->max_rows);
            return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_linear_gemv_rotated", msg);
        }
        return launch_job(&l, 1, s, &xh, &y, y_dtype, rows, ws, in, "fe_exl3_linear_gemv_rotated");
    }
    if (p.ver == 2 && rows >= 1 && rows <= kStreamRows) {
        if (rows > ws->max_rows || ws->z_len < (size_t)(l->programs + l->n / 128) * 128 * rows || ws->counters_len < l->n / 128) {
            snprintf(msg, sizeof msg, "%s: rows %u do not fit the workspace (max %u, z %zu)", l->name.c_str(), rows, ws->max_rows,
                     ws->z_len);
            return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_linear_gemv_rotated", msg);
        }
        uint32_t n = l->n, k = l->k, mode = (uint32_t)y_dtype, stride_k, stride_nb;
        view_strides(l->view, &stride_k, &stride_nb);
        fe_devptr_t tr = l->view.trellis, svh = l->view.svh, z = ws->z.p, cnt = ws->counters.p;
        void *args[] = {&xh, &tr, &svh, &y, &z, &cnt, &n, &k, &rows, &mode, &stride_k, &stride_nb};
        return fe_hip_launch(l->kern->gemv_stream[bits_slot(l->bits)], l->programs, 1, 1, 256, 1, 1, 0, s, args);
    }
    // linear.rs:302-307
    if (rows == 0 || rows > ws->max_rows || (p.sk > 1 && ws->z_len < (size_t)p.sk * rows * l->n)) {
        snprintf(msg, sizeof msg, "%s: rows %u do not fit the workspace (max %u, z %zu)", l->name.c_str(), rows, ws->max_rows,
                 ws->z_len);
        return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_linear_gemv_rotated", msg);
    }
    if (ws->counters_len < (size_t)((rows + 7) / 8) * (l->n / 128)) {
        snprintf(msg, sizeof msg, "%s: workspace counters too small for %u rows", l->name.c_str(), rows);
        return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_linear_gemv_rotated", msg);
    }
    const uint32_t rg = (rows + 15) / 16;
    const uint32_t steps = l->k / 64 / p.sk;
    uint32_t chunk = gemv_chunk(rows, steps);
    const uint32_t lds = std::max(rows * (chunk * 128 + 16), rows * kRedPitch * 4);
    uint32_t n = l->n, k = l->k, sk = p.sk, mode = (uint32_t)y_dtype, stride_k, stride_nb;
    view_strides(l->view, &stride_k, &stride_nb);
    fe_devptr_t tr = l->view.trellis, svh = l->view.svh, z = ws->z.p, cnt = ws->counters.p;
    fe_devptr_t suh = l->view.suh, x = in.x, x2 = in.x2;
    uint32_t x_mode = in.mode, ldx = in.ld;
    void *args[] = {&xh, &tr, &svh, &y, &z, &cnt, &n, &k, &rows, &sk, &mode, &stride_k, &stride_nb, &chunk, &x, &x_mode, &suh, &xh, &x2, &ldx};
    return fe_hip_launch(l->kern->gemv[bits_slot(l->bits)][rg - 1], n / 128 * sk, 1, 1, 256, 1, 1, lds, s, args);
}

int fe_exl3_linear_keep_decoded(fe_exl3_linear *l, fe_stream_t s, int on) {
    if (!l) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_keep_decoded", "null linear");
    if (!on) {
        l->hat.release();
        return 0;
    }
    if (l->hat.bytes) return 0;
    FE_TRY(l->hat.zeroed(hat_bytes(l)));  // zeroed: the unused half of the last tile of an odd count of column blocks is read
    int c = launch_decode(l, s, l->hat.p);
    if (c) l->hat.release();
    return c;
}

int fe_exl3_linear_forward_is_one_launch(const fe_exl3_linear *l, uint32_t rows) { return l && fused_rotation_fits(l, rows); }

// forward() on a described input: one launch where the GEMV rotates its own input, else the rotation and the linear.
static int forward_from(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, const RotInput &in, fe_devptr_t y,
                        int y_dtype, uint32_t rows, const fe_exl3_workspace *ws, const char *fn) {
    if (fused_rotation_fits(l, rows)) {
        if (rows > ws->max_rows || l->k > ws->max_k) {
            char msg[160];
            snprintf(msg, sizeof msg, "%s: rows %u (workspace %u x %u)", l->name.c_str(), rows, ws->max_rows, ws->max_k);
            return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
        }
        return launch_rows(l, s, ws->xh.p, y, y_dtype, rows, ws, in);
    }
    FE_TRY(launch_rot(l, kern, s, in, rows, ws, fn));
    return fe_exl3_linear_gemv_rotated(l, s, ws->xh.p, y, y_dtype, rows, ws);
}

int fe_exl3_linear_forward(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype,
                           fe_devptr_t y, int y_dtype, uint32_t rows, const fe_exl3_workspace *ws) {
    if (!l || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward", "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32)
        return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward", "x is bf16 or f32");
    RotInput in;
    in.x = x, in.mode = (uint32_t)x_dtype & 1, in.ld = l->k;
    return forward_from(l, kern, s, in, y, y_dtype, rows, ws, "fe_exl3_linear_forward");
}

}  // extern "C"

int fe_exl3_forward_over(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype,
                         fe_devptr_t y, int y_dtype, uint32_t rows, uint32_t max_rows, fe_devptr_t counters,
                         size_t counters_bytes, fe_devptr_t xh, size_t xh_bytes, fe_devptr_t z, size_t z_bytes, const char *fn) {
    if (!l || !kern || !x || !y) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32) return fe_set_error(FE_ERR_ARG, fn, "x is bf16 or f32");
    char msg[200];
    max_rows = std::min(max_rows, kMaxRowsPerPass);
    if (rows == 0 || rows > max_rows) {
        snprintf(msg, sizeof msg, "%s: %u rows (this entry point takes 1..%u)", l->name.c_str(), rows, max_rows);
        return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
    }
    const size_t need_xh = (size_t)rows * l->k * 2, need_cnt = (size_t)((rows + 7) / 8) * (l->n / 128) * 4;
    const size_t need_z = l->plan.ver == 3 ? job_z(l, rows) * 4
                          : l->plan.ver == 2 ? (size_t)(l->programs + l->n / 128) * 128 * rows * 4
                                           : (l->plan.sk > 1 ? (size_t)l->plan.sk * rows * l->n * 4 : 0);
    if (need_xh > xh_bytes || need_cnt > counters_bytes || need_z > z_bytes) {
        snprintf(msg, sizeof msg, "%s: %u rows of %ux%u need %zu B of rotated inputs (limit %zu), %zu B of partial sums (limit %zu), "
                 "%zu B of counters (limit %zu)", l->name.c_str(), rows, l->k, l->n, need_xh, xh_bytes, need_z, z_bytes, need_cnt,
                 counters_bytes);
        return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
    }
    fe_exl3_workspace ws;  // views only: nothing is allocated and nothing is freed
    ws.max_rows = rows, ws.max_k = l->k;
    ws.xh.view(xh, xh_bytes), ws.z.view(z, z_bytes), ws.counters.view(counters, counters_bytes);
    ws.z_len = z_bytes / 4, ws.counters_len = counters_bytes / 4;
    RotInput in;
    in.x = x, in.mode = (uint32_t)x_dtype & 1, in.ld = l->k;
    return forward_from(l, kern, s, in, y, y_dtype, rows, &ws, fn);
}

extern "C" {

int fe_exl3_linear_forward_swiglu(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t gate,
                                  fe_devptr_t up, uint32_t ld, fe_devptr_t y, int y_dtype, uint32_t rows,
                                  const fe_exl3_workspace *ws) {
    const char *fn = "fe_exl3_linear_forward_swiglu";
    if (!l || !kern || !ws || !gate || !up) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (ld < l->k || ld % 4 || gate % 8 || up % 8) return fe_set_error(FE_ERR_ARG, fn, "gate / up: rows of at least k elements, 8-byte aligned");
    RotInput in;
    in.x = gate, in.x2 = up, in.mode = 2, in.ld = ld;
    return forward_from(l, kern, s, in, y, y_dtype, rows, ws, fn);
}

// mirrors GemvGroup of k_exl3.hip
struct GemvGroupArgs {
    uint32_t count, first[kGroupMax + 1];
    struct Member {
        fe_devptr_t trellis, svh, suh, xh, y, z, counters;
        uint32_t n, sk, stride_k, stride_nb, chunk, pad;
    } m[kGroupMax];
};
struct RotGroupArgs {  // RotGroup
    fe_devptr_t suh[kGroupMax], xh[kGroupMax];
};

static uint32_t gemv_chunk(uint32_t rows, uint32_t steps) {
    // staged input chunk: as many load steps as the LDS budget holds for `rows` rows, a multiple of 4
    uint32_t chunk = (kLdsBudget / rows - 16) / 128 / 4 * 4;
    chunk = std::max(chunk, 4u);
    return std::min(chunk, (steps + 3) / 4 * 4);
}

// The grouped launch: the same input, width and kernel, and room in the workspace for every member's partials (and,
// where the members do not rotate their own input, rotated inputs) side by side. *fused: the GEMV rotates its own input.
static bool group_fits(const fe_exl3_linear *const *ls, size_t count, uint32_t rows, const fe_exl3_workspace *ws, bool *fused) {
    const char *e = getenv("FE_EXL3_NO_GROUP");  // read per call: tests compare both paths in one process
    if (e && atoi(e) != 0) return false;
    if (!ls || !ws || count < 2 || count > kGroupMax || rows < 1 || rows > kGroupRows || rows > ws->max_rows) return false;
    size_t z = 0, nb = 0;
    bool f = true;
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = ls[i];
        if (!l || l->k != ls[0]->k || l->bits != ls[0]->bits || l->kern != ls[0]->kern || l->plan.ver == 2 ||
            l->plan.ver != ls[0]->plan.ver)
            return false;
        f = f && fused_rotation_fits(l, rows);
        z += l->plan.ver == 3 ? job_z(l, rows) : (size_t)l->plan.sk * rows * l->n;
        nb += l->n / 128;
    }
    if (!f && count * (size_t)rows * ls[0]->k * 2 > ws->xh.bytes) return false;
    if (fused) *fused = f;
    return z <= ws->z_len && nb <= ws->counters_len && ls[0]->k <= ws->max_k;
}

int fe_exl3_linear_forward_group_launches(const fe_exl3_linear *const *ls, size_t count, uint32_t rows,
                                          const fe_exl3_workspace *ws) {
    bool fused = false;
    if (!group_fits(ls, count, rows, ws, &fused)) return 0;
    return fused ? 1 : 2;
}

int fe_exl3_linear_forward_group(const fe_exl3_linear *const *ls, size_t count, const fe_exl3_kernels *kern, fe_stream_t s,
                                 fe_devptr_t x, int x_dtype, const fe_devptr_t *ys, int y_dtype, uint32_t rows,
                                 const fe_exl3_workspace *ws) {
    if (!ls || !ys || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward_group", "null argument");
    bool fused = false;
    if (!group_fits(ls, count, rows, ws, &fused)) {  // member by member: the same bits, more launches
        for (size_t i = 0; i < count; i++) FE_TRY(fe_exl3_linear_forward(ls[i], kern, s, x, x_dtype, ys[i], y_dtype, rows, ws));
        return 0;
    }
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32)
        return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward_group", "x is bf16 or f32");
    if (y_dtype < 0 || y_dtype > 3) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward_group", "bad y dtype");
    if (ls[0]->plan.ver == 3) {
        RotGroupArgs r{};
        fe_devptr_t xhs[kGroupMax] = {};
        for (size_t i = 0; i < count; i++) {
            if (!ys[i]) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward_group", "null output");
            xhs[i] = ws->xh.p + i * (size_t)rows * ls[i]->k * 2;
            r.suh[i] = ls[i]->view.suh, r.xh[i] = xhs[i];
        }
        RotInput in;
        uint32_t x_mode = (uint32_t)x_dtype & 1, k = ls[0]->k;
        if (fused) {
            in.x = x, in.mode = x_mode, in.ld = k;
        } else {  // one launch rotates the input for every member
            void *rargs[] = {&r, &x, &x_mode, &k};
            FE_TRY(fe_hip_launch(kern->rot_in_group, (k + 511) / 512, rows, (uint32_t)count, 128, 1, 1, 0, s, rargs));
        }
        return launch_job(ls, count, s, xhs, ys, y_dtype, rows, ws, in, "fe_exl3_linear_forward_group");
    }
    GemvGroupArgs g{};
    RotGroupArgs r{};
    g.count = (uint32_t)count;
    uint32_t lds = 0, programs = 0;
    size_t z_at = 0, cnt_at = 0;
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = ls[i];
        if (!ys[i]) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward_group", "null output");
        GemvGroupArgs::Member &m = g.m[i];
        m.trellis = l->view.trellis, m.svh = l->view.svh, m.suh = l->view.suh, m.y = ys[i];
        m.xh = ws->xh.p + i * (size_t)rows * l->k * 2;
        r.suh[i] = m.suh, r.xh[i] = m.xh;
        m.z = ws->z.p + z_at * 4, m.counters = ws->counters.p + cnt_at * 4;
        m.n = l->n, m.sk = l->plan.sk;
        view_strides(l->view, &m.stride_k, &m.stride_nb);
        m.chunk = gemv_chunk(rows, l->k / 64 / m.sk);
        lds = std::max(lds, std::max(rows * (m.chunk * 128 + 16), rows * kRedPitch * 4));
        g.first[i] = programs;
        programs += l->n / 128 * m.sk;
        z_at += (size_t)m.sk * rows * l->n, cnt_at += l->n / 128;
    }
    for (size_t i = count; i <= kGroupMax; i++) g.first[i] = programs;
    uint32_t x_mode = (uint32_t)x_dtype & 1, k = ls[0]->k, mode = (uint32_t)y_dtype;
    if (!fused) {  // one launch rotates the input for every member, and the GEMV reads the members' rotated inputs
        void *rargs[] = {&r, &x, &x_mode, &k};
        FE_TRY(fe_hip_launch(kern->rot_in_group, (k + 511) / 512, rows, (uint32_t)count, 128, 1, 1, 0, s, rargs));
        x = 0;
    }
    void *args[] = {&g, &x, &x_mode, &k, &rows, &mode};
    return fe_hip_launch(kern->gemv_group[bits_slot(ls[0]->bits)][(rows + 15) / 16 - 1], programs, 1, 1, 256, 1, 1, lds, s, args);
}

int fe_exl3_reconstruct_hat_f16(const fe_exl3_kernels *kern, fe_stream_t s, const fe_exl3_view *w, fe_devptr_t out) {
    if (!kern || !w || !out) return fe_set_error(FE_ERR_ARG, "fe_exl3_reconstruct_hat_f16", "null argument");
    if (w->strips || w->k % 16 || w->n % 128 || w->bits < 1 || w->bits > 8)
        return fe_set_error(FE_ERR_SHAPE, "fe_exl3_reconstruct_hat_f16", "needs the stored layout, n % 128 == 0, 1..8 bits");
    uint32_t n_tiles = w->n / 16, nt0 = 0, ns = w->n, bits = w->bits;
    fe_devptr_t tr = w->trellis;
    void *args[] = {&out, &tr, &n_tiles, &nt0, &ns, &bits};
    return fe_hip_launch(kern->recon_hat_f16, w->n / 128, w->k / 16, 1, 256, 1, 1, 0, s, args);
}

int fe_exl3_reconstruct_bf16(const fe_exl3_kernels *kern, fe_stream_t s, const fe_exl3_view *w, fe_devptr_t out, int layout,
                             fe_devptr_t scratch, size_t scratch_bytes) {
    if (!kern || !w || !out || !scratch) return fe_set_error(FE_ERR_ARG, "fe_exl3_reconstruct_bf16", "null argument");
    const size_t k = w->k, n = w->n;
    if (k % 128 || n % 128 || w->strips || w->bits < 1 || w->bits > 8)
        return fe_set_error(FE_ERR_SHAPE, "fe_exl3_reconstruct_bf16", "not 128-aligned, or strips layout");
    const size_t max_ns = (scratch_bytes / (k * 4)) / 128 * 128;
    if (max_ns == 0) return fe_set_error(FE_ERR_WORKSPACE, "fe_exl3_reconstruct_bf16", "scratch smaller than k * 128 * 4 bytes");
    uint32_t ld = layout ? (uint32_t)k : (uint32_t)n, nk = layout ? 1u : 0u;
    for (size_t n0 = 0; n0 < n;) {
        uint32_t ns = (uint32_t)std::min(max_ns, n - n0), n032 = (uint32_t)n0, nt0 = n032 / 16, n_tiles = (uint32_t)n / 16;
        uint32_t bits = w->bits;
        fe_devptr_t tr = w->trellis, svh = w->svh, suh = w->suh;
        {
            void *args[] = {&scratch, &tr, &n_tiles, &nt0, &ns, &bits};
            FE_TRY(fe_hip_launch(kern->recon_hat_f32, ns / 128, (uint32_t)k / 16, 1, 256, 1, 1, 0, s, args));
        }
        {
            void *args[] = {&scratch, &ns, &svh, &n032};
            FE_TRY(fe_hip_launch(kern->had_rows, (ns / 128 + 1) / 2, (uint32_t)k, 1, 64, 1, 1, 0, s, args));
        }
        {
            void *args[] = {&scratch, &out, &ns, &suh, &n032, &ld, &nk};
            FE_TRY(fe_hip_launch(kern->had_cols_bf16, ns / 32, (uint32_t)k / 128, 1, 128, 1, 1, 0, s, args));
        }
        n0 += ns;
    }
    return 0;
}

static int time_launches(fe_stream_t s, uint32_t launches, float *ms, int (*launch)(void *), void *ctx) {
    fe_event_t a = nullptr, b = nullptr;
    FE_TRY(fe_hip_event_create(&a));
    int c = fe_hip_event_create(&b);
    if (!c) c = launch(ctx);  // warm-up
    if (!c) c = fe_hip_event_record(a, s);
    for (uint32_t i = 0; !c && i < launches; i++) c = launch(ctx);
    if (!c) c = fe_hip_event_record(b, s);
    if (!c) c = fe_hip_event_sync(b);
    float t = 0;
    if (!c) c = fe_hip_event_elapsed_ms(&t, a, b);
    fe_hip_event_destroy(a);
    fe_hip_event_destroy(b);
    if (!c && ms) *ms = t / (float)launches;
    return c;
}

int fe_exl3_probe_stream_read(const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t buf, size_t bytes, uint32_t grid,
                              uint32_t launches, float *ms) {
    if (!kern || !buf || !grid || !launches || bytes < 16) return fe_set_error(FE_ERR_ARG, "fe_exl3_probe_stream_read", "bad argument");
    struct Ctx {
        const fe_exl3_kernels *k;
        fe_stream_t s;
        fe_devptr_t buf, out;
        uint64_t vecs;
        uint32_t grid;
    } ctx{kern, s, buf, 0, bytes / 16, grid};
    FeBuf out;
    FE_TRY(out.zeroed(64));
    ctx.out = out.p;
    return time_launches(s, launches, ms,
                         [](void *p) {
                             Ctx *c = (Ctx *)p;
                             void *args[] = {&c->buf, &c->out, &c->vecs};
                             return fe_hip_launch(c->k->probe_v4, c->grid, 1, 1, 256, 1, 1, 0, c->s, args);
                         },
                         &ctx);
}

int fe_exl3_probe_decode(const fe_exl3_kernels *kern, fe_stream_t s, uint32_t bits, uint32_t grid, uint32_t iters,
                         uint32_t launches, float *ms) {
    if (!kern || bits < 3 || bits > 5 || !grid || !launches) return fe_set_error(FE_ERR_ARG, "fe_exl3_probe_decode", "bits 3..5");
    struct Ctx {
        const fe_exl3_kernels *k;
        fe_stream_t s;
        fe_devptr_t out;
        uint32_t bits, grid, iters, seed;
    } ctx{kern, s, 0, bits, grid, iters, 12345u};
    FeBuf out;
    FE_TRY(out.zeroed((size_t)grid * 256 * 4));
    ctx.out = out.p;
    return time_launches(s, launches, ms,
                         [](void *p) {
                             Ctx *c = (Ctx *)p;
                             void *args[] = {&c->out, &c->iters, &c->seed};
                             return fe_hip_launch(c->k->probe_decode[c->bits - 3], c->grid, 1, 1, 256, 1, 1, 0, c->s, args);
                         },
                         &ctx);
}

}  // extern "C"
