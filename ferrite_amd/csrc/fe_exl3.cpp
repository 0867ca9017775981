// fe_exl3: host side of the EXL3 linear (see include/fe_exl3.h). Launch geometry, workspaces and argument checks
// follow crates/fe-exl3/src/linear.rs and crates/fe-exl3/src/gpu/mod.rs; the kernels are ferrite_amd/csrc/kernels/k_exl3.hip.
#include "fe_exl3.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "fe_exl3_plans.h"
#include "fe_internal.h"

namespace {

constexpr uint32_t kMaxRowsPerPass = 64;       // 4 row groups of 16
constexpr uint32_t kHatRows = 3072;            // rows from which the prefill decodes once into fp16 tiles (12 output tile rows)
constexpr uint32_t kGroupMax = 4;              // FE_EXL3_GROUP_MAX: linears of one launch
// LDS of one GEMV program (sums of a segment + staged inputs of a chunk of the run): three programs fit a CU's 160 KB. Up
// to 16 rows a whole run fits in far less; from 17 rows on a larger budget (76 KB: longer chunks, two programs a CU) was
// measured slower: 37.8 against 30.9 us a linear at 32 rows on 5120 x 17408; at 64 rows 52.7 against 45.2 once the sums'
// buffer holds 32 rows at a time
constexpr uint32_t kJobLdsBudget = 53 * 1024;
constexpr uint32_t kRedPitch = 132;            // GEMV_RED_PITCH
constexpr uint32_t kGemmLds = 2 * (256 + 256) * 64 * 2;  // two k tiles of A and W, 256 rows each; the epilogue reuses it
constexpr uint32_t kCuLds = 160 * 1024;        // LDS of a CU
constexpr size_t kChainStride = 64;            // FE_CHAIN_STRIDE: u32 words between two ready words of the one-launch MLP

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

// Switches of the launch paths. Read from the environment once, when the kernels are loaded; fe_exl3_kernels_set_option
// changes them afterwards (tests compare both forms of a path in one process). No forward call reads the environment.
struct fe_exl3_options {
    uint32_t fused_rot = 1;        // the GEMV rotates its own input where that pays (FE_EXL3_NO_FUSED_ROT=1: never)
    uint32_t fused_rot_pairs = 16; // ... up to this many (row, 128-channel block) pairs a program (FE_EXL3_FUSED_ROT_PAIRS)
    uint32_t group = 1;            // linears of one input share a launch (FE_EXL3_NO_GROUP=1: one launch each)
    uint32_t hat_rows = kHatRows;  // rows from which the prefill decodes once (FE_EXL3_HAT_ROWS; 0: never)
    uint32_t lds_pad = 1;          // LDS request that pins the programs per CU to the plan's occ (FE_EXL3_NO_LDS_PAD=1: off)
    uint32_t fuse = 1;             // consecutive programs share a workgroup when a launch has more than the CUs hold (FE_EXL3_NO_FUSE=1: off)
    uint32_t gemm_group_m = 8;     // raster group of the prefill GEMM (FE_EXL3_GROUP)
    uint32_t gemm_splits = 8;      // most pieces a cut output tile of the prefill GEMM takes (FE_GEMM_SPLITS; 1: never cut)
    uint32_t gemm_sk = 1;          // stream-K schedule of the prefill GEMM: 0 never, 1 where measured faster, 2 always (FE_GEMM_SK)
    // fe_exl3_mlp_forward runs down in programs of this many units where that divides a column block: 0 (the default) the
    // linear's own partition; 2, 4, 8 shorter programs, which end the one launch sooner at one row and cost the two-launch
    // form of the call time from 8 rows on (FE_EXL3_CHAIN_DOWN_UNITS)
    uint32_t chain_down_units = 0;
    uint32_t handoff_fenced = 0;   // 1..16 rows through the kernels whose hand-off uses release / acquire fences (a slow cross-check)
    uint32_t mlp_chain = 1;        // the decode MLP (gate, up, down) as one launch where it applies (FE_EXL3_NO_CHAIN=1: off)
    uint32_t chain_rot_pairs = 32; // (row, 128-channel block) pairs a program rotates at most inside the one-launch MLP (FE_EXL3_CHAIN_ROT_PAIRS)
    uint32_t chain_perm = 1;       // the down stage's workgroups in the order in which their inputs get ready (FE_EXL3_CHAIN_PERM)
    uint32_t chain_spin = 1u << 16;  // polls a program of the down stage waits for the front stage's outputs (FE_EXL3_CHAIN_SPIN)
};

struct fe_exl3_kernels {
    fe_module_t module = nullptr;
    fe_function_t recon_hat_f32 = nullptr, recon_hat_f16 = nullptr, had_rows = nullptr, had_cols_bf16 = nullptr;
    fe_function_t rot_in = nullptr, rot_in_group = nullptr, probe_v4 = nullptr;
    fe_function_t probe_decode[3] = {nullptr, nullptr, nullptr};  // 3, 4, 5 bits
    fe_function_t gemvb[6][4] = {};                               // the decode GEMV, [bits slot][row groups - 1]
    fe_function_t gemvb_fenced[6] = {};                           // the same for 1..16 rows with the fenced hand-off
    fe_function_t mlp[6] = {};                                    // the decode MLP in one launch, [bits slot]
    uint32_t cus = 0;
    fe_function_t gemm[6] = {}, gemm_sk[6] = {};  // decode inside the GEMM: one piece a program / stream-K
    fe_function_t gemm_reduce = nullptr;
    fe_function_t hat_tiles[6] = {};  // trellis -> fp16 weights as the GEMM's LDS images
    fe_function_t gemm_hat = nullptr, gemm_hat_sk = nullptr;  // the GEMM over them
    fe_exl3_options opt;
};

struct fe_exl3_linear {
    std::string name;
    uint32_t k = 0, n = 0, bits = 0;
    fe_exl3_plan plan{};
    uint32_t programs = 0;  // grid of the decode GEMV under this plan
    fe_exl3_view view{};
    FeBuf trellis, suh, svh;  // owned copies (upload), empty for from_view
    FeBuf hat;                // decoded fp16 tiles kept with the linear (fe_exl3_linear_keep_decoded), else empty
    // The linear as the down projection of a one-launch MLP: its partition there (the linear's own, and partitions into
    // programs of 2, 4 and 8 units where that divides a column block) with u32[programs], the programs sorted by the last
    // channel block their run reads.
    struct ChainPart {
        uint32_t unit_len = 0, programs = 0;  // unit_len 0: the linear's own partition
        FeBuf order;
        // the same weights (no copies: the view) as a linear of this partition, for the launches of the MLP call that are
        // not the one launch: every row count then sums down's segments in the same order
        std::unique_ptr<fe_exl3_linear> as_linear;
    };
    std::vector<std::unique_ptr<ChainPart>> chain_parts;
    const fe_exl3_kernels *kern = nullptr;
};

struct fe_exl3_workspace {
    uint32_t max_rows = 0, max_k = 0;
    FeBuf xh, z, counters, part;  // part: partial tiles of the prefill GEMM (rows > 64 only)
    FeBuf hat;                    // decoded fp16 weights of one linear (workspaces of hat_rows rows or more)
    FeBuf chain;                  // state of the one-launch MLP: sequence, error, finished blocks, ready words (u32)
    size_t z_len = 0, counters_len = 0, chain_len = 0;
    bool chain_off = false;  // a bounded wait of the one-launch MLP ran out on this workspace: its calls are two launches from then on
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

static uint32_t env_u32(const char *name, uint32_t fallback) {
    const char *e = getenv(name);
    return e && *e ? (uint32_t)strtoul(e, nullptr, 0) : fallback;
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
            snprintf(nm, sizeof nm, "exl3_gemvb_b%d_r%d", kBits[i], rg);
            get(&k->gemvb[i][rg - 1], nm);
            if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemvb[i][rg - 1], 84 * 1024);
        }
        snprintf(nm, sizeof nm, "exl3_gemvb_b%d_r1_fenced", kBits[i]);
        get(&k->gemvb_fenced[i], nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemvb_fenced[i], 84 * 1024);
        snprintf(nm, sizeof nm, "exl3_mlp_b%d", kBits[i]);
        get(&k->mlp[i], nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->mlp[i], 84 * 1024);
        snprintf(nm, sizeof nm, "exl3_gemm_b%d", kBits[i]);
        get(&k->gemm[i], nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm[i], kGemmLds);
        snprintf(nm, sizeof nm, "exl3_gemm_b%d_sk", kBits[i]);
        get(&k->gemm_sk[i], nm);
        if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm_sk[i], kGemmLds);
        snprintf(nm, sizeof nm, "exl3_hat_tiles_b%d", kBits[i]);
        get(&k->hat_tiles[i], nm);
        if (i == 0) get(&k->gemm_reduce, "exl3_gemm_reduce");
    }
    get(&k->gemm_hat, "exl3_gemm_hat");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm_hat, kGemmLds);
    get(&k->gemm_hat_sk, "exl3_gemm_hat_sk");
    if (!c) c = fe_hip_func_set_max_dyn_lds(k->gemm_hat_sk, kGemmLds);
    fe_exl3_options &o = k->opt;
    o.fused_rot = env_u32("FE_EXL3_NO_FUSED_ROT", 0) ? 0 : 1;
    o.fused_rot_pairs = env_u32("FE_EXL3_FUSED_ROT_PAIRS", o.fused_rot_pairs);
    o.group = env_u32("FE_EXL3_NO_GROUP", 0) ? 0 : 1;
    if (getenv("FE_EXL3_HAT_ROWS")) fe_exl3_kernels_set_option(k, "hat_rows", (uint32_t)std::max(0, atoi(getenv("FE_EXL3_HAT_ROWS"))));
    o.lds_pad = env_u32("FE_EXL3_NO_LDS_PAD", 0) ? 0 : 1;
    o.fuse = env_u32("FE_EXL3_NO_FUSE", 0) ? 0 : 1;
    o.gemm_group_m = env_u32("FE_EXL3_GROUP", o.gemm_group_m);
    o.gemm_splits = env_u32("FE_GEMM_SPLITS", o.gemm_splits);
    o.gemm_sk = env_u32("FE_GEMM_SK", o.gemm_sk);
    o.mlp_chain = env_u32("FE_EXL3_NO_CHAIN", 0) ? 0 : 1;
    o.chain_spin = env_u32("FE_EXL3_CHAIN_SPIN", o.chain_spin);
    o.chain_perm = env_u32("FE_EXL3_CHAIN_PERM", o.chain_perm);
    o.chain_rot_pairs = env_u32("FE_EXL3_CHAIN_ROT_PAIRS", o.chain_rot_pairs);
    o.chain_down_units = env_u32("FE_EXL3_CHAIN_DOWN_UNITS", o.chain_down_units);
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

int fe_exl3_kernels_set_option(fe_exl3_kernels *k, const char *name, uint32_t value) {
    if (!k || !name) return fe_set_error(FE_ERR_ARG, "fe_exl3_kernels_set_option", "null argument");
    fe_exl3_options &o = k->opt;
    const std::string nm = name;
    if (nm == "chain_down_units") o.chain_down_units = value;
    else if (nm == "fused_rot") o.fused_rot = value;
    else if (nm == "fused_rot_pairs") o.fused_rot_pairs = value;
    else if (nm == "group") o.group = value;
    else if (nm == "hat_rows") o.hat_rows = value == 0 ? 0xffffffffu : std::max(value, kMaxRowsPerPass + 1);
    else if (nm == "lds_pad") o.lds_pad = value;
    else if (nm == "fuse") o.fuse = value;
    else if (nm == "gemm_group_m") o.gemm_group_m = value;
    else if (nm == "gemm_splits") o.gemm_splits = value;
    else if (nm == "gemm_sk") o.gemm_sk = value;
    else if (nm == "mlp_chain") o.mlp_chain = value;
    else if (nm == "handoff_fenced") o.handoff_fenced = value;
    else if (nm == "chain_spin") o.chain_spin = value;
    else if (nm == "chain_perm") o.chain_perm = value;
    else if (nm == "chain_rot_pairs") o.chain_rot_pairs = value;
    else return fe_set_error(FE_ERR_ARG, "fe_exl3_kernels_set_option", name);
    return 0;
}

// Launch plan for one shape. The decode GEMV deals 128-channel x 128-column units to `programs` programs in equal runs;
// what is chosen is how many programs: occ per CU (ver 3), each at least wk units long. The tuned table holds the measured
// choice for the shapes it knows on this CU count (FE_EXL3_UNTUNED=1 skips it: plans::tuned and its override,
// crates/fe-exl3/src/plans.rs:123-131, linear.rs:217-233); other shapes take the rule: the program target `blocks`
// (default 4 per CU, linear.rs:131-134) rounded to whole programs per CU, runs of at least 4 units, because programs of
// fewer than 8 load steps cost more in start-up and hand-off than their spread over the CUs gains. sk records the K splits
// per column block that this amounts to. FE_EXL3_NOSPLIT=1 / FE_EXL3_SPLIT=0: one program per column block (ver 1, sk 1).
int fe_exl3_plan_for(uint32_t k, uint32_t n, uint32_t bits, uint32_t blocks, fe_exl3_plan *out) {
    if (!out || !k || !n || k % 128 || n % 128) return fe_set_error(FE_ERR_SHAPE, "fe_exl3_plan_for", "k, n must be multiples of 128");
    if (env_is("FE_EXL3_NOSPLIT", "1") || env_is("FE_EXL3_SPLIT", "0")) {
        *out = fe_exl3_plan{1, 4, 1, 0};
        return 0;
    }
    int cus = 0;
    if (fe_hip_cu_count(&cus) || cus <= 0) cus = 256;  // planning without a device: the MI355X count
    uint32_t occ = blocks ? std::min(5u, std::max(1u, (blocks + (uint32_t)cus / 2) / (uint32_t)cus)) : 4, wk = 4;
    if (!env_is("FE_EXL3_UNTUNED", "1")) {
        for (const FeTunedPlan &t : kFeTunedPlans)
            if (t.k == k && t.n == n && t.bits == bits && t.cus == (uint32_t)cus) occ = t.occ, wk = t.min_units;
    }
    occ = env_u32("FE_EXL3_OCC", occ), wk = std::max(1u, env_u32("FE_EXL3_MIN_UNITS", wk));  // tuning runs
    const uint32_t units = (k / 128) * (n / 128), nb = n / 128;
    const uint32_t programs = std::max(1u, std::min(occ * (uint32_t)cus, units / wk));
    *out = fe_exl3_plan{(programs + nb - 1) / nb, wk, 3, occ};
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

}  // extern "C"

// Programs of the decode GEMV under a plan. ver 1 (the reference's meaning of a plan): sk programs per column block.
// ver 2 and 3: occ programs per CU, each a run of at least wk units. ver 4: sk programs in all (tests and tuners: any
// partition). Never more programs than units.
static uint32_t plan_programs(const fe_exl3_kernels *kern, const fe_exl3_plan &p, uint32_t k, uint32_t n) {
    const uint32_t units = (k / 128) * (n / 128);
    uint32_t progs;
    if (p.ver <= 1)
        progs = n / 128 * std::max(p.sk, 1u);
    else if (p.ver == 4)
        progs = std::max(p.sk, 1u);
    else
        progs = (p.occ ? p.occ : 4) * std::max(kern->cus, 1u), progs = std::min(progs, units / std::max(p.wk, 1u));
    return std::max(1u, std::min(progs, units));
}

// The programs of a partition of the linear in the order in which, as the down projection of a one-launch MLP, their
// inputs get ready: sorted by the last 128-channel block their run reads (a run that crosses into the next column block
// reads the last block of all), then by program number. A program of the down stage waits for lower-numbered programs'
// inputs only through this order, which keeps every program behind the ones that started earlier in K.
static int make_chain_part(fe_exl3_linear *l, uint32_t unit_len, uint32_t programs) {
    const uint32_t upb = l->k / 128, units = upb * (l->n / 128), base = units / programs, rem = units % programs;
    std::vector<uint32_t> order(programs), last(programs);
    for (uint32_t p = 0; p < programs; p++) {
        const uint32_t u0 = p * base + std::min(p, rem), len = base + (p < rem ? 1 : 0), kb0 = u0 % upb;
        order[p] = p;
        last[p] = kb0 + len > upb ? upb - 1 : kb0 + len - 1;
    }
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) { return last[a] < last[b]; });
    auto part = std::make_unique<fe_exl3_linear::ChainPart>();
    part->unit_len = unit_len, part->programs = programs;
    if (int c = part->order.from_host(order.data(), order.size() * 4)) return c;
    if (unit_len) {
        part->as_linear = std::make_unique<fe_exl3_linear>();
        fe_exl3_linear &sh = *part->as_linear;
        sh.name = l->name, sh.k = l->k, sh.n = l->n, sh.bits = l->bits, sh.plan = l->plan, sh.programs = programs;
        sh.view = l->view, sh.kern = l->kern;
    }
    l->chain_parts.push_back(std::move(part));
    return 0;
}

static int make_chain_order(fe_exl3_linear *l) {
    if (int c = make_chain_part(l, 0, l->programs)) return c;
    const uint32_t upb = l->k / 128, units = upb * (l->n / 128);
    for (uint32_t len : {2u, 4u, 8u})
        if (upb % len == 0 && units / len <= 8192 && units / len != l->programs)
            if (int c = make_chain_part(l, len, units / len)) return c;
    return 0;
}

// The partition the linear takes as the down stage of a one-launch MLP under the kernels' current options.
static const fe_exl3_linear::ChainPart *chain_part(const fe_exl3_linear *l) {
    const uint32_t want = l->kern->opt.chain_down_units;
    for (const auto &part : l->chain_parts)
        if (want && part->unit_len == want) return part.get();
    return l->chain_parts[0].get();
}

static int check_fit(const char *name, uint32_t k, uint32_t n, uint32_t bits, const fe_exl3_plan &p) {
    char msg[160];
    if (bits_slot(bits) < 0) {
        snprintf(msg, sizeof msg, "%s: %u bits (kernels exist for 2, 3, 4, 5, 6, 8)", name, bits);
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_linear", msg);
    }
    // linear.rs:244: k, n multiples of 128 and the K range divides into the plan's pieces (here: load steps of 64)
    if (!k || !n || k % 128 || n % 128 || p.sk == 0 || (p.ver <= 1 && (k / 64) % p.sk)) {
        snprintf(msg, sizeof msg, "%s: %ux%u does not fit plan sk %u", name, k, n, p.sk);
        return fe_set_error(FE_ERR_SHAPE, "fe_exl3_linear", msg);
    }
    return 0;
}

extern "C" {

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
    l->programs = plan_programs(kern, *plan, view->k, view->n);
    if (int c = make_chain_order(l)) {
        delete l;
        return c;
    }
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
    l->programs = plan_programs(kern, p, k, n);
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
    l->view = fe_exl3_view{k, n, bits, l->trellis.p, l->suh.p, l->svh.p, strips ? 1u : 0u};
    if (!c) c = make_chain_order(l);
    if (c) {
        delete l;
        return c;
    }
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

}  // extern "C"

// Many rows: decoding the trellis once into fp16 tiles and running the GEMM over them beats decoding inside the GEMM,
// where each 256-row tile of the output decodes its weights again. From opt.hat_rows rows on and only with a workspace
// created for that many rows, which then holds the largest linear's decoded weights (2 bytes a weight).
static size_t hat_bytes(const fe_exl3_linear *l) { return (size_t)((l->n / 128 + 1) / 2) * 256 * l->k * 2; }

// Room one linear's GEMV takes in a workspace at `rows` rows: a slot of 128 sums per (program, column block it touches).
static size_t job_z(const fe_exl3_linear *l, uint32_t rows) { return (size_t)(l->programs + l->n / 128) * 128 * rows; }
// ... as the down stage of a one-launch MLP
static size_t chain_z(const fe_exl3_linear *l, uint32_t rows) { return (size_t)(chain_part(l)->programs + l->n / 128) * 128 * rows; }

extern "C" {

int fe_exl3_workspace_create(fe_exl3_workspace **out, fe_exl3_linear *const *linears, size_t count, uint32_t max_rows) {
    if (!out || (count && !linears) || !max_rows) return fe_set_error(FE_ERR_ARG, "fe_exl3_workspace_create", "bad argument");
    size_t max_k = 128, max_hat = 0;
    uint32_t hat_rows = kHatRows;
    std::vector<size_t> zs, nbs;  // per linear; a launch of several linears needs room for the kGroupMax largest together
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = linears[i];
        zs.push_back(std::max(job_z(l, 1), chain_z(l, 1)));
        nbs.push_back(l->n / 128);
        max_hat = std::max(max_hat, hat_bytes(l));
        max_k = std::max<size_t>(max_k, l->k);
        hat_rows = l->kern->opt.hat_rows;
    }
    auto *ws = new fe_exl3_workspace;
    ws->max_rows = max_rows, ws->max_k = (uint32_t)max_k;
    auto top = [](std::vector<size_t> &v) {
        std::sort(v.begin(), v.end(), std::greater<size_t>());
        size_t t = 0;
        for (size_t i = 0; i < v.size() && i < kGroupMax; i++) t += v[i];
        return t;
    };
    const uint32_t gemv_rows = std::min(max_rows, kMaxRowsPerPass);
    ws->z_len = std::max<size_t>(top(zs) * gemv_rows, 4);
    int cus = 0, c = 0;
    if (max_rows > kMaxRowsPerPass) c = fe_hip_cu_count(&cus);
    // arrival counters: a word a column block of the linears of one launch (GEMV); a word an output tile (stream-K GEMM)
    ws->counters_len = std::max<size_t>({top(nbs), (size_t)32 * cus, 1});
    // (rotated inputs: one linear's at max_rows, or those of the linears of one launch at up to 64 rows each)
    if (!c) c = ws->xh.alloc((size_t)std::max(max_rows, kGroupMax * gemv_rows) * max_k * 2);
    if (!c) c = ws->z.alloc(ws->z_len * 4);
    if (!c) c = ws->counters.zeroed(ws->counters_len * 4);
    // one-launch MLP: 4 state words and a ready word per column block of two front members
    size_t max_nb = 1;
    for (size_t nb : nbs) max_nb = std::max(max_nb, nb);
    ws->chain_len = kChainStride * (1 + 2 * max_nb);
    if (!c) c = ws->chain.zeroed(ws->chain_len * 4);
    if (!c && cus > 0) c = ws->part.alloc((size_t)cus * kFeGemmSlotsPerCu * kFeGemmPartBytes);
    // zeroed once: the unused half of the last tile of an odd count of column blocks is read (and its sums discarded)
    if (!c && max_rows >= hat_rows && max_hat) c = ws->hat.zeroed(max_hat);
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

}  // extern "C"

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
    uint32_t n = l->n, k = l->k, mode = (uint32_t)y_dtype, stride_k, stride_nb, group = kern->opt.gemm_group_m;
    view_strides(l->view, &stride_k, &stride_nb);
    if ((uint64_t)rows * k * 2 >= (1ull << 32))
        return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_linear_gemv_rotated", "rotated input of 4 GB or more");
    const uint32_t tiles_m = (rows + 255) / 256, tiles_n = (n / 128 + 1) / 2;
    if (group == 0 || group > tiles_m) group = tiles_m;
    fe_devptr_t tr = l->view.trellis, svh = l->view.svh, part = ws->part.p;
    const bool kept = l->hat.bytes != 0;  // decoded once and kept: any row count above the GEMV's runs over it
    const bool over_hat = kept || (rows >= kern->opt.hat_rows && ws->hat.bytes >= hat_bytes(l));
    // (decoded tiles are a large weight operand: 32 KB a k tile against the trellis's 2 KB a bit)
    FeGemmSchedule sch = fe_gemm_schedule(tiles_m * tiles_n, k / 64, kern->cus, ws->part.p, ws->part.bytes, ws->counters.p,
                                          ws->counters_len, kern->opt.gemm_splits, kern->opt.gemm_sk, !over_hat);
    if (over_hat) {
        fe_devptr_t hat = kept ? l->hat.p : ws->hat.p;
        if (!kept) FE_TRY(launch_decode(l, s, hat));
        group = 0;  // the raster that deals column tiles to the XCDs: each decoded weight panel goes through one L2
        void *args[] = {&xh, &hat, &svh, &y, &n, &k, &rows, &mode, &group, &sch.args};
        FE_TRY(fe_hip_launch(sch.stream_k ? kern->gemm_hat_sk : kern->gemm_hat, sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args));
    } else {
        if (sch.stream_k) group = 1;  // column tiles fastest: the programs that are in step share a panel of inputs
        void *args[] = {&xh, &tr, &svh, &y, &n, &k, &rows, &mode, &stride_k, &stride_nb, &group, &sch.args};
        FE_TRY(fe_hip_launch((sch.stream_k ? kern->gemm_sk : kern->gemm)[bits_slot(l->bits)], sch.programs, 1, 1, 256, 1, 1, kGemmLds, s, args));
    }
    if (sch.stream_k || !sch.split.cut()) return 0;
    uint32_t full = sch.split.full, splits = sch.split.splits;
    void *rargs[] = {&part, &svh, &y, &n, &rows, &mode, &group, &full, &splits};
    return fe_hip_launch(kern->gemm_reduce, sch.split.cut() * 64, 1, 1, 256, 1, 1, 0, s, rargs);
}

// The GEMV can rotate its own input: every program rotates the channels of its own run, (row, 128-channel block) pairs,
// 8 at a time, so every column block repeats the rotation of its K range. Measured on 5120 x 17408: one launch wins up
// to a few rows, the separate rotation launch from about 8 rows on.
static uint32_t units_per_program(const fe_exl3_linear *l, uint32_t programs) {
    const uint32_t units = (l->k / 128) * (l->n / 128);
    return (units + programs - 1) / programs;
}

static bool fused_rotation_fits(const fe_exl3_linear *l, uint32_t rows) {
    const fe_exl3_options &o = l->kern->opt;
    if (!o.fused_rot || rows < 1 || rows > kMaxRowsPerPass) return false;
    const uint32_t units = (l->k / 128) * (l->n / 128);
    return rows * ((units + l->programs - 1) / l->programs) <= o.fused_rot_pairs;
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
struct RotGroupArgs {  // RotGroup
    fe_devptr_t suh[kGroupMax], xh[kGroupMax];
};

// The decode GEMV for 1..4 linears of one input in one launch, 1..64 rows: member i reads its rotated input at xhs[i]
// (in.x == 0) or rotates in.x itself and leaves the result at xhs[i]. The caller has checked rows, k and bits.
static int launch_job(const fe_exl3_linear *const *ls, size_t count, fe_stream_t s, const fe_devptr_t *xhs, const fe_devptr_t *ys,
                      int y_dtype, uint32_t rows, const fe_exl3_workspace *ws, const RotInput &in, const char *fn) {
    GemvJobArgs g{};
    g.count = (uint32_t)count;
    const fe_exl3_kernels *kern = ls[0]->kern;
    // Programs of the partition a workgroup runs one after the other (`fuse`): when the members' programs together are
    // more than the CUs hold at once, consecutive programs share a workgroup instead of waiting for a free place, which
    // saves the second one's start-up. The partition, and with it every sum, stays the member's own.
    uint32_t occ = 0, total = 0;
    for (size_t i = 0; i < count; i++) occ = std::max(occ, ls[i]->plan.occ), total += ls[i]->programs;
    const uint32_t places = std::max(1u, (occ ? occ : 4) * std::max(kern->cus, 1u));
    // (measured on gate + up, 4 bits: 34.1 against 35.6 us at 1 row, 36.8 / 38.2 at 4, even at 8, 44.8 / 41.9 at 16, where the
    // longer run's inputs no longer fit the staging buffer in one piece: up to 4 rows; 4-unit programs of 17408 x 5120 sharing a
    // workgroup at 8 / 16 rows: 61.6 / 77.1 us a block against 65.2 / 75.8 without)
    uint32_t fuse = kern->opt.fuse && rows <= 4 ? std::min(4u, std::max(1u, (total + places - 1) / places)) : 1;
    uint32_t programs = 0, run_steps = 0;  // (programs: workgroups of the launch)
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
        programs += (l->programs + fuse - 1) / fuse;
        z_at += job_z(l, rows), cnt_at += l->n / 128;
        const uint32_t units = (l->k / 128) * (l->n / 128);
        m.base = units / l->programs, m.rem = units % l->programs;
        m.inv_base = 0xffffffffu / m.base, m.inv_base1 = 0xffffffffu / (m.base + 1);
        run_steps = std::max(run_steps, 2 * fuse * ((units + l->programs - 1) / l->programs));
    }
    for (size_t i = count; i <= kGroupMax; i++) g.first[i] = programs;
    // staged inputs: the whole run where the LDS budget holds it for `rows` rows, else chunks of a multiple of 4 load steps
    const uint32_t red = std::min(rows, 32u) * kRedPitch * 4;  // (more than 32 rows pass through it in two halves)
    uint32_t chunk = std::max(4u, ((std::max(kJobLdsBudget, red + rows * 528) - red) / rows - 16) / 128 / 4 * 4);
    chunk = std::min(chunk, (run_steps + 3) / 4 * 4);
    uint32_t lds = red + rows * (chunk * 128 + 16);
    // Exactly occ programs a CU: the dispatcher fills a CU as far as registers and LDS allow (5 programs) before it moves
    // on, which would leave CUs empty while others hold 5; an LDS request that fits occ times into the CU's 160 KB, and
    // not occ + 1 times, makes the CUs take occ each.
    // (several linears: the most programs per CU any of them asks for)
    if (occ && kern->opt.lds_pad) lds = std::max(lds, kCuLds / (occ + 1) + 512);
    uint32_t k = ls[0]->k, mode = (uint32_t)y_dtype, x_mode = in.mode, ldx = in.ld, inv_spb = 0xffffffffu / (k / 64);
    fe_devptr_t x = in.x, x2 = in.x2;
    void *args[] = {&g, &x, &x2, &x_mode, &ldx, &k, &rows, &mode, &chunk, &inv_spb, &fuse};
    const fe_function_t f = kern->opt.handoff_fenced && rows <= 16 ? kern->gemvb_fenced[bits_slot(ls[0]->bits)]
                                                                   : kern->gemvb[bits_slot(ls[0]->bits)][(rows + 15) / 16 - 1];
    return fe_hip_launch(f, programs, 1, 1, 256, 1, 1, lds, s, args);
}

// Decode-sized rows run the GEMV (with in.x != 0 it rotates that input itself and leaves the rotated rows in xh; callers
// check fused_rotation_fits first), more rows the GEMM.
static int launch_rows(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype, uint32_t rows,
                       const fe_exl3_workspace *ws, const RotInput &in) {
    const char *fn = "fe_exl3_linear_gemv_rotated";
    if (!l || !ws || !xh || !y) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (y_dtype < 0 || y_dtype > 3) return fe_set_error(FE_ERR_ARG, fn, "bad y dtype");
    if (rows == 0 || rows > ws->max_rows) {  // linear.rs:302-307
        char msg[200];
        snprintf(msg, sizeof msg, "%s: rows %u do not fit the workspace (max %u)", l->name.c_str(), rows, ws->max_rows);
        return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
    }
    if (rows > kMaxRowsPerPass) return launch_gemm(l, s, xh, y, y_dtype, rows, ws);
    return launch_job(&l, 1, s, &xh, &y, y_dtype, rows, ws, in, fn);
}

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
    return launch_rows(l, s, ws->xh.p, y, y_dtype, rows, ws, RotInput{});
}

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
    const size_t need_xh = (size_t)rows * l->k * 2, need_cnt = (size_t)(l->n / 128) * 4, need_z = job_z(l, rows) * 4;
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

int fe_exl3_linear_rotate_input(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                int x_dtype, uint32_t rows, const fe_exl3_workspace *ws) {
    if (!l || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_rotate_input", "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32)
        return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_rotate_input", "x is bf16 or f32");
    RotInput in;
    in.x = x, in.mode = (uint32_t)x_dtype & 1, in.ld = l->k;
    return launch_rot(l, kern, s, in, rows, ws, "fe_exl3_linear_rotate_input");
}

int fe_exl3_linear_gemv_rotated(const fe_exl3_linear *l, fe_stream_t s, fe_devptr_t xh, fe_devptr_t y, int y_dtype,
                                uint32_t rows, const fe_exl3_workspace *ws) {
    return launch_rows(l, s, xh, y, y_dtype, rows, ws, RotInput{});
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

int fe_exl3_linear_decoded(const fe_exl3_linear *l, fe_devptr_t *tiles, size_t *bytes) {
    if (!l) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_decoded", "null linear");
    if (tiles) *tiles = l->hat.p;
    if (bytes) *bytes = l->hat.bytes;
    return 0;
}

int fe_exl3_linear_forward_is_one_launch(const fe_exl3_linear *l, uint32_t rows) { return l && fused_rotation_fits(l, rows); }

int fe_exl3_linear_forward(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype,
                           fe_devptr_t y, int y_dtype, uint32_t rows, const fe_exl3_workspace *ws) {
    if (!l || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward", "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32)
        return fe_set_error(FE_ERR_ARG, "fe_exl3_linear_forward", "x is bf16 or f32");
    RotInput in;
    in.x = x, in.mode = (uint32_t)x_dtype & 1, in.ld = l->k;
    return forward_from(l, kern, s, in, y, y_dtype, rows, ws, "fe_exl3_linear_forward");
}

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

}  // extern "C"

// One launch for several linears: the same input, width and kernel, and room in the workspace for every member's partial
// sums (and rotated inputs) side by side. *fused: the GEMV rotates its own input.
static bool group_fits(const fe_exl3_linear *const *ls, size_t count, uint32_t rows, const fe_exl3_workspace *ws, bool *fused) {
    if (!ls || !ws || count < 2 || count > kGroupMax || rows < 1 || rows > kMaxRowsPerPass || rows > ws->max_rows) return false;
    if (!ls[0] || !ls[0]->kern->opt.group) return false;
    size_t z = 0, nb = 0;
    bool f = true;
    for (size_t i = 0; i < count; i++) {
        const fe_exl3_linear *l = ls[i];
        if (!l || l->k != ls[0]->k || l->bits != ls[0]->bits || l->kern != ls[0]->kern) return false;
        f = f && fused_rotation_fits(l, rows);
        z += job_z(l, rows);
        nb += l->n / 128;
    }
    if (count * (size_t)rows * ls[0]->k * 2 > ws->xh.bytes) return false;
    if (fused) *fused = f;
    return z <= ws->z_len && nb <= ws->counters_len && ls[0]->k <= ws->max_k;
}

extern "C" {

int fe_exl3_linear_forward_group_launches(const fe_exl3_linear *const *ls, size_t count, uint32_t rows,
                                          const fe_exl3_workspace *ws) {
    bool fused = false;
    if (!group_fits(ls, count, rows, ws, &fused)) return 0;
    return fused ? 1 : 2;
}

int fe_exl3_linear_forward_group(const fe_exl3_linear *const *ls, size_t count, const fe_exl3_kernels *kern, fe_stream_t s,
                                 fe_devptr_t x, int x_dtype, const fe_devptr_t *ys, int y_dtype, uint32_t rows,
                                 const fe_exl3_workspace *ws) {
    const char *fn = "fe_exl3_linear_forward_group";
    if (!ls || !ys || !kern || !ws || !x) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    bool fused = false;
    if (!group_fits(ls, count, rows, ws, &fused)) {  // member by member: the same bits, more launches
        for (size_t i = 0; i < count; i++) FE_TRY(fe_exl3_linear_forward(ls[i], kern, s, x, x_dtype, ys[i], y_dtype, rows, ws));
        return 0;
    }
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32) return fe_set_error(FE_ERR_ARG, fn, "x is bf16 or f32");
    if (y_dtype < 0 || y_dtype > 3) return fe_set_error(FE_ERR_ARG, fn, "bad y dtype");
    RotGroupArgs r{};
    fe_devptr_t xhs[kGroupMax] = {};
    for (size_t i = 0; i < count; i++) {
        if (!ys[i]) return fe_set_error(FE_ERR_ARG, fn, "null output");
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
    return launch_job(ls, count, s, xhs, ys, y_dtype, rows, ws, in, fn);
}

}  // extern "C"

// mirrors MlpChain of k_exl3.hip
struct MlpChainArgs {
    GemvJobArgs front;
    GemvJobArgs::Member down;
    fe_devptr_t state, perm;
    uint32_t front_wgs, interleave;
    uint32_t k1, chunk1, inv_spb1, fuse1;
    uint32_t k2, chunk2, inv_spb2, fuse2;
    uint32_t spin_limit, pad;
};
static_assert(sizeof(MlpChainArgs) == 24 + kGroupMax * 88 + 88 + 16 + 12 * 4, "MlpChain layout");

static void fill_member(GemvJobArgs::Member &m, const fe_exl3_linear *l, uint32_t programs, fe_devptr_t xh, fe_devptr_t y,
                        fe_devptr_t z, fe_devptr_t counters) {
    m.trellis = l->view.trellis, m.svh = l->view.svh, m.suh = l->view.suh, m.xh = xh, m.y = y, m.z = z, m.counters = counters;
    m.n = l->n, m.programs = programs;
    view_strides(l->view, &m.stride_k, &m.stride_nb);
    const uint32_t units = (l->k / 128) * (l->n / 128);
    m.base = units / programs, m.rem = units % programs;
    m.inv_base = 0xffffffffu / m.base, m.inv_base1 = 0xffffffffu / (m.base + 1);
}



// Whether the decode MLP gate, up -> SwiGLU -> down runs as one launch: trellis linears of one width, gate and up of one
// shape whose outputs are down's input, every stage rotating its own input at this row count, a run of the down stage
// within the 32 units a wavefront watches, and a workspace with room for the three side by side.
static bool mlp_chain_fits(const fe_exl3_linear *g, const fe_exl3_linear *u, const fe_exl3_linear *d, uint32_t rows,
                           const fe_exl3_workspace *ws, int y_dtype) {
    if (!g || !u || !d || !ws || ws->chain_off || !g->kern->opt.mlp_chain || g->kern->opt.handoff_fenced) return false;
    if (g->kern != u->kern || g->kern != d->kern || g->bits != u->bits || g->bits != d->bits) return false;
    if (g->k != u->k || g->n != u->n || d->k != g->n) return false;
    if (rows < 1 || rows > 16 || rows > ws->max_rows || y_dtype < 0 || y_dtype > 3) return false;
    // every stage rotates its own input inside the launch: (row, 128-channel block) pairs a program. As separate launches
    // that pays up to 16 pairs (fused_rotation_fits); inside the one launch up to 32, i.e. up to 4 rows on the 27B-shaped
    // MLP (measured at 4 bits, cold weights: 4 rows 53.6 us against 56.8 us for rotation and GEMV launches; 8 rows 65.1 / 60.1)
    const fe_exl3_options &o = g->kern->opt;
    const uint32_t d_units = units_per_program(d, chain_part(d)->programs);
    if (!o.fused_rot || rows * std::max({units_per_program(g, g->programs), units_per_program(u, u->programs), d_units}) > o.chain_rot_pairs)
        return false;
    if (d_units > 32) return false;
    if (std::max(g->k, d->k) > ws->max_k || (size_t)2 * rows * g->k * 2 > ws->xh.bytes) return false;
    if (job_z(g, rows) + job_z(u, rows) + chain_z(d, rows) > ws->z_len) return false;
    if ((size_t)(2 * (g->n / 128) + d->n / 128) > ws->counters_len || kChainStride * (1 + 2 * (size_t)(g->n / 128)) > ws->chain_len) return false;
    return true;
}

static int launch_mlp(const fe_exl3_linear *g, const fe_exl3_linear *u, const fe_exl3_linear *d, fe_stream_t s, fe_devptr_t x,
                      int x_dtype, fe_devptr_t yg, fe_devptr_t yu, fe_devptr_t y, int y_dtype, uint32_t rows,
                      const fe_exl3_workspace *ws) {
    const fe_exl3_kernels *kern = g->kern;
    MlpChainArgs a{};
    const fe_exl3_linear *front[2] = {g, u};
    const fe_devptr_t ys[2] = {yg, yu};
    const uint32_t occ = std::max({g->plan.occ, u->plan.occ, d->plan.occ});
    const uint32_t places = std::max(1u, (occ ? occ : 4) * std::max(kern->cus, 1u));
    // (as launch_job: consecutive programs of the front stage share a workgroup when they are more than the CUs hold)
    a.fuse1 = kern->opt.fuse && rows <= 4 ? std::min(4u, std::max(1u, (g->programs + u->programs + places - 1) / places)) : 1;
    a.fuse2 = 1;
    size_t z_at = 0, cnt_at = 0;
    uint32_t wgs = 0;
    a.front.count = 2;
    for (int i = 0; i < 2; i++) {
        const fe_exl3_linear *l = front[i];
        fill_member(a.front.m[i], l, l->programs, ws->xh.p + (size_t)i * rows * l->k * 2, ys[i], ws->z.p + z_at * 4,
                    ws->counters.p + cnt_at * 4);
        a.front.first[i] = wgs;
        wgs += (l->programs + a.fuse1 - 1) / a.fuse1;
        z_at += job_z(l, rows), cnt_at += l->n / 128;
    }
    for (size_t i = 2; i <= kGroupMax; i++) a.front.first[i] = wgs;
    a.front_wgs = wgs;
    a.interleave = g->programs == u->programs ? 1 : 0;
    const fe_exl3_linear::ChainPart *dp = chain_part(d);
    fill_member(a.down, d, dp->programs, ws->xh.p, y, ws->z.p + z_at * 4, ws->counters.p + cnt_at * 4);
    a.state = ws->chain.p;
    a.k1 = g->k, a.k2 = d->k;
    a.inv_spb1 = 0xffffffffu / (a.k1 / 64), a.inv_spb2 = 0xffffffffu / (a.k2 / 64);
    const uint32_t red = rows * kRedPitch * 4;
    auto chunk_of = [&](uint32_t run_steps) {
        const uint32_t c = std::max(4u, ((std::max(kJobLdsBudget, red + rows * 528) - red) / rows - 16) / 128 / 4 * 4);
        return std::min(c, (run_steps + 3) / 4 * 4);
    };
    a.chunk1 = chunk_of(2 * a.fuse1 * std::max(units_per_program(g, g->programs), units_per_program(u, u->programs)));
    a.chunk2 = chunk_of(2 * a.fuse2 * units_per_program(d, dp->programs));
    uint32_t lds = red + rows * (std::max(a.chunk1, a.chunk2) * 128 + 16);
    if (occ && kern->opt.lds_pad) lds = std::max(lds, kCuLds / (occ + 1) + 512);
    // the down stage's programs in the order in which their inputs get ready (the linear's table)
    a.perm = kern->opt.chain_perm ? dp->order.p : 0;
    a.spin_limit = kern->opt.chain_spin;
    const uint32_t grid = a.front_wgs + (dp->programs + a.fuse2 - 1) / a.fuse2;
    uint32_t x_mode = (uint32_t)x_dtype & 1, ldx = g->k, mode = (uint32_t)y_dtype;
    void *args[] = {&a, &x, &x_mode, &ldx, &rows, &mode};
    return fe_hip_launch(kern->mlp[bits_slot(g->bits)], grid, 1, 1, 256, 1, 1, lds, s, args);
}

extern "C" {

int fe_exl3_mlp_forward_launches(const fe_exl3_linear *gate, const fe_exl3_linear *up, const fe_exl3_linear *down, uint32_t rows,
                                 int y_dtype, const fe_exl3_workspace *ws) {
    return mlp_chain_fits(gate, up, down, rows, ws, y_dtype) ? 1 : 0;
}

int fe_exl3_mlp_forward(const fe_exl3_linear *gate, const fe_exl3_linear *up, const fe_exl3_linear *down,
                        const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x, int x_dtype, fe_devptr_t yg, fe_devptr_t yu,
                        fe_devptr_t y, int y_dtype, uint32_t rows, const fe_exl3_workspace *ws) {
    const char *fn = "fe_exl3_mlp_forward";
    if (!gate || !up || !down || !kern || !ws || !x || !yg || !yu || !y) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (x_dtype != FE_DTYPE_BF16 && x_dtype != FE_DTYPE_F32) return fe_set_error(FE_ERR_ARG, fn, "x is bf16 or f32");
    if (gate->n != up->n || down->k != gate->n) return fe_set_error(FE_ERR_SHAPE, fn, "gate and up must produce down's input");
    if (yg % 8 || yu % 8) return fe_set_error(FE_ERR_ARG, fn, "gate / up outputs: 8-byte aligned");
    if (mlp_chain_fits(gate, up, down, rows, ws, y_dtype))
        return launch_mlp(gate, up, down, s, x, x_dtype, yg, yu, y, y_dtype, rows, ws);
    const fe_exl3_linear *front[2] = {gate, up};
    const fe_devptr_t ys[2] = {yg, yu};
    FE_TRY(fe_exl3_linear_forward_group(front, 2, kern, s, x, x_dtype, ys, FE_DTYPE_BF16, rows, ws));
    // down in the partition it has in the one launch (where the GEMV runs and the workspace has the room), so that a row's
    // bits are the same at every row count of this call
    const fe_exl3_linear *dl = down;
    if (rows <= kMaxRowsPerPass) {
        const fe_exl3_linear::ChainPart *part = chain_part(down);
        if (part->as_linear && job_z(part->as_linear.get(), rows) <= ws->z_len) dl = part->as_linear.get();
    }
    return fe_exl3_linear_forward_swiglu(dl, kern, s, yg, yu, gate->n, y, y_dtype, rows, ws);
}

int fe_exl3_workspace_chain_status(fe_exl3_workspace *ws, uint32_t *error) {
    if (!ws || !error) return fe_set_error(FE_ERR_ARG, "fe_exl3_workspace_chain_status", "null argument");
    uint32_t st[4] = {};
    FE_TRY(fe_hip_synchronize());
    FE_TRY(fe_hip_memcpy_dtoh(st, ws->chain.p, sizeof st));
    *error = st[1];
    if (st[1] || st[2]) {  // a wait ran out: the ready words and the count of that launch are void
        ws->chain_off = true;  // (workgroups were not dispatched in grid order here: no further one-launch calls on this workspace)
        FE_TRY(fe_hip_memset_d8(ws->chain.p, 0, ws->chain_len * 4, nullptr));
        FE_TRY(fe_hip_memset_d8(ws->counters.p, 0, ws->counters_len * 4, nullptr));
        FE_TRY(fe_hip_synchronize());
    }
    return 0;
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

int fe_exl3_probe_op(const fe_exl3_kernels *kern, fe_stream_t s, const char *op, uint32_t grid, uint32_t iters,
                     uint32_t launches, float *ms) {
    if (!kern || !op || !grid || !launches || strlen(op) > 32) return fe_set_error(FE_ERR_ARG, "fe_exl3_probe_op", "bad argument");
    char nm[64];
    snprintf(nm, sizeof nm, "exl3_probe_op_%s", op);
    struct Ctx {
        fe_function_t f;
        fe_stream_t s;
        fe_devptr_t out;
        uint32_t grid, iters, seed;
    } ctx{nullptr, s, 0, grid, iters, 7u};
    FE_TRY(fe_hip_module_get_function(&ctx.f, kern->module, nm));
    FeBuf out;
    FE_TRY(out.zeroed(64));
    ctx.out = out.p;
    return time_launches(s, launches, ms,
                         [](void *p) {
                             Ctx *c = (Ctx *)p;
                             void *args[] = {&c->out, &c->iters, &c->seed};
                             return fe_hip_launch(c->f, c->grid, 1, 1, 256, 1, 1, 0, c->s, args);
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
