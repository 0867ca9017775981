// fe_route: how rows of a batch reach the two quantized linears (see include/fe_route.h). Follows
// crates/fe-model/src/model.rs:172-203, 260-403, 3160-3203; the two elementwise kernels are kernels/k_route.hip.
#include "fe_route.h"

#include <algorithm>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#include "fe_internal.h"

namespace {
// The code object with fe_silu_mul and fe_copy2d, loaded once per process at first use.
struct RouteKernels {
    fe_module_t module = nullptr;
    fe_function_t silu_mul = nullptr, copy2d = nullptr;
    int code = 0;
};
RouteKernels g_kern;
std::once_flag g_kern_once;

int route_kernels(const RouteKernels **out) {
    std::call_once(g_kern_once, [] {
        int c = fe_load_module(&g_kern.module, "FE_ROUTE_HSACO", fe_k_route_hsaco, fe_k_route_hsaco_end);
        if (!c) c = fe_hip_module_get_function(&g_kern.silu_mul, g_kern.module, "fe_silu_mul");
        if (!c) c = fe_hip_module_get_function(&g_kern.copy2d, g_kern.module, "fe_copy2d");
        g_kern.code = c;
    });
    if (g_kern.code) return fe_set_error(g_kern.code, "fe_route", "the routing kernels did not load");
    *out = &g_kern;
    return 0;
}

int fail(int code, const char *call, const std::string &msg) { return fe_set_error(code, call, msg.c_str()); }
}  // namespace

struct fe_route_ctx {
    const fe_exl3_kernels *xk = nullptr;
    const fe_exl3_workspace *xws = nullptr;
    const fe_fp4_kernels *fk = nullptr;
    const fe_fp4_workspace *fws = nullptr;
    const fe_bf16_kernels *bk = nullptr;
    fe_stream_t s = nullptr;
    FeBuf tmp;  // [FE_DEC_MAX][max_proj] bf16
    uint32_t max_proj = 0, dec = 0;
    bool x3_gemm = true;
    bool x3() const { return xk && xws; }
    bool fp4() const { return fk && fws; }
};

struct fe_route_linear {
    std::string name;
    uint32_t n = 0, k = 0;
    const fe_exl3_linear *q = nullptr;
    const fe_fp4_linear *p = nullptr;
    fe_devptr_t w = 0;  // bf16 weights [n][k]
};

struct fe_route_proj {
    std::vector<std::pair<const fe_route_linear *, std::vector<uint32_t>>> lins;
    const fe_fp4_linear *prompt = nullptr;
    uint32_t prompt_n = 0, cover = 0;
};

// Linear::forward with an explicit count of decode rows (the reference copies its LinCtx with another `dec`).
static int linear_forward(const fe_route_linear *l, const fe_route_ctx *c, uint32_t dec, fe_devptr_t y, uint32_t ldy,
                          fe_devptr_t x, uint32_t lda, uint32_t m, fe_devptr_t res) {
    const char *fn = "fe_route_linear_forward";
    if (m == 0) return 0;
    if (l->q && c->x3()) {
        // decode rows (all rows of a small batch): the trellis GEMV, FE_X3_PASS rows a call (model.rs:277-303)
        uint32_t d = m <= FE_X3_ROWS ? m : std::min(dec, m);
        if (d > 0 && lda == l->k && ldy == l->n) {
            if (res && res != y) return fail(FE_ERR_ARG, fn, l->name + ": residual must be in place");
            // the residual is added in the GEMV's epilogue: y = bf16(f32(y) + x . W)
            const int yd = res ? FE_DTYPE_BF16_ADD : FE_DTYPE_BF16;
            for (uint32_t r = 0; r < d;) {
                uint32_t n = std::min<uint32_t>(d - r, FE_X3_PASS);
                FE_TRY(fe_exl3_linear_forward(l->q, c->xk, c->s, x + (size_t)r * lda * 2, FE_DTYPE_BF16,
                                              y + (size_t)r * ldy * 2, yd, n, c->xws));
                r += n;
            }
            if (d == m) return 0;
            // the prompt rows after them
            return linear_forward(l, c, 0, y + (size_t)d * ldy * 2, ldy, x + (size_t)d * lda * 2, lda, m - d,
                                  res ? res + (size_t)d * ldy * 2 : 0);
        }
    }
    if (l->p && c->fp4()) return fe_fp4_linear_forward(l->p, c->fk, c->s, c->fws, y, ldy, x, lda, m, res);
    if (!l->w && l->q && c->x3() && m > FE_X3_ROWS) {
        // no prompt weights and no bf16 weights: every row through the trellis linear (model.rs:305-309); with bf16
        // weights beside the trellis the prompt rows take the bf16 GEMM below, as in the reference
        if (lda != l->k || ldy != l->n) return fail(FE_ERR_ARG, fn, l->name + ": the trellis linear needs lda == k and ldy == n");
        uint32_t ws_rows = 0;
        FE_TRY(fe_exl3_workspace_xh(c->xws, nullptr, &ws_rows, nullptr));
        if (c->x3_gemm && m > FE_X3_PASS && ws_rows >= m) {
            // one call: above 64 rows the library runs its MFMA GEMM
            if (res && res != y) return fail(FE_ERR_ARG, fn, l->name + ": residual must be in place");
            return fe_exl3_linear_forward(l->q, c->xk, c->s, x, FE_DTYPE_BF16, y, res ? FE_DTYPE_BF16_ADD : FE_DTYPE_BF16, m, c->xws);
        }
        return linear_forward(l, c, m, y, ldy, x, lda, m, res);
    }
    if (!l->w || !c->bk) {
        char msg[200];
        snprintf(msg, sizeof msg, "%s: no bf16 weights for %u rows", l->name.c_str(), m);
        return fe_set_error(FE_ERR_UNSUPPORTED, fn, msg);
    }
    // plain bf16 weights: GEMV passes for the decode rows, the GEMM for the rest (model.rs:310-345)
    return fe_bf16_linear_forward(c->bk, c->s, y, ldy, x, lda, l->w, res, m, l->n, l->k, dec);
}

extern "C" {

int fe_route_ctx_create(fe_route_ctx **out, const fe_exl3_kernels *xk, const fe_exl3_workspace *xws,
                        const fe_fp4_kernels *fk, const fe_fp4_workspace *fws, fe_stream_t s, uint32_t max_proj) {
    if (!out) return fe_set_error(FE_ERR_ARG, "fe_route_ctx_create", "null out");
    if ((xk == nullptr) != (xws == nullptr) || (fk == nullptr) != (fws == nullptr))
        return fe_set_error(FE_ERR_ARG, "fe_route_ctx_create", "kernels and workspace come together");
    const RouteKernels *rk;
    FE_TRY(route_kernels(&rk));
    auto *c = new fe_route_ctx;
    c->xk = xk, c->xws = xws, c->fk = fk, c->fws = fws, c->s = s, c->max_proj = max_proj;
    if (max_proj) {
        int e = c->tmp.alloc((size_t)FE_DEC_MAX * max_proj * 2);
        if (e) {
            delete c;
            return e;
        }
    }
    *out = c;
    return 0;
}

int fe_route_ctx_destroy(fe_route_ctx *c) {
    delete c;
    return 0;
}

int fe_route_ctx_set_dec(fe_route_ctx *c, uint32_t dec) {
    if (!c) return fe_set_error(FE_ERR_ARG, "fe_route_ctx_set_dec", "null context");
    c->dec = dec;
    return 0;
}

int fe_route_ctx_set_bf16(fe_route_ctx *c, const fe_bf16_kernels *bk) {
    if (!c) return fe_set_error(FE_ERR_ARG, "fe_route_ctx_set_bf16", "null context");
    c->bk = bk;
    return 0;
}

int fe_route_linear_set_bf16(fe_route_linear *l, fe_devptr_t w) {
    if (!l) return fe_set_error(FE_ERR_ARG, "fe_route_linear_set_bf16", "null linear");
    if (w % 16) return fe_set_error(FE_ERR_ARG, "fe_route_linear_set_bf16", "weights must be 16-byte aligned");
    l->w = w;
    return 0;
}

int fe_route_ctx_set_x3_gemm(fe_route_ctx *c, int on) {
    if (!c) return fe_set_error(FE_ERR_ARG, "fe_route_ctx_set_x3_gemm", "null context");
    c->x3_gemm = on != 0;
    return 0;
}

int fe_route_linear_create(fe_route_linear **out, const char *name, uint32_t n, uint32_t k, const fe_exl3_linear *q,
                           const fe_fp4_linear *p) {
    const char *fn = "fe_route_linear_create";
    if (!out || !name) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (q) {
        fe_exl3_view v;
        FE_TRY(fe_exl3_linear_view(q, &v, nullptr));
        if (v.k != k || v.n != n) return fail(FE_ERR_SHAPE, fn, std::string(name) + ": the trellis linear has another shape");
    }
    if (p) {
        uint32_t pn = 0, pk = 0;
        FE_TRY(fe_fp4_linear_shape(p, &pn, &pk, nullptr));
        if (pk != k || pn != n) return fail(FE_ERR_SHAPE, fn, std::string(name) + ": the prompt linear has another shape");
    }
    auto *l = new fe_route_linear;
    l->name = name, l->n = n, l->k = k, l->q = q, l->p = p;
    *out = l;
    return 0;
}

int fe_route_linear_destroy(fe_route_linear *l) {
    delete l;
    return 0;
}

int fe_route_linear_forward(const fe_route_linear *l, const fe_route_ctx *c, fe_devptr_t y, uint32_t ldy, fe_devptr_t x,
                            uint32_t lda, uint32_t m, fe_devptr_t res) {
    if (!l || !c || !y || !x) return fe_set_error(FE_ERR_ARG, "fe_route_linear_forward", "null argument");
    return linear_forward(l, c, c->dec, y, ldy, x, lda, m, res);
}

int fe_route_proj_create(fe_route_proj **out, const fe_route_linear *const *lins, const uint32_t *const *widths,
                         const uint32_t *widths_len, size_t count, const fe_fp4_linear *prompt, uint32_t cover) {
    const char *fn = "fe_route_proj_create";
    if (!out || !lins || !widths || !widths_len || !count) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    auto *p = new fe_route_proj;
    for (size_t i = 0; i < count; i++) {
        std::vector<uint32_t> w(widths[i], widths[i] + widths_len[i]);
        uint32_t sum = 0;
        for (uint32_t v : w) sum += v;
        if (!lins[i] || sum != lins[i]->n) {
            delete p;
            return fe_set_error(FE_ERR_SHAPE, fn, "the widths of a linear's parts do not sum to its n");
        }
        p->lins.emplace_back(lins[i], std::move(w));
    }
    if (prompt) {
        uint32_t pn = 0, pk = 0, covered = 0;
        int e = fe_fp4_linear_shape(prompt, &pn, &pk, nullptr);
        if (!e && (cover == 0 || cover > count)) e = fe_set_error(FE_ERR_ARG, fn, "cover out of range");
        for (uint32_t i = 0; !e && i < cover; i++) {
            covered += lins[i]->n;
            if (lins[i]->k != pk) e = fe_set_error(FE_ERR_SHAPE, fn, "the fused prompt linear has another k");
        }
        if (!e && covered != pn) e = fe_set_error(FE_ERR_SHAPE, fn, "the fused prompt linear does not cover its linears");
        if (e) {
            delete p;
            return e;
        }
        p->prompt = prompt, p->prompt_n = pn, p->cover = cover;
    }
    *out = p;
    return 0;
}

int fe_route_proj_destroy(fe_route_proj *p) {
    delete p;
    return 0;
}

uint32_t fe_route_proj_total_n(const fe_route_proj *p) {
    uint32_t n = 0;
    if (p)
        for (auto &l : p->lins) n += l.first->n;
    return n;
}

int fe_route_copy2d(fe_stream_t s, fe_devptr_t dst, uint32_t ldd, fe_devptr_t src, uint32_t lds, uint32_t cols, uint32_t rows) {
    if (!dst || !src || (cols & 1) || cols > ldd || cols > lds) return fe_set_error(FE_ERR_ARG, "fe_route_copy2d", "bad argument");
    if (!rows || !cols) return 0;
    const RouteKernels *rk;
    FE_TRY(route_kernels(&rk));
    void *args[] = {&dst, &ldd, &src, &lds, &cols};
    return fe_hip_launch(rk->copy2d, rows, (cols / 2 + 255) / 256, 1, 256, 1, 1, 0, s, args);
}

int fe_route_silu_mul(fe_stream_t s, fe_devptr_t out, fe_devptr_t gate, fe_devptr_t up, uint32_t ld, uint32_t inter,
                      uint32_t rows) {
    if (!out || !gate || !up || (inter & 1) || inter > ld) return fe_set_error(FE_ERR_ARG, "fe_route_silu_mul", "bad argument");
    if (!rows || !inter) return 0;
    const RouteKernels *rk;
    FE_TRY(route_kernels(&rk));
    void *args[] = {&out, &gate, &up, &ld, &inter};
    return fe_hip_launch(rk->silu_mul, (inter / 2 + 255) / 256, rows, 1, 256, 1, 1, 0, s, args);
}

// Proj::forward with an explicit count of decode rows.
static int proj_forward(const fe_route_proj *p, const fe_route_ctx *c, uint32_t dec, fe_devptr_t out, fe_devptr_t x,
                        uint32_t lda, uint32_t m, fe_devptr_t *part_ptr, uint32_t *part_ld, size_t parts_cap, size_t *parts_n) {
    const char *fn = "fe_route_proj_forward";
    size_t np = 0;
    auto push = [&](fe_devptr_t ptr, uint32_t ld) {
        if (np < parts_cap) {
            if (part_ptr) part_ptr[np] = ptr;
            if (part_ld) part_ld[np] = ld;
        }
        np++;
    };
    size_t off = 0, first = 0;  // elements into `out`
    if (p->prompt && c->fp4() && m > FE_X3_ROWS) {
        const uint32_t pn = p->prompt_n, d = std::min(dec, m);
        if (d < m)
            FE_TRY(fe_fp4_linear_forward(p->prompt, c->fk, c->s, c->fws, out + (size_t)d * pn * 2, pn, x + (size_t)d * lda * 2,
                                         lda, m - d, 0));
        uint32_t col = 0;
        for (uint32_t i = 0; i < p->cover; i++) {
            const fe_route_linear *l = p->lins[i].first;
            if (d > 0) {
                // decode rows: the linear's own GEMV into scratch, then into the fused layout (model.rs:373-382)
                if (d > FE_DEC_MAX || l->n > c->max_proj) {
                    char msg[160];
                    snprintf(msg, sizeof msg, "%s: %u decode rows", l->name.c_str(), d);
                    return fe_set_error(FE_ERR_WORKSPACE, fn, msg);
                }
                FE_TRY(linear_forward(l, c, d, c->tmp.p, l->n, x, lda, d, 0));
                FE_TRY(fe_route_copy2d(c->s, out + (size_t)col * 2, pn, c->tmp.p, l->n, l->n, d));
            }
            for (uint32_t w : p->lins[i].second) {
                push(out + (size_t)col * 2, pn);
                col += w;
            }
        }
        off = (size_t)m * pn;
        first = p->cover;
    }
    for (size_t i = first; i < p->lins.size();) {
        // Trellis linears of this input, for a batch the GEMV takes whole in one pass: one grouped launch for up to four of them
        // (the bits of each linear's own forward). The reference runs them one after the other (model.rs:384-392).
        size_t j = i;
        if ((m <= FE_X3_ROWS || (dec >= m && m <= FE_X3_PASS)) && c->x3())
            while (j < p->lins.size() && j - i < 4 && p->lins[j].first->q && p->lins[j].first->k == lda) j++;
        if (j - i >= 2) {
            const fe_exl3_linear *qs[4];
            fe_devptr_t ys[4];
            size_t o = off;
            for (size_t t = i; t < j; t++) {
                qs[t - i] = p->lins[t].first->q, ys[t - i] = out + o * 2;
                o += (size_t)m * p->lins[t].first->n;
            }
            FE_TRY(fe_exl3_linear_forward_group(qs, j - i, c->xk, c->s, x, FE_DTYPE_BF16, ys, FE_DTYPE_BF16, m, c->xws));
        } else {
            j = i + 1;
            FE_TRY(linear_forward(p->lins[i].first, c, dec, out + off * 2, p->lins[i].first->n, x, lda, m, 0));
        }
        for (; i < j; i++) {
            const fe_route_linear *l = p->lins[i].first;
            const fe_devptr_t y = out + off * 2;
            uint32_t col = 0;
            for (uint32_t w : p->lins[i].second) {
                push(y + (size_t)col * 2, l->n);
                col += w;
            }
            off += (size_t)m * l->n;
        }
    }
    if (parts_n) *parts_n = np;
    if (np > parts_cap && (part_ptr || part_ld)) return fe_set_error(FE_ERR_ARG, fn, "more parts than the caller made room for");
    return 0;
}

int fe_route_proj_forward(const fe_route_proj *p, const fe_route_ctx *c, fe_devptr_t out, fe_devptr_t x, uint32_t lda,
                          uint32_t m, fe_devptr_t *part_ptr, uint32_t *part_ld, size_t parts_cap, size_t *parts_n) {
    if (!p || !c || !out || !x) return fe_set_error(FE_ERR_ARG, "fe_route_proj_forward", "null argument");
    return proj_forward(p, c, c->dec, out, x, lda, m, part_ptr, part_ld, parts_cap, parts_n);
}

int fe_route_mlp_forward(const fe_route_ctx *c, const fe_route_proj *gate_up, const fe_route_linear *down,
                         const fe_fp4_linear *swiglu, const fe_fp4_workspace *act_ws, fe_devptr_t x, fe_devptr_t xn,
                         fe_devptr_t big, fe_devptr_t act, uint32_t rows, uint32_t hidden, uint32_t inter) {
    return fe_route_mlp_forward_w(c, gate_up, down, swiglu, act_ws, 0, x, xn, big, act, rows, hidden, inter);
}

int fe_route_mlp_forward_w(const fe_route_ctx *c, const fe_route_proj *gate_up, const fe_route_linear *down,
                           const fe_fp4_linear *swiglu, const fe_fp4_workspace *act_ws, fe_devptr_t swiglu_w, fe_devptr_t x,
                           fe_devptr_t xn, fe_devptr_t big, fe_devptr_t act, uint32_t rows, uint32_t hidden, uint32_t inter) {
    const char *fn = "fe_route_mlp_forward";
    if (!c || !gate_up || !down || !x || !xn || !big || !act) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    if (down->n != hidden || down->k != inter) return fe_set_error(FE_ERR_SHAPE, fn, "down is not hidden x inter");
    if (rows == 0) return 0;
    // prompt rows [d, rows) may take the fused SwiGLU path; decode rows [0, d) always the per-linear one
    const uint32_t d = rows > FE_X3_ROWS ? std::min(c->dec, rows) : rows;
    const uint32_t pr_rows = rows - d;
    bool fused = false;
    if (pr_rows > FE_X3_ROWS && swiglu && down->p && c->fp4() && act_ws) {
        const fe_devptr_t xn_p = xn + (size_t)d * hidden * 2, x_p = x + (size_t)d * hidden * 2;
        float down_g = 1.0f;
        FE_TRY(fe_fp4_linear_shape(down->p, nullptr, nullptr, &down_g));
        // gate|up GEMM + SwiGLU + NVFP4 quantization in one kernel, then down on the quantized activation with the
        // residual in place (model.rs:3166-3178)
        FE_TRY(fe_fp4_linear_forward_swiglu(swiglu, c->fk, c->s, c->fws, act_ws, xn_p, hidden, pr_rows, down_g));
        FE_TRY(fe_fp4_linear_gemm(down->p, c->fk, c->s, act_ws, x_p, hidden, pr_rows, x_p));
        fused = true;
    } else if (pr_rows > FE_X3_ROWS && swiglu_w && c->bk) {
        // interleaved bf16 gate|up weights: one GEMM with SwiGLU in its epilogue, then down over the prompt rows with the
        // residual (model.rs:3179-3188)
        const fe_devptr_t xn_p = xn + (size_t)d * hidden * 2, x_p = x + (size_t)d * hidden * 2;
        const fe_devptr_t act_p = act + (size_t)d * inter * 2;
        FE_TRY(fe_bf16_gemm_swiglu(c->bk, c->s, act_p, xn_p, hidden, swiglu_w, pr_rows, inter, hidden));
        FE_TRY(linear_forward(down, c, 0, x_p, hidden, act_p, inter, pr_rows, x_p));
        fused = true;
    }
    const uint32_t n_rest = fused ? d : rows;
    if (n_rest > 0 && gate_up->lins.size() == 2 && !(gate_up->prompt && c->fp4() && n_rest > FE_X3_ROWS) && c->x3() && down->q) {
        // Decode rows through three trellis linears, gate and up each one part, every row in one GEMV pass: the block
        // through fe_exl3_mlp_forward at every such row count (one launch where that applies, else the grouped gate + up
        // launch and down's forward_swiglu with down partitioned as in the one launch), so that a row's bits do not
        // depend on the batch it is in
        const fe_route_linear *g = gate_up->lins[0].first, *u = gate_up->lins[1].first;
        if (g->q && u->q && g->k == hidden && u->k == hidden && g->n == inter && u->n == inter &&
            gate_up->lins[0].second.size() == 1 && gate_up->lins[1].second.size() == 1 && n_rest <= FE_X3_PASS &&
            (n_rest <= FE_X3_ROWS || d >= n_rest))
            return fe_exl3_mlp_forward(g->q, u->q, down->q, c->xk, c->s, xn, FE_DTYPE_BF16, big, big + (size_t)n_rest * inter * 2, x,
                                       FE_DTYPE_BF16_ADD, n_rest, c->xws);
    }
    if (n_rest > 0) {
        fe_devptr_t ptr[8] = {};
        uint32_t ld[8] = {};
        size_t parts = 0;
        FE_TRY(proj_forward(gate_up, c, d, big, xn, hidden, n_rest, ptr, ld, 8, &parts));
        if (parts < 2) return fe_set_error(FE_ERR_SHAPE, fn, "gate_up has fewer than two parts");
        if (ld[0] != ld[1]) return fe_set_error(FE_ERR_SHAPE, fn, "gate/up strides differ");
        if (down->q && c->x3() && n_rest <= FE_X3_PASS && (n_rest <= FE_X3_ROWS || d >= n_rest)) {
            // every row through down's trellis GEMV in one pass: SwiGLU is applied as the GEMV's input rotation reads
            // gate and up (the bits of fe_silu_mul followed by the linear; the reference launches both, model.rs:3184-3199)
            FE_TRY(fe_exl3_linear_forward_swiglu(down->q, c->xk, c->s, ptr[0], ptr[1], ld[0], x, FE_DTYPE_BF16_ADD, n_rest, c->xws));
        } else {
            FE_TRY(fe_route_silu_mul(c->s, act, ptr[0], ptr[1], ld[0], inter, n_rest));
            FE_TRY(linear_forward(down, c, d, x, hidden, act, inter, n_rest, x));
        }
    }
    return 0;
}

}  // extern "C"
