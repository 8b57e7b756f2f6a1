// host_dropins.hip — host-pointer entry points with the reference's own signatures.
//
// Each stages its operands through cached device buffers (H2D, kernels, D2H) and returns when the
// result is in host memory, so a caller of the reference's CPU ops swaps the symbol only:
//   rmsnorm / rmsnorm_bwd            training/stories_cpu_ops.h:6-53
//   cross_entropy_loss               training/stories_cpu_ops.h:71-108, training/training_dynamic/cpu_ops.h:68-93
//   embed_lookup / embed_backward    training/stories_cpu_ops.h:112-131
//   rope_backward_inplace            training/training_dynamic/cpu_ops.h:168-184
// Failures print one "mi355_bridge: ..." line and leave the outputs untouched.
#include "common.h"

#include <stdlib.h>
#include <algorithm>
#include <vector>

namespace {

constexpr int NSLOT = 8;
struct Slot {
    void *dev;
    size_t bytes;
};
Slot g_slot[NSLOT] = {};

// grow-only staging buffer number `i`
void *slot(int i, size_t bytes) {
    Slot &s = g_slot[i];
    if (s.dev && s.bytes >= bytes) return s.dev;
    if (s.dev) { (void)hipStreamSynchronize(g_ctx.stream); (void)hipFree(s.dev); s.dev = nullptr; s.bytes = 0; }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) { mi355_fail("staging hipMalloc(%zu): %s", bytes, hipGetErrorString(e)); return nullptr; }
    s.dev = p;
    s.bytes = bytes;
    return p;
}

bool h2d(void *dst, const void *src, size_t bytes) {
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_ctx.stream);
    if (e != hipSuccess) { mi355_fail("H2D copy: %s", hipGetErrorString(e)); return false; }
    return true;
}
bool d2h(void *dst, const void *src, size_t bytes) {
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_ctx.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_ctx.stream);
    if (e != hipSuccess) { mi355_fail("D2H copy: %s", hipGetErrorString(e)); return false; }
    return true;
}

// resident embedding tables, keyed by host address
struct Table {
    const float *host;
    float *dev;
    int V, D;
    bool dirty;
};
Table g_tab[4] = {};
int g_tab_n = 0;

}   // namespace

void mi355_free_rope_cache(void);

void mi355_free_caches(void) {
    for (auto &s : g_slot) { if (s.dev) (void)hipFree(s.dev); s = Slot{}; }
    for (int i = 0; i < g_tab_n; i++) if (g_tab[i].dev) (void)hipFree(g_tab[i].dev);
    g_tab_n = 0;
    mi355_free_rope_cache();
}

MI355_API void mi355_rmsnorm(float *out, const float *x, const float *w, int d, int S) {
    if (!mi355_ready("rmsnorm")) return;
    if (!out || !x || !w || d <= 0 || S <= 0) { mi355_fail("rmsnorm: bad arguments"); return; }
    const size_t nb = (size_t)d * S * sizeof(float);
    float *dx = (float *)slot(0, nb), *dy = (float *)slot(1, nb), *dw = (float *)slot(2, (size_t)d * sizeof(float));
    if (!dx || !dy || !dw) return;
    if (!h2d(dx, x, nb) || !h2d(dw, w, (size_t)d * sizeof(float))) return;
    if (mi355_rmsnorm_fwd_dev(dy, dx, dw, d, S, 1, 1e-5f)) return;
    d2h(out, dy, nb);
}

MI355_API void mi355_rmsnorm_bwd(float *dx, float *dw, const float *dy, const float *x, const float *w, int d, int S) {
    if (!mi355_ready("rmsnorm_bwd")) return;
    if (!dx || !dw || !dy || !x || !w || d <= 0 || S <= 0) { mi355_fail("rmsnorm_bwd: bad arguments"); return; }
    const size_t nb = (size_t)d * S * sizeof(float), wb = (size_t)d * sizeof(float);
    float *x_d = (float *)slot(0, nb), *dy_d = (float *)slot(1, nb), *w_d = (float *)slot(2, wb);
    float *dx_d = (float *)slot(3, nb), *dw_d = (float *)slot(4, wb);
    if (!x_d || !dy_d || !w_d || !dx_d || !dw_d) return;
    if (!h2d(x_d, x, nb) || !h2d(dy_d, dy, nb) || !h2d(w_d, w, wb) || !h2d(dw_d, dw, wb)) return;
    if (mi355_rmsnorm_bwd_dev(dx_d, dw_d, dy_d, x_d, w_d, d, S, 1, 1e-5f, 0)) return;
    std::vector<float> dw_new(d);
    if (!d2h(dw_new.data(), dw_d, wb)) return;
    if (!d2h(dx, dx_d, nb)) return;
    memcpy(dw, dw_new.data(), wb);
}

MI355_API float mi355_cross_entropy_loss(float *dlogits, const float *logits, const uint16_t *targets, int V, int S) {
    if (!mi355_ready("cross_entropy_loss")) return NAN;
    if (!dlogits || !logits || !targets || V <= 0 || S <= 0) { mi355_fail("cross_entropy_loss: bad arguments"); return NAN; }
    const size_t nb = (size_t)V * S * sizeof(float);
    float *l_d = (float *)slot(0, nb);
    int32_t *t_d = (int32_t *)slot(1, (size_t)S * sizeof(int32_t));
    float *loss_d = (float *)slot(2, 256);
    if (!l_d || !t_d || !loss_d) return NAN;
    std::vector<int32_t> t32(S);
    for (int t = 0; t < S; t++) t32[t] = targets[t];
    if (!h2d(l_d, logits, nb) || !h2d(t_d, t32.data(), (size_t)S * sizeof(int32_t))) return NAN;
    // the copy of t32 must finish before the vector dies; the loss read-back below synchronises
    if (mi355_softmax_ce_dev(l_d, loss_d, l_d, t_d, V, S, 1.0f)) { (void)hipStreamSynchronize(g_ctx.stream); return NAN; }
    float loss = NAN;
    if (!d2h(&loss, loss_d, sizeof(float))) return NAN;
    if (!d2h(dlogits, l_d, nb)) return NAN;
    for (int t = 0; t < S; t++)
        if (targets[t] >= V)
            fprintf(stderr, "WARN: target token %d out of vocab range [0,%d), skipping\n", (int)targets[t], V);
    return loss;
}

MI355_API void mi355_host_table_invalidate(const float *embed) {
    for (int i = 0; i < g_tab_n; i++)
        if (g_tab[i].host == embed) g_tab[i].dirty = true;
}

MI355_API void mi355_embed_lookup(float *x, const float *embed, const uint16_t *tokens, int vocab, int dim, int seq) {
    if (!mi355_ready("embed_lookup")) return;
    if (!x || !embed || !tokens || vocab <= 0 || dim <= 0 || seq <= 0) { mi355_fail("embed_lookup: bad arguments"); return; }
    Table *tb = nullptr;
    for (int i = 0; i < g_tab_n; i++)
        if (g_tab[i].host == embed && g_tab[i].V == vocab && g_tab[i].D == dim) tb = &g_tab[i];
    const size_t eb = (size_t)vocab * dim * sizeof(float);
    if (!tb) {
        if (g_tab_n == 4) { mi355_fail("embed_lookup: resident-table cache full (4 tables)"); return; }
        float *dev = nullptr;
        hipError_t e = hipMalloc((void **)&dev, eb);
        if (e != hipSuccess) { mi355_fail("embed_lookup: table hipMalloc(%zu): %s", eb, hipGetErrorString(e)); return; }
        g_tab[g_tab_n] = Table{embed, dev, vocab, dim, true};
        tb = &g_tab[g_tab_n++];
    }
    if (tb->dirty) {
        if (!h2d(tb->dev, embed, eb)) return;
        tb->dirty = false;
    }
    const size_t xb = (size_t)dim * seq * sizeof(float);
    float *x_d = (float *)slot(0, xb);
    int32_t *t_d = (int32_t *)slot(1, (size_t)seq * sizeof(int32_t));
    if (!x_d || !t_d) return;
    std::vector<int32_t> t32(seq);
    bool any_oob = false;
    for (int t = 0; t < seq; t++) {
        t32[t] = tokens[t];
        if (tokens[t] >= vocab) {
            any_oob = true;
            fprintf(stderr, "WARN: token %d out of range [0,%d)\n", (int)tokens[t], vocab);
        }
    }
    // skipped columns must keep the caller's values, so those are staged in first
    if (any_oob && !h2d(x_d, x, xb)) return;
    if (!h2d(t_d, t32.data(), (size_t)seq * sizeof(int32_t))) { (void)hipStreamSynchronize(g_ctx.stream); return; }
    if (mi355_embed_gather_dev(x_d, tb->dev, t_d, vocab, dim, seq, 1)) { (void)hipStreamSynchronize(g_ctx.stream); return; }
    d2h(x, x_d, xb);
}

MI355_API void mi355_embed_backward(float *d_embed, const float *dx, const uint16_t *tokens, int vocab, int dim,
                                    int seq) {
    if (!mi355_ready("embed_backward")) return;
    if (!d_embed || !dx || !tokens || vocab <= 0 || dim <= 0 || seq <= 0) { mi355_fail("embed_backward: bad arguments"); return; }
    // Only the rows that are touched travel: unique tokens are numbered 0..U-1 in ascending order,
    // their current rows are uploaded, summed into on the device (same order as the reference
    // loop, starting from the old values) and copied back.
    std::vector<int> uniq;
    uniq.reserve(seq);
    for (int t = 0; t < seq; t++)
        if (tokens[t] < vocab) uniq.push_back(tokens[t]);
    std::sort(uniq.begin(), uniq.end());
    uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
    const int U = (int)uniq.size();
    if (U == 0) return;
    std::vector<int32_t> cid(seq);
    for (int t = 0; t < seq; t++) {
        if (tokens[t] < vocab) cid[t] = (int32_t)(std::lower_bound(uniq.begin(), uniq.end(), (int)tokens[t]) - uniq.begin());
        else cid[t] = -1;
    }
    const size_t rb = (size_t)dim * sizeof(float);
    std::vector<float> rows((size_t)U * dim);
    for (int u = 0; u < U; u++) memcpy(&rows[(size_t)u * dim], d_embed + (size_t)uniq[u] * dim, rb);
    const size_t xb = (size_t)dim * seq * sizeof(float);
    float *dx_d = (float *)slot(0, xb), *rows_d = (float *)slot(3, (size_t)U * rb);
    int32_t *t_d = (int32_t *)slot(1, (size_t)seq * sizeof(int32_t));
    if (!dx_d || !rows_d || !t_d) return;
    bool ok = h2d(dx_d, dx, xb) && h2d(rows_d, rows.data(), (size_t)U * rb) &&
              h2d(t_d, cid.data(), (size_t)seq * sizeof(int32_t));
    if (ok) ok = mi355_embed_scatter_add_dev(rows_d, dx_d, t_d, U, dim, seq, 1) == 0;
    if (!ok) { (void)hipStreamSynchronize(g_ctx.stream); return; }
    if (!d2h(rows.data(), rows_d, (size_t)U * rb)) return;
    for (int u = 0; u < U; u++) memcpy(d_embed + (size_t)uniq[u] * dim, &rows[(size_t)u * dim], rb);
}

MI355_API void mi355_rope_backward_inplace(float *dx, int seq, int dim, int hd) {
    if (!mi355_ready("rope_backward_inplace")) return;
    if (!dx || seq <= 0 || dim <= 0 || hd <= 0 || (hd & 1) || dim % hd) { mi355_fail("rope_backward_inplace: bad arguments"); return; }
    const float *c_d, *s_d;
    if (mi355_rope_tables_dev(&c_d, &s_d, seq, hd, 10000.0f)) return;
    const size_t nb = (size_t)dim * seq * sizeof(float);
    float *x_d = (float *)slot(0, nb);
    if (!x_d) return;
    if (!h2d(x_d, dx, nb)) return;
    if (mi355_rope_dev(x_d, nullptr, x_d, nullptr, dim / hd, 0, hd, seq, 1, c_d, s_d, -1)) return;
    d2h(dx, x_d, nb);
}

// SiLU-gate backward as one call: the 13 vDSP/vForce calls of training/training_dynamic/train.m:537-554.
MI355_API void mi355_swiglu_bwd(float *dh1, float *dh3, const float *dsilu, const float *h1, const float *h3, size_t n) {
    if (!mi355_ready("swiglu_bwd")) return;
    if (!dh1 || !dh3 || !dsilu || !h1 || !h3 || n == 0) { mi355_fail("swiglu_bwd: bad arguments"); return; }
    const size_t nb = n * sizeof(float);
    float *d = (float *)slot(0, nb), *a = (float *)slot(1, nb), *b = (float *)slot(2, nb);
    float *o1 = (float *)slot(3, nb), *o3 = (float *)slot(4, nb);
    if (!d || !a || !b || !o1 || !o3) return;
    if (!h2d(d, dsilu, nb) || !h2d(a, h1, nb) || !h2d(b, h3, nb)) return;
    if (mi355_swiglu_bwd_dev(o1, o3, d, a, b, n)) return;
    if (!d2h(dh1, o1, nb)) return;
    d2h(dh3, o3, nb);
}

// SiLU-gate forward: out = (h1*sigmoid(h1))*h3 (training/forward.h:101,149-151).
MI355_API void mi355_swiglu_fwd(float *out, const float *h1, const float *h3, size_t n) {
    if (!mi355_ready("swiglu_fwd")) return;
    if (!out || !h1 || !h3 || n == 0) { mi355_fail("swiglu_fwd: bad arguments"); return; }
    const size_t nb = n * sizeof(float);
    float *a = (float *)slot(0, nb), *b = (float *)slot(1, nb), *o = (float *)slot(2, nb);
    if (!a || !b || !o) return;
    if (!h2d(a, h1, nb) || !h2d(b, h3, nb)) return;
    if (mi355_swiglu_fwd_dev(o, a, b, n)) return;
    d2h(out, o, nb);
}

// Residual family on host pointers: vDSP_vsma / vDSP_vsmul / vDSP_vadd
// (training/training_dynamic/train.m:460,523,595; training/train_large.m:427,442).
MI355_API void mi355_axpby(float *y, const float *a, const float *b, float alpha, size_t n, int mode) {
    if (!mi355_ready("axpby")) return;
    if (!y || !a || (mode != 1 && !b) || n == 0 || mode < 0 || mode > 2) { mi355_fail("axpby: bad arguments"); return; }
    const size_t nb = n * sizeof(float);
    float *ad = (float *)slot(0, nb), *bd = (float *)slot(1, nb), *yd = (float *)slot(2, nb);
    if (!ad || !bd || !yd) return;
    if (!h2d(ad, a, nb)) return;
    if (mode != 1 && !h2d(bd, b, nb)) return;
    if (mi355_axpby_dev(yd, ad, mode != 1 ? bd : nullptr, alpha, n, mode)) return;
    d2h(y, yd, nb);
}

// adam_update (training/training_dynamic/cpu_ops.h:56-64) on host arrays.
MI355_API void mi355_adam_update(float *w, const float *g, float *m, float *v, size_t n, int t, float lr, float b1,
                                 float b2, float eps, float wd) {
    if (!mi355_ready("adam_update")) return;
    if (!w || !g || !m || !v || n == 0 || t < 1) { mi355_fail("adam_update: bad arguments"); return; }
    const size_t nb = n * sizeof(float);
    float *wd_ = (float *)slot(0, nb), *gd = (float *)slot(1, nb), *md = (float *)slot(2, nb), *vd = (float *)slot(3, nb);
    if (!wd_ || !gd || !md || !vd) return;
    if (!h2d(wd_, w, nb) || !h2d(gd, g, nb) || !h2d(md, m, nb) || !h2d(vd, v, nb)) return;
    if (mi355_adam_update_dev(wd_, gd, md, vd, n, t, lr, b1, b2, eps, wd, 1.0f, nullptr, 0)) return;
    std::vector<float> w2(n), m2(n);
    if (!d2h(w2.data(), wd_, nb) || !d2h(m2.data(), md, nb)) return;
    if (!d2h(v, vd, nb)) return;
    memcpy(w, w2.data(), nb);
    memcpy(m, m2.data(), nb);
}
