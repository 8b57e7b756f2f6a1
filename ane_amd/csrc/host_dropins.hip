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

// Host-pointer entry points copy and wait, so they cannot run while a graph is being recorded.
bool host_ready(const char *who) { return mi355_ready(who) && mi355_outside_capture(who); }

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

// A drop-in has written the host range [p, p+bytes): any resident table that overlaps it is stale.
void host_written(const void *p, size_t bytes) {
    const char *lo = (const char *)p, *hi = lo + bytes;
    for (int i = 0; i < g_tab_n; i++) {
        const char *tlo = (const char *)g_tab[i].host;
        const char *thi = tlo + (size_t)g_tab[i].V * g_tab[i].D * sizeof(float);
        if (lo < thi && tlo < hi) g_tab[i].dirty = true;
    }
}

// A drop-in has written the host range [p, p+bytes) and its device staging buffer `dev_src` holds the same bytes: a
// resident table that contains the whole range takes them from there (a copy on the device, in stream order) and
// stays current; one that only overlaps it is stale.  The embedding table that adam_update steps every iteration
// (training/training_dynamic/train.m:869) is then not uploaded again by the vocab_compact_embed that follows (:871).
void host_written_from(const void *p, const void *dev_src, size_t bytes) {
    const char *lo = (const char *)p, *hi = lo + bytes;
    for (int i = 0; i < g_tab_n; i++) {
        const char *tlo = (const char *)g_tab[i].host;
        const char *thi = tlo + (size_t)g_tab[i].V * g_tab[i].D * sizeof(float);
        if (!(lo < thi && tlo < hi)) continue;
        if (!g_tab[i].dirty && tlo <= lo && hi <= thi &&
            hipMemcpyAsync((char *)g_tab[i].dev + (lo - tlo), dev_src, bytes, hipMemcpyDeviceToDevice, g_ctx.stream) == hipSuccess)
            continue;
        g_tab[i].dirty = true;
    }
}

// The device copy of the host table `embed` [vocab][dim], uploaded if new or stale.  NULL on failure.
Table *resident_table(const char *who, const float *embed, int vocab, int dim) {
    Table *tb = nullptr;
    for (int i = 0; i < g_tab_n; i++)
        if (g_tab[i].host == embed && g_tab[i].V == vocab && g_tab[i].D == dim) tb = &g_tab[i];
    const size_t eb = (size_t)vocab * dim * sizeof(float);
    if (!tb) {
        if (g_tab_n == 4) { mi355_fail("%s: resident-table cache full (4 tables)", who); return nullptr; }
        float *dev = nullptr;
        hipError_t e = hipMalloc((void **)&dev, eb);
        if (e != hipSuccess) { mi355_fail("%s: table hipMalloc(%zu): %s", who, eb, hipGetErrorString(e)); return nullptr; }
        g_tab[g_tab_n] = Table{embed, dev, vocab, dim, true};
        tb = &g_tab[g_tab_n++];
    }
    if (tb->dirty) {
        if (!h2d(tb->dev, embed, eb)) return nullptr;
        tb->dirty = false;
    }
    return tb;
}

}   // namespace

void mi355_free_rope_cache(void);
void mi355_free_scatter_report(void);

void mi355_free_caches(void) {
    for (auto &s : g_slot) { if (s.dev) (void)hipFree(s.dev); s = Slot{}; }
    for (int i = 0; i < g_tab_n; i++) if (g_tab[i].dev) (void)hipFree(g_tab[i].dev);
    g_tab_n = 0;
    mi355_free_rope_cache();
    mi355_free_scatter_report();
}

MI355_API void mi355_rmsnorm(float *out, const float *x, const float *w, int d, int S) {
    if (!host_ready("rmsnorm")) return;
    if (!out || !x || !w || d <= 0 || S <= 0) { mi355_fail("rmsnorm: bad arguments"); return; }
    const size_t nb = (size_t)d * S * sizeof(float);
    float *dx = (float *)slot(0, nb), *dy = (float *)slot(1, nb), *dw = (float *)slot(2, (size_t)d * sizeof(float));
    if (!dx || !dy || !dw) return;
    if (!h2d(dx, x, nb) || !h2d(dw, w, (size_t)d * sizeof(float))) return;
    if (mi355_rmsnorm_fwd_dev(dy, dx, dw, d, S, 1, 1e-5f)) return;
    d2h(out, dy, nb);
}

MI355_API void mi355_rmsnorm_bwd(float *dx, float *dw, const float *dy, const float *x, const float *w, int d, int S) {
    if (!host_ready("rmsnorm_bwd")) return;
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
    if (!host_ready("cross_entropy_loss")) return NAN;
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
    if (!host_ready("embed_lookup")) return;
    if (!x || !embed || !tokens || vocab <= 0 || dim <= 0 || seq <= 0) { mi355_fail("embed_lookup: bad arguments"); return; }
    Table *tb = resident_table("embed_lookup", embed, vocab, dim);
    if (!tb) return;
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
    if (!host_ready("embed_backward")) return;
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
    if (!host_ready("rope_backward_inplace")) return;
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
    if (!host_ready("swiglu_bwd")) return;
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
    if (!host_ready("swiglu_fwd")) return;
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
    if (!host_ready("axpby")) return;
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
    if (!host_ready("adam_update")) return;
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
    host_written_from(w, wd_, nb);      // a resident embedding table that lives in w follows on the device
}

// ---- vocabulary compaction on host arrays: training/training_dynamic/cpu_ops.h:96-148 ----

// vocab_map_build (cpu_ops.h:102-126): both maps are caller-allocated ([full_vocab] ints each; the first
// compact_vocab entries of compact_to_full are written).  Returns compact_vocab, or -1.
MI355_API int mi355_vocab_map_build(int *full_to_compact, int *compact_to_full, const uint16_t *data, size_t n_tokens,
                                    int full_vocab) {
    if (!host_ready("vocab_map_build")) return -1;
    if (!full_to_compact || !compact_to_full || (!data && n_tokens) || full_vocab <= 0)
        return mi355_fail("vocab_map_build: bad arguments");
    const size_t mb = (size_t)full_vocab * sizeof(int32_t), db = n_tokens * sizeof(uint16_t);
    int32_t *f2c = (int32_t *)slot(0, mb), *c2f = (int32_t *)slot(1, mb), *cnt = (int32_t *)slot(2, 256);
    uint16_t *dat = (uint16_t *)slot(3, db ? db : 2);
    if (!f2c || !c2f || !cnt || !dat) return -1;
    if (db && !h2d(dat, data, db)) return -1;
    if (mi355_vocab_map_build_dev(f2c, c2f, cnt, dat, n_tokens, full_vocab)) return -1;
    int32_t cv = -1;
    if (!d2h(&cv, cnt, sizeof(cv))) return -1;
    if (cv < 0 || cv > full_vocab) return mi355_fail("vocab_map_build: device count %d out of range", cv);
    std::vector<int32_t> f(full_vocab);
    if (!d2h(f.data(), f2c, mb)) return -1;
    if (cv && !d2h(compact_to_full, c2f, (size_t)cv * sizeof(int32_t))) return -1;
    memcpy(full_to_compact, f.data(), mb);
    return cv;
}

// vocab_compact_embed (cpu_ops.h:127-132) into a caller-allocated [compact_vocab][dim] array.  The full table
// is kept resident on the device, keyed by its host address, as for embed_lookup.
MI355_API void mi355_vocab_compact_embed(float *compact, const float *full_embed, const int *compact_to_full,
                                         int compact_vocab, int full_vocab, int dim) {
    if (!host_ready("vocab_compact_embed")) return;
    if (!compact || !full_embed || !compact_to_full || compact_vocab <= 0 || full_vocab <= 0 || dim <= 0) {
        mi355_fail("vocab_compact_embed: bad arguments");
        return;
    }
    Table *tb = resident_table("vocab_compact_embed", full_embed, full_vocab, dim);
    if (!tb) return;
    const size_t cb = (size_t)compact_vocab * dim * sizeof(float), ib = (size_t)compact_vocab * sizeof(int32_t);
    float *c_d = (float *)slot(0, cb);
    int32_t *i_d = (int32_t *)slot(1, ib);
    if (!c_d || !i_d) return;
    // a map entry outside the table is skipped on the device: such rows keep the caller's values
    bool any_oob = false;
    for (int c = 0; c < compact_vocab; c++) any_oob |= compact_to_full[c] < 0 || compact_to_full[c] >= full_vocab;
    if (any_oob && !h2d(c_d, compact, cb)) return;
    if (!h2d(i_d, compact_to_full, ib)) return;
    if (mi355_vocab_compact_embed_dev(c_d, tb->dev, i_d, compact_vocab, full_vocab, dim)) return;
    d2h(compact, c_d, cb);
}

namespace {
// Host rows full[map[c]] <-> a packed [CV][dim] staging array (only the rows an op touches travel).
void pack_rows(std::vector<float> &rows, const float *full, const int *map, int cv, int full_vocab, int dim) {
    for (int c = 0; c < cv; c++)
        if (map[c] >= 0 && map[c] < full_vocab)
            memcpy(&rows[(size_t)c * dim], full + (size_t)map[c] * dim, (size_t)dim * sizeof(float));
}
void unpack_rows(float *full, const std::vector<float> &rows, const int *map, int cv, int full_vocab, int dim) {
    for (int c = 0; c < cv; c++)
        if (map[c] >= 0 && map[c] < full_vocab)
            memcpy(full + (size_t)map[c] * dim, &rows[(size_t)c * dim], (size_t)dim * sizeof(float));
}
}   // namespace

// vocab_scatter_grads (cpu_ops.h:135-142): full_gembed[map[c]] += compact_gembed[c].  The touched rows of the
// full gradient are uploaded packed, summed into on the device and copied back.
MI355_API void mi355_vocab_scatter_grads(float *full_gembed, const float *compact_gembed, const int *compact_to_full,
                                         int compact_vocab, int full_vocab, int dim) {
    if (!host_ready("vocab_scatter_grads")) return;
    if (!full_gembed || !compact_gembed || !compact_to_full || compact_vocab <= 0 || full_vocab <= 0 || dim <= 0) {
        mi355_fail("vocab_scatter_grads: bad arguments");
        return;
    }
    const size_t cb = (size_t)compact_vocab * dim * sizeof(float);
    std::vector<float> rows((size_t)compact_vocab * dim, 0.0f);
    pack_rows(rows, full_gembed, compact_to_full, compact_vocab, full_vocab, dim);
    std::vector<int32_t> ident(compact_vocab);
    for (int c = 0; c < compact_vocab; c++)
        ident[c] = (compact_to_full[c] >= 0 && compact_to_full[c] < full_vocab) ? c : -1;
    float *rows_d = (float *)slot(0, cb), *g_d = (float *)slot(1, cb);
    int32_t *i_d = (int32_t *)slot(2, (size_t)compact_vocab * sizeof(int32_t));
    if (!rows_d || !g_d || !i_d) return;
    if (!h2d(rows_d, rows.data(), cb) || !h2d(g_d, compact_gembed, cb) ||
        !h2d(i_d, ident.data(), (size_t)compact_vocab * sizeof(int32_t))) { (void)hipStreamSynchronize(g_ctx.stream); return; }
    if (mi355_vocab_scatter_grads_dev(rows_d, g_d, i_d, compact_vocab, compact_vocab, dim)) { (void)hipStreamSynchronize(g_ctx.stream); return; }
    if (!d2h(rows.data(), rows_d, cb)) return;
    unpack_rows(full_gembed, rows, compact_to_full, compact_vocab, full_vocab, dim);
    host_written(full_gembed, (size_t)full_vocab * dim * sizeof(float));
}

// vocab_update_full (cpu_ops.h:145-148): full_embed[map[c]] = compact_embed[c].  The rows are written into the
// resident device copy of the table (which therefore stays current) and the host rows are filled from it.
MI355_API void mi355_vocab_update_full(float *full_embed, const float *compact_embed, const int *compact_to_full,
                                       int compact_vocab, int full_vocab, int dim) {
    if (!host_ready("vocab_update_full")) return;
    if (!full_embed || !compact_embed || !compact_to_full || compact_vocab <= 0 || full_vocab <= 0 || dim <= 0) {
        mi355_fail("vocab_update_full: bad arguments");
        return;
    }
    Table *tb = resident_table("vocab_update_full", full_embed, full_vocab, dim);
    if (!tb) return;
    const size_t cb = (size_t)compact_vocab * dim * sizeof(float), ib = (size_t)compact_vocab * sizeof(int32_t);
    float *c_d = (float *)slot(0, cb), *back_d = (float *)slot(2, cb);
    int32_t *i_d = (int32_t *)slot(1, ib);
    if (!c_d || !i_d || !back_d) return;
    bool ok = h2d(c_d, compact_embed, cb) && h2d(i_d, compact_to_full, ib);
    if (ok) ok = mi355_vocab_update_full_dev(tb->dev, c_d, i_d, compact_vocab, full_vocab, dim) == 0;
    if (ok) ok = mi355_vocab_compact_embed_dev(back_d, tb->dev, i_d, compact_vocab, full_vocab, dim) == 0;
    if (!ok) { (void)hipStreamSynchronize(g_ctx.stream); tb->dirty = true; return; }
    std::vector<float> rows((size_t)compact_vocab * dim);
    if (!d2h(rows.data(), back_d, cb)) { tb->dirty = true; return; }
    unpack_rows(full_embed, rows, compact_to_full, compact_vocab, full_vocab, dim);
}
