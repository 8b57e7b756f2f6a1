/*
 * mi355_cpu_ops.h — the reference's CPU-op names on top of the MI355X bridge.
 *
 * The training loops call their CPU ops by these names and signatures:
 *   rmsnorm, rmsnorm_bwd, cross_entropy_loss, embed_lookup, embed_backward
 *       (training/stories_cpu_ops.h:6,23,71,112,123; training/training_dynamic/cpu_ops.h:7,24,68,150,158)
 *   rope_backward_inplace (training/training_dynamic/cpu_ops.h:168)
 * Including this header INSTEAD of the reference's cpu-ops header gives the same names, argument
 * order and ownership rules (host float pointers in, host float pointers out, dx assigned,
 * dw and d_embed accumulated), with the work done on the GPU through mi355_bridge.h.
 *
 * The vocabulary size for the range checks comes from the VOCAB macro, as in the reference
 * (training/stories_cpu_ops.h:115); define it before including this header.
 *
 * C99; usable from C, C++ and Objective-C translation units.
 */
#ifndef MI355_CPU_OPS_H
#define MI355_CPU_OPS_H

#include "mi355_bridge.h"

#ifndef VOCAB
#error "define VOCAB (the vocabulary size of the model header) before including mi355_cpu_ops.h"
#endif

static inline void rmsnorm(float *out, const float *x, const float *w, int d, int S) {
    mi355_rmsnorm(out, x, w, d, S);
}

static inline void rmsnorm_bwd(float *dx, float *dw, const float *dy, const float *x, const float *w, int d, int S) {
    mi355_rmsnorm_bwd(dx, dw, dy, x, w, d, S);
}

static inline float cross_entropy_loss(float *dlogits, const float *logits, const uint16_t *targets, int V, int S) {
    return mi355_cross_entropy_loss(dlogits, logits, targets, V, S);
}

static inline void embed_lookup(float *x, const float *embed, const uint16_t *tokens, int dim, int seq) {
    mi355_embed_lookup(x, embed, tokens, VOCAB, dim, seq);
}

static inline void embed_backward(float *d_embed, const float *dx, const uint16_t *tokens, int dim, int seq) {
    mi355_embed_backward(d_embed, dx, tokens, VOCAB, dim, seq);
}

static inline void rope_backward_inplace(float *dx, int seq, int dim, int hd) {
    mi355_rope_backward_inplace(dx, seq, dim, hd);
}

/* adam_update — training/training_dynamic/cpu_ops.h:56-64 (the static loop's version,
 * training/stories_cpu_ops.h:55-63, is the same with wd = 0).  AdamState as in
 * training/training_dynamic/config.h:46; define MI355_HAVE_ADAMSTATE if the including file already has it. */
#ifndef MI355_HAVE_ADAMSTATE
typedef struct { float *m, *v; size_t n; } AdamState;
#endif
static inline void adam_update(float *w, const float *g, AdamState *s, int t, float lr, float b1, float b2, float eps,
                               float wd) {
    mi355_adam_update(w, g, s->m, s->v, s->n, t, lr, b1, b2, eps, wd);
}

/* The loops' inline Accelerate blocks, as calls with the same operand order:
 *   vDSP_vsma(b, 1, &alpha, a, 1, y, 1, n)   -> mi355_vsma(b, alpha, a, y, n)     train.m:460
 *   vDSP_vsmul(a, 1, &alpha, y, 1, n)        -> mi355_vsmul(a, alpha, y, n)       train.m:497,523,595
 *   vDSP_vadd(a, 1, b, 1, y, 1, n)           -> mi355_vadd(a, b, y, n)            train_large.m:427,442 */
static inline void mi355_vsma(const float *b, float alpha, const float *a, float *y, size_t n) {
    mi355_axpby(y, a, b, alpha, n, 0);
}
static inline void mi355_vsmul(const float *a, float alpha, float *y, size_t n) { mi355_axpby(y, a, NULL, alpha, n, 1); }
static inline void mi355_vadd(const float *a, const float *b, float *y, size_t n) { mi355_axpby(y, a, b, 0.0f, n, 2); }

#endif /* MI355_CPU_OPS_H */
