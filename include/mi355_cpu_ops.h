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
 * The two pipelines declare adam_update differently: the dynamic loop's takes a weight decay
 * (training/training_dynamic/cpu_ops.h:56, nine arguments), the static loops' does not
 * (training/stories_cpu_ops.h:55, eight arguments: train_large.m:638-652, train_large_ane.m:694-707).
 * Define MI355_STATIC_PIPELINE before including this header to get the eight-argument form.
 *
 * C99; usable from C, C++ and Objective-C translation units.
 */
#ifndef MI355_CPU_OPS_H
#define MI355_CPU_OPS_H

#include <stdlib.h>
#include <string.h>

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

/* adam_update — training/training_dynamic/cpu_ops.h:56-64 (AdamW), or with MI355_STATIC_PIPELINE
 * training/stories_cpu_ops.h:55-63 (no weight decay).  AdamState as in training/training_dynamic/config.h:46 and
 * training/stories_config.h:57-59; define MI355_HAVE_ADAMSTATE if the including file already has it. */
#ifndef MI355_HAVE_ADAMSTATE
typedef struct { float *m, *v; size_t n; } AdamState;
#endif
#ifdef MI355_STATIC_PIPELINE
static inline void adam_update(float *w, const float *g, AdamState *s, int t, float lr, float b1, float b2, float eps) {
    mi355_adam_update(w, g, s->m, s->v, s->n, t, lr, b1, b2, eps, 0.0f);
}
#else
static inline void adam_update(float *w, const float *g, AdamState *s, int t, float lr, float b1, float b2, float eps,
                               float wd) {
    mi355_adam_update(w, g, s->m, s->v, s->n, t, lr, b1, b2, eps, wd);
}
#endif

/* Vocabulary compaction — training/training_dynamic/cpu_ops.h:96-148, called at
 * training/training_dynamic/train.m:300 (vocab_map_build), :304 and :871 (vocab_compact_embed), :766
 * (vocab_scatter_grads).  Same struct, same ownership: the maps and the compact table are malloc'd here and
 * freed by the caller.  The size of the full table, which the reference's vocab_compact_embed does not
 * take, comes from VOCAB.  Tokens >= full_vocab in the data, which the reference's scan would write out of
 * bounds for, are ignored.  If the GPU cannot be used compact_vocab is 0. */
typedef struct {
    int compact_vocab;          /* number of tokens that occur */
    int *full_to_compact;       /* [full_vocab] -> compact id, -1 if unused */
    int *compact_to_full;       /* [compact_vocab] -> id in the full vocabulary */
} VocabMap;

static inline VocabMap vocab_map_build(const uint16_t *data, size_t n_tokens, int full_vocab) {
    VocabMap vm;
    vm.full_to_compact = (int *)malloc((size_t)full_vocab * sizeof(int));
    vm.compact_to_full = (int *)malloc((size_t)full_vocab * sizeof(int));
    memset(vm.full_to_compact, -1, (size_t)full_vocab * sizeof(int));
    vm.compact_vocab = mi355_vocab_map_build(vm.full_to_compact, vm.compact_to_full, data, n_tokens, full_vocab);
    if (vm.compact_vocab < 0) vm.compact_vocab = 0;
    return vm;
}

static inline float *vocab_compact_embed(const float *full_embed, const VocabMap *vm, int dim) {
    float *ce = (float *)calloc((size_t)vm->compact_vocab * dim + 1, sizeof(float));
    mi355_vocab_compact_embed(ce, full_embed, vm->compact_to_full, vm->compact_vocab, VOCAB, dim);
    return ce;
}

static inline void vocab_scatter_grads(float *full_gembed, const float *compact_gembed, const VocabMap *vm, int dim) {
    mi355_vocab_scatter_grads(full_gembed, compact_gembed, vm->compact_to_full, vm->compact_vocab, VOCAB, dim);
}

static inline void vocab_update_full(float *full_embed, const float *compact_embed, const VocabMap *vm, int dim) {
    mi355_vocab_update_full(full_embed, compact_embed, vm->compact_to_full, vm->compact_vocab, VOCAB, dim);
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
