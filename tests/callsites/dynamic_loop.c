/*
 * Every CPU-op call of the reference's dynamic training loop, with the loop's own argument lists
 * (training/training_dynamic/train.m:300-306, 403-405, 417, 460-461, 487, 492, 497, 513, 523, 589-595, 659-660,
 * 714-728, 766, 839-871), compiled against include/mi355_cpu_ops.h in place of the loop's cpu_ops.h.
 * A translation unit that compiles with -Wall -Werror shows that the include swap needs no edit at the call sites;
 * the loop's inline vDSP calls map to the mi355_v* helpers named beside them.  Not run: ane_amd/host/train_step_mirror.c
 * is the program that runs the sequence.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* models/qwen3_06b.h:6-16 */
#define DIM 1024
#define HIDDEN 3072
#define HEADS 16
#define KV_HEADS 8
#define HD 128
#define SEQ 256
#define NLAYERS 28
#define VOCAB 151936
#define Q_DIM (HEADS * HD)
#define KV_DIM (KV_HEADS * HD)

#include "mi355_cpu_ops.h"

typedef struct { float *Wq, *rms_att, *rms_ffn; } LayerWeights;
typedef struct { AdamState Wq, rms_att, rms_ffn; } LayerAdam;
typedef struct { float *Wq, *rms_att, *rms_ffn; } LayerGrads;
typedef struct { float *layer_in, *x2, *x2norm, *h1, *h3; } LayerActs;

float run_step(const uint16_t *token_data, size_t n_tokens, float *embed, LayerWeights *lw, LayerAdam *la,
               LayerGrads *grads, LayerActs *acts, float *rms_final, AdamState arms_final, AdamState aembed,
               float *scratch) {
    float *x_cur = scratch, *xnorm_buf = scratch, *x_final = scratch, *logits = scratch, *dlogits = scratch;
    float *dy = scratch, *dffn = scratch, *dsilu = scratch, *dh1 = scratch, *dh3 = scratch, *dx_ffn = scratch;
    float *dx2 = scratch, *dx2_scaled = scratch, *dq = scratch, *dk_buf = scratch, *dx_attn = scratch;
    float *dx_rms1 = scratch, *dx_rms_final = scratch, *grms_final = scratch, *gembed = scratch, *o_out = scratch;
    const float res_alpha = 1.0f / sqrtf(2.0f * NLAYERS), loss_scale = 256.0f;
    const float lr = 3e-4f, adam_b1 = 0.9f, adam_b2 = 0.95f, adam_eps = 1e-8f, wd = 0.1f;
    const int adam_t = 1, L = 0;

    VocabMap vm = vocab_map_build(token_data, n_tokens, VOCAB);                                   /* :300 */
    int CV = vm.compact_vocab;
    float *cembed = vocab_compact_embed(embed, &vm, DIM);                                         /* :304 */
    float *gcembed = (float *)calloc((size_t)CV * DIM, 4);

    const uint16_t *input_tokens = token_data, *target_tokens_raw = token_data + 1;
    uint16_t ctargets[SEQ];
    for (int t = 0; t < SEQ; t++) ctargets[t] = (uint16_t)vm.full_to_compact[target_tokens_raw[t]];   /* :403 */

    embed_lookup(x_cur, embed, input_tokens, DIM, SEQ);                                           /* :405 */
    LayerActs *ac = &acts[L];
    LayerGrads *gr = &grads[L], *g = &grads[L];
    rmsnorm(xnorm_buf, x_cur, lw[L].rms_att, DIM, SEQ);                                           /* :417 */
    mi355_vsma(o_out, res_alpha, x_cur, ac->x2, (size_t)SEQ * DIM);                               /* :460 vDSP_vsma */
    rmsnorm(ac->x2norm, ac->x2, lw[L].rms_ffn, DIM, SEQ);                                         /* :461 */
    rmsnorm(x_final, x_cur, rms_final, DIM, SEQ);                                                 /* :487 */
    float loss = cross_entropy_loss(dlogits, logits, ctargets, CV, SEQ);                          /* :492 */
    mi355_vsmul(dlogits, loss_scale, dlogits, (size_t)SEQ * CV);                                  /* :497 vDSP_vsmul */
    rmsnorm_bwd(dx_rms_final, grms_final, dy, x_cur, rms_final, DIM, SEQ);                        /* :513 */
    mi355_vsmul(dy, res_alpha, dffn, (size_t)SEQ * DIM);                                          /* :523 */
    mi355_swiglu_bwd(dh1, dh3, dsilu, ac->h1, ac->h3, (size_t)HIDDEN * SEQ);                      /* :537-554 */
    rmsnorm_bwd(dx2, gr->rms_ffn, dx_ffn, ac->x2, lw[L].rms_ffn, DIM, SEQ);                       /* :589 */
    mi355_vadd(dx2, dy, dx2, (size_t)SEQ * DIM);                                                  /* :590 */
    mi355_vsmul(dx2, res_alpha, dx2_scaled, (size_t)SEQ * DIM);                                   /* :595 */
    rope_backward_inplace(dq, SEQ, Q_DIM, HD);                                                    /* :659 */
    rope_backward_inplace(dk_buf, SEQ, KV_DIM, HD);                                               /* :660 */
    rmsnorm_bwd(dx_rms1, gr->rms_att, dx_attn, ac->layer_in, lw[L].rms_att, DIM, SEQ);            /* :720 */
    mi355_vadd(dx_rms1, dx2, dy, (size_t)SEQ * DIM);                                              /* :721 */
    embed_backward(gembed, dy, input_tokens, DIM, SEQ);                                           /* :728 */

    vocab_scatter_grads(gembed, gcembed, &vm, DIM);                                               /* :766 */
    adam_update(lw[L].Wq, g->Wq, &la[L].Wq, adam_t, lr, adam_b1, adam_b2, adam_eps, wd);          /* :839 */
    adam_update(lw[L].rms_att, g->rms_att, &la[L].rms_att, adam_t, lr, adam_b1, adam_b2, adam_eps, 0.0f);   /* :846 */
    adam_update(lw[L].rms_ffn, g->rms_ffn, &la[L].rms_ffn, adam_t, lr, adam_b1, adam_b2, adam_eps, 0.0f);   /* :847 */
    adam_update(rms_final, grms_final, &arms_final, adam_t, lr, adam_b1, adam_b2, adam_eps, 0.0f);          /* :868 */
    adam_update(embed, gembed, &aembed, adam_t, lr, adam_b1, adam_b2, adam_eps, wd);              /* :869 */
    free(cembed);
    cembed = vocab_compact_embed(embed, &vm, DIM);                                                /* :871 */
    vocab_update_full(embed, cembed, &vm, DIM);                                                   /* cpu_ops.h:145 (no caller in the loop) */
    free(cembed); free(gcembed); free(vm.full_to_compact); free(vm.compact_to_full);
    return loss;
}

int main(void) { return 0; }
