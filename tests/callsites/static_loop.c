/*
 * Every CPU-op call of the reference's static training loops, with the loops' own argument lists
 * (training/train_large.m:405, 427, 442, 448, 458, 480, 519-521, 568, 597, 603, 638-652; the same calls in
 * training/train_large_ane.m:439, 500, 549, 596, 659, 671, 694-707), compiled against include/mi355_cpu_ops.h with
 * MI355_STATIC_PIPELINE (eight-argument adam_update, training/stories_cpu_ops.h:55) in place of stories_cpu_ops.h.
 * Compiled with -Wall -Werror, not run.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* training/stories_config.h:18-25 */
#define DIM 768
#define HIDDEN 2048
#define HEADS 12
#define SEQ 256
#define NLAYERS 12
#define VOCAB 32000

#define MI355_STATIC_PIPELINE
#include "mi355_cpu_ops.h"

typedef struct { float *Wq, *rms_att, *rms_ffn; } LayerWeights;
typedef struct { AdamState Wq, rms_att, rms_ffn; } LayerAdam;
typedef struct { float *Wq, *rms_att, *rms_ffn; } LayerGrads;
typedef struct { float *layer_in, *x2; } LayerActs;

float run_step(const uint16_t *input_tokens, const uint16_t *target_tokens, float *embed, LayerWeights *lw,
               LayerAdam *la, LayerGrads *grads, LayerActs *acts, float *rms_final, AdamState arms_final,
               AdamState aembed, float *scratch) {
    float *x_cur = scratch, *x_final = scratch, *logits = scratch, *dlogits = scratch, *dy = scratch, *o_out = scratch;
    float *x2 = scratch, *ffn_out = scratch, *dx_ffn = scratch, *dx2 = scratch, *dx_attn = scratch, *dx_rms1 = scratch;
    float *dx_rms_final = scratch, *grms_final = scratch, *gembed = scratch;
    const float lr = 3e-4f, adam_b1 = 0.9f, adam_b2 = 0.999f, adam_eps = 1e-8f;
    const int adam_t = 1, L = 0;
    LayerActs *ac = &acts[L];
    LayerGrads *gr = &grads[L], *g = &grads[L];

    embed_lookup(x_cur, embed, input_tokens, DIM, SEQ);                                           /* :405 */
    mi355_vadd(x_cur, o_out, x2, (size_t)SEQ * DIM);                                              /* :427 vDSP_vadd */
    mi355_vadd(x2, ffn_out, x_cur, (size_t)SEQ * DIM);                                            /* :442 */
    rmsnorm(x_final, x_cur, rms_final, DIM, SEQ);                                                 /* :448 */
    float loss = cross_entropy_loss(dlogits, logits, target_tokens, VOCAB, SEQ);                  /* :458 */
    rmsnorm_bwd(dx_rms_final, grms_final, dy, x_cur, rms_final, DIM, SEQ);                        /* :480 */
    rmsnorm_bwd(dx2, gr->rms_ffn, dx_ffn, ac->x2, lw[L].rms_ffn, DIM, SEQ);                       /* :519 */
    mi355_vadd(dx2, dy, dx2, (size_t)SEQ * DIM);                                                  /* :521 */
    rmsnorm_bwd(dx_rms1, gr->rms_att, dx_attn, ac->layer_in, lw[L].rms_att, DIM, SEQ);            /* :568 */
    mi355_vadd(dx_rms1, dx2, dy, (size_t)SEQ * DIM);                                              /* :597 */
    embed_backward(gembed, dy, input_tokens, DIM, SEQ);                                           /* :603 */
    adam_update(lw[L].Wq, g->Wq, &la[L].Wq, adam_t, lr, adam_b1, adam_b2, adam_eps);              /* :638 */
    adam_update(lw[L].rms_att, g->rms_att, &la[L].rms_att, adam_t, lr, adam_b1, adam_b2, adam_eps);   /* :645 */
    adam_update(lw[L].rms_ffn, g->rms_ffn, &la[L].rms_ffn, adam_t, lr, adam_b1, adam_b2, adam_eps);   /* :646 */
    adam_update(rms_final, grms_final, &arms_final, adam_t, lr, adam_b1, adam_b2, adam_eps);      /* :649 */
    adam_update(embed, gembed, &aembed, adam_t, lr, adam_b1, adam_b2, adam_eps);                  /* :652 */
    return loss;
}

int main(void) { return 0; }
