/*
 * train_step_mirror.c — the CPU-op sequence of the reference's dynamic training loop
 * (training/training_dynamic/train.m:300-306, 396-877), two consecutive steps, written in C against the reference's own
 * op names (include/mi355_cpu_ops.h), so every op runs on the GPU through the bridge.
 *
 * The stages the reference runs on the ANE (QKV/SDPA, Wo, FFN matmuls and their backward twins) are out of this
 * library's scope; they are replaced here by a fixed, cheap mixing function (`stage`) that only keeps data flowing
 * with the right shapes.  The classifier products (cblas_sgemm at train.m:490, :501, :507) are plain host loops with a
 * double accumulator.  Everything else is the reference's call order, operand order and accumulate-vs-assign rules,
 * including the vocabulary compaction (vocab_map_build, vocab_compact_embed, the target remap of :403,
 * vocab_scatter_grads) and the optimizer tail whose adam_update rewrites the embedding table that the next step's
 * embed_lookup reads.
 *
 * Model shape comes from compile-time macros, as the reference's models/*.h headers do.
 * Output (argv[1]): per step a binary dump (floats) of the loss, the embedded input x, the final dy, the scaled
 * RMSNorm weight gradients, the scaled embedding gradient, and the RMSNorm weights, the embedding table and the
 * re-compacted classifier table after the Adam step.
 *
 *   gcc -O2 -ffp-contract=off -Iinclude ane_amd/host/train_step_mirror.c -Lane_amd -lmi355_ops -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifndef DIM
#define DIM 64
#define HIDDEN 160
#define HEADS 4
#define KV_HEADS 2
#define HD 16
#define SEQ 32
#define NLAYERS 2
#define VOCAB 500
#endif
#define Q_DIM (HEADS * HD)
#define KV_DIM (KV_HEADS * HD)
#define NSTEPS 2
#define NTOKENS (4 * SEQ + 1)
#define CLS_GAIN 16.0f        /* keeps the stand-in classifier's softmax away from uniform */

#include "mi355_cpu_ops.h"

/* stand-in for an ANE stage: out[i] = 0.5*in[(7i+salt) % n_in] + 0.25*in[(13i+3salt) % n_in] */
static void stage(float *out, size_t n_out, const float *in, size_t n_in, unsigned salt) {
    for (size_t i = 0; i < n_out; i++) {
        float a = in[(i * 7u + salt) % n_in] * 0.5f;
        float b = 0.25f * in[(i * 13u + 3u * salt) % n_in];
        out[i] = a + b;
    }
}

/* C[M,N] (+)= gain * op(A)·op(B) with a double accumulator: the loop's cblas_sgemm calls, row-major */
static void host_gemm(int ta, int tb, int M, int N, int K, const float *A, int lda, const float *B, int ldb, float *Cm,
                      int ldc, int accumulate) {
    for (int i = 0; i < M; i++)
        for (int j = 0; j < N; j++) {
            double acc = 0.0;
            for (int k = 0; k < K; k++) {
                const float a = ta ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k];
                const float b = tb ? B[(size_t)j * ldb + k] : B[(size_t)k * ldb + j];
                acc += (double)a * (double)b;
            }
            const float v = (float)acc * CLS_GAIN;
            Cm[(size_t)i * ldc + j] = accumulate ? Cm[(size_t)i * ldc + j] + v : v;
        }
}

/* inputs: a small LCG so the Python replay can regenerate them */
static uint32_t g_lcg = 12345u;
static float frand(void) {
    g_lcg = g_lcg * 1664525u + 1013904223u;
    return (float)(g_lcg >> 8) * (1.0f / 16777216.0f) - 0.5f;   /* [-0.5, 0.5) */
}
static float *fmalloc(size_t n) { return (float *)calloc(n, sizeof(float)); }
static AdamState adam_alloc(size_t n) { AdamState s; s.m = fmalloc(n); s.v = fmalloc(n); s.n = n; return s; }

typedef struct {
    float *layer_in, *xnorm, *attn_out, *o_out, *x2, *x2norm, *h1, *h3, *silu_out;
} LayerActs;

int main(int argc, char **argv) {
    if (argc < 2) { fprintf(stderr, "usage: %s out.bin\n", argv[0]); return 2; }
    if (mi355_init() != 0) { fprintf(stderr, "no GPU: %s\n", mi355_last_error()); return 3; }
    const size_t DS = (size_t)DIM * SEQ, HS = (size_t)HIDDEN * SEQ, QS = (size_t)Q_DIM * SEQ, KS = (size_t)KV_DIM * SEQ;
    const size_t VD = (size_t)VOCAB * DIM;
    const float res_alpha = 1.0f / sqrtf(2.0f * NLAYERS);     /* train.m:188 */
    const float loss_scale = 256.0f;                          /* train.m:190 */

    /* weights and data */
    float *embed = fmalloc(VD), *gembed = fmalloc(VD);
    for (size_t i = 0; i < VD; i++) embed[i] = 0.04f * frand();
    float *rms_att[NLAYERS], *rms_ffn[NLAYERS], *g_rms_att[NLAYERS], *g_rms_ffn[NLAYERS];
    AdamState a_att[NLAYERS], a_ffn[NLAYERS];
    for (int L = 0; L < NLAYERS; L++) {
        rms_att[L] = fmalloc(DIM); rms_ffn[L] = fmalloc(DIM);
        g_rms_att[L] = fmalloc(DIM); g_rms_ffn[L] = fmalloc(DIM);
        a_att[L] = adam_alloc(DIM); a_ffn[L] = adam_alloc(DIM);
        for (int i = 0; i < DIM; i++) { rms_att[L][i] = 1.0f + 0.1f * frand(); rms_ffn[L][i] = 1.0f + 0.1f * frand(); }
    }
    float *rms_final = fmalloc(DIM), *grms_final = fmalloc(DIM);
    for (int i = 0; i < DIM; i++) rms_final[i] = 1.0f + 0.1f * frand();
    AdamState arms_final = adam_alloc(DIM), aembed = adam_alloc(VD);
    uint16_t token_data[NTOKENS];
    for (int t = 0; t < NTOKENS; t++) token_data[t] = (uint16_t)((7 * t + 13) % 256 + 1);   /* pattern of training/train.m:50-51 */
    token_data[5] = token_data[2];                            /* a duplicate id: embed_backward accumulates */

    /* vocabulary compaction (train.m:300-306) */
    VocabMap vm = vocab_map_build(token_data, NTOKENS, VOCAB);
    const int CV = vm.compact_vocab;
    if (CV <= 0) { fprintf(stderr, "vocab_map_build failed\n"); return 5; }
    float *cembed = vocab_compact_embed(embed, &vm, DIM);
    float *gcembed = fmalloc((size_t)CV * DIM);
    const size_t VS = (size_t)CV * SEQ;

    LayerActs acts[NLAYERS];
    for (int L = 0; L < NLAYERS; L++) {
        acts[L].layer_in = fmalloc(DS); acts[L].xnorm = fmalloc(DS); acts[L].attn_out = fmalloc(QS);
        acts[L].o_out = fmalloc(DS); acts[L].x2 = fmalloc(DS); acts[L].x2norm = fmalloc(DS);
        acts[L].h1 = fmalloc(HS); acts[L].h3 = fmalloc(HS); acts[L].silu_out = fmalloc(HS);
    }
    float *x_cur = fmalloc(DS), *x_final = fmalloc(DS), *ffn_out = fmalloc(DS);
    float *logits = fmalloc(VS), *dlogits = fmalloc(VS);
    float *dy = fmalloc(DS), *dffn = fmalloc(DS), *dsilu = fmalloc(HS), *dh1 = fmalloc(HS), *dh3 = fmalloc(HS);
    float *dh13 = fmalloc(2 * HS), *dx_ffn = fmalloc(DS), *dx2 = fmalloc(DS), *dx2_scaled = fmalloc(DS);
    float *da = fmalloc(QS), *dq = fmalloc(QS), *dk = fmalloc(KS), *dx_attn = fmalloc(DS), *dx_kv = fmalloc(DS);
    float *dx_rms = fmalloc(DS);

    FILE *f = fopen(argv[1], "wb");
    if (!f) { perror(argv[1]); return 4; }
    { float cvf = (float)CV; fwrite(&cvf, 4, 1, f); }

    for (int step = 0; step < NSTEPS; step++) {
        const uint16_t *input_tokens = token_data + 17 * step;                          /* train.m:398-400 */
        const uint16_t *target_tokens_raw = input_tokens + 1;
        uint16_t ctargets[SEQ];
        for (int t = 0; t < SEQ; t++) ctargets[t] = (uint16_t)vm.full_to_compact[target_tokens_raw[t]];   /* :403 */

        /* ===== forward (train.m:405-492) ===== */
        embed_lookup(x_cur, embed, input_tokens, DIM, SEQ);                                 /* :405 */
        fwrite(x_cur, 4, DS, f);
        for (int L = 0; L < NLAYERS; L++) {
            LayerActs *ac = &acts[L];
            memcpy(ac->layer_in, x_cur, DS * 4);
            rmsnorm(ac->xnorm, x_cur, rms_att[L], DIM, SEQ);                                /* :417 */
            stage(ac->attn_out, QS, ac->xnorm, DS, 1u + L);                                 /* sdpaFwd (ANE) */
            stage(ac->o_out, DS, ac->attn_out, QS, 2u + L);                                 /* woFwd (ANE) */
            mi355_vsma(ac->o_out, res_alpha, x_cur, ac->x2, DS);                            /* :460 */
            rmsnorm(ac->x2norm, ac->x2, rms_ffn[L], DIM, SEQ);                              /* :461 */
            stage(ac->h1, HS, ac->x2norm, DS, 3u + L);                                      /* ffnFused (ANE): W1, W3 */
            stage(ac->h3, HS, ac->x2norm, DS, 4u + L);
            mi355_swiglu_fwd(ac->silu_out, ac->h1, ac->h3, HS);                             /* SiLU gate (mil_dynamic.h:264-266) */
            stage(ffn_out, DS, ac->silu_out, HS, 5u + L);                                   /* W2 */
            mi355_vsma(ffn_out, res_alpha, ac->x2, x_cur, DS);                              /* mil_dynamic.h:279-283 */
        }
        rmsnorm(x_final, x_cur, rms_final, DIM, SEQ);                                       /* :487 */
        host_gemm(0, 0, CV, SEQ, DIM, cembed, DIM, x_final, SEQ, logits, SEQ, 0);           /* :490 */
        float loss = cross_entropy_loss(dlogits, logits, ctargets, CV, SEQ);                /* :492 */

        /* ===== backward (train.m:497-728) ===== */
        mi355_vsmul(dlogits, loss_scale, dlogits, VS);                                      /* :497 */
        host_gemm(1, 0, DIM, SEQ, CV, cembed, DIM, dlogits, SEQ, dy, SEQ, 0);               /* :501 */
        host_gemm(0, 1, CV, DIM, SEQ, dlogits, SEQ, x_final, SEQ, gcembed, DIM, 1);         /* :507 */
        rmsnorm_bwd(dx_rms, grms_final, dy, x_cur, rms_final, DIM, SEQ);                    /* :513 */
        memcpy(dy, dx_rms, DS * 4);
        for (int L = NLAYERS - 1; L >= 0; L--) {
            LayerActs *ac = &acts[L];
            mi355_vsmul(dy, res_alpha, dffn, DS);                                           /* :523 */
            stage(dsilu, HS, dffn, DS, 8u + L);                                             /* ffnBwdW2t (ANE) */
            mi355_swiglu_bwd(dh1, dh3, dsilu, ac->h1, ac->h3, HS);                          /* :537-554 */
            memcpy(dh13, dh1, HS * 4); memcpy(dh13 + HS, dh3, HS * 4);
            stage(dx_ffn, DS, dh13, 2 * HS, 9u + L);                                        /* ffnBwdW13t (ANE) */
            memset(dx2, 0, DS * 4);
            rmsnorm_bwd(dx2, g_rms_ffn[L], dx_ffn, ac->x2, rms_ffn[L], DIM, SEQ);           /* :589 */
            mi355_vadd(dx2, dy, dx2, DS);                                                   /* :590 */
            mi355_vsmul(dx2, res_alpha, dx2_scaled, DS);                                    /* :595 */
            stage(da, QS, dx2_scaled, DS, 10u + L);                                         /* wotBwd (ANE) */
            stage(dq, QS, da, QS, 11u + L);                                                 /* sdpaBwd1/2 (ANE) */
            stage(dk, KS, da, QS, 12u + L);
            rope_backward_inplace(dq, SEQ, Q_DIM, HD);                                      /* :659 */
            rope_backward_inplace(dk, SEQ, KV_DIM, HD);                                     /* :660 */
            stage(dx_attn, DS, dq, QS, 13u + L);                                            /* qBwd (ANE) */
            stage(dx_kv, DS, dk, KS, 14u + L);                                              /* kvBwd (ANE) */
            mi355_vadd(dx_attn, dx_kv, dx_attn, DS);                                        /* :714 */
            rmsnorm_bwd(dx_rms, g_rms_att[L], dx_attn, ac->layer_in, rms_att[L], DIM, SEQ); /* :720 */
            mi355_vadd(dx_rms, dx2, dy, DS);                                                /* :721 */
        }
        embed_backward(gembed, dy, input_tokens, DIM, SEQ);                                 /* :728 */

        /* ===== optimizer tail (train.m:748-877), accum_steps = 1 ===== */
        const float gsc = 1.0f / loss_scale;                                                /* :750 */
        const float lr = 3e-4f, b1 = 0.9f, b2 = 0.95f, eps = 1e-8f, wd = 0.1f;
        const int adam_t = step + 1;
        for (int L = 0; L < NLAYERS; L++)
            for (int i = 0; i < DIM; i++) { g_rms_att[L][i] *= gsc; g_rms_ffn[L][i] *= gsc; }     /* :763 */
        for (int i = 0; i < DIM; i++) grms_final[i] *= gsc;                                       /* :765 */
        vocab_scatter_grads(gembed, gcembed, &vm, DIM);                                           /* :766 */
        for (size_t i = 0; i < VD; i++) gembed[i] *= gsc;                                         /* :767 */

        fwrite(&loss, 4, 1, f);
        fwrite(dy, 4, DS, f);
        fwrite(grms_final, 4, DIM, f);
        for (int L = 0; L < NLAYERS; L++) { fwrite(g_rms_att[L], 4, DIM, f); fwrite(g_rms_ffn[L], 4, DIM, f); }
        fwrite(gembed, 4, VD, f);

        for (int L = 0; L < NLAYERS; L++) {
            adam_update(rms_att[L], g_rms_att[L], &a_att[L], adam_t, lr, b1, b2, eps, 0.0f);      /* :846 */
            adam_update(rms_ffn[L], g_rms_ffn[L], &a_ffn[L], adam_t, lr, b1, b2, eps, 0.0f);      /* :847 */
        }
        adam_update(rms_final, grms_final, &arms_final, adam_t, lr, b1, b2, eps, 0.0f);           /* :868 */
        adam_update(embed, gembed, &aembed, adam_t, lr, b1, b2, eps, wd);                         /* :869 */
        free(cembed);
        cembed = vocab_compact_embed(embed, &vm, DIM);                                            /* :871 */
        for (int L = 0; L < NLAYERS; L++) { memset(g_rms_att[L], 0, DIM * 4); memset(g_rms_ffn[L], 0, DIM * 4); }   /* :874 */
        memset(grms_final, 0, DIM * 4);                                                           /* :875 */
        memset(gembed, 0, VD * 4);                                                                /* :876 */
        memset(gcembed, 0, (size_t)CV * DIM * 4);                                                 /* :877 */

        /* weights after the Adam step */
        fwrite(rms_final, 4, DIM, f);
        for (int L = 0; L < NLAYERS; L++) { fwrite(rms_att[L], 4, DIM, f); fwrite(rms_ffn[L], 4, DIM, f); }
        fwrite(embed, 4, VD, f);
        fwrite(cembed, 4, (size_t)CV * DIM, f);
        printf("step %d loss=%.6f\n", step, loss);
    }
    fclose(f);
    mi355_shutdown();
    return 0;
}
