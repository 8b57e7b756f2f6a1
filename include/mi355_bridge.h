/*
 * mi355_bridge.h — C-callable bridge to the MI355X (gfx950) implementations of the per-layer
 * CPU ops of the maderix/ANE training loops.
 *
 * Pure C, includable from C, C++ and Objective-C.  The interface style follows the reference's
 * own C-ABI, bridge/ane_bridge.h:11-98: an idempotent `int ..._init(void)` returning 0 / -1,
 * opaque handles that are NULL on failure, NULL-safe `..._free`, `write`/`read` calls that
 * silently ignore bad arguments, and one "mi355_bridge: ..." line on stderr per failure.
 *
 * All tensors are fp32 in the reference's channel-first layout x[c*S + s]
 * (training/stories_cpu_ops.h:110-118).  "batch B" means B consecutive [C,S] slabs — the
 * reference processes one sequence per call, so batch B equals B reference calls in slab order.
 *
 * Threading: one process-global context and one HIP stream; entry points are not re-entrant
 * (the reference's ops share a global scratch buffer the same way,
 * training/training_dynamic/cpu_ops.h:5).  Device-resident calls (`*_dev`) are asynchronous on
 * the bridge stream until mi355_sync() / mi355_buf_read(); host-pointer drop-ins are synchronous.
 *
 * Device-resident calls return 0 on success and -1 on failure (bad shape, NULL pointer, no
 * device); on failure no kernel is launched and the outputs are untouched.
 */
#ifndef MI355_BRIDGE_H
#define MI355_BRIDGE_H

#include <stddef.h>
#include <stdint.h>
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Lifecycle.  Replaces ane_bridge_init (bridge/ane_bridge.h:20, bridge/ane_bridge.m:33-57).
 * ---------------------------------------------------------------------------------------- */

/* Select device 0, create the context.  Idempotent.  0 on success, -1 if no usable GPU. */
int mi355_init(void);
/* Release every cached device allocation and the context.  Safe to call twice. */
void mi355_shutdown(void);
/* Text of the most recent failure ("" if none).  Static storage, never NULL. */
const char *mi355_last_error(void);
/* Device name, its peak HBM bandwidth in GB/s as reported by the driver (memory clock x bus
 * width; 0 when not reported), and the number of compute units.  Any pointer may be NULL. */
int mi355_device_info(char *name, size_t name_len, double *peak_hbm_gbs, int *compute_units);
/* Run every later device-resident call on the given hipStream_t (NULL = the default stream). */
int mi355_set_stream(void *hip_stream);
/* Wait for everything queued on the bridge stream.  0 / -1. */
int mi355_sync(void);
/* Grow the internal workspace (sort buffers, reduction partials) to at least `bytes` now, so
 * that later calls of up to that need allocate nothing. */
int mi355_workspace_reserve(size_t bytes);
/* Present size of that workspace: run a step once, read this, reserve as much at the next start. */
size_t mi355_workspace_size(void);
/* Tuning knobs for experiments; 0 = choose per shape (the default), unknown names return -1:
 * "rms_lpr" (lanes per strip row, 4/8/16) and "rms_threads" (256/512/1024) of the RMSNorm tiles, "qk_lpr" and
 * "qk_threads" (256/512) of the QK-norm + RoPE tiles, "ew_unroll" (accesses per lane of the streaming ops, 1/2/4),
 * "ce_rows" / "ce_rows2" (rows of logits per workgroup in the first / second pass of softmax-CE),
 * "gemm_splitk" (K slices of mi355_sgemm_dev; 1 = never split),
 * "scatter_tree" (1: mi355_embed_scatter_add_dev sums long segments by a fixed tree instead of the reference's
 * sequential order: still deterministic and within 1e-5 of each row's scale, faster, no longer bit-identical to
 * the CPU loop), "scatter_cols" (the form of mi355_embed_scatter_add_dev in which every workgroup owns a few columns
 * of the gradient table and reads its rows of dx in place: 1 = for any number of positions, -1 = never),
 * "buf_phase" (where mi355_buf_alloc starts buffers of 1 MiB and more within a 1 KiB group:
 * 0 = a multiple of 128 bytes that rotates from one allocation to the next, 1..8 = always (value-1)*128),
 * "rms_cluster" (channel split of the RMSNorm over cooperating workgroups: -1 = never, and mi355_int8_scale_dev and
 * mi355_int8_quantize_dynamic_dev then run as two launches each; 2/4/8 = forced),
 * "ce_resident" (one-launch softmax-CE: 1 = for any V, -1 = never), "rms_cluster_spin" (how long a workgroup of those
 * kernels and of mi355_int8_scale_dev waits for a partner's partial result before it computes it itself, in ticks
 * of 10 ns: 0 = 2 ms; -1 = do not wait), "xch_take_nothing" (1: those kernels take no partner's value at
 * all, present or not, so every workgroup goes the way of an expired wait).  The last two settings are for tests: the
 * results are the same to the bit. */
int mi355_tune_set(const char *key, int value);

/* How often, since the library was loaded, a workgroup of a kernel whose workgroups hand partial results to one
 * another inside one launch gave up its bounded wait for a partner and computed the partner's part itself:
 * *shared_area counts the clustered RMSNorm family and mi355_int8_scale_dev, *softmax_ce the one-launch
 * softmax-CE (either pointer may be NULL).  No counterpart in the reference, whose ops are single loops
 * (training/stories_cpu_ops.h:6-53, bridge/ane_bridge.m:346-353).  The results are identical to the bit whichever way
 * a value was obtained, so these counts are the only sign that the cooperating workgroups do not run together (a GPU
 * shared with other work): every expiry costs the wait ("rms_cluster_spin") plus the recomputation.  A caller that
 * sees them grow can switch the cooperating forms off with mi355_tune_set("rms_cluster", -1) and ("ce_resident", -1);
 * mi355_sync() does so by itself (one stderr line) when the counts have grown at three of its calls in a row with no
 * knob changed in between, and setting the two knobs back to 0 switches the forms on again.
 * Waits for the stream and copies two words to the host: not possible during a graph capture.  0 / -1. */
int mi355_exchange_stats(long long *shared_area, long long *softmax_ce);

/* ------------------------------------------------------------------------------------------
 * Device buffers (opaque).  Replace the IOSurface-backed tensors behind
 * ane_bridge_write_input / ane_bridge_read_output / ane_bridge_free
 * (bridge/ane_bridge.h:54-62, bridge/ane_bridge.m:233-251).
 * ---------------------------------------------------------------------------------------- */
typedef struct mi355_buf mi355_buf;

/* The device address is 128-byte aligned (see "buf_phase" above: buffers that one op reads together should not
 * all start at the same offset within 1 KiB, and by default they do not). */
mi355_buf *mi355_buf_alloc(size_t bytes);                 /* NULL on failure; contents zeroed */
void mi355_buf_free(mi355_buf *b);                        /* NULL-safe */
void *mi355_buf_devptr(mi355_buf *b);                     /* raw device address (NULL if b NULL) */
size_t mi355_buf_bytes(mi355_buf *b);
/* Synchronous copies; out-of-range or NULL arguments are ignored, as in the reference. */
void mi355_buf_write(mi355_buf *b, size_t offset, const void *src, size_t bytes);
void mi355_buf_read(mi355_buf *b, size_t offset, void *dst, size_t bytes);
int mi355_buf_zero(mi355_buf *b);                         /* asynchronous fill on the bridge stream */

/* Optional bfloat16-storage variants (no counterpart in the reference, whose CPU ops are fp32): the same
 * arithmetic in fp32 registers, activations in device memory as bfloat16 bit patterns (uint16_t, the upper half
 * of the fp32 pattern), results rounded to nearest even on store; norm weights and weight gradients stay fp32.
 * They agree with the fp32 entry points run on the same bf16-representable inputs to within 5e-3.
 * Arguments as the fp32 entry points of the same name. */
int mi355_cvt_f32_bf16_dev(uint16_t *dst, size_t dst_ld, const float *src, size_t src_ld, size_t rows, size_t cols);
int mi355_cvt_bf16_f32_dev(float *dst, size_t dst_ld, const uint16_t *src, size_t src_ld, size_t rows, size_t cols);
int mi355_rmsnorm_fwd_bf16_dev(uint16_t *y, const uint16_t *x, const float *w, int C, int S, int batch, float eps);
int mi355_rmsnorm_bwd_bf16_dev(uint16_t *dx, float *dw, const uint16_t *dy, const uint16_t *x, const float *w, int C,
                               int S, int batch, float eps, int variant);
/* bf16-storage twins of mi355_residual_rmsnorm_fwd_dev and mi355_rmsnorm_bwd_residual_dev (the residual add and the
 * RMSNorm after it, training/training_dynamic/train.m:460-461; the RMSNorm backward with the backward residual and the
 * scaled copy, train.m:586-595, :714-721).  y, dx and dx_scaled are each rounded once, from fp32 values; yn is the norm
 * of the rounded y.  Aliasing as for the fp32 entry points. */
int mi355_residual_rmsnorm_fwd_bf16_dev(uint16_t *y, uint16_t *yn, const uint16_t *a, const uint16_t *b, float alpha,
                                        const float *w, int C, int S, int batch, float eps);
int mi355_rmsnorm_bwd_residual_bf16_dev(uint16_t *dx, uint16_t *dx_scaled, float *dw, const uint16_t *dy,
                                        const uint16_t *x, const float *w, const uint16_t *res, float alpha, int C,
                                        int S, int batch, float eps, int variant);
int mi355_swiglu_fwd_bf16_dev(uint16_t *out, const uint16_t *h1, const uint16_t *h3, size_t n);
int mi355_swiglu_bwd_bf16_dev(uint16_t *dh1, uint16_t *dh3, const uint16_t *dsilu, const uint16_t *h1,
                              const uint16_t *h3, size_t n);
int mi355_axpby_bf16_dev(uint16_t *y, const uint16_t *a, const uint16_t *b, float alpha, size_t n, int mode);
int mi355_softmax_ce_bf16_dev(uint16_t *dlogits, float *loss_dev, const uint16_t *logits, const int32_t *targets,
                              int V, int S, float grad_scale);
int mi355_rope_bf16_dev(uint16_t *q_out, uint16_t *k_out, const uint16_t *q_in, const uint16_t *k_in, int heads,
                        int kv_heads, int hd, int S, int batch, const float *cos_dev, const float *sin_dev, int dir);
/* The head size must fit the register tile: hd <= 1024 with rows of a multiple of 8 columns and 16-byte aligned
 * pointers, hd <= 128 otherwise (the fp32 entry points have no such limit). */
int mi355_qknorm_rope_fwd_bf16_dev(uint16_t *q_out, uint16_t *k_out, const uint16_t *q, const uint16_t *k,
                                   const float *wq, const float *wk, int heads, int kv_heads, int hd, int S, int batch,
                                   const float *cos_dev, const float *sin_dev, float eps);
int mi355_qknorm_rope_bwd_bf16_dev(uint16_t *dq, uint16_t *dk, float *dwq, float *dwk, const uint16_t *dq_out,
                                   const uint16_t *dk_out, const uint16_t *q, const uint16_t *k, const float *wq,
                                   const float *wk, int heads, int kv_heads, int hd, int S, int batch,
                                   const float *cos_dev, const float *sin_dev, float eps, int variant);

/* Graphs: record a launch-bound sequence of device-resident ops once, replay it as one submission.  No
 * counterpart in the reference (its ops are synchronous CPU calls).  Between begin and end the *_dev ops are
 * recorded instead of run; calls that allocate, wait or touch the host (buf_alloc/free/read/write, sync,
 * set_stream, workspace growth, a first-time RoPE table, the first clustered RMSNorm or INT8 scale of the process
 * (their exchange area is allocated then), embed_scatter_add beyond 16384 positions, sgemm, ckpt_*, the
 * host-pointer drop-ins) fail with -1 and end in a failed capture, so run the sequence once eagerly first.  mi355_graph_launch
 * enqueues the replay on the bridge stream; it fails if a workspace was reallocated since the recording (record
 * again).  Accumulating ops (dw +=) accumulate on every replay. */
typedef struct mi355_graph mi355_graph;
int mi355_graph_begin(void);
mi355_graph *mi355_graph_end(void);          /* NULL on failure */
int mi355_graph_launch(mi355_graph *g);
void mi355_graph_free(mi355_graph *g);       /* NULL-safe */

/* Timing on the bridge stream (HIP events). */
typedef struct mi355_event mi355_event;
mi355_event *mi355_event_create(void);
void mi355_event_destroy(mi355_event *e);
int mi355_event_record(mi355_event *e);
/* Waits for `stop`, returns milliseconds between the two records (-1 on failure). */
float mi355_event_elapsed_ms(mi355_event *start, mi355_event *stop);

/* Synthetic data, generated on the device (counter-based splitmix64 + Box-Muller). */
int mi355_fill_normal_dev(float *p, size_t n, uint64_t seed, float mean, float std);
int mi355_fill_randint_dev(int32_t *p, size_t n, uint64_t seed, int32_t lo, int32_t hi /*excl.*/);

/* ------------------------------------------------------------------------------------------
 * Device-resident ops (the measured path).  Every pointer is a device address.
 * ---------------------------------------------------------------------------------------- */

/* RMSNorm forward.  Replaces rmsnorm — training/stories_cpu_ops.h:6-21,
 * training/training_dynamic/cpu_ops.h:7-22.  y = (x * rsqrt(mean_c x^2 + eps)) * w[c].
 * x, y: [batch][C][S]; w: [C].  The reference hard-codes eps = 1e-5f. */
int mi355_rmsnorm_fwd_dev(float *y, const float *x, const float *w, int C, int S, int batch,
                          float eps);

/* RMSNorm backward.  Replaces rmsnorm_bwd — training/stories_cpu_ops.h:23-53,
 * training/training_dynamic/cpu_ops.h:24-54.  dx is assigned, dw[C] is accumulated (+=).
 * variant 0 = the reference CPU op: dx = ((dy - x*dot)*rr)*w;
 * variant 1 = the textbook gradient (training/backward.h:28-42, training/ane_rmsnorm_bwd.h:56-74):
 * dx = (dy*w)*rr - (x*dot)*rr.  Both use dot = rr^2/C * sum_c dy*x*w.  dx may alias dy; it must not alias x. */
int mi355_rmsnorm_bwd_dev(float *dx, float *dw, const float *dy, const float *x, const float *w,
                          int C, int S, int batch, float eps, int variant);

/* Introspection, host-only (needs no GPU): the register tile that the RMSNorm entry points choose for a shape —
 * op 0 = mi355_rmsnorm_fwd_dev, 1 = mi355_rmsnorm_bwd_dev, 2 = mi355_rmsnorm_bwd_residual_dev; aligned != 0 means
 * 16-byte aligned tensors.  tile5 (may be NULL) receives {columns per lane, lanes per row piece, threads per
 * workgroup, rows per lane held in registers (0 = rows are read twice), workgroups that share the rows of one strip
 * (0 = one workgroup owns all C rows; 2, 4 or 8 = the clustered kernels, which out-of-place calls of tall shapes
 * run)}.  0, or -1 if no kernel exists for the choice (a defect: the entry point would fail the same way). */
int mi355_rmsnorm_tile(int op, int C, int S, int batch, int aligned, int *tile5);

/* Weight-gradient accumulation mode.  By default dw / dwq / dwk are up to date (in stream order) when
 * the backward call that adds into them returns.  The loops read these gradients only at the optimizer
 * step, after the whole backward pass (training/training_dynamic/train.m:748-869); with
 * mi355_dw_defer(1) the library uses that: each backward op queues its reduction and
 * mi355_dw_flush() runs everything queued in a few launches.  mi355_sync(), mi355_buf_read(),
 * mi355_set_stream() and mi355_dw_defer(0) flush too.  Results are bit-identical in both modes.
 * Gradient pointers passed while deferred must be distinct or identical, not partially overlapping. */
int mi355_dw_defer(int on);
int mi355_dw_flush(void);

/* RMSNorm backward with the residual of the backward pass riding along, one launch:
 *   dx = rmsnorm_bwd(dy, x, w) + res;  dx_scaled = alpha * dx  (dx_scaled may be NULL);  dw += as rmsnorm_bwd.
 * Replaces memset + rmsnorm_bwd + the add loop + vDSP_vsmul — training/training_dynamic/train.m:586-595 — and
 * rmsnorm_bwd + the add loop of train.m:714-721.  The adds and the scale are the separate passes' own, in their
 * order: the result equals mi355_rmsnorm_bwd_dev followed by mi355_axpby_dev (modes 2 and 1) bit for bit when
 * both run on the same tile shape (they do below 32 x 256 columns), and to the rounding of the column sums
 * otherwise.  dx may alias res or dy; it must not alias x. */
int mi355_rmsnorm_bwd_residual_dev(float *dx, float *dx_scaled, float *dw, const float *dy, const float *x,
                                   const float *w, const float *res, float alpha, int C, int S, int batch, float eps,
                                   int variant);

/* Residual add fused with the RMSNorm that follows it in the loops: vDSP_vsma + rmsnorm at
 * training/training_dynamic/train.m:460-461 (and a layer's x_next feeding the next rmsnorm at :417).
 * y = a + alpha*b (as mode 0 of mi355_axpby_dev); yn = rmsnorm(y, w).  One launch instead of two; y is bit-identical
 * to the separate call, yn too when y aliases neither input (in place another tile shape is used, and yn then
 * agrees to the rounding of the column sums).  y may alias a or b; yn must not alias anything. */
int mi355_residual_rmsnorm_fwd_dev(float *y, float *yn, const float *a, const float *b, float alpha,
                                   const float *w, int C, int S, int batch, float eps);

/* SwiGLU gate forward: out = (h1*sigmoid(h1))*h3.  Replaces the MIL sigmoid/mul/mul of
 * training/training_dynamic/mil_dynamic.h:264-266 and training/forward.h:101,149-151. */
int mi355_swiglu_fwd_dev(float *out, const float *h1, const float *h3, size_t n);

/* SwiGLU gate backward.  Replaces the 13 vDSP/vForce calls of
 * training/training_dynamic/train.m:537-554: dh3 = dsilu*(h1*sig), dh1 = (dsilu*h3)*(sig*(1+h1*(1-sig))). */
int mi355_swiglu_bwd_dev(float *dh1, float *dh3, const float *dsilu, const float *h1,
                         const float *h3, size_t n);

/* cos/sin tables [hd/2][S] (pair-major, positions contiguous), built on the host with libm from
 * angle = p * (1/powf(theta, 2i/hd)) — the expression of training/training_dynamic/cpu_ops.h:172-175
 * (theta is 10000 there).  Host pointers. */
int mi355_rope_tables(float *cos_host, float *sin_host, int S, int hd, float theta);
/* The same tables resident on the device, cached per (S, hd, theta).  The pointers stay valid until mi355_shutdown; the
 * cache holds up to 1024 tables and 256 MiB and the call fails beyond that. */
int mi355_rope_tables_dev(const float **cos_dev, const float **sin_dev, int S, int hd, float theta);

/* RoPE on Q [batch][heads*hd][S] and K [batch][kv_heads*hd][S], interleaved row pairs (2i,2i+1).
 * dir = -1 replaces rope_backward_inplace — training/training_dynamic/cpu_ops.h:168-184, called at
 * training/training_dynamic/train.m:659-660 for dQ (Q_DIM) and dK (KV_DIM); dir = +1 is the forward
 * rotation (training/forward.h:55-70; training/training_dynamic/mil_dynamic.h:131-168).
 * In place when q_out == q_in / k_out == k_in.  k_* may be NULL (kv_heads = 0). */
int mi355_rope_dev(float *q_out, float *k_out, const float *q_in, const float *k_in, int heads,
                   int kv_heads, int hd, int S, int batch, const float *cos_dev,
                   const float *sin_dev, int dir);

/* Qwen3 per-head QK-RMSNorm fused with RoPE (one HBM pass).  Not in the reference: equals rmsnorm
 * (stories_cpu_ops.h:6-21) applied to each head's [hd,S] slab with a [hd] weight shared by the
 * heads, followed by the forward RoPE above. */
int mi355_qknorm_rope_fwd_dev(float *q_out, float *k_out, const float *q, const float *k,
                              const float *wq, const float *wk, int heads, int kv_heads, int hd,
                              int S, int batch, const float *cos_dev, const float *sin_dev,
                              float eps);
/* Backward of the above: inverse rotation (cpu_ops.h:168-184) then rmsnorm_bwd per head
 * (stories_cpu_ops.h:23-53).  dq/dk assigned; dwq/dwk [hd] accumulated over heads and batch.
 * q, k are the saved pre-norm inputs. */
int mi355_qknorm_rope_bwd_dev(float *dq, float *dk, float *dwq, float *dwk, const float *dq_out,
                              const float *dk_out, const float *q, const float *k, const float *wq,
                              const float *wk, int heads, int kv_heads, int hd, int S, int batch,
                              const float *cos_dev, const float *sin_dev, float eps, int variant);

/* Residual family.  mode 0: y = a + alpha*b (vDSP_vsma, training/training_dynamic/train.m:460);
 * mode 1: y = alpha*a (vDSP_vsmul, train.m:497,523,595); mode 2: y = a + b (vDSP_vadd,
 * training/train_large.m:427,442; loops at train.m:590,714,721).  y may alias a or b. */
int mi355_axpby_dev(float *y, const float *a, const float *b, float alpha, size_t n, int mode);

/* Embedding gather.  Replaces embed_lookup — training/stories_cpu_ops.h:112-120,
 * training/training_dynamic/cpu_ops.h:150-156.  x[b][d][t] = E[ids[b][t]][d]; an id outside
 * [0,V) leaves its column untouched (the static loop's policy).  Bit-exact copy. */
int mi355_embed_gather_dev(float *x, const float *E, const int32_t *ids, int V, int D, int S,
                           int batch);

/* Embedding backward.  Replaces embed_backward — training/stories_cpu_ops.h:123-131,
 * training/training_dynamic/cpu_ops.h:158-164.  dE[ids[b][t]][d] += dx[b][d][t], each (row, d) sum
 * taken in ascending (b, t) order starting from the value already in dE, so the result is
 * bit-identical to the reference loop and run-to-run deterministic.  Ids outside [0,V) are skipped.
 * Two forms give the same bits: up to 16384 positions (S a multiple of 4, V < 2^19, D within one round of workgroups)
 * every workgroup owns a few columns of dE and reads its rows of dx in place; otherwise dx is first copied
 * token-major and summed row by row (the "scatter_cols" knob names a form).  The first form costs by the number of
 * distinct (token, block of 8192 positions) pairs and is the default; every call leaves that number in a word of
 * pinned host memory, and the next call with the same number of positions and D takes the second form if the ids
 * repeated too little for the first (and returns when they repeat again): same bits, only the time differs.
 * While a graph is recorded, inputs beyond 16384 positions take the first form too (the library sort of the second
 * cannot be recorded). */
int mi355_embed_scatter_add_dev(float *dE, const float *dx, const int32_t *ids, int V, int D,
                                int S, int batch);
/* Which form the next mi355_embed_scatter_add_dev call of this shape would take under the current knobs and the last
 * call's report: 1 = columns of dE owned by workgroups, -1 = token-major copy and row sums, 0 = bad shape.  `aligned`:
 * dx is 16-byte aligned.  No counterpart in the reference (its op is one loop); for tests and tuning. */
int mi355_embed_scatter_add_form(int V, int D, int S, int batch, int aligned);

/* Fused softmax + cross-entropy forward/backward on logits [V][S].  Replaces cross_entropy_loss —
 * training/training_dynamic/cpu_ops.h:68-93, training/stories_cpu_ops.h:71-108 — and the loss-scale
 * pass at training/training_dynamic/train.m:497 (grad_scale; 1.0f = none).
 * dlogits = (softmax - onehot) * (1/S) * grad_scale; *loss_dev = mean_t -logf(p[tgt]+1e-10f).
 * A target outside [0,V) contributes no loss and leaves its column as the unscaled softmax
 * (stories_cpu_ops.h:98).  dlogits may alias logits.
 * Logits with S a multiple of 64 (at most 1024), V >= 4096, 16-byte aligned and not in place run as ONE launch
 * that keeps the logits in registers and LDS between the two passes (one workgroup per compute unit; partial
 * sums exchanged inside the launch through a device array of the library, bounded wait as for the RMSNorm); every
 * other call runs as three launches that read the logits twice.  Both forms are deterministic; they sum in
 * different orders, so their results differ in the last bits.  Tuning knob "ce_resident": 0 = as described,
 * 1 = the one-launch form for any V, -1 = never. */
int mi355_softmax_ce_dev(float *dlogits, float *loss_dev, const float *logits,
                         const int32_t *targets, int V, int S, float grad_scale);

/* mi355_softmax_ce_dev for callers that may not allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and the same
 * bits out, but the scratch lives in a fixed 3 MiB device array of the library, located once by mi355_init (call
 * it first): the call performs no hipMalloc, no hipFree and no workspace growth.  The array holds the exchange
 * slots of the one-launch form (which mi355_softmax_ce_dev uses from there as well) and 2 MiB for the three-launch
 * form's first-pass partials and per-column max / sum / loss.
 * Limit, for calls that take the three-launch form: 2 * ceil(V / rows per workgroup) * S * 4 + 3 * S * 4 bytes
 * (rounded up to 256 each) must fit 2 MiB, otherwise the call fails with a message and launches nothing.  Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race. */
int mi355_softmax_ce_noalloc_dev(float *dlogits, float *loss_dev, const float *logits, const int32_t *targets,
                                 int V, int S, float grad_scale);

/* The two halves of that op as the static loop with ANE extras runs them when the classifier stays on the CPU
 * (training/train_large_ane.m:499-530).
 * mi355_softmax_cols_dev: probs[v][t] = exp(logits[v][t] - max_v) / sum_v exp(...), per column t — the scalar loop of
 * train_large_ane.m:508-516 (which divides by the sum).  probs may alias logits.
 * mi355_nll_from_probs_dev: *loss_dev = mean_t -logf(probs[tgt_t][t] + 1e-10f); dlogits = (probs - onehot) * (1/S) —
 * train_large_ane.m:519-530.  The reference indexes with the target unchecked; here a target outside [0,V) adds no
 * loss term and no one-hot (its column is still scaled by 1/S).  dlogits may alias probs. */
int mi355_softmax_cols_dev(float *probs, const float *logits, int V, int S);
int mi355_nll_from_probs_dev(float *dlogits, float *loss_dev, const float *probs, const int32_t *targets, int V,
                             int S);

/* Range diagnostics of the loops: out3_dev = {min x, max x, max |x|}.  Replaces vDSP_minv / vDSP_maxv /
 * vDSP_maxmgv — training/training_dynamic/train.m:664-666 (dq, dk, dv magnitudes) and :738-742 (range of x and
 * dy).  Exact in any order; NaNs are skipped. */
int mi355_minmax_dev(float *out3_dev, const float *x, size_t n);

/* Per-tensor symmetric INT8.  Replaces the quantizer of ane_bridge_build_weight_blob_quantized —
 * bridge/ane_bridge.m:346-365 — and the MIL quantize/dequantize pair of ane_int8_bench.m:83-92.
 * scale = max|x|/127 (1.0 when the tensor is all zero); q = clamp(x/scale, -128, 127) rounded
 * half-to-even (rounding 0) or half away from zero (rounding 1, the reference's); x^ = q*scale. */
int mi355_int8_scale_dev(float *scale_dev, const float *x, size_t n);
int mi355_int8_quant_dev(int8_t *q, const float *x, const float *scale_dev, size_t n, int rounding);
/* The quantizer of bridge/ane_bridge.m:346-365 as one call (the activation path of W8A8): scale = max|x|/127 (written
 * to scale_dev) and q = quantize(x, scale); one launch that reads x once up to 8.4 M floats, two beyond; the same
 * bytes out as mi355_int8_scale_dev + mi355_int8_quant_dev. */
int mi355_int8_quantize_dynamic_dev(int8_t *q, float *scale_dev, const float *x, size_t n, int rounding);
int mi355_int8_dequant_dev(float *x, const int8_t *q, const float *scale_dev, size_t n);

/* Optimizer tail — training/training_dynamic/train.m:748-877 in two sweeps instead of five.
 * mi355_sumsq_accum_dev: *acc_dev += sum_i (pre_scale*g_i)^2 — the gradient-scale loop (:754-769) and the
 * vDSP_dotpr per tensor (:771-787) in one read; deterministic for a given n.
 * mi355_clip_scale_dev: *scale_dev = grad_clip/sqrt(*sumsq_dev) if grad_clip > 0 and the norm exceeds it,
 * else 1 (:806-808); stays on the device, so no host round trip sits between norm and update.
 * mi355_adam_update_dev: adam_update — training/training_dynamic/cpu_ops.h:56-64 (AdamW; wd = 0 is
 * training/stories_cpu_ops.h:55-63) — on g' = (g*scale1)*scale2 (scale2_dev may be NULL = 1), i.e. with
 * the scale pass (:754-769) and the clip pass (:806-821) folded in; zero_grad != 0 also clears g
 * (layer_grads_zero / memset, :873-877).  t >= 1 is the Adam step count. */
int mi355_sumsq_accum_dev(float *acc_dev, const float *g, size_t n, float pre_scale);
int mi355_clip_scale_dev(float *scale_dev, const float *sumsq_dev, float grad_clip);
int mi355_adam_update_dev(float *w, float *g, float *m, float *v, size_t n, int t, float lr, float b1,
                          float b2, float eps, float wd, float scale1, const float *scale2_dev,
                          int zero_grad);

/* The same two sweeps over several tensors per launch (the loop updates 9 tensors per layer, train.m:843-852):
 * host arrays of `count` device pointers / sizes / per-tensor weight decay; tensors must be 16-byte aligned.
 * Results equal the per-tensor calls (the norm up to summation order). */
int mi355_sumsq_accum_multi_dev(float *acc_dev, const float *const *g, const size_t *n, int count,
                                float pre_scale);
int mi355_adam_update_multi_dev(float *const *w, float *const *g, float *const *m, float *const *v,
                                const size_t *n, const float *wd, int count, int t, float lr, float b1,
                                float b2, float eps, float scale1, const float *scale2_dev, int zero_grad);

/* GQA helpers of the dynamic loop — training/training_dynamic/io.h:330-351 (calls at
 * training/training_dynamic/train.m:620-621,653-654).  tile: out[batch][kv_heads*ratio*hd][S] gets each KV
 * head `ratio` times; reduce: out[batch][kv_heads*hd][S] = sum over the `ratio` query heads of each group,
 * added in head order (the reference's memset + += loop). */
int mi355_gqa_tile_dev(float *out, const float *in, int kv_heads, int ratio, int hd, int S, int batch);
int mi355_gqa_reduce_dev(float *out, const float *in, int kv_heads, int ratio, int hd, int S, int batch);

/* fp32 <-> fp16 staging converts — cvt_f32_f16 / cvt_f16_f32, training/training_dynamic/io.h:33-50, as used by
 * io_write_fp16 / io_read_fp16 / io_write_fp16_at / io_write_dyn / io_read_dyn (io.h:53-96) and the per-kernel
 * packers (io.h:160-310).  A rectangle of `rows` runs of `cols` contiguous elements; dst_ld / src_ld are the
 * row pitches in elements (>= cols; equal to cols for one contiguous run).  fp16 values travel as uint16_t bit
 * patterns (IEEE binary16).  fp32 -> fp16 rounds to nearest even, overflows to infinity and keeps subnormals,
 * as the reference's vcvt_f16_f32 does. */
int mi355_cvt_f32_f16_dev(uint16_t *dst, size_t dst_ld, const float *src, size_t src_ld, size_t rows, size_t cols);
int mi355_cvt_f16_f32_dev(float *dst, size_t dst_ld, const uint16_t *src, size_t src_ld, size_t rows, size_t cols);

/* What the dynamic loop does between the attention backward kernels and the QKV backward —
 * training/training_dynamic/train.m:646-660: io_read_fp16 of dQ, dK, dV (all at `heads` query heads),
 * gqa_reduce_kv of dK and dV to `kv_heads`, the copy of dQ, rope_backward_inplace of dQ and dK — in one pass.
 * Inputs [batch][heads*hd][S], fp16 bit patterns (in_f16 = 1) or fp32 (in_f16 = 0); q/k/v_stride = elements
 * between consecutive sequences of each input (0 = heads*hd*S, i.e. packed), so that the three may be channel
 * ranges of larger surfaces.  Outputs fp32: dq [batch][heads*hd][S], dk and dv [batch][kv_heads*hd][S].
 * cos/sin: tables of mi355_rope_tables(_dev), or both NULL for no rotation.  dq may alias dq_full when fp32.
 * Results equal the separate calls bit for bit. */
int mi355_attn_grads_finish_dev(float *dq, float *dk, float *dv, const void *dq_full, const void *dk_full,
                                const void *dv_full, int in_f16, size_t q_stride, size_t k_stride, size_t v_stride,
                                int heads, int kv_heads, int hd, int S, int batch, const float *cos_dev,
                                const float *sin_dev);

/* cblas_sgemm(CblasRowMajor, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc) on device memory —
 * the classifier products training/training_dynamic/train.m:490-491 (logits), :501-502 (dy), :507-508 (gcembed +=)
 * and the weight-gradient products :577-581, :613, :681-685.  Same argument order and meaning as the cblas call
 * without the layout argument (always row-major); trans flags take 0/1 or CblasNoTrans/CblasTrans (111/112).
 * Runs on the bridge stream through rocBLAS, which is opened on the first call. */
int mi355_sgemm_dev(int trans_a, int trans_b, int M, int N, int K, float alpha, const float *A, int lda,
                    const float *B, int ldb, float beta, float *C, int ldc);

/* Checkpoints of the two big loops — header CkptHdr training/stories_config.h:90-105 (version 2) and
 * training/training_dynamic/config.h:78-86 (version 4: the trailing pad carries the GQA fields); tensor order of
 * save_checkpoint / load_checkpoint training/train_large.m:110-181, training/training_dynamic/train.m:104-172
 * (the dashboard reads the same layout, training/dashboard.py:141-174).  The struct below IS the 96 on-disk
 * bytes.  read_header / locate / file_bytes / create are host-only and need no GPU; load / store move one
 * tensor between the file and device memory on the bridge stream and return when it is done. */
typedef struct mi355_ckpt_hdr {
    int magic, version, step, total_steps;                 /* magic 0x424C5A54, version 2 or 4 */
    int n_layers, vocab_size, dim, hidden_dim, n_heads, seq_len;
    float lr, loss;
    double cum_compile, cum_train, cum_wall;
    int cum_steps, cum_batches, adam_t;
    int kv_heads, head_dim, q_dim;                         /* version 4; zero padding in version 2 */
} mi355_ckpt_hdr;
enum { MI355_CK_WQ = 0, MI355_CK_WK, MI355_CK_WV, MI355_CK_WO, MI355_CK_W1, MI355_CK_W2, MI355_CK_W3,
       MI355_CK_RMS_ATT, MI355_CK_RMS_FFN,                 /* per layer */
       MI355_CK_RMS_FINAL, MI355_CK_EMBED };               /* once per file (layer argument ignored) */
enum { MI355_CK_WEIGHT = 0, MI355_CK_ADAM_M = 1, MI355_CK_ADAM_V = 2 };
/* 0, or -1 when the file is missing, short, or not a version 2 / 4 checkpoint (load_checkpoint's `return false`). */
int mi355_ckpt_read_header(const char *path, mi355_ckpt_hdr *hdr);
/* Byte offset in the file and element count of one tensor (part: the weight or its Adam m / v). */
int mi355_ckpt_locate(const mi355_ckpt_hdr *hdr, int layer, int tensor, int part, uint64_t *byte_offset,
                      uint64_t *count);
uint64_t mi355_ckpt_file_bytes(const mi355_ckpt_hdr *hdr);                 /* 0 on a bad header */
/* Writes the header and sizes the file; tensors are then stored in any order. */
int mi355_ckpt_create(const char *path, const mi355_ckpt_hdr *hdr);
int mi355_ckpt_load_dev(const char *path, uint64_t byte_offset, float *dst_dev, uint64_t count);
int mi355_ckpt_store_dev(const char *path, uint64_t byte_offset, const float *src_dev, uint64_t count);

/* Vocabulary map.  Replaces vocab_map_build — training/training_dynamic/cpu_ops.h:102-126: full_to_compact[V]
 * gets the compact id of every token that occurs in data[0..n_tokens) (numbered in ascending token order) and
 * -1 for the others; compact_to_full (room for V entries) gets the inverse; *compact_vocab_dev their number.
 * Tokens >= V in the data are ignored.  mi355_vocab_remap_dev maps ids of the full vocabulary to compact ids
 * (the loop at training/training_dynamic/train.m:403); an id outside [0,V) or without a compact id gives -1. */
int mi355_vocab_map_build_dev(int32_t *full_to_compact, int32_t *compact_to_full, int32_t *compact_vocab_dev,
                              const uint16_t *data, size_t n_tokens, int V);
int mi355_vocab_remap_dev(int32_t *out, const int32_t *ids, const int32_t *full_to_compact, size_t n, int V);

/* Vocabulary compaction — training/training_dynamic/cpu_ops.h:127-148.  compact_to_full[CV] is the map that
 * vocab_map_build (cpu_ops.h:103-125; above, or the host code unchanged) produces: distinct row numbers of the
 * full table.
 *   compact_embed: compact[c] = full[map[c]]           (vocab_compact_embed, cpu_ops.h:127-132)
 *   update_full:   full[map[c]] = compact[c]           (vocab_update_full,   cpu_ops.h:145-148)
 *   scatter_grads: full_grad[map[c]] += compact_grad[c] (vocab_scatter_grads, cpu_ops.h:135-142)
 * Rows are [D] floats; a map entry outside [0,V) is skipped.  Pure copies: bit-exact. */
int mi355_vocab_compact_embed_dev(float *compact, const float *full, const int32_t *compact_to_full, int CV,
                                  int V, int D);
int mi355_vocab_update_full_dev(float *full, const float *compact, const int32_t *compact_to_full, int CV,
                                int V, int D);
int mi355_vocab_scatter_grads_dev(float *full_grad, const float *compact_grad, const int32_t *compact_to_full,
                                  int CV, int V, int D);

/* ------------------------------------------------------------------------------------------
 * Host-pointer drop-ins: the reference signatures verbatim (host float* in, host float* out),
 * so a caller swaps the symbol only.  Each call stages through cached device buffers
 * (H2D, kernel, D2H) and returns when the result is in host memory.  On failure they print one
 * line to stderr and leave the outputs untouched.
 * ---------------------------------------------------------------------------------------- */
/* rmsnorm — training/stories_cpu_ops.h:6 */
void mi355_rmsnorm(float *out, const float *x, const float *w, int d, int S);
/* rmsnorm_bwd — training/stories_cpu_ops.h:23 */
void mi355_rmsnorm_bwd(float *dx, float *dw, const float *dy, const float *x, const float *w,
                       int d, int S);
/* cross_entropy_loss — training/stories_cpu_ops.h:71, training/training_dynamic/cpu_ops.h:68 */
float mi355_cross_entropy_loss(float *dlogits, const float *logits, const uint16_t *targets, int V,
                               int S);
/* embed_lookup — training/stories_cpu_ops.h:112.  The reference reads the vocabulary size from the
 * compile-time VOCAB macro; it is an argument here.  The table is kept resident on the device, keyed
 * by its host address.  It is uploaded again after any host-pointer call of this library has written into
 * that host array (mi355_adam_update on the table, as training/training_dynamic/train.m:869 does) and after
 * mi355_host_table_invalidate(embed), which is for callers that change the array with code of their own. */
void mi355_embed_lookup(float *x, const float *embed, const uint16_t *tokens, int vocab, int dim,
                        int seq);
void mi355_host_table_invalidate(const float *embed);
/* embed_backward — training/stories_cpu_ops.h:123 */
void mi355_embed_backward(float *d_embed, const float *dx, const uint16_t *tokens, int vocab,
                          int dim, int seq);
/* rope_backward_inplace — training/training_dynamic/cpu_ops.h:168 (theta = 10000) */
void mi355_rope_backward_inplace(float *dx, int seq, int dim, int hd);
/* The inline vDSP blocks of the dynamic loop as calls: SiLU-gate backward
 * (training/training_dynamic/train.m:537-554), its forward (training/forward.h:101,149-151), and the
 * residual family vDSP_vsma / vDSP_vsmul / vDSP_vadd (train.m:460,523,595; modes as mi355_axpby_dev). */
void mi355_swiglu_bwd(float *dh1, float *dh3, const float *dsilu, const float *h1, const float *h3,
                      size_t n);
void mi355_swiglu_fwd(float *out, const float *h1, const float *h3, size_t n);
void mi355_axpby(float *y, const float *a, const float *b, float alpha, size_t n, int mode);
/* adam_update — training/training_dynamic/cpu_ops.h:56 with the AdamState fields spelled out */
void mi355_adam_update(float *w, const float *g, float *m, float *v, size_t n, int t, float lr, float b1,
                       float b2, float eps, float wd);

/* Vocabulary compaction on host arrays — training/training_dynamic/cpu_ops.h:96-148, with the VocabMap fields
 * and the size of the full table spelled out (include/mi355_cpu_ops.h wraps them in the reference's own
 * names and struct).  The maps are caller-allocated: full_to_compact [full_vocab]; compact_to_full with room for
 * full_vocab entries, of which the first compact_vocab are written.  mi355_vocab_map_build returns compact_vocab
 * (-1 on failure); tokens >= full_vocab in the data are ignored.  compact_embed and update_full keep the full
 * table resident on the device, keyed by its host address, like mi355_embed_lookup (and update_full keeps that
 * copy current).  Map entries outside [0, full_vocab) are skipped. */
int mi355_vocab_map_build(int *full_to_compact, int *compact_to_full, const uint16_t *data, size_t n_tokens,
                          int full_vocab);
/* vocab_compact_embed — cpu_ops.h:127-132: compact[c] = full_embed[compact_to_full[c]] */
void mi355_vocab_compact_embed(float *compact, const float *full_embed, const int *compact_to_full, int compact_vocab,
                               int full_vocab, int dim);
/* vocab_scatter_grads — cpu_ops.h:135-142: full_gembed[compact_to_full[c]] += compact_gembed[c] */
void mi355_vocab_scatter_grads(float *full_gembed, const float *compact_gembed, const int *compact_to_full,
                               int compact_vocab, int full_vocab, int dim);
/* vocab_update_full — cpu_ops.h:145-148: full_embed[compact_to_full[c]] = compact_embed[c] */
void mi355_vocab_update_full(float *full_embed, const float *compact_embed, const int *compact_to_full,
                             int compact_vocab, int full_vocab, int dim);

#ifdef __cplusplus
}
#endif

#endif /* MI355_BRIDGE_H */
