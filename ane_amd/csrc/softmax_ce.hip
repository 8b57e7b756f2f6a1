// softmax_ce.hip — fused classifier softmax + cross-entropy forward/backward on logits [V][S].
//
// Reference op: cross_entropy_loss (training/training_dynamic/cpu_ops.h:68-93; transpose form
// training/stories_cpu_ops.h:71-108) plus the loss-scale pass of training/training_dynamic/train.m:497.
//
// The softmax runs down the STRIDED axis v (columns t are contiguous), so a wave reads whole rows
// with 128-bit loads and every lane owns four columns; no cross-lane traffic is needed until the
// four waves of a workgroup are combined through LDS.
//   pass 1  each workgroup reduces a block of rows to per-column (max, sum exp) partials
//           (online rescaling between 64-row register tiles);
//   combine per column, partials are merged in a fixed order, the target logit is read and the
//           per-column loss term is formed (the mean is taken, by a fixed tree, by one workgroup of pass 2);
//   pass 2  dlogits = (exp(l - M) * (1/L) - onehot) * (1/S) * grad_scale.  Row blocks are visited
//           in the reverse order of pass 1 so the most recently read rows are re-read first
//           (they are the most likely to still sit in the last-level cache).
#include "common.h"

#include <math.h>

namespace {

constexpr int CE_THREADS = 256;
constexpr int CE_WAVES = CE_THREADS / 64;
constexpr int CE_CAP = 16;                       // register tile: 16 steps x 4 waves = 64 rows
constexpr int CE_TILE_ROWS = CE_CAP * CE_WAVES;

template <int VEC>
__device__ __forceinline__ void ld_cols(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        v4f t = ld4(p);
        r[0] = t.x; r[1] = t.y; r[2] = t.z; r[3] = t.w;
    } else {
        r[0] = *p;
    }
}

template <int VEC>
__device__ __forceinline__ void ld_cols_nt(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        v4f t = ld4_nt(p);
        r[0] = t.x; r[1] = t.y; r[2] = t.z; r[3] = t.w;
    } else {
        r[0] = __builtin_nontemporal_load(p);
    }
}

// bfloat16 logits (the optional bf16-storage variant): four columns = one 64-bit access; widened to fp32 here,
// so everything below is the same arithmetic for both storage types.
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float bf_widen(unsigned bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ unsigned bf_narrow(float f) {       // round to nearest even; NaN stays NaN
    const unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
template <int VEC>
__device__ __forceinline__ void ld_cols(float (&r)[VEC], const uint16_t *p) {
    if constexpr (VEC == 4) {
        const v2u w = *reinterpret_cast<const v2u *>(p);
        r[0] = bf_widen(w[0] & 0xffffu); r[1] = bf_widen(w[0] >> 16);
        r[2] = bf_widen(w[1] & 0xffffu); r[3] = bf_widen(w[1] >> 16);
    } else {
        r[0] = bf_widen(*p);
    }
}
template <int VEC>
__device__ __forceinline__ void ld_cols_nt(float (&r)[VEC], const uint16_t *p) {
    if constexpr (VEC == 4) {
        const v2u w = __builtin_nontemporal_load(reinterpret_cast<const v2u *>(p));
        r[0] = bf_widen(w[0] & 0xffffu); r[1] = bf_widen(w[0] >> 16);
        r[2] = bf_widen(w[1] & 0xffffu); r[3] = bf_widen(w[1] >> 16);
    } else {
        r[0] = bf_widen(*p);
    }
}
__device__ __forceinline__ float ld_one(const float *p) { return *p; }
__device__ __forceinline__ float ld_one(const uint16_t *p) { return bf_widen(*p); }
template <int VEC>
__device__ __forceinline__ void st_cols(float *p, const float (&o)[VEC]) {
    if constexpr (VEC == 4) {
        v4f t = {o[0], o[1], o[2], o[3]};
        st4_nt(p, t);
    } else {
        *p = o[0];
    }
}
template <int VEC>
__device__ __forceinline__ void st_cols(uint16_t *p, const float (&o)[VEC]) {
    if constexpr (VEC == 4) {
        v2u w = {bf_narrow(o[0]) | (bf_narrow(o[1]) << 16), bf_narrow(o[2]) | (bf_narrow(o[3]) << 16)};
        __builtin_nontemporal_store(w, reinterpret_cast<v2u *>(p));
    } else {
        *p = (uint16_t)bf_narrow(o[0]);
    }
}

// grid: (row blocks, column strips of 64*VEC)
template <int VEC, typename T>
__global__ __launch_bounds__(CE_THREADS) void ce_partial_kernel(float *__restrict__ pm, float *__restrict__ pl,
                                                                const T *__restrict__ logits, int V, int S,
                                                                int rows_per_block) {
    __shared__ float sm[CE_WAVES][64 * VEC], sl[CE_WAVES][64 * VEC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = (blockIdx.y * 64 + lane) * VEC;
    const bool col_ok = col < S;
    const int v_lo = blockIdx.x * rows_per_block;
    const int v_hi = min(V, v_lo + rows_per_block);

    float m[VEC], l[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) { m[j] = -INFINITY; l[j] = 0.f; }

    for (int base = v_lo; base < v_hi; base += CE_TILE_ROWS) {
        float x[CE_CAP][VEC];
#pragma unroll
        for (int k = 0; k < CE_CAP; k++) {
            const int v = base + k * CE_WAVES + wave;
            if (v < v_hi && col_ok) ld_cols<VEC>(x[k], logits + (size_t)v * S + col);   // cached: pass 2 re-reads these rows (non-temporal here costs 30 %)
            else {
#pragma unroll
                for (int j = 0; j < VEC; j++) x[k][j] = -INFINITY;
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            float tm = x[0][j];
#pragma unroll
            for (int k = 1; k < CE_CAP; k++) tm = fmaxf(tm, x[k][j]);
            const float nm = fmaxf(m[j], tm);
            if (nm > -INFINITY) {
                float s = 0.f;
#pragma unroll
                for (int k = 0; k < CE_CAP; k++) s += exp_neg_fast(x[k][j] - nm);   // exp(-inf) = 0 for masked rows
                l[j] = l[j] * exp_neg(m[j] - nm) + s;
                m[j] = nm;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) { sm[wave][lane * VEC + j] = m[j]; sl[wave][lane * VEC + j] = l[j]; }
    __syncthreads();
    if (wave == 0 && col_ok) {
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            float M = sm[0][lane * VEC + j];
#pragma unroll
            for (int w = 1; w < CE_WAVES; w++) M = fmaxf(M, sm[w][lane * VEC + j]);
            float L = 0.f;
#pragma unroll
            for (int w = 0; w < CE_WAVES; w++) {
                const float mw = sm[w][lane * VEC + j];
                if (mw > -INFINITY) L += sl[w][lane * VEC + j] * exp_neg(mw - M);
            }
            pm[(size_t)blockIdx.x * S + col + j] = M;
            pl[(size_t)blockIdx.x * S + col + j] = L;
        }
    }
}

// One workgroup per 16 columns: 64 groups of threads each merge an interleaved subset of the row blocks (few
// rounds of loads per thread, S/16 workgroups in flight), then the 64 partial results are merged by a fixed
// tree.  The merge of two (max, sum) pairs is the online-softmax rescaling.
constexpr int CB_COLS = 16, CB_GROUPS = 1024 / CB_COLS;
// PLAIN: the stand-alone column softmax; there are no targets, and colInv receives the sum itself (that op divides).
template <typename T, bool PLAIN = false>
__global__ __launch_bounds__(1024) void ce_combine_kernel(float *__restrict__ colM, float *__restrict__ colInv,
                                                          float *__restrict__ colLoss, const float *__restrict__ pm,
                                                          const float *__restrict__ pl,
                                                          const T *__restrict__ logits,
                                                          const int32_t *__restrict__ targets, int V, int S,
                                                          int nblk) {
    __shared__ float sm[CB_GROUPS][CB_COLS], sl[CB_GROUPS][CB_COLS];
    const int cl = threadIdx.x % CB_COLS, g = threadIdx.x / CB_COLS;
    const int t = blockIdx.x * CB_COLS + cl;
    float m = -INFINITY, l = 0.f;
    if (t < S)
        for (int r0 = g; r0 < nblk; r0 += CB_GROUPS * 4) {
            float mr[4], lr[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {     // four independent loads in flight
                const int r = r0 + CB_GROUPS * u;
                mr[u] = r < nblk ? pm[(size_t)r * S + t] : -INFINITY;
                lr[u] = r < nblk ? pl[(size_t)r * S + t] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const float nm = fmaxf(m, mr[u]);
                if (nm > -INFINITY) {
                    l = l * exp_neg(m - nm) + lr[u] * exp_neg(mr[u] - nm);
                    m = nm;
                }
            }
        }
    sm[g][cl] = m;
    sl[g][cl] = l;
    __syncthreads();
    for (int half = CB_GROUPS / 2; half > 0; half >>= 1) {
        if (g < half) {
            const float m0 = sm[g][cl], m1 = sm[g + half][cl];
            const float nm = fmaxf(m0, m1);
            if (nm > -INFINITY) {
                sl[g][cl] = sl[g][cl] * exp_neg(m0 - nm) + sl[g + half][cl] * exp_neg(m1 - nm);
                sm[g][cl] = nm;
            }
        }
        __syncthreads();
    }
    if (g == 0 && t < S) {
        const float M = sm[0][cl];
        colM[t] = M;
        if constexpr (PLAIN) {
            colInv[t] = sl[0][cl];
            return;
        }
        const float inv = 1.0f / sl[0][cl];
        colInv[t] = inv;
        const int tgt = targets[t];
        float loss = 0.f;
        if (tgt >= 0 && tgt < V) {
            const float p = exp_neg(ld_one(logits + (size_t)tgt * S + t) - M) * inv;
            loss = -logf(p + 1e-10f);
        }
        colLoss[t] = loss;
    }
}

template <int VEC, typename T>
__global__ __launch_bounds__(CE_THREADS) void ce_grad_kernel(T *dlogits, const T *logits,
                                                             const float *__restrict__ colM,
                                                             const float *__restrict__ colInv,
                                                             const int32_t *__restrict__ targets, int V, int S,
                                                             int rows_per_block, float invS, float grad_scale,
                                                             float *__restrict__ loss_out,
                                                             const float *__restrict__ colLoss) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        // loss = (sum_t colLoss[t]) / S with a fixed summation tree; one workgroup does it on the side
        __shared__ float red[CE_THREADS];
        float sl = 0.f;
        for (int t = threadIdx.x; t < S; t += CE_THREADS) sl += colLoss[t];
        red[threadIdx.x] = sl;
        __syncthreads();
        for (int off = CE_THREADS / 2; off > 0; off >>= 1) {
            if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
            __syncthreads();
        }
        if (threadIdx.x == 0) *loss_out = red[0] / (float)S;
    }
    const int col = (blockIdx.y * 64 + lane) * VEC;
    if (col >= S) return;
    const int rb = gridDim.x - 1 - blockIdx.x;           // reverse order of pass 1
    const int v_lo = rb * rows_per_block;
    const int v_hi = min(V, v_lo + rows_per_block);
    float M[VEC], inv[VEC], sc[VEC];
    int tgt[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        M[j] = colM[col + j];
        inv[j] = colInv[col + j];
        const int tg = targets[col + j];
        const bool ok = tg >= 0 && tg < V;
        tgt[j] = ok ? tg : -1;
        sc[j] = ok ? invS : 1.0f;      // an out-of-range target leaves the column unscaled (stories_cpu_ops.h:98)
    }
    for (int base = v_lo; base < v_hi; base += CE_TILE_ROWS) {
        float x[CE_CAP][VEC];
#pragma unroll
        for (int k = 0; k < CE_CAP; k++) {
            const int v = base + k * CE_WAVES + wave;
            if (v < v_hi) ld_cols_nt<VEC>(x[k], logits + (size_t)v * S + col);
        }
#pragma unroll
        for (int k = 0; k < CE_CAP; k++) {
            const int v = base + k * CE_WAVES + wave;
            if (v < v_hi) {
                float o[VEC];
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    float p = exp_neg(x[k][j] - M[j]) * inv[j];
                    if (v == tgt[j]) p -= 1.0f;
                    p = p * sc[j];
                    if (grad_scale != 1.0f) p = p * grad_scale;
                    o[j] = p;
                }
                st_cols<VEC>(dlogits + (size_t)v * S + col, o);
            }
        }
    }
}

// probs = exp(l - M) / L: the second pass of the stand-alone column softmax (training/train_large_ane.m:508-516)
template <int VEC>
__global__ __launch_bounds__(CE_THREADS) void softmax_out_kernel(float *probs, const float *logits,
                                                                 const float *__restrict__ colM,
                                                                 const float *__restrict__ colL, int V, int S,
                                                                 int rows_per_block) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = (blockIdx.y * 64 + lane) * VEC;
    if (col >= S) return;
    const int rb = gridDim.x - 1 - blockIdx.x;
    const int v_lo = rb * rows_per_block;
    const int v_hi = min(V, v_lo + rows_per_block);
    float M[VEC], L[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) { M[j] = colM[col + j]; L[j] = colL[col + j]; }
    for (int v = v_lo + wave; v < v_hi; v += CE_WAVES) {
        float x[VEC], o[VEC];
        ld_cols_nt<VEC>(x, logits + (size_t)v * S + col);
#pragma unroll
        for (int j = 0; j < VEC; j++) o[j] = exp_neg(x[j] - M[j]) / L[j];
        st_cols<VEC>(probs + (size_t)v * S + col, o);
    }
}

// NLL on given probabilities (training/train_large_ane.m:519-530).  The loss is formed first, by one workgroup and
// a fixed tree, so that the gradient pass may overwrite the probabilities in place.
__global__ __launch_bounds__(CE_THREADS) void nll_loss_kernel(float *__restrict__ loss_out, const float *__restrict__ probs,
                                                              const int32_t *__restrict__ targets, int V, int S) {
    __shared__ float red[CE_THREADS];
    float sl = 0.f;
    for (int t = threadIdx.x; t < S; t += CE_THREADS) {
        const int tg = targets[t];
        if (tg >= 0 && tg < V) sl -= logf(probs[(size_t)tg * S + t] + 1e-10f);
    }
    red[threadIdx.x] = sl;
    __syncthreads();
    for (int off = CE_THREADS / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss_out = red[0] / (float)S;
}

// dlogits = (probs - onehot) * (1/S), one 128-bit access per lane; n4 = V*S/4 when VEC = 4
template <int VEC>
__global__ __launch_bounds__(256) void nll_grad_kernel(float *dlogits, const float *probs,
                                                       const int32_t *__restrict__ targets, int V, int S, size_t n,
                                                       float invS) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    const int v = (int)(i / (size_t)S), t0 = (int)(i - (size_t)v * S);
    float x[VEC], o[VEC];
    ld_cols_nt<VEC>(x, probs + i);
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        float p = x[j];
        if (targets[t0 + j] == v) p -= 1.0f;
        o[j] = p * invS;
    }
    st_cols<VEC>(dlogits + i, o);
}

// resident workgroups of the second pass per compute unit (asked of the runtime once per storage type)
template <typename T>
int grad_blocks_per_cu() {
    static int cached = 0;
    if (cached == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, ce_grad_kernel<4, T>, CE_THREADS, 0) != hipSuccess || n <= 0)
            n = 4;
        cached = n;
    }
    return cached;
}

// Scratch of mi355_softmax_ce_noalloc_dev: the first-pass partials and the three per-column arrays, in a
// file-scope device array, so that the call needs no allocation.  One copy per GPU, held until the process ends.
// In host code the array's name is only a handle for the symbol lookup below; kernels and copies use the address
// that the lookup returns for the current device.
constexpr size_t CE_SCRATCH_BYTES = (size_t)2 << 20;
constexpr int CE_MAX_DEVICES = 16;
}   // namespace
static __device__ __align__(256) unsigned char scratch[CE_SCRATCH_BYTES];
namespace {
unsigned char *g_scratch_ptr[CE_MAX_DEVICES] = {};

template <typename T>
int ce_run(const char *who, T *dlogits, float *loss_dev, const T *logits, const int32_t *targets, int V, int S,
           float grad_scale, bool no_alloc = false) {
    if (!mi355_ready(who)) return -1;
    if (!dlogits || !loss_dev || !logits || !targets) return mi355_fail("%s: NULL pointer", who);
    if (V <= 0 || S <= 0) return mi355_fail("%s: bad shape V=%d S=%d", who, V, S);
    // Rows per workgroup: one to six 64-row register tiles, chosen so that the workgroups of a column strip fill the
    // compute units evenly (at least 1.75 per unit, and the last round of them as full as possible); ties go to
    // the larger block, which leaves fewer partials to merge.  At V = 151936 on 256 units: 320 rows, 475
    // workgroups (87 us for the op; 256 rows and 594 workgroups: 91 us; 384 rows and 396: 97 us).
    int rpb = g_ctx.ce_rows;
    if (rpb <= 0) {
        const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
        double best = -1.0;
        rpb = CE_TILE_ROWS;
        for (int t = 1; t <= 6; t++) {
            const long nb = (long)ceil_div((size_t)V, (size_t)t * CE_TILE_ROWS);
            if (t > 1 && nb * 4 < (long)cu * 7) break;
            const long rounds = (nb + cu - 1) / cu;
            const double score = (double)nb / (double)(rounds * cu) + 0.002 * t;
            if (score > best) { best = score; rpb = t * CE_TILE_ROWS; }
        }
    }
    const int nblk = (int)ceil_div((size_t)V, (size_t)rpb);
    // The second pass has no partials to merge and its own blocks: a multiple of 16 rows between 64 and 384 that
    // fills the resident workgroup slots of the chip in as few rounds as it can (four workgroups fit a compute
    // unit: at V = 151936, 160 rows = 950 workgroups for 1024 slots, 83 us for the op; 144 rows = 1056 workgroups,
    // a second round for 32 of them, 98 us; 320 rows, less than half the slots, 88 us).
    int rpb2 = g_ctx.ce_rows2;
    if (rpb2 <= 0) {
        const long slots = (long)(g_ctx.num_cu > 0 ? g_ctx.num_cu : 256) * grad_blocks_per_cu<T>();
        double best = -1.0;
        rpb2 = CE_TILE_ROWS;
        for (int m = CE_TILE_ROWS / 16; m <= 6 * CE_TILE_ROWS / 16; m++) {
            const long nb = (long)ceil_div((size_t)V, (size_t)m * 16);
            const long rounds = (nb + slots - 1) / slots;
            const double score = (double)nb / (double)(rounds * slots) - 0.05 * (double)(rounds - 1) + 1e-4 * m;
            if (score > best) { best = score; rpb2 = m * 16; }
        }
    }
    const int nblk2 = (int)ceil_div((size_t)V, (size_t)rpb2);
    // four columns per lane: 16 bytes of fp32, 8 bytes of bf16
    const uintptr_t mask = 4 * sizeof(T) - 1;
    const bool vec_ok = (S % 4 == 0) && (((uintptr_t)logits | (uintptr_t)dlogits) & mask) == 0;
    const int vec = vec_ok ? 4 : 1;
    const int strips = (int)ceil_div((size_t)S, (size_t)64 * vec);
    if (strips > 65535) return mi355_fail("%s: S too large", who);

    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t part_b = al((size_t)nblk * S * sizeof(float)), col_b = al((size_t)S * sizeof(float));
    char *ws;
    if (no_alloc) {
        if (2 * part_b + 3 * col_b > CE_SCRATCH_BYTES)
            return mi355_fail("%s: V=%d S=%d needs %zu bytes of scratch, the fixed scratch holds %zu "
                              "(use mi355_softmax_ce_dev, whose workspace grows)", who, V, S, 2 * part_b + 3 * col_b,
                              CE_SCRATCH_BYTES);
        ws = (g_ctx.device >= 0 && g_ctx.device < CE_MAX_DEVICES) ? (char *)g_scratch_ptr[g_ctx.device] : nullptr;
        if (!ws) return mi355_fail("%s: the scratch array was not located at init", who);
    } else {
        ws = (char *)mi355_ws(2 * part_b + 3 * col_b);
    }
    if (!ws) return -1;
    float *pm = (float *)ws, *pl = (float *)(ws + part_b);
    float *colM = (float *)(ws + 2 * part_b), *colInv = (float *)(ws + 2 * part_b + col_b);
    float *colLoss = (float *)(ws + 2 * part_b + 2 * col_b);

    const dim3 grid((unsigned)nblk, (unsigned)strips);
    if (vec_ok) hipLaunchKernelGGL((ce_partial_kernel<4, T>), grid, dim3(CE_THREADS), 0, g_ctx.stream, pm, pl, logits, V, S, rpb);
    else hipLaunchKernelGGL((ce_partial_kernel<1, T>), grid, dim3(CE_THREADS), 0, g_ctx.stream, pm, pl, logits, V, S, rpb);
    LAUNCH_OK("softmax_ce partial");
    hipLaunchKernelGGL(ce_combine_kernel<T>, dim3((unsigned)ceil_div((size_t)S, CB_COLS)), dim3(1024), 0, g_ctx.stream, colM,
                       colInv, colLoss, pm, pl, logits, targets, V, S, nblk);
    LAUNCH_OK("softmax_ce combine");
    const dim3 grid2((unsigned)nblk2, (unsigned)strips);
    if (vec_ok)
        hipLaunchKernelGGL((ce_grad_kernel<4, T>), grid2, dim3(CE_THREADS), 0, g_ctx.stream, dlogits, logits, colM, colInv,
                           targets, V, S, rpb2, 1.0f / (float)S, grad_scale, loss_dev, colLoss);
    else
        hipLaunchKernelGGL((ce_grad_kernel<1, T>), grid2, dim3(CE_THREADS), 0, g_ctx.stream, dlogits, logits, colM, colInv,
                           targets, V, S, rpb2, 1.0f / (float)S, grad_scale, loss_dev, colLoss);
    LAUNCH_OK("softmax_ce grad");
    return 0;
}

}   // namespace

// Called by mi355_init with the device current: finds this device's copy of the scratch array, and asks the
// runtime for the second pass's occupancy now so that the entry point below never has to.
int mi355_ce_setup(void) {
    const int dev = g_ctx.device;
    if (dev < 0 || dev >= CE_MAX_DEVICES) return mi355_fail("init: device index %d beyond %d", dev, CE_MAX_DEVICES);
    unsigned char *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return mi355_fail("init: hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
    (void)grad_blocks_per_cu<float>();
    return 0;
}

// The same op with its scratch in the fixed device array: no hipMalloc, no hipFree, no workspace growth.
MI355_API int mi355_softmax_ce_noalloc_dev(float *dlogits, float *loss_dev, const float *logits, const int32_t *targets,
                                           int V, int S, float grad_scale) {
    return ce_run<float>("softmax_ce_noalloc", dlogits, loss_dev, logits, targets, V, S, grad_scale, true);
}

MI355_API int mi355_softmax_cols_dev(float *probs, const float *logits, int V, int S) {
    if (!mi355_ready("softmax_cols")) return -1;
    if (!probs || !logits) return mi355_fail("softmax_cols: NULL pointer");
    if (V <= 0 || S <= 0) return mi355_fail("softmax_cols: bad shape V=%d S=%d", V, S);
    const int rpb = 4 * CE_TILE_ROWS;
    const int nblk = (int)ceil_div((size_t)V, (size_t)rpb);
    const bool vec_ok = (S % 4 == 0) && aligned16(logits) && aligned16(probs);
    const int vec = vec_ok ? 4 : 1;
    const int strips = (int)ceil_div((size_t)S, (size_t)64 * vec);
    if (strips > 65535) return mi355_fail("softmax_cols: S too large");
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t part_b = al((size_t)nblk * S * sizeof(float)), col_b = al((size_t)S * sizeof(float));
    char *ws = (char *)mi355_ws(2 * part_b + 2 * col_b);
    if (!ws) return -1;
    float *pm = (float *)ws, *pl = (float *)(ws + part_b);
    float *colM = (float *)(ws + 2 * part_b), *colL = (float *)(ws + 2 * part_b + col_b);
    const dim3 grid((unsigned)nblk, (unsigned)strips);
    if (vec_ok) hipLaunchKernelGGL((ce_partial_kernel<4, float>), grid, dim3(CE_THREADS), 0, g_ctx.stream, pm, pl, logits, V, S, rpb);
    else hipLaunchKernelGGL((ce_partial_kernel<1, float>), grid, dim3(CE_THREADS), 0, g_ctx.stream, pm, pl, logits, V, S, rpb);
    LAUNCH_OK("softmax_cols partial");
    hipLaunchKernelGGL((ce_combine_kernel<float, true>), dim3((unsigned)ceil_div((size_t)S, CB_COLS)), dim3(1024), 0,
                       g_ctx.stream, colM, colL, nullptr, pm, pl, logits, nullptr, V, S, nblk);
    LAUNCH_OK("softmax_cols combine");
    if (vec_ok) hipLaunchKernelGGL(softmax_out_kernel<4>, grid, dim3(CE_THREADS), 0, g_ctx.stream, probs, logits, colM, colL, V, S, rpb);
    else hipLaunchKernelGGL(softmax_out_kernel<1>, grid, dim3(CE_THREADS), 0, g_ctx.stream, probs, logits, colM, colL, V, S, rpb);
    LAUNCH_OK("softmax_cols out");
    return 0;
}

MI355_API int mi355_nll_from_probs_dev(float *dlogits, float *loss_dev, const float *probs, const int32_t *targets, int V,
                                       int S) {
    if (!mi355_ready("nll_from_probs")) return -1;
    if (!dlogits || !loss_dev || !probs || !targets) return mi355_fail("nll_from_probs: NULL pointer");
    if (V <= 0 || S <= 0) return mi355_fail("nll_from_probs: bad shape V=%d S=%d", V, S);
    const size_t n = (size_t)V * S;
    hipLaunchKernelGGL(nll_loss_kernel, dim3(1), dim3(CE_THREADS), 0, g_ctx.stream, loss_dev, probs, targets, V, S);
    LAUNCH_OK("nll_from_probs loss");
    const bool vec_ok = (S % 4 == 0) && aligned16(probs) && aligned16(dlogits);
    if (vec_ok)
        hipLaunchKernelGGL(nll_grad_kernel<4>, dim3((unsigned)ceil_div(n / 4, 256)), dim3(256), 0, g_ctx.stream, dlogits,
                           probs, targets, V, S, n, 1.0f / (float)S);
    else
        hipLaunchKernelGGL(nll_grad_kernel<1>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, g_ctx.stream, dlogits, probs,
                           targets, V, S, n, 1.0f / (float)S);
    LAUNCH_OK("nll_from_probs grad");
    return 0;
}

MI355_API int mi355_softmax_ce_dev(float *dlogits, float *loss_dev, const float *logits, const int32_t *targets, int V,
                                   int S, float grad_scale) {
    return ce_run<float>("softmax_ce", dlogits, loss_dev, logits, targets, V, S, grad_scale);
}

// bfloat16 logits and gradient (bit patterns as uint16_t); the loss and every intermediate stay fp32.
MI355_API int mi355_softmax_ce_bf16_dev(uint16_t *dlogits, float *loss_dev, const uint16_t *logits, const int32_t *targets,
                                        int V, int S, float grad_scale) {
    return ce_run<uint16_t>("softmax_ce_bf16", dlogits, loss_dev, logits, targets, V, S, grad_scale);
}
