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
#include "tile.h"

#include <math.h>
#include <type_traits>

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
__device__ __forceinline__ float bf_widen(unsigned bits16) { return bf_to_f(bits16); }
__device__ __forceinline__ unsigned bf_narrow(float f) { return f_to_bf(f); }      // round to nearest even; NaN stays NaN
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

// ---- the one-launch form: logits stay on the chip between the two passes ---------------------------------------
// The register files and the LDS of the chip together hold more than the logits of the classifier
// ([151936][256] fp32 = 156 MB; 256 compute units x (512 KB of registers + 160 KB of LDS) = 172 MB), so one launch
// with ONE workgroup of 1024 threads per compute unit can read most rows once: a workgroup owns a block of rows of
// one 64-column strip (256-byte row pieces), keeps its last 16 row steps in registers and the 9 before them in LDS
// (25 of the 38 steps of the Qwen3 vocabulary; all of them for 32000 rows, and for bfloat16 storage, whose rows take
// half the space), and reads only the remainder a second time.  Measured at [151936][256]: 69 us against 84 us for
// the three launches (bfloat16: 61 against 99).  The (max, sum exp) partials of the workgroups of a strip (its members)
// are exchanged through tagged 8-byte slots as in the clustered RMSNorm (norm_cluster.h): one relaxed agent-scope
// atomic {fp32 value, launch tag} per slot, a launch counter per workgroup number, nothing to clear, a bounded
// wait.  A member whose wait for a partner expires recomputes that partner's partial from memory with the same
// operations in the same order (same bits), so every member of a strip normalises with identical column sums.
constexpr int CR_THREADS = 1024;
constexpr int CR_W = 64;                     // columns per strip
constexpr int CR_RPS = CR_THREADS / 16;      // rows per step: 16 lanes x 16 B per row piece
constexpr int CR_NW = CR_THREADS / 64;
constexpr int CR_MAX_SPLIT = 64;             // members per strip
constexpr int CR_MAX_STRIPS = 16;
constexpr int CR_LOSS_SLOT = 2 * CR_W;       // after the 64 maxima and 64 sums
constexpr int CR_STRIDE = 136;               // slots per workgroup number
constexpr int CR_MAX_WG = 512;
constexpr int CR_SUB = 4;                    // rows per lane and online step beyond the register rows
constexpr int CR_MAX_STEPS = 64;             // beyond that most rows would be read twice anyway
constexpr size_t CR_XCH_BYTES = (size_t)CR_MAX_WG * CR_STRIDE * 8 + (size_t)CR_MAX_WG * 4 + 256;

struct CeXch {
    unsigned long long *slots;     // [CR_MAX_WG][CR_STRIDE]
    unsigned *cnt;                 // [CR_MAX_WG] launches completed by each workgroup number
    int *fallbacks;                // workgroups whose bounded wait expired, ever (diagnostic)
};
// Storage of the logits: element type, the register form of a lane's four columns of one row (fp32: 16 bytes;
// bfloat16: two packed words, widened at each use), loads, the store that rounds, and how many row steps a
// workgroup keeps in registers (64 of a lane's 128 in both cases) and in LDS (144 KB in both cases).
struct CrF32 {
    typedef float T;
    typedef v4f Raw;
    static constexpr int K_REG = 16, K_LDS = 9;
    static __device__ __forceinline__ Raw ld(const T *p) { return ld4(p); }
    static __device__ __forceinline__ Raw ld_nt(const T *p) { return ld4_nt(p); }
    static __device__ __forceinline__ Raw ninf() { Raw r = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}; return r; }
    static __device__ __forceinline__ float at(const Raw &r, int j) { return r[j]; }
    static __device__ __forceinline__ void st_nt(T *p, const float (&o)[4]) { Raw r = {o[0], o[1], o[2], o[3]}; st4_nt(p, r); }
    static __device__ __forceinline__ void forget(Raw &) {}
};
struct CrBf16 {
    typedef uint16_t T;
    typedef v2u Raw;
    static constexpr int K_REG = 32, K_LDS = 18;
    static __device__ __forceinline__ Raw ld(const T *p) { return *reinterpret_cast<const v2u *>(p); }
    static __device__ __forceinline__ Raw ld_nt(const T *p) { return __builtin_nontemporal_load(reinterpret_cast<const v2u *>(p)); }
    static __device__ __forceinline__ Raw ninf() { Raw r = {0xff80ff80u, 0xff80ff80u}; return r; }
    static __device__ __forceinline__ float at(const Raw &r, int j) { return bf_to_f((j & 1) ? r[j >> 1] >> 16 : r[j >> 1] & 0xffffu); }
    static __device__ __forceinline__ void st_nt(T *p, const float (&o)[4]) {
        Raw r = {f2_to_bf2(o[0], o[1]), f2_to_bf2(o[2], o[3])};
        __builtin_nontemporal_store(r, reinterpret_cast<v2u *>(p));
    }
    // Tells the compiler nothing about the words' contents from here on, so that the widened copies made for the
    // first pass are dropped instead of being kept alive for the second (they would double the register rows).
    static __device__ __forceinline__ void forget(Raw &r) {
        unsigned a = r[0], b = r[1];
        asm volatile("" : "+v"(a), "+v"(b));
        r[0] = a; r[1] = b;
    }
};
template <typename T>
struct CrGeo {
    const T *logits;
    int V, S, strips, csplit, Rm, K;   // Rm rows per member, K = ceil(Rm / CR_RPS) row steps
};

// (m, l) <- (m, l) merged with N more values: the online-softmax step
template <int N>
__device__ __forceinline__ void online_update(float &m, float &l, const float (&x)[N]) {
    float tm = x[0];
#pragma unroll
    for (int k = 1; k < N; k++) tm = fmaxf(tm, x[k]);
    const float nm = fmaxf(m, tm);
    if (nm > -INFINITY) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < N; k++) s += exp_neg_fast(x[k] - nm);     // exp(-inf) = 0 for masked rows
        l = l * exp_neg(m - nm) + s;
        m = nm;
    }
}
__device__ __forceinline__ void merge_pair(float &m, float &l, float m1, float l1) {
    const float nm = fmaxf(m, m1);
    if (nm > -INFINITY) {
        l = l * exp_neg(m - nm) + l1 * exp_neg(m1 - nm);
        m = nm;
    }
}

// Sixteen (max, sum) pairs of one column -> their merge: the maximum, then the sums rescaled to it (sixteen
// independent exponentials) and added in order.
__device__ __forceinline__ void cr_merge16(const float (*wm)[CR_W], const float (*wl)[CR_W], int c, float &M, float &L) {
    float mm[CR_NW];
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < CR_NW; w++) { mm[w] = wm[w][c]; mx = fmaxf(mx, mm[w]); }
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < CR_NW; w++) acc += wl[w][c] * exp_neg(mm[w] - mx);     // an empty part has sum 0
    M = mx;
    L = acc;
}

// The (max, sum exp) partial of member p of a strip over its rows, for the 64 columns of the strip: valid in
// threads 0..63 (thread t = column t) on return.  Of a member's K row steps the last K_REG are the register rows,
// the K_LDS before them the LDS rows, and the first kL = K - K_REG - K_LDS the rows that are read twice.  A lane
// folds its rows into its running (max, sum) four at a time, in row order: the rows before the register rows, then
// the register rows.  KEEP: this workgroup's own rows; the loads run ahead of the arithmetic.
// Otherwise nothing is kept: one column and one
// group of four rows at a time, the same operations on the same values in the same order (same bits) in a handful
// of registers, because the caller's own rows stay live in theirs.
template <typename ST, bool KEEP, bool NT = false>
__device__ __forceinline__ void cr_member_partial(const CrGeo<typename ST::T> &g, int strip, int p, typename ST::Raw (&xr)[ST::K_REG],
                                                  typename ST::Raw (*lrow)[CR_THREADS],
                                                  float (*wm)[CR_W], float (*wl)[CR_W], float &Mout, float &Lout) {
    typedef typename ST::Raw Raw;
    constexpr int K_REG = ST::K_REG, K_LDS = ST::K_LDS;
    static_assert(K_REG % CR_SUB == 0, "the register rows fold four at a time");
    const int lc = threadIdx.x & 15, row0 = threadIdx.x >> 4, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int v_lo = p * g.Rm;
    constexpr int rs = CR_RPS;                                    // rows between a lane's consecutive rows
    // this lane holds the member's rows row0 + rs*k; they exist while rs*k < lim
    const int lim = min(g.V, v_lo + g.Rm) - v_lo - row0;
    const int kR = max(0, g.K - K_REG), kL = max(0, kR - K_LDS);
    // a row piece = (uniform address of row v_lo + rs*k of the strip) + (this lane's fixed 32-bit offset)
    const typename ST::T *base = g.logits + ((size_t)v_lo * g.S + (size_t)strip * CR_W);
    const unsigned loff = (unsigned)row0 * (unsigned)g.S + (unsigned)lc * 4u;
    const size_t step = (size_t)rs * g.S;
    const Raw ninf = ST::ninf();
    float m[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; j++) { m[j] = -INFINITY; l[j] = 0.f; }
    if constexpr (KEEP) {
        // rows that stay on the chip may be read past the cache (they are not read again); the others stay cached
        auto loadg = [&](Raw (&t)[CR_SUB], int k0) {
#pragma unroll
            for (int u = 0; u < CR_SUB; u++) {
                const int k = k0 + u;
                if (k < kR && rs * k < lim) t[u] = (NT && k >= kL) ? ST::ld_nt(base + k * step + loff) : ST::ld(base + k * step + loff);
                else t[u] = ninf;
            }
        };
        auto foldg = [&](const Raw (&t)[CR_SUB]) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float x4[CR_SUB];
#pragma unroll
                for (int u = 0; u < CR_SUB; u++) x4[u] = ST::at(t[u], j);
                online_update<CR_SUB>(m[j], l[j], x4);
            }
        };
        auto keepg = [&](const Raw (&t)[CR_SUB], int k0) {
#pragma unroll
            for (int u = 0; u < CR_SUB; u++)
                if (k0 + u >= kL && k0 + u < kR) lrow[k0 + u - kL][threadIdx.x] = t[u];
        };
        // the register rows are asked for first and folded last: they are in flight while the other rows stream
        // through two groups of four
#pragma unroll
        for (int i = 0; i < K_REG; i++) {
            const int k = kR + i;
            xr[i] = rs * k < lim ? (NT ? ST::ld_nt(base + k * step + loff) : ST::ld(base + k * step + loff)) : ninf;
        }
        {
            Raw ta[CR_SUB], tb[CR_SUB];
            loadg(ta, 0);
            loadg(tb, CR_SUB);
            for (int k0 = 0; k0 < kR; k0 += 2 * CR_SUB) {
                keepg(ta, k0);
                foldg(ta);
                loadg(ta, k0 + 2 * CR_SUB);
                if (k0 + CR_SUB < kR) {
                    keepg(tb, k0 + CR_SUB);
                    foldg(tb);
                }
                loadg(tb, k0 + 3 * CR_SUB);
            }
        }
#pragma unroll
        for (int c = 0; c < K_REG / CR_SUB; c++) {
            // (a member with fewer row steps than registers for them: the groups past its last step hold nothing,
            // and folding nothing leaves (max, sum) as they are: skipped, for the exponentials' sake)
            if (kR + c * CR_SUB >= g.K) continue;
            Raw t[CR_SUB];
#pragma unroll
            for (int u = 0; u < CR_SUB; u++) t[u] = xr[c * CR_SUB + u];
            foldg(t);
        }
#pragma unroll
        for (int i = 0; i < K_REG; i++) ST::forget(xr[i]);
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float mj = -INFINITY, lj = 0.f;
            auto part = [&](int kbeg, int kend) {
#pragma unroll 1
                for (int k0 = kbeg; k0 < kend; k0 += CR_SUB) {
                    float x4[CR_SUB];
#pragma unroll
                    for (int u = 0; u < CR_SUB; u++) {
                        const int k = k0 + u;
                        x4[u] = (k < kend && rs * k < lim) ? ld_one(base + k * step + loff + j) : -INFINITY;
                    }
                    online_update<CR_SUB>(mj, lj, x4);
                }
            };
            part(0, kR);
            part(kR, kR + K_REG);
            m[j] = mj;
            l[j] = lj;
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the four row groups of a wave, then the sixteen waves in order
#pragma unroll
    for (int j = 0; j < 4; j++) {
        merge_pair(m[j], l[j], lane_xor<16>(m[j]), lane_xor<16>(l[j]));
        merge_pair(m[j], l[j], lane_xor<32>(m[j]), lane_xor<32>(l[j]));
    }
    if (lane < 16) {
#pragma unroll
        for (int j = 0; j < 4; j++) { wm[wave][lc * 4 + j] = m[j]; wl[wave][lc * 4 + j] = l[j]; }
    }
    __syncthreads();
    if (threadIdx.x < CR_W) cr_merge16(wm, wl, threadIdx.x, Mout, Lout);
    __syncthreads();
}

constexpr int CR_MPG = CR_MAX_SPLIT / CR_NW;     // members per group of 64 threads (thread = group, column)

// The members' partials, four members per thread (pm, pl: member grp * mpg + q of column c) -> the strip's column
// maxima and sums: the maximum first, then every member's sum rescaled to it and added in a fixed order (within the
// sixteen groups, then the groups); valid in threads 0..63 on return.
__device__ __forceinline__ void cr_merge_members(const float (&pm)[CR_MPG], const float (&pl)[CR_MPG], float (*wm)[CR_W],
                                                 float (*wl)[CR_W], float &Mout, float &Lout) {
    const int c = threadIdx.x & 63, grp = threadIdx.x >> 6;
    float M = pm[0];
#pragma unroll
    for (int q = 1; q < CR_MPG; q++) M = fmaxf(M, pm[q]);
    wm[grp][c] = M;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < CR_NW; w++) M = fmaxf(M, wm[w][c]);
    float L = 0.f;
#pragma unroll
    for (int q = 0; q < CR_MPG; q++) L += pl[q] * exp_neg(pm[q] - M);      // a member that is absent has sum 0
    wl[grp][c] = L;
    __syncthreads();
    if (threadIdx.x < CR_W) {
        L = wl[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < CR_NW; w++) L += wl[w][threadIdx.x];
        Mout = M;
        Lout = L;
    }
    __syncthreads();
}

// Sum over the strip's columns of -log(p[target] + 1e-10), by wave 0 (every lane of it ends with the sum).
template <typename T>
__device__ __forceinline__ float cr_strip_loss(const CrGeo<T> &g, int strip, const int32_t *targets, float M, float inv) {
    const int t = strip * CR_W + threadIdx.x;
    const int tg = targets[t];
    float loss = 0.f;
    if (tg >= 0 && tg < g.V) {
        const float p = exp_neg(ld_one(g.logits + (size_t)tg * g.S + t) - M) * inv;
        loss = -logf(p + 1e-10f);
    }
    return wave_sum_far_first(loss);
}

// One bounded wait for a tagged slot.  false: the tag did not arrive within spin_ticks.
__device__ __forceinline__ bool cr_wait_slot(const unsigned long long *sp, unsigned want, int spin_ticks, float &value) {
    const long long t0 = wall_clock64();
    for (;;) {
        const unsigned long long pk = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((unsigned)(pk >> 32) == want) { value = __uint_as_float((unsigned)pk); return true; }
        if (wall_clock64() - t0 >= (long long)spin_ticks) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}

// grid: strips * csplit workgroups, all resident at once (one per compute unit).  Workgroup b: strip b % strips,
// member b / strips, so that the workgroups that read the pieces of one row are neighbours in time.
template <typename ST, bool NT>
__global__ __launch_bounds__(CR_THREADS) void ce_resident_kernel(typename ST::T *__restrict__ dlogits,
                                                                 const typename ST::T *__restrict__ logits,
                                                                 const int32_t *__restrict__ targets, int V, int S,
                                                                 int strips, int csplit, int Rm, int K, float invS,
                                                                 float grad_scale, float *__restrict__ loss_out, CeXch ws,
                                                                 int spin_ticks, int take_nothing) {
    typedef typename ST::Raw Raw;
    constexpr int K_REG = ST::K_REG, K_LDS = ST::K_LDS;
    __shared__ Raw lrow[K_LDS][CR_THREADS];
    __shared__ float wm[CR_NW][CR_W], wl[CR_NW][CR_W];
    __shared__ float fb[2][CR_W];                  // one member's partial on its way to the threads that hold it
    __shared__ float fM[CR_W], fInv[CR_W];
    __shared__ float strip_loss[CR_MAX_STRIPS];
    __shared__ unsigned want[CR_MAX_SPLIT], want_leader[CR_MAX_STRIPS];
    __shared__ int failed[CR_MAX_SPLIT];
    __shared__ int any_failed;
    const int tid = threadIdx.x;
    // Workgroups are dealt to the eight XCDs in turn.  The workgroups that read the pieces of one row run at the
    // same time and, where the split allows, on one XCD, so that each L2 sees whole rows.
    int strip = blockIdx.x % strips, me = blockIdx.x / strips;
    if (csplit % 8 == 0) {
        const int xcd = blockIdx.x % 8, q = blockIdx.x / 8;
        strip = q % strips;
        me = xcd + 8 * (q / strips);
    }
    const int b = me * strips + strip;           // the workgroup number that owns slots and counter
    const CrGeo<typename ST::T> g = {logits, V, S, strips, csplit, Rm, K};
    if (tid < csplit) { want[tid] = ws.cnt[tid * strips + strip] + 1u; failed[tid] = 0; }
    if (tid < strips) want_leader[tid] = ws.cnt[tid] + 1u;          // member 0 of strip s is workgroup s
    if (tid == 0) any_failed = 0;
    const unsigned my_tag = ws.cnt[b] + 1u;
    __syncthreads();

    // ---- pass 1: this member's rows, kept; its partial published
    Raw xr[K_REG];
    float Mp = -INFINITY, Lp = 0.f;
    cr_member_partial<ST, true, NT>(g, strip, me, xr, lrow, wm, wl, Mp, Lp);
    if (tid < CR_W) {
        unsigned long long *mine = ws.slots + (size_t)b * CR_STRIDE;
        __hip_atomic_store(mine + tid, ((unsigned long long)my_tag << 32) | __float_as_uint(Mp), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + CR_W + tid, ((unsigned long long)my_tag << 32) | __float_as_uint(Lp), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    // ---- every member's partial.  Thread (group, column) fetches the (max, sum) slots of the group's members for
    // its column: eight slots.  The loads of a round go out together, so a round costs one trip to the memory side
    // however many of the eight are still missing.
    const int mc = tid & 63, mgrp = tid >> 6;
    const int mpg = (csplit + CR_NW - 1) / CR_NW;                      // members per group, at most CR_MPG
    float pm[CR_MPG], pl[CR_MPG];
    {
        unsigned pend = 0;
#pragma unroll
        for (int q = 0; q < CR_MPG; q++) {
            pm[q] = -INFINITY;
            pl[q] = 0.f;
            if (q < mpg && mgrp * mpg + q < csplit) pend |= 3u << (2 * q);
        }
        const long long t0 = wall_clock64();
        if (take_nothing) {                    // test mode: every partner counts as late, whatever its slots hold
#pragma unroll
            for (int f = 0; f < 2 * CR_MPG; f++)
                if ((pend >> f) & 1u) failed[mgrp * mpg + (f >> 1)] = 1;
            any_failed = 1;
            pend = 0;
        }
        while (pend) {
            unsigned long long pk[2 * CR_MPG];
#pragma unroll
            for (int f = 0; f < 2 * CR_MPG; f++) {
                const int p = mgrp * mpg + (f >> 1);
                if ((pend >> f) & 1u)
                    pk[f] = __hip_atomic_load(ws.slots + (size_t)(p * strips + strip) * CR_STRIDE + (f & 1) * CR_W + mc,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int f = 0; f < 2 * CR_MPG; f++) {
                const int p = mgrp * mpg + (f >> 1);
                if (((pend >> f) & 1u) && (unsigned)(pk[f] >> 32) == want[p]) {
                    if (f & 1) pl[f >> 1] = __uint_as_float((unsigned)pk[f]);
                    else pm[f >> 1] = __uint_as_float((unsigned)pk[f]);
                    pend &= ~(1u << f);
                }
            }
            if (pend) {
                if (wall_clock64() - t0 >= (long long)spin_ticks) {
#pragma unroll
                    for (int f = 0; f < 2 * CR_MPG; f++)
                        if ((pend >> f) & 1u) failed[mgrp * mpg + (f >> 1)] = 1;
                    any_failed = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        }
    }
    __syncthreads();
    if (any_failed) {                                                // the same for every thread: read after the barrier
        if (tid == 0) atomicAdd(ws.fallbacks, 1);
        for (int p = 0; p < csplit; p++) {
            if (failed[p]) {
                float M2 = -INFINITY, L2 = 0.f;
                cr_member_partial<ST, false>(g, strip, p, xr, lrow, wm, wl, M2, L2);
                if (tid < CR_W) { fb[0][tid] = M2; fb[1][tid] = L2; }
                __syncthreads();
#pragma unroll
                for (int q = 0; q < CR_MPG; q++)
                    if (q < mpg && mgrp * mpg + q == p) { pm[q] = fb[0][mc]; pl[q] = fb[1][mc]; }
                __syncthreads();
            }
        }
    }
    float Mc = 0.f, Lc = 1.f;
    cr_merge_members(pm, pl, wm, wl, Mc, Lc);
    if (tid < CR_W) {
        const float inv = 1.0f / Lc;
        fM[tid] = Mc;
        fInv[tid] = inv;
        if (me == 0) {                                               // the strip's leader also forms its loss term
            const float ls = cr_strip_loss(g, strip, targets, Mc, inv);
            if (tid == 0) {
                strip_loss[strip] = ls;
                __hip_atomic_store(ws.slots + (size_t)b * CR_STRIDE + CR_LOSS_SLOT,
                                   ((unsigned long long)my_tag << 32) | __float_as_uint(ls), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();

    // ---- pass 2: dlogits = (exp(l - M) / L - onehot) / S * grad_scale
    {
        const int lc = tid & 15;
        int row0 = tid >> 4;
        asm volatile("" : "+v"(row0));     // the row masks are formed again here instead of being kept from pass 1
        const int v_lo = me * Rm;
        constexpr int rs = CR_RPS;
        const int lim = min(V, v_lo + Rm) - v_lo - row0;           // this lane's rows row0 + rs*k exist while rs*k < lim
        const int kR = max(0, K - K_REG), kL = max(0, kR - K_LDS);
        const typename ST::T *src = logits + ((size_t)v_lo * S + (size_t)strip * CR_W);
        typename ST::T *dst = dlogits + ((size_t)v_lo * S + (size_t)strip * CR_W);
        const unsigned loff = (unsigned)row0 * (unsigned)S + (unsigned)lc * 4u;
        const size_t step = (size_t)rs * S;
        float M[4], inv[4], sc[4];
        int tk[4];                         // the target's row is this lane's row 64k when tk == 64k
#pragma unroll
        for (int j = 0; j < 4; j++) {
            M[j] = fM[lc * 4 + j];
            inv[j] = fInv[lc * 4 + j];
            const int tg = targets[strip * CR_W + lc * 4 + j];
            const bool ok = tg >= 0 && tg < V;
            tk[j] = ok ? tg - v_lo - row0 : -1;
            sc[j] = ok ? invS : 1.0f;      // an out-of-range target leaves the column unscaled (stories_cpu_ops.h:98)
        }
        auto emit = [&](int k, const Raw &x) {
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float pj = exp_neg(ST::at(x, j) - M[j]) * inv[j];
                if (tk[j] == rs * k) pj -= 1.0f;
                pj = pj * sc[j];
                if (grad_scale != 1.0f) pj = pj * grad_scale;
                o[j] = pj;
            }
            ST::st_nt(dst + k * step + loff, o);
        };
        // the rows read a second time run up to sixteen ahead of their use, in the registers that the register
        // rows leave as they are written out
        auto loadg = [&](Raw (&t)[CR_SUB], int k0) {
#pragma unroll
            for (int u = 0; u < CR_SUB; u++)
                if (k0 + u < kL && rs * (k0 + u) < lim) t[u] = ST::ld_nt(src + (k0 + u) * step + loff);
        };
        auto emitg = [&](const Raw (&t)[CR_SUB], int k0) {
#pragma unroll
            for (int u = 0; u < CR_SUB; u++)
                if (k0 + u < kL && rs * (k0 + u) < lim) emit(k0 + u, t[u]);
        };
        Raw t0[CR_SUB], t1[CR_SUB], t2[CR_SUB], t3[CR_SUB];
        loadg(t0, 0);
#pragma unroll
        for (int i = 0; i < K_REG; i++) {
            if (rs * (kR + i) < lim) emit(kR + i, xr[i]);
            __builtin_amdgcn_sched_barrier(0);       // one row at a time: the scheduler would otherwise hold them all
        }
        loadg(t1, CR_SUB);
        loadg(t2, 2 * CR_SUB);
        loadg(t3, 3 * CR_SUB);
#pragma unroll
        for (int i = 0; i < K_LDS; i++) {
            if (kL + i < kR && rs * (kL + i) < lim) emit(kL + i, lrow[i][tid]);
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int k0 = 0; k0 < kL; k0 += 4 * CR_SUB) {
            emitg(t0, k0);
            loadg(t0, k0 + 4 * CR_SUB);
            emitg(t1, k0 + CR_SUB);
            loadg(t1, k0 + 5 * CR_SUB);
            emitg(t2, k0 + 2 * CR_SUB);
            loadg(t2, k0 + 6 * CR_SUB);
            emitg(t3, k0 + 3 * CR_SUB);
            loadg(t3, k0 + 7 * CR_SUB);
        }
    }

    // ---- the loss: workgroup 0 adds the strips' terms in order; by now the other leaders have long published
    if (b == 0) {
        __syncthreads();
        if (tid < strips) failed[tid] = 0;
        __syncthreads();
        if (tid > 0 && tid < strips) {
            float val = 0.f;
            if (take_nothing || !cr_wait_slot(ws.slots + (size_t)tid * CR_STRIDE + CR_LOSS_SLOT, want_leader[tid], spin_ticks, val))
                failed[tid] = 1;
            strip_loss[tid] = val;
        }
        __syncthreads();
        for (int s2 = 1; s2 < strips; s2++) {
            if (failed[s2]) {                                        // that strip's loss term from memory, the same way
                float qm[CR_MPG], ql[CR_MPG];
#pragma unroll
                for (int q = 0; q < CR_MPG; q++) { qm[q] = -INFINITY; ql[q] = 0.f; }
                for (int p = 0; p < csplit; p++) {
                    float M2 = -INFINITY, L2 = 0.f;
                    cr_member_partial<ST, false>(g, s2, p, xr, lrow, wm, wl, M2, L2);
                    if (tid < CR_W) { fb[0][tid] = M2; fb[1][tid] = L2; }
                    __syncthreads();
#pragma unroll
                    for (int q = 0; q < CR_MPG; q++)
                        if (q < mpg && mgrp * mpg + q == p) { qm[q] = fb[0][mc]; ql[q] = fb[1][mc]; }
                    __syncthreads();
                }
                float M3 = 0.f, L3 = 1.f;
                cr_merge_members(qm, ql, wm, wl, M3, L3);
                if (tid < CR_W) {
                    const float ls = cr_strip_loss(g, s2, targets, M3, 1.0f / L3);
                    if (tid == 0) strip_loss[s2] = ls;
                }
                __syncthreads();
            }
        }
        if (tid == 0) {
            float total = 0.f;
            for (int s2 = 0; s2 < strips; s2++) total += strip_loss[s2];
            *loss_out = total / (float)S;
        }
    }
    if (tid == 0) ws.cnt[b] = my_tag;
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
// Behind them, in the same array, lies the exchange area of the one-launch kernel (slots and launch counters, which
// must start at zero: the array is zero-initialised when the code object is loaded, and nothing ever clears it).
constexpr size_t CE_SCRATCH_BYTES = (size_t)2 << 20;
constexpr size_t CE_XCH_AREA = (size_t)1 << 20;
static_assert(CR_XCH_BYTES <= CE_XCH_AREA, "the exchange area must fit behind the partials");
constexpr int CE_MAX_DEVICES = 16;
}   // namespace
static __device__ __align__(256) unsigned char scratch[CE_SCRATCH_BYTES + CE_XCH_AREA];
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
    {
        // The one-launch form: whole 64-column strips, a lane's four columns in one aligned access, out of place (a
        // member that recomputes a partner's partial reads the partner's logits), and a vocabulary for which it
        // pays (ce_resident: 0 = V >= 4096, 1 = any V, -1 = never).  One workgroup per compute unit at most, so that
        // all of them are resident at once.
        typedef typename std::conditional<std::is_same<T, float>::value, CrF32, CrBf16>::type ST;
        const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
        const int strips_r = S / CR_W;
        const uintptr_t amask = 4 * sizeof(T) - 1;
        unsigned char *base = (g_ctx.device >= 0 && g_ctx.device < CE_MAX_DEVICES) ? g_scratch_ptr[g_ctx.device] : nullptr;
        if (g_ctx.ce_resident >= 0 && base && S % CR_W == 0 && strips_r <= CR_MAX_STRIPS && (const void *)dlogits != (const void *)logits &&
            (((uintptr_t)logits | (uintptr_t)dlogits) & amask) == 0 && (V >= 4096 || g_ctx.ce_resident > 0)) {
            const int csplit = cu / strips_r < CR_MAX_SPLIT ? cu / strips_r : CR_MAX_SPLIT;
            const int Rm = csplit > 0 ? (int)ceil_div((size_t)V, (size_t)csplit) : 0;
            const int K = (int)ceil_div((size_t)Rm, (size_t)CR_RPS);
            if (csplit >= 2 && csplit * strips_r <= CR_MAX_WG && csplit * strips_r <= cu && K <= CR_MAX_STEPS) {
                CeXch xch;
                xch.slots = (unsigned long long *)(base + CE_SCRATCH_BYTES);
                xch.cnt = (unsigned *)(base + CE_SCRATCH_BYTES + (size_t)CR_MAX_WG * CR_STRIDE * 8);
                xch.fallbacks = (int *)(base + CE_SCRATCH_BYTES + (size_t)CR_MAX_WG * CR_STRIDE * 8 + (size_t)CR_MAX_WG * 4);
                hipLaunchKernelGGL((ce_resident_kernel<ST, true>), dim3((unsigned)(csplit * strips_r)), dim3(CR_THREADS), 0,
                                   g_ctx.stream, dlogits, logits, targets, V, S, strips_r, csplit, Rm, K, 1.0f / (float)S,
                                   grad_scale, loss_dev, xch, mi355_exchange_spin_ticks() < 0 ? 0 : mi355_exchange_spin_ticks(),
                                   g_ctx.xch_take_nothing > 0 ? 1 : 0);
                LAUNCH_OK("softmax_ce (one launch)");
                return 0;
            }
        }
    }
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

int *mi355_ce_fallbacks_dev(void) {
    unsigned char *base = (g_ctx.ready && g_ctx.device >= 0 && g_ctx.device < CE_MAX_DEVICES) ? g_scratch_ptr[g_ctx.device] : nullptr;
    return base ? (int *)(base + CE_SCRATCH_BYTES + (size_t)CR_MAX_WG * CR_STRIDE * 8 + (size_t)CR_MAX_WG * 4) : nullptr;
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
