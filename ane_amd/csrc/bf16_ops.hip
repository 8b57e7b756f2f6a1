// bf16_ops.hip — optional bfloat16-storage variants of the streaming and normalisation ops.
//
// Same arithmetic as the fp32 kernels (every value is widened to fp32 on load, all sums and the
// weight gradients stay fp32, norm weights stay fp32); only the activations in HBM are bfloat16, which
// halves the bytes these memory-bound ops move.  Results round to nearest even on store, so they agree
// with the fp32 ops run on the same (bf16-representable) inputs to within bf16 rounding, 2^-9 relative.
// bf16 values travel through the C-ABI as uint16_t bit patterns: the upper half of the fp32 pattern.
//
// One lane handles 8 contiguous elements: one 128-bit access on the bf16 side.
#include "common.h"
#include "tile.h"
#include "norm_cluster.h"

#include <math.h>

namespace {

constexpr int BT = 256;

// ---- converts (rectangles, as the fp16 staging converts) ----
template <int VEC>
__global__ __launch_bounds__(BT) void cvt_f32_bf16_kernel(bf16_t *__restrict__ dst, size_t dst_ld,
                                                          const float *__restrict__ src, size_t src_ld, size_t colg,
                                                          size_t total) {
    const size_t i = (size_t)blockIdx.x * BT + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / colg, g = i - r * colg;
    float v[VEC];
    if constexpr (VEC == 8) {
        const v4f a = ld4_nt(src + r * src_ld + 8 * g), b = ld4_nt(src + r * src_ld + 8 * g + 4);
#pragma unroll
        for (int j = 0; j < 4; j++) { v[j] = a[j]; v[4 + j] = b[j]; }
    } else {
        v[0] = src[r * src_ld + g];
    }
    stb<VEC>(dst + r * dst_ld + VEC * g, v);
}

template <int VEC>
__global__ __launch_bounds__(BT) void cvt_bf16_f32_kernel(float *__restrict__ dst, size_t dst_ld,
                                                          const bf16_t *__restrict__ src, size_t src_ld, size_t colg,
                                                          size_t total) {
    const size_t i = (size_t)blockIdx.x * BT + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / colg, g = i - r * colg;
    float v[VEC];
    ldb<VEC, true>(v, src + r * src_ld + VEC * g);
    if constexpr (VEC == 8) {
        v4f a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
        st4_nt(dst + r * dst_ld + 8 * g, a);
        st4_nt(dst + r * dst_ld + 8 * g + 4, b);
    } else {
        dst[r * dst_ld + g] = v[0];
    }
}

// ---- SwiGLU and the residual family ----
__device__ __forceinline__ float sigmoid_ref(float h) { return 1.0f / (1.0f + expf(-h)); }

template <int VEC>
__global__ __launch_bounds__(BT) void swiglu_fwd_bf16_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ h1,
                                                             const bf16_t *__restrict__ h3, size_t nv) {
    const size_t i = (size_t)blockIdx.x * BT + threadIdx.x;
    if (i >= nv) return;
    float a[VEC], b[VEC], o[VEC];
    ldb<VEC, true>(a, h1 + VEC * i);
    ldb<VEC, true>(b, h3 + VEC * i);
#pragma unroll
    for (int j = 0; j < VEC; j++) o[j] = (a[j] * sigmoid_ref(a[j])) * b[j];
    stb<VEC>(out + VEC * i, o);
}

template <int VEC>
__global__ __launch_bounds__(BT) void swiglu_bwd_bf16_kernel(bf16_t *__restrict__ dh1, bf16_t *__restrict__ dh3,
                                                             const bf16_t *__restrict__ ds,
                                                             const bf16_t *__restrict__ h1,
                                                             const bf16_t *__restrict__ h3, size_t nv) {
    const size_t i = (size_t)blockIdx.x * BT + threadIdx.x;
    if (i >= nv) return;
    float d[VEC], a[VEC], b[VEC], o1[VEC], o3[VEC];
    ldb<VEC, true>(d, ds + VEC * i);
    ldb<VEC, true>(a, h1 + VEC * i);
    ldb<VEC, true>(b, h3 + VEC * i);
#pragma unroll
    for (int j = 0; j < VEC; j++) {      // the op order of training/training_dynamic/train.m:541-553
        const float sig = sigmoid_ref(a[j]);
        o3[j] = d[j] * (a[j] * sig);
        float u = -(sig + -1.0f);
        u = a[j] * u;
        u = u + 1.0f;
        u = sig * u;
        o1[j] = (d[j] * b[j]) * u;
    }
    stb<VEC>(dh1 + VEC * i, o1);
    stb<VEC>(dh3 + VEC * i, o3);
}

template <int VEC, int MODE>
__global__ __launch_bounds__(BT) void axpby_bf16_kernel(bf16_t *y, const bf16_t *a, const bf16_t *b, float alpha,
                                                        size_t nv) {
    const size_t i = (size_t)blockIdx.x * BT + threadIdx.x;
    if (i >= nv) return;
    float x[VEC], z[VEC], o[VEC];
    ldb<VEC, true>(x, a + VEC * i);
    if (MODE != 1) ldb<VEC, true>(z, b + VEC * i);
#pragma unroll
    for (int j = 0; j < VEC; j++) o[j] = MODE == 0 ? z[j] * alpha + x[j] : MODE == 1 ? x[j] * alpha : x[j] + z[j];
    stb<VEC>(y + VEC * i, o);
}

// ---- RMSNorm forward / backward: the fp32 tile (workgroup = all C rows x a strip of columns) with 8-column lanes ----
template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void rms_fwd_bf16_kernel(bf16_t *__restrict__ y, const bf16_t *__restrict__ x,
                                                               const float *__restrict__ w, int C, int S, int strips,
                                                               int nblk, float eps, float invC) {
    constexpr int RPS = THREADS / LPR;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * (LPR < 64 ? LPR : 64) * VEC];
    const int blk = xcd_remap(blockIdx.x, nblk);
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, row0 = threadIdx.x / LPR;
    const int col = (strip * LPR + lc) * VEC;
    const bool col_ok = col < S;
    const size_t base = (size_t)slab * C * S + col;
    float acc[1][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = 0.f;
    if constexpr (CAP > 0) {
        typename RawT<VEC>::type xr[CAP];
        float wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            const bool ok = c < C && col_ok;
            xr[k] = ok ? ld_raw<VEC, true>(x + base + (size_t)c * S) : raw_zero<VEC>();
            wv[k] = ok ? w[c] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            float xv[VEC];
            unpack<VEC>(xv, xr[k]);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[0][j] += xv[j] * xv[j];
        }
        strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
#pragma unroll
        for (int k = 0; k < CAP; k++) forget<VEC>(xr[k]);
        float rr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                float xv[VEC], o[VEC];
                unpack<VEC>(xv, xr[k]);
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = (xv[j] * rr[j]) * wv[k];
                stb<VEC>(y + base + (size_t)c * S, o);
            }
        }
    } else {
        if (col_ok)
            for (int c = row0; c < C; c += RPS) {
                float t[VEC];
                ldb<VEC, false>(t, x + base + (size_t)c * S);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc[0][j] += t[j] * t[j];
            }
        strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
        float rr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
        if (col_ok)
            for (int c = row0; c < C; c += RPS) {
                float t[VEC], o[VEC];
                ldb<VEC, true>(t, x + base + (size_t)c * S);
                const float wc = w[c];
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = (t[j] * rr[j]) * wc;
                stb<VEC>(y + base + (size_t)c * S, o);
            }
    }
}

// dx by the reference's formula (variant 0, training/stories_cpu_ops.h:35-46) or the textbook one (variant 1);
// per-workgroup partial rows of dw (fp32) go to dw_part[blk][C].
template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void rms_bwd_bf16_kernel(bf16_t *dx, float *__restrict__ dw_part, const bf16_t *dy,
                                                               const bf16_t *__restrict__ x,
                                                               const float *__restrict__ w, int C, int S, int strips,
                                                               int nblk, float eps, float invC, int variant,
                                                               const bf16_t *res, bf16_t *dx2, float alpha2) {
    constexpr int RPS = THREADS / LPR;
    constexpr int NW = THREADS / 64;
    constexpr int G = LPR < 64 ? LPR : 64;
    __shared__ float lds[NW * 2 * G * VEC];
    const int blk = xcd_remap(blockIdx.x, nblk);
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, row0 = threadIdx.x / LPR;
    const int col = (strip * LPR + lc) * VEC;
    const bool col_ok = col < S;
    const size_t base = (size_t)slab * C * S + col;
    float *part = dw_part + (size_t)blk * C;
    float acc[2][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = acc[1][j] = 0.f;

    auto row_out = [&](int c, const float (&xr)[VEC], const float (&dyr)[VEC], float wc, const float (&rr)[VEC],
                       const float (&dotn)[VEC]) {
        float o[VEC];
        float p = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            if (variant == 0) o[j] = ((dyr[j] - xr[j] * dotn[j]) * rr[j]) * wc;
            else o[j] = (dyr[j] * wc) * rr[j] - (xr[j] * dotn[j]) * rr[j];
            p += (dyr[j] * xr[j]) * rr[j];
        }
        if (col_ok) {
            // res != NULL: the backward residual rides along, dx = rmsnorm_bwd + res, and dx2 = alpha2 * dx if asked
            // for (training/training_dynamic/train.m:586-595); res is read here, by the thread that then writes the
            // same elements of dx, so dx may lie over res
            if (res) {
                float rv[VEC];
                ldb<VEC, true>(rv, res + base + (size_t)c * S);
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = o[j] + rv[j];
            }
            stb<VEC>(dx + base + (size_t)c * S, o);
            if (dx2) {
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = o[j] * alpha2;
                stb<VEC>(dx2 + base + (size_t)c * S, o);
            }
        }
        p = group_sum<G>(p);
        if (lc == 0) part[c] = p;
    };

    if constexpr (CAP > 0) {
        typename RawT<VEC>::type xr[CAP], dr[CAP];
        float wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            const bool ok = c < C && col_ok;
            xr[k] = ok ? ld_raw<VEC, true>(x + base + (size_t)c * S) : raw_zero<VEC>();
            dr[k] = ok ? ld_raw<VEC, true>(dy + base + (size_t)c * S) : raw_zero<VEC>();
            wv[k] = ok ? w[c] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            float xv[VEC], dv[VEC];
            unpack<VEC>(xv, xr[k]);
            unpack<VEC>(dv, dr[k]);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                acc[0][j] += xv[j] * xv[j];
                acc[1][j] += (dv[j] * xv[j]) * wv[k];
            }
        }
        strip_reduce<VEC, LPR, THREADS, 2>(acc, lds);
#pragma unroll
        for (int k = 0; k < CAP; k++) { forget<VEC>(xr[k]); forget<VEC>(dr[k]); }
        float rr[VEC], dotn[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
            dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invC);
        }
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C) {                                                  // uniform per group of LPR lanes
                float xv[VEC], dv[VEC];
                unpack<VEC>(xv, xr[k]);
                unpack<VEC>(dv, dr[k]);
                row_out(c, xv, dv, wv[k], rr, dotn);
            }
        }
    } else {
        if (col_ok)
            for (int c = row0; c < C; c += RPS) {
                float a[VEC], b[VEC];
                ldb<VEC, false>(a, x + base + (size_t)c * S);
                ldb<VEC, false>(b, dy + base + (size_t)c * S);
                const float wc = w[c];
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    acc[0][j] += a[j] * a[j];
                    acc[1][j] += (b[j] * a[j]) * wc;
                }
            }
        strip_reduce<VEC, LPR, THREADS, 2>(acc, lds);
        float rr[VEC], dotn[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
            dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invC);
        }
        for (int c = row0; c < C; c += RPS) {                           // uniform per group of LPR lanes
            float a[VEC], b[VEC];
            if (col_ok) {
                ldb<VEC, true>(a, x + base + (size_t)c * S);
                ldb<VEC, true>(b, dy + base + (size_t)c * S);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) a[j] = b[j] = 0.f;
            }
            row_out(c, a, b, w[c], rr, dotn);
        }
    }
}

// ---- RoPE and per-head QK-RMSNorm + RoPE ----
// fp32 table row -> VEC floats (tables are shared by all heads and sequences: cached loads)
template <int VEC>
__device__ __forceinline__ void ldtab(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 8) {
        const v4f a = ld4(p), b = ld4(p + 4);
#pragma unroll
        for (int j = 0; j < 4; j++) { r[j] = a[j]; r[4 + j] = b[j]; }
    } else {
        r[0] = *p;
    }
}

// one lane = one interleaved row pair of one head x VEC columns; Q pair rows first, then K
template <int VEC>
__global__ __launch_bounds__(BT) void rope_bf16_kernel(bf16_t *q_out, bf16_t *k_out, const bf16_t *q_in,
                                                       const bf16_t *k_in, int heads, int /*kv_heads*/, int hd, int S,
                                                       int batch, const float *__restrict__ cos_t,
                                                       const float *__restrict__ sin_t, float sgn, size_t total) {
    const size_t idx = (size_t)blockIdx.x * BT + threadIdx.x;
    if (idx >= total) return;
    const int cols = S / VEC;
    const int cg = (int)(idx % cols);
    size_t pr = idx / cols;
    const int half = hd >> 1;
    const size_t q_rows = (size_t)batch * heads * half;
    const bf16_t *in = q_in;
    bf16_t *out = q_out;
    if (pr >= q_rows) { pr -= q_rows; in = k_in; out = k_out; }
    const int i = (int)(pr % half);
    const size_t row = (pr / half) * hd + 2 * i;
    const int s = cg * VEC;
    const size_t o0 = row * S + s;
    float v0[VEC], v1[VEC], c[VEC], sn[VEC], r0[VEC], r1[VEC];
    ldb<VEC, true>(v0, in + o0);
    ldb<VEC, true>(v1, in + o0 + S);
    ldtab<VEC>(c, cos_t + (size_t)i * S + s);
    ldtab<VEC>(sn, sin_t + (size_t)i * S + s);
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        const float sj = sn[j] * sgn;
        r0[j] = v0[j] * c[j] - v1[j] * sj;
        r1[j] = v0[j] * sj + v1[j] * c[j];
    }
    stb<VEC>(out + o0, r0);
    stb<VEC>(out + o0 + S, r1);
}

template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void qknorm_rope_fwd_bf16_kernel(
    bf16_t *__restrict__ q_out, bf16_t *__restrict__ k_out, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const float *__restrict__ wq, const float *__restrict__ wk, int hd, int S, int strips, int nq,
    const float *__restrict__ cos_t, const float *__restrict__ sin_t, float eps, float invhd) {
    constexpr int PPS = THREADS / LPR;   // row pairs per step
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * (LPR < 64 ? LPR : 64) * VEC];
    int blk = blockIdx.x;
    const bf16_t *in = q;
    const float *w = wq;
    bf16_t *out = q_out;
    if (blk >= nq) { blk -= nq; in = k; out = k_out; w = wk; }
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, p0 = threadIdx.x / LPR;
    const int col = (strip * LPR + lc) * VEC;
    const bool col_ok = col < S;
    const int half = hd >> 1;
    const size_t base = (size_t)slab * hd * S + col;
    typename RawT<VEC>::type r0[CAP], r1[CAP];
    float w0[CAP], w1[CAP];
    float acc[1][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = 0.f;
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        const bool ok = rp < half && col_ok;
        r0[kk] = ok ? ld_raw<VEC, true>(in + base + (size_t)(2 * rp) * S) : raw_zero<VEC>();
        r1[kk] = ok ? ld_raw<VEC, true>(in + base + (size_t)(2 * rp + 1) * S) : raw_zero<VEC>();
        w0[kk] = ok ? w[2 * rp] : 0.f;
        w1[kk] = ok ? w[2 * rp + 1] : 0.f;
        float x0[VEC], x1[VEC];
        unpack<VEC>(x0, r0[kk]);
        unpack<VEC>(x1, r1[kk]);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            acc[0][j] += x0[j] * x0[j];
            acc[0][j] += x1[j] * x1[j];
        }
    }
    strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) { forget<VEC>(r0[kk]); forget<VEC>(r1[kk]); }
    float rr[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invhd + eps);
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half && col_ok) {
            float x0[VEC], x1[VEC], cs[VEC], sn[VEC], o0[VEC], o1[VEC];
            unpack<VEC>(x0, r0[kk]);
            unpack<VEC>(x1, r1[kk]);
            ldtab<VEC>(cs, cos_t + (size_t)rp * S + col);
            ldtab<VEC>(sn, sin_t + (size_t)rp * S + col);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                const float y0 = (x0[j] * rr[j]) * w0[kk], y1 = (x1[j] * rr[j]) * w1[kk];
                o0[j] = y0 * cs[j] - y1 * sn[j];
                o1[j] = y0 * sn[j] + y1 * cs[j];
            }
            stb<VEC>(out + base + (size_t)(2 * rp) * S, o0);
            stb<VEC>(out + base + (size_t)(2 * rp + 1) * S, o1);
        }
    }
}

template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void qknorm_rope_bwd_bf16_kernel(
    bf16_t *dq, bf16_t *dk, float *__restrict__ part, const bf16_t *dq_out, const bf16_t *dk_out,
    const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const float *__restrict__ wq,
    const float *__restrict__ wk, int hd, int S, int strips, int nq, const float *__restrict__ cos_t,
    const float *__restrict__ sin_t, float eps, float invhd, int variant) {
    constexpr int PPS = THREADS / LPR;
    constexpr int NW = THREADS / 64;
    constexpr int G = LPR < 64 ? LPR : 64;
    __shared__ float lds[NW * 2 * G * VEC];
    int blk = blockIdx.x;
    float *prt = part + (size_t)blk * hd;
    const bf16_t *gin = dq_out, *xin = q;
    const float *w = wq;
    bf16_t *out = dq;
    if (blk >= nq) { blk -= nq; gin = dk_out; xin = k; out = dk; w = wk; }
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, p0 = threadIdx.x / LPR;
    const int col = (strip * LPR + lc) * VEC;
    const bool col_ok = col < S;
    const int half = hd >> 1;
    const size_t base = (size_t)slab * hd * S + col;
    typename RawT<VEC>::type rx0[CAP], rx1[CAP], rg0[CAP], rg1[CAP];
    float w0[CAP], w1[CAP];
    float acc[2][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = acc[1][j] = 0.f;

    // un-rotated upstream gradient of pair kk (training/training_dynamic/cpu_ops.h:179-180); zero where masked
    auto unrotate = [&](int kk, int rp, float (&d0)[VEC], float (&d1)[VEC]) {
        float g0[VEC], g1[VEC], c[VEC], sn[VEC];
        unpack<VEC>(g0, rg0[kk]);
        unpack<VEC>(g1, rg1[kk]);
        // (loaded from a valid address in every lane and zeroed by selects: with the loads under a branch the
        // compiler merges the two paths through scratch memory, and a kernel with scratch is dispatched later)
        const bool ok = rp < half && col_ok;
        const size_t to = ok ? (size_t)rp * S + col : 0;
        ldtab<VEC>(c, cos_t + to);
        ldtab<VEC>(sn, sin_t + to);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            c[j] = ok ? c[j] : 0.f;
            sn[j] = ok ? sn[j] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            d0[j] = g0[j] * c[j] + g1[j] * sn[j];
            d1[j] = (-g0[j]) * sn[j] + g1[j] * c[j];
        }
    };

#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        const bool ok = rp < half && col_ok;
        const size_t o = base + (size_t)(2 * rp) * S;
        rx0[kk] = ok ? ld_raw<VEC, true>(xin + o) : raw_zero<VEC>();
        rx1[kk] = ok ? ld_raw<VEC, true>(xin + o + S) : raw_zero<VEC>();
        rg0[kk] = ok ? ld_raw<VEC, true>(gin + o) : raw_zero<VEC>();
        rg1[kk] = ok ? ld_raw<VEC, true>(gin + o + S) : raw_zero<VEC>();
        w0[kk] = ok ? w[2 * rp] : 0.f;
        w1[kk] = ok ? w[2 * rp + 1] : 0.f;
        float x0[VEC], x1[VEC], d0[VEC], d1[VEC];
        unpack<VEC>(x0, rx0[kk]);
        unpack<VEC>(x1, rx1[kk]);
        unrotate(kk, rp, d0, d1);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            acc[0][j] += x0[j] * x0[j];
            acc[0][j] += x1[j] * x1[j];
            acc[1][j] += (d0[j] * x0[j]) * w0[kk];
            acc[1][j] += (d1[j] * x1[j]) * w1[kk];
        }
    }
    strip_reduce<VEC, LPR, THREADS, 2>(acc, lds);
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) { forget<VEC>(rx0[kk]); forget<VEC>(rx1[kk]); forget<VEC>(rg0[kk]); forget<VEC>(rg1[kk]); }
    float rr[VEC], dotn[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        rr[j] = 1.0f / sqrtf(acc[0][j] * invhd + eps);
        dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invhd);
    }
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half) {   // uniform over each group of LPR lanes
            float x0[VEC], x1[VEC], d0[VEC], d1[VEC], o0[VEC], o1[VEC];
            unpack<VEC>(x0, rx0[kk]);
            unpack<VEC>(x1, rx1[kk]);
            unrotate(kk, rp, d0, d1);
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                if (variant == 0) {
                    o0[j] = ((d0[j] - x0[j] * dotn[j]) * rr[j]) * w0[kk];
                    o1[j] = ((d1[j] - x1[j] * dotn[j]) * rr[j]) * w1[kk];
                } else {
                    o0[j] = (d0[j] * w0[kk]) * rr[j] - (x0[j] * dotn[j]) * rr[j];
                    o1[j] = (d1[j] * w1[kk]) * rr[j] - (x1[j] * dotn[j]) * rr[j];
                }
                s0 += (d0[j] * x0[j]) * rr[j];
                s1 += (d1[j] * x1[j]) * rr[j];
            }
            if (col_ok) {
                stb<VEC>(out + base + (size_t)(2 * rp) * S, o0);
                stb<VEC>(out + base + (size_t)(2 * rp + 1) * S, o1);
            }
            s0 = group_sum<G>(s0);
            s1 = group_sum<G>(s1);
            if (lc == 0) {
                prt[2 * rp] = s0;
                prt[2 * rp + 1] = s1;
            }
        }
    }
}

struct QkBf {
    int vec, lpr, threads, cap;
};

// Widest strip whose row pairs fit the (packed) register tile: 16 lanes x 8 columns = 256-byte row segments first;
// 64-byte segments run at little more than half the rate.  One-column lanes (ragged S, unaligned pointers) hold
// at most four pairs.
bool pick_qk_bf(int hd, bool vec_ok, bool backward, QkBf &cfg) {
    const int half = hd / 2;
    if (!vec_ok) {
        cfg = QkBf{1, 64, 1024, 4};
        return half <= 64;
    }
    const int thr = backward ? 512 : 256;
    for (int lpr : {16, 8, 4})
        for (int cap : {1, 2, 4})
            if ((thr / lpr) * cap >= half) { cfg = QkBf{8, lpr, thr, cap}; return true; }
    if (512 >= half) { cfg = QkBf{8, 4, 1024, 2}; return true; }
    return false;
}

#define QKBF_CASE(KERNEL, V, L, T, CP, grid, ...)                                                                    \
    case (V) * 1000000 + (L) * 10000 + ((T) / 256) * 100 + (CP):                                                     \
        hipLaunchKernelGGL((KERNEL<V, L, T, CP>), grid, dim3(T), 0, g_ctx.stream, __VA_ARGS__);                      \
        break;
#define QKBF_DISPATCH(KERNEL, cfg, grid, ...)                                                                        \
    do {                                                                                                             \
        switch ((cfg).vec * 1000000 + (cfg).lpr * 10000 + ((cfg).threads / 256) * 100 + (cfg).cap) {                 \
            QKBF_CASE(KERNEL, 1, 64, 1024, 4, grid, __VA_ARGS__)                                                     \
            QKBF_CASE(KERNEL, 8, 16, 256, 1, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 16, 256, 2, grid, __VA_ARGS__)  \
            QKBF_CASE(KERNEL, 8, 16, 256, 4, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 16, 512, 1, grid, __VA_ARGS__)  \
            QKBF_CASE(KERNEL, 8, 16, 512, 2, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 16, 512, 4, grid, __VA_ARGS__)  \
            QKBF_CASE(KERNEL, 8, 8, 256, 1, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 8, 256, 2, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 8, 256, 4, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 8, 512, 1, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 8, 512, 2, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 8, 512, 4, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 4, 256, 1, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 4, 256, 2, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 4, 256, 4, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 4, 512, 1, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 4, 512, 2, grid, __VA_ARGS__) QKBF_CASE(KERNEL, 8, 4, 512, 4, grid, __VA_ARGS__)    \
            QKBF_CASE(KERNEL, 8, 4, 1024, 2, grid, __VA_ARGS__)                                                      \
            default: return mi355_fail("bf16 qknorm_rope: no kernel for this tile");                                 \
        }                                                                                                            \
    } while (0)

int qk_shape(const char *who, int heads, int kv_heads, int hd, int S, int batch) {
    if (hd <= 0 || (hd & 1) || S <= 0 || batch <= 0 || heads < 0 || kv_heads < 0 || heads + kv_heads == 0)
        return mi355_fail("%s: bad shape heads=%d kv_heads=%d hd=%d S=%d batch=%d", who, heads, kv_heads, hd, S, batch);
    return 0;
}

struct BfCfg {
    int vec, lpr, threads, cap;
};

// 8-column lanes when the rows allow 128-bit accesses; rows in (packed) registers when one workgroup can hold
// them, else two sweeps.  The rms_lpr / rms_threads knobs override the strip width and workgroup size.
BfCfg pick_bf(int C, bool vec_ok, int S, int batch) {
    if (!vec_ok) return BfCfg{1, 64, 256, 0};
    // 128-byte strips (8 lanes x 8 columns) once they still give every compute unit a workgroup
    const long strips8 = (long)ceil_div((size_t)S, 64) * batch;
    int lpr = g_ctx.rms_lpr == 8 || (!g_ctx.rms_lpr && strips8 >= (g_ctx.num_cu > 0 ? g_ctx.num_cu : 256)) ? 8 : 4;
    int threads = g_ctx.rms_threads == 256 || g_ctx.rms_threads == 512 || g_ctx.rms_threads == 1024
                      ? g_ctx.rms_threads
                      : (C >= 512 ? 1024 : 256);   // measured at C = 1024, 16 x 256 columns: 11.0 / 20.5 us forward / backward with
                                                   // 16 waves, 12.6 / 23.0 with 8, 15.1 / 25.7 with 128-byte strips
    const int rps = threads / lpr;
    for (int cap : {2, 4, 8})
        if (rps * cap >= C) return BfCfg{8, lpr, threads, cap};
    return BfCfg{8, lpr, threads, 0};
}

// Clustered variants (norm_cluster.h, bf16 storage: strips of 128 columns, 2 or 4 rows per lane).  Not when the
// single-workgroup tile is chosen by hand through the rms_lpr / rms_threads knobs.
Mi355Exchange g_bf_cluster_ws = {nullptr, nullptr, nullptr};
ClusterPlan plan_cluster_bf(int C, int S, int batch, bool vec_ok) {
    if (g_ctx.rms_lpr || g_ctx.rms_threads) return NO_CLUSTER;
    return cluster_plan(C, S, batch, vec_ok, StoreBf16::VEC, 2, 4, 1);
}
#define BF_CLUSTER_FWD(RPT, EXACT)                                                                                   \
    hipLaunchKernelGGL((rms_fwd_cluster_kernel<StoreBf16, RPT, 1024, false, EXACT>), dim3(cp.nblk), dim3(1024), 0,   \
                       g_ctx.stream, y, (uint16_t *)nullptr, x, (const uint16_t *)nullptr, 0.f, w, C, S, cp.strips,  \
                       cp.nblk, cp.csplit, cp.rows_pm, eps, 1.0f / (float)C, g_bf_cluster_ws,                        \
                       mi355_exchange_spin_ticks())
#define BF_CLUSTER_BWD(RPT, EXACT)                                                                                   \
    hipLaunchKernelGGL((rms_bwd_cluster_kernel<StoreBf16, RPT, 1024, false, EXACT>), dim3(cp.nblk), dim3(1024), 0,   \
                       g_ctx.stream, dx, part, dy, x, w, C, S, cp.strips, cp.nblk, cp.csplit, cp.rows_pm, eps,       \
                       1.0f / (float)C, variant, (const uint16_t *)nullptr, (uint16_t *)nullptr, 0.f,                \
                       g_bf_cluster_ws, mi355_exchange_spin_ticks())

#define BF_CASE(KERNEL, V, L, T, CP, nblk, ...)                                                                      \
    case (V) * 1000000 + (L) * 10000 + ((T) / 256) * 100 + (CP):                                                     \
        hipLaunchKernelGGL((KERNEL<V, L, T, CP>), dim3(nblk), dim3(T), 0, g_ctx.stream, __VA_ARGS__);                \
        break;
#define BF_CASES4(KERNEL, L, T, nblk, ...)                                                                           \
    BF_CASE(KERNEL, 8, L, T, 0, nblk, __VA_ARGS__) BF_CASE(KERNEL, 8, L, T, 2, nblk, __VA_ARGS__)                    \
    BF_CASE(KERNEL, 8, L, T, 4, nblk, __VA_ARGS__) BF_CASE(KERNEL, 8, L, T, 8, nblk, __VA_ARGS__)
#define BF_DISPATCH(KERNEL, cfg, nblk, ...)                                                                          \
    do {                                                                                                             \
        switch ((cfg).vec * 1000000 + (cfg).lpr * 10000 + ((cfg).threads / 256) * 100 + (cfg).cap) {                 \
            BF_CASE(KERNEL, 1, 64, 256, 0, nblk, __VA_ARGS__)                                                        \
            BF_CASES4(KERNEL, 4, 256, nblk, __VA_ARGS__) BF_CASES4(KERNEL, 4, 512, nblk, __VA_ARGS__)                \
            BF_CASES4(KERNEL, 4, 1024, nblk, __VA_ARGS__) BF_CASES4(KERNEL, 8, 256, nblk, __VA_ARGS__)               \
            BF_CASES4(KERNEL, 8, 512, nblk, __VA_ARGS__) BF_CASES4(KERNEL, 8, 1024, nblk, __VA_ARGS__)               \
            default: return mi355_fail("bf16 rmsnorm: no kernel for this tile");                                     \
        }                                                                                                            \
    } while (0)

int cvt_check(const char *who, const void *dst, const void *src, size_t dst_ld, size_t src_ld, size_t rows,
              size_t cols) {
    if (!mi355_ready(who)) return -1;
    if (!dst || !src) return mi355_fail("%s: NULL pointer", who);
    if (rows == 0 || cols == 0) return mi355_fail("%s: empty rectangle rows=%zu cols=%zu", who, rows, cols);
    if (dst_ld < cols || src_ld < cols)
        return mi355_fail("%s: row pitch below the row length (cols=%zu dst_ld=%zu src_ld=%zu)", who, cols, dst_ld, src_ld);
    return 0;
}

inline unsigned blocks_for(size_t work) { return (unsigned)ceil_div(work, (size_t)BT); }

}   // namespace

MI355_API int mi355_cvt_f32_bf16_dev(uint16_t *dst, size_t dst_ld, const float *src, size_t src_ld, size_t rows,
                                     size_t cols) {
    if (cvt_check("cvt_f32_bf16", dst, src, dst_ld, src_ld, rows, cols)) return -1;
    const bool vec = cols % 8 == 0 && dst_ld % 8 == 0 && src_ld % 4 == 0 && aligned16(dst) && aligned16(src);
    if (vec) {
        const size_t colg = cols / 8, total = rows * colg;
        hipLaunchKernelGGL(cvt_f32_bf16_kernel<8>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, dst, dst_ld, src, src_ld, colg, total);
    } else {
        const size_t total = rows * cols;
        hipLaunchKernelGGL(cvt_f32_bf16_kernel<1>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, dst, dst_ld, src, src_ld, cols, total);
    }
    LAUNCH_OK("cvt_f32_bf16");
    return 0;
}

MI355_API int mi355_cvt_bf16_f32_dev(float *dst, size_t dst_ld, const uint16_t *src, size_t src_ld, size_t rows,
                                     size_t cols) {
    if (cvt_check("cvt_bf16_f32", dst, src, dst_ld, src_ld, rows, cols)) return -1;
    const bool vec = cols % 8 == 0 && dst_ld % 4 == 0 && src_ld % 8 == 0 && aligned16(dst) && aligned16(src);
    if (vec) {
        const size_t colg = cols / 8, total = rows * colg;
        hipLaunchKernelGGL(cvt_bf16_f32_kernel<8>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, dst, dst_ld, src, src_ld, colg, total);
    } else {
        const size_t total = rows * cols;
        hipLaunchKernelGGL(cvt_bf16_f32_kernel<1>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, dst, dst_ld, src, src_ld, cols, total);
    }
    LAUNCH_OK("cvt_bf16_f32");
    return 0;
}

MI355_API int mi355_swiglu_fwd_bf16_dev(uint16_t *out, const uint16_t *h1, const uint16_t *h3, size_t n) {
    if (!mi355_ready("swiglu_fwd_bf16")) return -1;
    if (!out || !h1 || !h3) return mi355_fail("swiglu_fwd_bf16: NULL pointer");
    if (n == 0) return mi355_fail("swiglu_fwd_bf16: empty tensor");
    if (n % 8 == 0 && aligned16(out) && aligned16(h1) && aligned16(h3))
        hipLaunchKernelGGL(swiglu_fwd_bf16_kernel<8>, dim3(blocks_for(n / 8)), dim3(BT), 0, g_ctx.stream, out, h1, h3, n / 8);
    else
        hipLaunchKernelGGL(swiglu_fwd_bf16_kernel<1>, dim3(blocks_for(n)), dim3(BT), 0, g_ctx.stream, out, h1, h3, n);
    LAUNCH_OK("swiglu_fwd_bf16");
    return 0;
}

MI355_API int mi355_swiglu_bwd_bf16_dev(uint16_t *dh1, uint16_t *dh3, const uint16_t *dsilu, const uint16_t *h1,
                                        const uint16_t *h3, size_t n) {
    if (!mi355_ready("swiglu_bwd_bf16")) return -1;
    if (!dh1 || !dh3 || !dsilu || !h1 || !h3) return mi355_fail("swiglu_bwd_bf16: NULL pointer");
    if (n == 0) return mi355_fail("swiglu_bwd_bf16: empty tensor");
    if (n % 8 == 0 && aligned16(dh1) && aligned16(dh3) && aligned16(dsilu) && aligned16(h1) && aligned16(h3))
        hipLaunchKernelGGL(swiglu_bwd_bf16_kernel<8>, dim3(blocks_for(n / 8)), dim3(BT), 0, g_ctx.stream, dh1, dh3, dsilu, h1, h3, n / 8);
    else
        hipLaunchKernelGGL(swiglu_bwd_bf16_kernel<1>, dim3(blocks_for(n)), dim3(BT), 0, g_ctx.stream, dh1, dh3, dsilu, h1, h3, n);
    LAUNCH_OK("swiglu_bwd_bf16");
    return 0;
}

MI355_API int mi355_axpby_bf16_dev(uint16_t *y, const uint16_t *a, const uint16_t *b, float alpha, size_t n, int mode) {
    if (!mi355_ready("axpby_bf16")) return -1;
    if (mode < 0 || mode > 2) return mi355_fail("axpby_bf16: mode must be 0, 1 or 2");
    if (!y || !a || (mode != 1 && !b)) return mi355_fail("axpby_bf16: NULL pointer");
    if (n == 0) return mi355_fail("axpby_bf16: empty tensor");
    const bool vec = n % 8 == 0 && aligned16(y) && aligned16(a) && (mode == 1 || aligned16(b));
    const size_t nv = vec ? n / 8 : n;
#define AX(V, M) hipLaunchKernelGGL((axpby_bf16_kernel<V, M>), dim3(blocks_for(nv)), dim3(BT), 0, g_ctx.stream, y, a, b, alpha, nv)
    if (vec) { if (mode == 0) AX(8, 0); else if (mode == 1) AX(8, 1); else AX(8, 2); }
    else { if (mode == 0) AX(1, 0); else if (mode == 1) AX(1, 1); else AX(1, 2); }
#undef AX
    LAUNCH_OK("axpby_bf16");
    return 0;
}

MI355_API int mi355_rmsnorm_fwd_bf16_dev(uint16_t *y, const uint16_t *x, const float *w, int C, int S, int batch,
                                         float eps) {
    if (!mi355_ready("rmsnorm_fwd_bf16")) return -1;
    if (!y || !x || !w) return mi355_fail("rmsnorm_fwd_bf16: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0) return mi355_fail("rmsnorm_fwd_bf16: bad shape C=%d S=%d batch=%d", C, S, batch);
    const bool vec_ok = S % 8 == 0 && aligned16(x) && aligned16(y);
    // tall shapes whose strips would leave compute units idle split the channel axis over clusters of workgroups,
    // as the fp32 op does (norm_cluster.h); in place the single-workgroup tile is used
    const ClusterPlan cp = y == x ? NO_CLUSTER : plan_cluster_bf(C, S, batch, vec_ok);
    if (cp.csplit) {
        if (!mi355_exchange(&g_bf_cluster_ws)) return -1;
        if (cp.rpt == 2 && cp.exact) BF_CLUSTER_FWD(2, true);
        else if (cp.rpt == 2) BF_CLUSTER_FWD(2, false);
        else if (cp.exact) BF_CLUSTER_FWD(4, true);
        else BF_CLUSTER_FWD(4, false);
        LAUNCH_OK("rmsnorm_fwd_bf16");
        return 0;
    }
    const BfCfg cfg = pick_bf(C, vec_ok, S, batch);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    BF_DISPATCH(rms_fwd_bf16_kernel, cfg, nblk, y, x, w, C, S, strips, nblk, eps, 1.0f / (float)C);
    LAUNCH_OK("rmsnorm_fwd_bf16");
    return 0;
}

MI355_API int mi355_rmsnorm_bwd_bf16_dev(uint16_t *dx, float *dw, const uint16_t *dy, const uint16_t *x, const float *w,
                                         int C, int S, int batch, float eps, int variant) {
    if (!mi355_ready("rmsnorm_bwd_bf16")) return -1;
    if (!dx || !dw || !dy || !x || !w) return mi355_fail("rmsnorm_bwd_bf16: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0) return mi355_fail("rmsnorm_bwd_bf16: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (variant != 0 && variant != 1) return mi355_fail("rmsnorm_bwd_bf16: variant must be 0 or 1");
    if (dx == x) return mi355_fail("rmsnorm_bwd_bf16: dx must not alias x (dx may alias dy)");      // as the fp32 op
    const bool vec_ok = S % 8 == 0 && aligned16(x) && aligned16(dy) && aligned16(dx);
    const ClusterPlan cp = dx == dy ? NO_CLUSTER : plan_cluster_bf(C, S, batch, vec_ok);
    if (cp.csplit) {
        if (!mi355_exchange(&g_bf_cluster_ws)) return -1;
        const int nrows = cp.nblk / cp.csplit;
        float *part = mi355_dw_partials((size_t)nrows * C, dw, nullptr);
        if (!part) return -1;
        // (four rows per lane without the masks would need more than the 128 registers a lane has)
        if (cp.rpt == 2 && cp.exact) BF_CLUSTER_BWD(2, true);
        else if (cp.rpt == 2) BF_CLUSTER_BWD(2, false);
        else BF_CLUSTER_BWD(4, false);
        LAUNCH_OK("rmsnorm_bwd_bf16");
        if (mi355_dw_submit(dw, part, nrows, C)) return -1;
        return mi355_dw_op_end();
    }
    const BfCfg cfg = pick_bf(C, vec_ok, S, batch);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    float *part = mi355_dw_partials((size_t)nblk * C, dw, nullptr);
    if (!part) return -1;
    BF_DISPATCH(rms_bwd_bf16_kernel, cfg, nblk, dx, part, dy, x, w, C, S, strips, nblk, eps, 1.0f / (float)C, variant,
                (const uint16_t *)nullptr, (uint16_t *)nullptr, 0.f);
    LAUNCH_OK("rmsnorm_bwd_bf16");
    if (mi355_dw_submit(dw, part, nblk, C)) return -1;
    return mi355_dw_op_end();
}

// The two fusions of the RMSNorm with the residual around it, for bfloat16 storage: the clustered kernels of
// norm_cluster.h with the storage policy StoreBf16 where the shape clusters, otherwise the composition (forward) or
// the single-workgroup tile with the residual riding along (backward).
MI355_API int mi355_residual_rmsnorm_fwd_bf16_dev(uint16_t *y, uint16_t *yn, const uint16_t *a, const uint16_t *b,
                                                  float alpha, const float *w, int C, int S, int batch, float eps) {
    if (!mi355_ready("residual_rmsnorm_fwd_bf16")) return -1;
    if (!y || !yn || !a || !b || !w) return mi355_fail("residual_rmsnorm_fwd_bf16: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("residual_rmsnorm_fwd_bf16: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (yn == y || yn == a || yn == b) return mi355_fail("residual_rmsnorm_fwd_bf16: yn must not alias y, a or b");
    const bool vec_ok = S % 8 == 0 && aligned16(y) && aligned16(yn) && aligned16(a) && aligned16(b);
    const ClusterPlan cp = (y == a || y == b) ? NO_CLUSTER : plan_cluster_bf(C, S, batch, vec_ok);
    if (cp.csplit) {
        if (!mi355_exchange(&g_bf_cluster_ws)) return -1;
#define BF_CLUSTER_RES_FWD(RPT, EXACT)                                                                               \
    hipLaunchKernelGGL((rms_fwd_cluster_kernel<StoreBf16, RPT, 1024, true, EXACT>), dim3(cp.nblk), dim3(1024), 0,    \
                       g_ctx.stream, yn, y, a, b, alpha, w, C, S, cp.strips, cp.nblk, cp.csplit, cp.rows_pm, eps,    \
                       1.0f / (float)C, g_bf_cluster_ws, mi355_exchange_spin_ticks())
        if (cp.rpt == 2 && cp.exact) BF_CLUSTER_RES_FWD(2, true);
        else if (cp.rpt == 2) BF_CLUSTER_RES_FWD(2, false);
        else if (cp.exact) BF_CLUSTER_RES_FWD(4, true);
        else BF_CLUSTER_RES_FWD(4, false);
#undef BF_CLUSTER_RES_FWD
        LAUNCH_OK("residual_rmsnorm_fwd_bf16");
        return 0;
    }
    // two launches: y is rounded to bfloat16 either way and the norm is taken of the rounded values, as above
    if (mi355_axpby_bf16_dev(y, a, b, alpha, (size_t)batch * C * S, 0)) return -1;
    return mi355_rmsnorm_fwd_bf16_dev(yn, y, w, C, S, batch, eps);
}

MI355_API int mi355_rmsnorm_bwd_residual_bf16_dev(uint16_t *dx, uint16_t *dx_scaled, float *dw, const uint16_t *dy,
                                                  const uint16_t *x, const float *w, const uint16_t *res, float alpha,
                                                  int C, int S, int batch, float eps, int variant) {
    if (!mi355_ready("rmsnorm_bwd_residual_bf16")) return -1;
    if (!dx || !dw || !dy || !x || !w || !res) return mi355_fail("rmsnorm_bwd_residual_bf16: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("rmsnorm_bwd_residual_bf16: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (variant != 0 && variant != 1) return mi355_fail("rmsnorm_bwd_residual_bf16: variant must be 0 or 1");
    if (dx_scaled && (dx_scaled == dx || dx_scaled == dy || dx_scaled == x || dx_scaled == res))
        return mi355_fail("rmsnorm_bwd_residual_bf16: dx_scaled must not alias another operand");
    if (dx == x) return mi355_fail("rmsnorm_bwd_residual_bf16: dx must not alias x (dx may alias res or dy)");
    const bool vec_ok = S % 8 == 0 && aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(res) &&
                        (!dx_scaled || aligned16(dx_scaled));
    const ClusterPlan cp = dx == dy ? NO_CLUSTER : plan_cluster_bf(C, S, batch, vec_ok);
    if (cp.csplit) {
        if (!mi355_exchange(&g_bf_cluster_ws)) return -1;
        const int nrows = cp.nblk / cp.csplit;
        float *part = mi355_dw_partials((size_t)nrows * C, dw, nullptr);
        if (!part) return -1;
#define BF_CLUSTER_RES_BWD(RPT)                                                                                      \
    hipLaunchKernelGGL((rms_bwd_cluster_kernel<StoreBf16, RPT, 1024, true, false>), dim3(cp.nblk), dim3(1024), 0,    \
                       g_ctx.stream, dx, part, dy, x, w, C, S, cp.strips, cp.nblk, cp.csplit, cp.rows_pm, eps,       \
                       1.0f / (float)C, variant, res, dx_scaled, alpha, g_bf_cluster_ws, mi355_exchange_spin_ticks())
        if (cp.rpt == 2) BF_CLUSTER_RES_BWD(2);
        else BF_CLUSTER_RES_BWD(4);
#undef BF_CLUSTER_RES_BWD
        LAUNCH_OK("rmsnorm_bwd_residual_bf16");
        if (mi355_dw_submit(dw, part, nrows, C)) return -1;
        return mi355_dw_op_end();
    }
    const BfCfg cfg = pick_bf(C, vec_ok, S, batch);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    float *part = mi355_dw_partials((size_t)nblk * C, dw, nullptr);
    if (!part) return -1;
    BF_DISPATCH(rms_bwd_bf16_kernel, cfg, nblk, dx, part, dy, x, w, C, S, strips, nblk, eps, 1.0f / (float)C, variant, res,
                dx_scaled, alpha);
    LAUNCH_OK("rmsnorm_bwd_residual_bf16");
    if (mi355_dw_submit(dw, part, nblk, C)) return -1;
    return mi355_dw_op_end();
}

MI355_API int mi355_rope_bf16_dev(uint16_t *q_out, uint16_t *k_out, const uint16_t *q_in, const uint16_t *k_in, int heads,
                                  int kv_heads, int hd, int S, int batch, const float *cos_dev, const float *sin_dev,
                                  int dir) {
    if (!mi355_ready("rope_bf16")) return -1;
    if (qk_shape("rope_bf16", heads, kv_heads, hd, S, batch)) return -1;
    if (!cos_dev || !sin_dev || (heads > 0 && (!q_out || !q_in)) || (kv_heads > 0 && (!k_out || !k_in)))
        return mi355_fail("rope_bf16: NULL pointer");
    if (dir != 1 && dir != -1) return mi355_fail("rope_bf16: dir must be +1 or -1");
    const bool vec = S % 8 == 0 && aligned16(cos_dev) && aligned16(sin_dev) &&
                     (heads == 0 || (aligned16(q_in) && aligned16(q_out))) &&
                     (kv_heads == 0 || (aligned16(k_in) && aligned16(k_out)));
    const size_t pair_rows = (size_t)batch * (heads + kv_heads) * (hd / 2);
    const size_t total = pair_rows * (size_t)(vec ? S / 8 : S);
    if (vec) hipLaunchKernelGGL(rope_bf16_kernel<8>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, q_out, k_out, q_in, k_in, heads, kv_heads, hd, S, batch, cos_dev, sin_dev, (float)dir, total);
    else hipLaunchKernelGGL(rope_bf16_kernel<1>, dim3(blocks_for(total)), dim3(BT), 0, g_ctx.stream, q_out, k_out, q_in, k_in, heads, kv_heads, hd, S, batch, cos_dev, sin_dev, (float)dir, total);
    LAUNCH_OK("rope_bf16");
    return 0;
}

MI355_API int mi355_qknorm_rope_fwd_bf16_dev(uint16_t *q_out, uint16_t *k_out, const uint16_t *q, const uint16_t *k,
                                             const float *wq, const float *wk, int heads, int kv_heads, int hd, int S,
                                             int batch, const float *cos_dev, const float *sin_dev, float eps) {
    if (!mi355_ready("qknorm_rope_fwd_bf16")) return -1;
    if (qk_shape("qknorm_rope_fwd_bf16", heads, kv_heads, hd, S, batch)) return -1;
    if (!cos_dev || !sin_dev || (heads > 0 && (!q_out || !q || !wq)) || (kv_heads > 0 && (!k_out || !k || !wk)))
        return mi355_fail("qknorm_rope_fwd_bf16: NULL pointer");
    const bool vec_ok = S % 8 == 0 && aligned16(cos_dev) && aligned16(sin_dev) &&
                        (heads == 0 || (aligned16(q) && aligned16(q_out))) &&
                        (kv_heads == 0 || (aligned16(k) && aligned16(k_out)));
    QkBf cfg;
    if (!pick_qk_bf(hd, vec_ok, false, cfg))
        return mi355_fail("qknorm_rope_fwd_bf16: head size %d does not fit the register tile for this layout", hd);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nq = batch * heads * strips, nk = batch * kv_heads * strips;
    QKBF_DISPATCH(qknorm_rope_fwd_bf16_kernel, cfg, dim3(nq + nk), q_out, k_out, q, k, wq, wk, hd, S, strips, nq, cos_dev,
                  sin_dev, eps, 1.0f / (float)hd);
    LAUNCH_OK("qknorm_rope_fwd_bf16");
    return 0;
}

MI355_API int mi355_qknorm_rope_bwd_bf16_dev(uint16_t *dq, uint16_t *dk, float *dwq, float *dwk, const uint16_t *dq_out,
                                             const uint16_t *dk_out, const uint16_t *q, const uint16_t *k,
                                             const float *wq, const float *wk, int heads, int kv_heads, int hd, int S,
                                             int batch, const float *cos_dev, const float *sin_dev, float eps,
                                             int variant) {
    if (!mi355_ready("qknorm_rope_bwd_bf16")) return -1;
    if (qk_shape("qknorm_rope_bwd_bf16", heads, kv_heads, hd, S, batch)) return -1;
    if (variant != 0 && variant != 1) return mi355_fail("qknorm_rope_bwd_bf16: variant must be 0 or 1");
    if (!cos_dev || !sin_dev || (heads > 0 && (!dq || !dwq || !dq_out || !q || !wq)) ||
        (kv_heads > 0 && (!dk || !dwk || !dk_out || !k || !wk)))
        return mi355_fail("qknorm_rope_bwd_bf16: NULL pointer");
    const bool vec_ok = S % 8 == 0 && aligned16(cos_dev) && aligned16(sin_dev) &&
                        (heads == 0 || (aligned16(q) && aligned16(dq) && aligned16(dq_out))) &&
                        (kv_heads == 0 || (aligned16(k) && aligned16(dk) && aligned16(dk_out)));
    QkBf cfg;
    if (!pick_qk_bf(hd, vec_ok, true, cfg))
        return mi355_fail("qknorm_rope_bwd_bf16: head size %d does not fit the register tile for this layout", hd);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nq = batch * heads * strips, nk = batch * kv_heads * strips;
    float *part = mi355_dw_partials((size_t)(nq + nk) * hd, nq > 0 ? dwq : nullptr, nk > 0 ? dwk : nullptr);
    if (!part) return -1;
    QKBF_DISPATCH(qknorm_rope_bwd_bf16_kernel, cfg, dim3(nq + nk), dq, dk, part, dq_out, dk_out, q, k, wq, wk, hd, S,
                  strips, nq, cos_dev, sin_dev, eps, 1.0f / (float)hd, variant);
    LAUNCH_OK("qknorm_rope_bwd_bf16");
    if (nq > 0 && mi355_dw_submit(dwq, part, nq, hd)) return -1;
    if (nk > 0 && mi355_dw_submit(dwk, part + (size_t)nq * hd, nk, hd)) return -1;
    return mi355_dw_op_end();
}
