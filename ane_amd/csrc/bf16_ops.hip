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

#include <math.h>

namespace {

typedef uint16_t bf16_t;
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

constexpr int BT = 256;

__device__ __forceinline__ float bf_to_f(unsigned bits16) { return __uint_as_float(bits16 << 16); }
// round to nearest even; NaN stays NaN (quiet bit forced)
__device__ __forceinline__ unsigned f_to_bf(float f) {
    const unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// VEC bf16 values -> VEC floats.  VEC = 8: one 128-bit access, element 2j in the low half of word j.
template <int VEC, bool NT>
__device__ __forceinline__ void ldb(float (&r)[VEC], const bf16_t *p) {
    if constexpr (VEC == 8) {
        const v4u *q = reinterpret_cast<const v4u *>(p);
        const v4u w = NT ? __builtin_nontemporal_load(q) : *q;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            r[2 * j] = bf_to_f(w[j] & 0xffffu);
            r[2 * j + 1] = bf_to_f(w[j] >> 16);
        }
    } else {
        static_assert(VEC == 1, "bf16 rows are read 8 columns or 1 column at a time");
        r[0] = bf_to_f(*p);
    }
}
template <int VEC>
__device__ __forceinline__ void stb(bf16_t *p, const float (&r)[VEC]) {
    if constexpr (VEC == 8) {
        v4u w;
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = f_to_bf(r[2 * j]) | (f_to_bf(r[2 * j + 1]) << 16);
        __builtin_nontemporal_store(w, reinterpret_cast<v4u *>(p));
    } else {
        *p = (bf16_t)f_to_bf(r[0]);
    }
}

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
        float xv[CAP][VEC], wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                ldb<VEC, true>(xv[k], x + base + (size_t)c * S);
                wv[k] = w[c];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) xv[k][j] = 0.f;
                wv[k] = 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < CAP; k++)
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[0][j] += xv[k][j] * xv[k][j];
        strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
        float rr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                float o[VEC];
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = (xv[k][j] * rr[j]) * wv[k];
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
                                                               int nblk, float eps, float invC, int variant) {
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
        if (col_ok) stb<VEC>(dx + base + (size_t)c * S, o);
        p = group_sum<G>(p);
        if (lc == 0) part[c] = p;
    };

    if constexpr (CAP > 0) {
        float xv[CAP][VEC], dv[CAP][VEC], wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                ldb<VEC, true>(xv[k], x + base + (size_t)c * S);
                ldb<VEC, true>(dv[k], dy + base + (size_t)c * S);
                wv[k] = w[c];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) xv[k][j] = dv[k][j] = 0.f;
                wv[k] = 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < CAP; k++)
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                acc[0][j] += xv[k][j] * xv[k][j];
                acc[1][j] += (dv[k][j] * xv[k][j]) * wv[k];
            }
        strip_reduce<VEC, LPR, THREADS, 2>(acc, lds);
        float rr[VEC], dotn[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
            dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invC);
        }
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C) row_out(c, xv[k], dv[k], wv[k], rr, dotn);      // uniform per group of LPR lanes
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

struct BfCfg {
    int vec, lpr, threads, cap;
};

// 8-column lanes when the rows allow 128-bit accesses; 4 lanes (64 bytes) per strip row; rows in registers
// when one workgroup can hold them.
BfCfg pick_bf(int C, bool vec_ok, bool backward) {
    if (!vec_ok) return BfCfg{1, 64, 256, 0};
    const int threads = C >= 512 ? 1024 : 256;
    const int rps = threads / 4;
    const int max_cap = backward ? 4 : 8;            // 8 floats per row and operand: 2 x 4 x 8 data registers backward
    for (int cap : {2, 4, 8})
        if (cap <= max_cap && rps * cap >= C) return BfCfg{8, 4, threads, cap};
    return BfCfg{8, 4, threads, 0};
}

#define BF_DISPATCH(KERNEL, cfg, nblk, ...)                                                                          \
    do {                                                                                                             \
        const int key = (cfg).vec * 100000 + (cfg).threads * 10 + (cfg).cap;                                         \
        switch (key) {                                                                                               \
            case 102560: hipLaunchKernelGGL((KERNEL<1, 64, 256, 0>), dim3(nblk), dim3(256), 0, g_ctx.stream, __VA_ARGS__); break;   \
            case 802560: hipLaunchKernelGGL((KERNEL<8, 4, 256, 0>), dim3(nblk), dim3(256), 0, g_ctx.stream, __VA_ARGS__); break;    \
            case 802562: hipLaunchKernelGGL((KERNEL<8, 4, 256, 2>), dim3(nblk), dim3(256), 0, g_ctx.stream, __VA_ARGS__); break;    \
            case 802564: hipLaunchKernelGGL((KERNEL<8, 4, 256, 4>), dim3(nblk), dim3(256), 0, g_ctx.stream, __VA_ARGS__); break;    \
            case 802568: hipLaunchKernelGGL((KERNEL<8, 4, 256, 8>), dim3(nblk), dim3(256), 0, g_ctx.stream, __VA_ARGS__); break;    \
            case 810240: hipLaunchKernelGGL((KERNEL<8, 4, 1024, 0>), dim3(nblk), dim3(1024), 0, g_ctx.stream, __VA_ARGS__); break;  \
            case 810242: hipLaunchKernelGGL((KERNEL<8, 4, 1024, 2>), dim3(nblk), dim3(1024), 0, g_ctx.stream, __VA_ARGS__); break;  \
            case 810244: hipLaunchKernelGGL((KERNEL<8, 4, 1024, 4>), dim3(nblk), dim3(1024), 0, g_ctx.stream, __VA_ARGS__); break;  \
            case 810248: hipLaunchKernelGGL((KERNEL<8, 4, 1024, 8>), dim3(nblk), dim3(1024), 0, g_ctx.stream, __VA_ARGS__); break;  \
            default: return mi355_fail("bf16 rmsnorm: no kernel for tile key %d", key);                              \
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
    const BfCfg cfg = pick_bf(C, S % 8 == 0 && aligned16(x) && aligned16(y), false);
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
    const BfCfg cfg = pick_bf(C, S % 8 == 0 && aligned16(x) && aligned16(dy) && aligned16(dx), true);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    float *part = mi355_dw_partials((size_t)nblk * C, dw, nullptr);
    if (!part) return -1;
    BF_DISPATCH(rms_bwd_bf16_kernel, cfg, nblk, dx, part, dy, x, w, C, S, strips, nblk, eps, 1.0f / (float)C, variant);
    LAUNCH_OK("rmsnorm_bwd_bf16");
    if (mi355_dw_submit(dw, part, nblk, C)) return -1;
    return mi355_dw_op_end();
}
