// optim.hip — the optimizer tail of the training loops: gradient scale, global L2 norm, clip, Adam/AdamW.
//
// Reference: training/training_dynamic/train.m:748-877 — a scale pass over every gradient (:754-769),
// vDSP_dotpr per tensor for the global norm (:771-787), a clip pass (:806-821), adam_update per tensor
// (training/training_dynamic/cpu_ops.h:56-64; wd = 0 is training/stories_cpu_ops.h:55-63) and a zeroing
// pass (:873-877).  That is five sweeps over the gradients; here it is two: one read for the norm
// (with the scale folded in) and one fused update that applies both scales, updates m, v, w and can
// clear the gradient in the same pass.  Pure HBM streams: 16 B read + 12-16 B written per parameter.
#include "common.h"

#include <math.h>

namespace {

constexpr int OPT_THREADS = 256;

// fixed grid -> fixed assignment of elements to lanes -> deterministic sum
__global__ __launch_bounds__(OPT_THREADS) void sumsq_partial_kernel(float *__restrict__ part,
                                                                    const float *__restrict__ g, size_t n, size_t n4,
                                                                    float pre, bool vec) {
    __shared__ float red[OPT_THREADS / 64];
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    const size_t tid = (size_t)blockIdx.x * OPT_THREADS + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * OPT_THREADS;
    if (vec) {
        for (size_t i = tid; i < n4; i += stride) {
            v4f v = ld4_nt(g + 4 * i) * pre;            // the scale pass of train.m:755-769, folded in
            s0 += v.x * v.x; s1 += v.y * v.y; s2 += v.z * v.z; s3 += v.w * v.w;
        }
        if (blockIdx.x == 0)
            for (size_t i = n4 * 4 + threadIdx.x; i < n; i += OPT_THREADS) { float t = g[i] * pre; s0 += t * t; }
    } else {
        for (size_t i = tid; i < n; i += stride) { float t = g[i] * pre; s0 += t * t; }
    }
    float s = (s0 + s1) + (s2 + s3);
    s = wave_sum_far_first(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(1024) void sumsq_final_kernel(float *__restrict__ acc, const float *__restrict__ part,
                                                           int nblk) {
    __shared__ float red[1024];
    float s = 0.f;
    for (int i = threadIdx.x; i < nblk; i += 1024) s += part[i];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int off = 512; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) *acc = *acc + red[0];
}

// clip_scale = grad_clip / sqrt(sumsq) when clipping applies, else 1 (train.m:806-808)
__global__ void clip_scale_kernel(float *scale, const float *sumsq, float grad_clip) {
    const float norm = sqrtf(*sumsq);
    *scale = (grad_clip > 0.f && norm > grad_clip) ? grad_clip / norm : 1.0f;
}

__device__ __forceinline__ void adam1(float &w, float &m, float &v, float g, float lr, float b1, float b2,
                                      float omb1, float omb2, float eps, float wd, float bc1, float bc2) {
    // cpu_ops.h:59-62, one rounding per operation
    m = b1 * m + omb1 * g;
    v = b2 * v + (omb2 * g) * g;
    const float mh = m / bc1, vh = v / bc2;
    w -= lr * (mh / (sqrtf(vh) + eps) + wd * w);
}

template <bool ZERO>
__global__ __launch_bounds__(OPT_THREADS) void adam_kernel(float *__restrict__ w, float *__restrict__ g,
                                                           float *__restrict__ m, float *__restrict__ v, size_t n,
                                                           size_t n4, float lr, float b1, float b2, float eps,
                                                           float wd, float bc1, float bc2, float scale1,
                                                           const float *__restrict__ scale2_p, bool vec) {
    const float scale2 = scale2_p ? *scale2_p : 1.0f;
    const float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    const size_t i = (size_t)blockIdx.x * OPT_THREADS + threadIdx.x;
    if (vec) {
        if (i < n4) {
            v4f wv = ld4_nt(w + 4 * i), gv = ld4_nt(g + 4 * i), mv = ld4_nt(m + 4 * i), vv = ld4_nt(v + 4 * i);
            gv = (gv * scale1) * scale2;                 // the two scale passes (train.m:755-769, 806-821)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float a = wv[j], b = mv[j], c = vv[j];
                adam1(a, b, c, gv[j], lr, b1, b2, omb1, omb2, eps, wd, bc1, bc2);
                wv[j] = a; mv[j] = b; vv[j] = c;
            }
            st4_nt(w + 4 * i, wv);
            st4_nt(m + 4 * i, mv);
            st4_nt(v + 4 * i, vv);
            if (ZERO) { const v4f z = {0.f, 0.f, 0.f, 0.f}; st4_nt(g + 4 * i, z); }
        }
        if (blockIdx.x == 0 && threadIdx.x < n - n4 * 4) {
            const size_t k = n4 * 4 + threadIdx.x;
            float gg = (g[k] * scale1) * scale2;
            adam1(w[k], m[k], v[k], gg, lr, b1, b2, omb1, omb2, eps, wd, bc1, bc2);
            if (ZERO) g[k] = 0.f;
        }
    } else if (i < n) {
        float gg = (g[i] * scale1) * scale2;
        adam1(w[i], m[i], v[i], gg, lr, b1, b2, omb1, omb2, eps, wd, bc1, bc2);
        if (ZERO) g[i] = 0.f;
    }
}

// ---- several tensors per launch: blockIdx.y selects the tensor ----
constexpr int MT_MAX = 16;
struct MtSumsq {
    const float *g[MT_MAX];
    size_t n[MT_MAX];
};
struct MtAdam {
    float *w[MT_MAX], *g[MT_MAX], *m[MT_MAX], *v[MT_MAX];
    size_t n[MT_MAX];
    float wd[MT_MAX];
};

// partials laid out [tensor][gridDim.x]; every tensor uses the same fixed grid, so the sum is deterministic
__global__ __launch_bounds__(OPT_THREADS) void sumsq_partial_mt_kernel(float *__restrict__ part, MtSumsq a, float pre) {
    __shared__ float red[OPT_THREADS / 64];
    const float *__restrict__ g = a.g[blockIdx.y];
    const size_t n = a.n[blockIdx.y], n4 = n / 4;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    const size_t tid = (size_t)blockIdx.x * OPT_THREADS + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * OPT_THREADS;
    for (size_t i = tid; i < n4; i += stride) {
        v4f v = ld4_nt(g + 4 * i) * pre;
        s0 += v.x * v.x; s1 += v.y * v.y; s2 += v.z * v.z; s3 += v.w * v.w;
    }
    if (blockIdx.x == 0)
        for (size_t i = n4 * 4 + threadIdx.x; i < n; i += OPT_THREADS) { float t = g[i] * pre; s0 += t * t; }
    float s = (s0 + s1) + (s2 + s3);
    s = wave_sum_far_first(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

template <bool ZERO>
__global__ __launch_bounds__(OPT_THREADS) void adam_mt_kernel(MtAdam a, float lr, float b1, float b2, float eps,
                                                              float bc1, float bc2, float scale1,
                                                              const float *__restrict__ scale2_p) {
    const size_t n = a.n[blockIdx.y], n4 = n / 4;
    const size_t i = (size_t)blockIdx.x * OPT_THREADS + threadIdx.x;
    if (i >= n4 && !(blockIdx.x == 0 && threadIdx.x < n - n4 * 4)) return;
    float *__restrict__ w = a.w[blockIdx.y], *__restrict__ g = a.g[blockIdx.y];
    float *__restrict__ m = a.m[blockIdx.y], *__restrict__ v = a.v[blockIdx.y];
    const float wd = a.wd[blockIdx.y];
    const float scale2 = scale2_p ? *scale2_p : 1.0f;
    const float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    if (i < n4) {
        v4f wv = ld4_nt(w + 4 * i), gv = ld4_nt(g + 4 * i), mv = ld4_nt(m + 4 * i), vv = ld4_nt(v + 4 * i);
        gv = (gv * scale1) * scale2;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float x = wv[j], y = mv[j], z = vv[j];
            adam1(x, y, z, gv[j], lr, b1, b2, omb1, omb2, eps, wd, bc1, bc2);
            wv[j] = x; mv[j] = y; vv[j] = z;
        }
        st4_nt(w + 4 * i, wv);
        st4_nt(m + 4 * i, mv);
        st4_nt(v + 4 * i, vv);
        if (ZERO) { const v4f z4 = {0.f, 0.f, 0.f, 0.f}; st4_nt(g + 4 * i, z4); }
    }
    if (blockIdx.x == 0 && threadIdx.x < n - n4 * 4) {
        const size_t k = n4 * 4 + threadIdx.x;
        float gg = (g[k] * scale1) * scale2;
        adam1(w[k], m[k], v[k], gg, lr, b1, b2, omb1, omb2, eps, wd, bc1, bc2);
        if (ZERO) g[k] = 0.f;
    }
}

}   // namespace

MI355_API int mi355_sumsq_accum_multi_dev(float *acc_dev, const float *const *g, const size_t *n, int count,
                                          float pre_scale) {
    if (!mi355_ready("sumsq_accum_multi")) return -1;
    if (!acc_dev || !g || !n || count <= 0) return mi355_fail("sumsq_accum_multi: bad arguments");
    for (int i = 0; i < count; i++)
        if (!g[i] || n[i] == 0 || !aligned16(g[i])) return mi355_fail("sumsq_accum_multi: tensor %d is NULL, empty or not 16-byte aligned", i);
    for (int i0 = 0; i0 < count; i0 += MT_MAX) {
        const int k = count - i0 < MT_MAX ? count - i0 : MT_MAX;
        MtSumsq a = {};
        size_t nmax = 0;
        for (int i = 0; i < k; i++) { a.g[i] = g[i0 + i]; a.n[i] = n[i0 + i]; if (n[i0 + i] > nmax) nmax = n[i0 + i]; }
        size_t blocks = ceil_div(nmax / 4 + 1, (size_t)OPT_THREADS * 4);
        if (blocks > 1024) blocks = 1024;
        float *part = (float *)mi355_ws((size_t)k * blocks * sizeof(float));
        if (!part) return -1;
        hipLaunchKernelGGL(sumsq_partial_mt_kernel, dim3((unsigned)blocks, (unsigned)k), dim3(OPT_THREADS), 0, g_ctx.stream,
                           part, a, pre_scale);
        hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(1024), 0, g_ctx.stream, acc_dev, part, (int)(k * blocks));
        LAUNCH_OK("sumsq_accum_multi");
    }
    return 0;
}

MI355_API int mi355_adam_update_multi_dev(float *const *w, float *const *g, float *const *m, float *const *v,
                                          const size_t *n, const float *wd, int count, int t, float lr, float b1,
                                          float b2, float eps, float scale1, const float *scale2_dev, int zero_grad) {
    if (!mi355_ready("adam_update_multi")) return -1;
    if (!w || !g || !m || !v || !n || !wd || count <= 0 || t < 1) return mi355_fail("adam_update_multi: bad arguments");
    for (int i = 0; i < count; i++)
        if (!w[i] || !g[i] || !m[i] || !v[i] || n[i] == 0 || !aligned16(w[i]) || !aligned16(g[i]) || !aligned16(m[i]) ||
            !aligned16(v[i]))
            return mi355_fail("adam_update_multi: tensor %d is NULL, empty or not 16-byte aligned", i);
    const float bc1 = 1.0f - powf(b1, (float)t), bc2 = 1.0f - powf(b2, (float)t);
    for (int i0 = 0; i0 < count; i0 += MT_MAX) {
        const int k = count - i0 < MT_MAX ? count - i0 : MT_MAX;
        MtAdam a = {};
        size_t nmax = 0;
        for (int i = 0; i < k; i++) {
            a.w[i] = w[i0 + i]; a.g[i] = g[i0 + i]; a.m[i] = m[i0 + i]; a.v[i] = v[i0 + i];
            a.n[i] = n[i0 + i]; a.wd[i] = wd[i0 + i];
            if (n[i0 + i] > nmax) nmax = n[i0 + i];
        }
        const dim3 grid((unsigned)ceil_div(nmax / 4 + 1, (size_t)OPT_THREADS), (unsigned)k);
        if (zero_grad)
            hipLaunchKernelGGL((adam_mt_kernel<true>), grid, dim3(OPT_THREADS), 0, g_ctx.stream, a, lr, b1, b2, eps, bc1,
                               bc2, scale1, scale2_dev);
        else
            hipLaunchKernelGGL((adam_mt_kernel<false>), grid, dim3(OPT_THREADS), 0, g_ctx.stream, a, lr, b1, b2, eps, bc1,
                               bc2, scale1, scale2_dev);
        LAUNCH_OK("adam_update_multi");
    }
    return 0;
}

MI355_API int mi355_sumsq_accum_dev(float *acc_dev, const float *g, size_t n, float pre_scale) {
    if (!mi355_ready("sumsq_accum")) return -1;
    if (!acc_dev || !g) return mi355_fail("sumsq_accum: NULL pointer");
    if (n == 0) return mi355_fail("sumsq_accum: empty tensor");
    const bool vec = aligned16(g);
    const size_t n4 = vec ? n / 4 : 0;
    size_t blocks = ceil_div(vec ? (n4 ? n4 : 1) : n, (size_t)OPT_THREADS * 4);
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
    float *part = (float *)mi355_ws(blocks * sizeof(float));
    if (!part) return -1;
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3((unsigned)blocks), dim3(OPT_THREADS), 0, g_ctx.stream, part, g, n, n4,
                       pre_scale, vec);
    hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(1024), 0, g_ctx.stream, acc_dev, part, (int)blocks);
    LAUNCH_OK("sumsq_accum");
    return 0;
}

MI355_API int mi355_clip_scale_dev(float *scale_dev, const float *sumsq_dev, float grad_clip) {
    if (!mi355_ready("clip_scale")) return -1;
    if (!scale_dev || !sumsq_dev) return mi355_fail("clip_scale: NULL pointer");
    hipLaunchKernelGGL(clip_scale_kernel, dim3(1), dim3(1), 0, g_ctx.stream, scale_dev, sumsq_dev, grad_clip);
    LAUNCH_OK("clip_scale");
    return 0;
}

MI355_API int mi355_adam_update_dev(float *w, float *g, float *m, float *v, size_t n, int t, float lr, float b1,
                                    float b2, float eps, float wd, float scale1, const float *scale2_dev,
                                    int zero_grad) {
    if (!mi355_ready("adam_update")) return -1;
    if (!w || !g || !m || !v) return mi355_fail("adam_update: NULL pointer");
    if (n == 0 || t < 1) return mi355_fail("adam_update: empty tensor or step < 1");
    // bias corrections as the reference computes them (cpu_ops.h:57)
    const float bc1 = 1.0f - powf(b1, (float)t), bc2 = 1.0f - powf(b2, (float)t);
    const bool vec = aligned16(w) && aligned16(g) && aligned16(m) && aligned16(v);
    const size_t n4 = vec ? n / 4 : 0;
    const size_t work = vec ? (n4 ? n4 : 1) : n;
    const unsigned blocks = (unsigned)ceil_div(work, (size_t)OPT_THREADS);
    if (zero_grad)
        hipLaunchKernelGGL((adam_kernel<true>), dim3(blocks), dim3(OPT_THREADS), 0, g_ctx.stream, w, g, m, v, n, n4, lr,
                           b1, b2, eps, wd, bc1, bc2, scale1, scale2_dev, vec);
    else
        hipLaunchKernelGGL((adam_kernel<false>), dim3(blocks), dim3(OPT_THREADS), 0, g_ctx.stream, w, g, m, v, n, n4, lr,
                           b1, b2, eps, wd, bc1, bc2, scale1, scale2_dev, vec);
    LAUNCH_OK("adam_update");
    return 0;
}
