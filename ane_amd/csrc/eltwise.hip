// eltwise.hip — streaming elementwise ops: SwiGLU gate fwd/bwd, residual family, RoPE, INT8.
//
// All of these are pure HBM streams (<= ~30 flops per 12-20 bytes), so the design is the same
// for each: 128-bit loads and stores, every load instruction of a wave covering one contiguous
// 1 KiB run, UNROLL independent loads in flight per lane before the first use, and enough
// workgroups (one pass, no grid-stride loop) to cover the 256 compute units many times over.
#include "common.h"

#include <math.h>

namespace {

constexpr int EW_THREADS = 256;

__device__ __forceinline__ float sigmoid_ref(float h) {
    // 1/(1+exp(-h)) with the library expf and an IEEE division, as the reference's
    // vvexpf + vvrecf sequence (training/training_dynamic/train.m:541-544)
    return 1.0f / (1.0f + expf(-h));
}

// ---- SwiGLU forward: out = (h1*sig(h1))*h3  (mil_dynamic.h:264-266) ----
template <int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void swiglu_fwd_kernel(float *__restrict__ out, const float *__restrict__ h1,
                                                                const float *__restrict__ h3, size_t n4) {
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    v4f a[UNROLL], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            a[u] = ld4_nt(h1 + 4 * i);
            b[u] = ld4_nt(h3 + 4 * i);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            v4f o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = (a[u][j] * sigmoid_ref(a[u][j])) * b[u][j];
            st4_nt(out + 4 * i, o);
        }
    }
}

__global__ void swiglu_fwd_scalar(float *out, const float *h1, const float *h3, size_t lo, size_t n) {
    size_t i = lo + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (h1[i] * sigmoid_ref(h1[i])) * h3[i];
}

// ---- SwiGLU backward (train.m:537-554) ----
__device__ __forceinline__ void swiglu_bwd_elem(float d, float h, float g, float &dh1, float &dh3) {
    float sig = sigmoid_ref(h);
    dh3 = d * (h * sig);
    float u = -(sig + -1.0f);
    u = h * u;
    u = u + 1.0f;
    u = sig * u;
    dh1 = (d * g) * u;
}

template <int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void swiglu_bwd_kernel(float *__restrict__ dh1, float *__restrict__ dh3,
                                                                const float *__restrict__ ds,
                                                                const float *__restrict__ h1,
                                                                const float *__restrict__ h3, size_t n4) {
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    v4f a[UNROLL], b[UNROLL], d[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            d[u] = ld4_nt(ds + 4 * i);
            a[u] = ld4_nt(h1 + 4 * i);
            b[u] = ld4_nt(h3 + 4 * i);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            v4f o1, o3;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float x1, x3;
                swiglu_bwd_elem(d[u][j], a[u][j], b[u][j], x1, x3);
                o1[j] = x1;
                o3[j] = x3;
            }
            st4_nt(dh1 + 4 * i, o1);
            st4_nt(dh3 + 4 * i, o3);
        }
    }
}

__global__ void swiglu_bwd_scalar(float *dh1, float *dh3, const float *ds, const float *h1, const float *h3,
                                  size_t lo, size_t n) {
    size_t i = lo + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float x1, x3;
        swiglu_bwd_elem(ds[i], h1[i], h3[i], x1, x3);
        dh1[i] = x1;
        dh3[i] = x3;
    }
}

// ---- residual family ----
template <int MODE, int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void axpby_kernel(float *y, const float *a, const float *b, float alpha,
                                                           size_t n4) {
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    v4f av[UNROLL], bv[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            av[u] = ld4_nt(a + 4 * i);
            if (MODE != 1) bv[u] = ld4_nt(b + 4 * i);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            v4f o;
            if (MODE == 0) o = bv[u] * alpha + av[u];
            else if (MODE == 1) o = av[u] * alpha;
            else o = av[u] + bv[u];
            st4_nt(y + 4 * i, o);
        }
    }
}

template <int MODE>
__global__ void axpby_scalar(float *y, const float *a, const float *b, float alpha, size_t lo, size_t n) {
    size_t i = lo + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        if (MODE == 0) y[i] = b[i] * alpha + a[i];
        else if (MODE == 1) y[i] = a[i] * alpha;
        else y[i] = a[i] + b[i];
    }
}

// ---- RoPE on interleaved row pairs; one thread = one pair of rows x VEC columns ----
// rows: all (batch, head, pair) triples of Q then of K; tables [hd/2][S].
template <int VEC>
__global__ __launch_bounds__(EW_THREADS) void rope_kernel(float *q_out, float *k_out, const float *q_in,
                                                          const float *k_in, int heads, int /*kv_heads*/, int hd, int S,
                                                          int batch, const float *__restrict__ cos_t,
                                                          const float *__restrict__ sin_t, float sgn, size_t total) {
    const int cols = (S + VEC - 1) / VEC;   // column groups per row
    const size_t idx = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (idx >= total) return;
    const int cg = (int)(idx % cols);
    size_t pr = idx / cols;   // pair-row index
    const int half = hd >> 1;
    const size_t q_rows = (size_t)batch * heads * half;
    const float *in;
    float *out;
    int i;
    size_t row;
    if (pr < q_rows) {
        i = (int)(pr % half);
        row = (pr / half) * hd + 2 * i;   // (b*heads + h)*hd + 2i
        in = q_in; out = q_out;
    } else {
        pr -= q_rows;
        i = (int)(pr % half);
        row = (pr / half) * hd + 2 * i;
        in = k_in; out = k_out;
    }
    const int s = cg * VEC;
    const size_t o0 = row * S + s, o1 = o0 + S;
    const size_t t = (size_t)i * S + s;
    if constexpr (VEC == 4) {
        v4f v0 = ld4(in + o0), v1 = ld4(in + o1);
        v4f c = ld4(cos_t + t), sn = ld4(sin_t + t) * sgn;
        // forward (sgn=+1): x0*c - x1*s, x0*s + x1*c ; backward (sgn=-1): x0*c + x1*s, -x0*s + x1*c
        v4f r0 = v0 * c - v1 * sn;
        v4f r1 = v0 * sn + v1 * c;
        st4(out + o0, r0);
        st4(out + o1, r1);
    } else {
        float v0 = in[o0], v1 = in[o1];
        float c = cos_t[t], sn = sin_t[t] * sgn;
        out[o0] = v0 * c - v1 * sn;
        out[o1] = v0 * sn + v1 * c;
    }
}

// ---- INT8 ----
// max|x| over the tensor in two launches: per-workgroup maxima, then one workgroup folds them and
// writes scale = max/127 (1.0 for an all-zero tensor).  max is exact whatever the order.
__global__ __launch_bounds__(EW_THREADS) void absmax_kernel(float *__restrict__ part, const float *__restrict__ x,
                                                            size_t n, size_t n4, bool vec) {
    __shared__ float red[EW_THREADS / 64];
    float m = 0.f;
    const size_t stride = (size_t)gridDim.x * EW_THREADS;
    const size_t tid = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (vec) {
        for (size_t i = tid; i < n4; i += stride) {
            v4f v = ld4(x + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; j++) m = fmaxf(m, fabsf(v[j]));
        }
        if (blockIdx.x == 0)
            for (size_t i = n4 * 4 + threadIdx.x; i < n; i += EW_THREADS) m = fmaxf(m, fabsf(x[i]));
    } else {
        for (size_t i = tid; i < n; i += stride) m = fmaxf(m, fabsf(x[i]));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < EW_THREADS / 64; k++) m = fmaxf(m, red[k]);
        part[blockIdx.x] = m;
    }
}

// The per-tensor scale in ONE launch: every workgroup publishes its maximum through the exchange area (an 8-byte
// relaxed agent-scope atomic {value, launch tag}; the protocol is described in norm_cluster.h) and workgroup 0
// gathers them and writes scale = max|x|/127 (1 for an all-zero tensor).  At most 1024 workgroups, one per compute
// unit in practice, so all of them are resident together; if a maximum does not arrive within the bounded wait,
// workgroup 0 takes the maximum of the whole tensor itself.  The maximum is exact in any order.
// (Workgroup 0 reads the others' launch counters when it starts.  The others do not wait for it, so one that had
// finished before workgroup 0 started would be taken for absent and cost the bounded wait; workgroups are
// dispatched in index order and need microseconds for their share, so workgroup 0 is running long before.)
__global__ __launch_bounds__(1024) void absmax_scale_kernel(float *__restrict__ scale, const float *__restrict__ x,
                                                            size_t n, size_t n4, bool vec, Mi355Exchange ws,
                                                            int spin_ticks) {
    __shared__ float red[16];
    __shared__ int failed;
    const int nblk = (int)gridDim.x, blk = (int)blockIdx.x, t = (int)threadIdx.x;
    if (t == 0) failed = 0;
    unsigned want = 0;
    if (blk == 0 && t < nblk) want = ws.cnt[t] + 1u;
    const unsigned my_tag = ws.cnt[blk] + 1u;
    auto tensor_max = [&](size_t first, size_t stride) {
        float m = 0.f;
        if (vec) {
            for (size_t i = first; i < n4; i += stride) {
                const v4f v = ld4_nt(x + 4 * i);
#pragma unroll
                for (int j = 0; j < 4; j++) m = fmaxf(m, fabsf(v[j]));
            }
            if (first < 1024)       // the few elements behind the last whole group of four
                for (size_t i = n4 * 4 + first; i < n; i += 1024) m = fmaxf(m, fabsf(x[i]));
        } else {
            for (size_t i = first; i < n; i += stride) m = fmaxf(m, fabsf(x[i]));
        }
        return m;
    };
    auto block_max = [&](float m) {          // maximum over the workgroup, in every thread
        m = wave_max(m);
        __syncthreads();
        if ((t & 63) == 0) red[t >> 6] = m;
        __syncthreads();
        float r = red[0];
#pragma unroll
        for (int k = 1; k < 16; k++) r = fmaxf(r, red[k]);
        return r;
    };
    float m = block_max(tensor_max((size_t)blk * 1024 + t, (size_t)nblk * 1024));
    if (t == 0)
        __hip_atomic_store(&ws.slots[(size_t)blk * XCH_SLOT_STRIDE], ((unsigned long long)my_tag << 32) | __float_as_uint(m),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (blk == 0) {
        float g = 0.f;
        if (t < nblk) {
            const unsigned long long *sp = &ws.slots[(size_t)t * XCH_SLOT_STRIDE];
            const long long t0 = wall_clock64();
            unsigned long long pk;
            bool ok = false;
            for (;;) {
                pk = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (spin_ticks < 0) break;                        // test mode: whatever the slot holds is refused
                if ((unsigned)(pk >> 32) == want) { ok = true; break; }
                if (wall_clock64() - t0 >= (long long)spin_ticks) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (!ok) failed = 1;
            g = __uint_as_float((unsigned)pk);
        }
        g = block_max(g);
        if (failed) {
            if (t == 0) atomicAdd(ws.fallbacks, 1);
            g = block_max(tensor_max((size_t)t, 1024));
        }
        if (t == 0) {
            float s = g / 127.0f;
            if (s == 0.0f) s = 1.0f;
            *scale = s;
        }
    }
    if (t == 0) ws.cnt[blk] = my_tag;
}

__global__ __launch_bounds__(1024) void scale_from_partials_kernel(float *scale, const float *__restrict__ part,
                                                                   int nblk) {
    __shared__ float red[16];
    float m = 0.f;
    for (int i = threadIdx.x; i < nblk; i += 1024) m = fmaxf(m, part[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 16; k++) m = fmaxf(m, red[k]);
        float s = m / 127.0f;
        if (s == 0.0f) s = 1.0f;
        *scale = s;
    }
}

// min, max and max|x| over the tensor (the loop's range diagnostics, vDSP_minv / vDSP_maxv / vDSP_maxmgv at
// training/training_dynamic/train.m:664-666,738-742): per-workgroup triples, then one workgroup folds them.
// All three are exact whatever the order; NaNs are skipped (fminf/fmaxf).
__global__ __launch_bounds__(EW_THREADS) void minmax_kernel(float *__restrict__ part, const float *__restrict__ x,
                                                            size_t n, size_t n4, bool vec) {
    __shared__ float red[3][EW_THREADS / 64];
    float lo = INFINITY, hi = -INFINITY;
    const size_t stride = (size_t)gridDim.x * EW_THREADS;
    const size_t tid = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (vec) {
        for (size_t i = tid; i < n4; i += stride) {
            v4f v = ld4_nt(x + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; j++) { lo = fminf(lo, v[j]); hi = fmaxf(hi, v[j]); }
        }
        if (blockIdx.x == 0)
            for (size_t i = n4 * 4 + threadIdx.x; i < n; i += EW_THREADS) { lo = fminf(lo, x[i]); hi = fmaxf(hi, x[i]); }
    } else {
        for (size_t i = tid; i < n; i += stride) { lo = fminf(lo, x[i]); hi = fmaxf(hi, x[i]); }
    }
    lo = wave_min(lo);
    hi = wave_max(hi);
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = lo; red[1][threadIdx.x >> 6] = hi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < EW_THREADS / 64; k++) { lo = fminf(lo, red[0][k]); hi = fmaxf(hi, red[1][k]); }
        part[2 * blockIdx.x] = lo;
        part[2 * blockIdx.x + 1] = hi;
    }
}

__global__ __launch_bounds__(1024) void minmax_final_kernel(float *out, const float *__restrict__ part, int nblk) {
    __shared__ float red[2][16];
    float lo = INFINITY, hi = -INFINITY;
    for (int i = threadIdx.x; i < nblk; i += 1024) { lo = fminf(lo, part[2 * i]); hi = fmaxf(hi, part[2 * i + 1]); }
    lo = wave_min(lo);
    hi = wave_max(hi);
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = lo; red[1][threadIdx.x >> 6] = hi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 16; k++) { lo = fminf(lo, red[0][k]); hi = fmaxf(hi, red[1][k]); }
        out[0] = lo;
        out[1] = hi;
        out[2] = fmaxf(fabsf(lo), fabsf(hi));       // max |x| is |min| or |max|
    }
}

__device__ __forceinline__ int quant1(float x, float scale, int rounding) {
    float v = x / scale;              // IEEE division, as the reference (bridge/ane_bridge.m:361)
    v = fminf(v, 127.0f);
    v = fmaxf(v, -128.0f);
    if (rounding == 1) return (int)(v + (v >= 0 ? 0.5f : -0.5f));   // half away from zero, then truncate
    return (int)rintf(v);                                            // half to even
}

template <int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void quant_kernel(int *__restrict__ q4, const float *__restrict__ x,
                                                           const float *__restrict__ scale_p, size_t n4,
                                                           int rounding) {
    const float scale = *scale_p;
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    v4f a[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) a[u] = ld4(x + 4 * i);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            unsigned int pk = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) pk |= ((unsigned int)(quant1(a[u][j], scale, rounding) & 0xFF)) << (8 * j);
            q4[i] = (int)pk;
        }
    }
}

__global__ void quant_scalar(int8_t *q, const float *x, const float *scale_p, size_t lo, size_t n, int rounding) {
    size_t i = lo + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) q[i] = (int8_t)quant1(x[i], *scale_p, rounding);
}

// Quantize with the scale taken from the per-workgroup maxima of absmax_kernel: every workgroup folds the maxima
// itself, which saves the launch that would do it once; workgroup 0 also writes the scale out.
template <int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void quant_dyn_kernel(int *__restrict__ q4, const float *__restrict__ x,
                                                               const float *__restrict__ part, int nblk,
                                                               float *__restrict__ scale_out, size_t n4, int rounding) {
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    v4f a[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) a[u] = ld4(x + 4 * i);
    }
    // the maxima (at most 256: a few cache lines, read by one wave per workgroup so that the thousand workgroups
    // do not queue on them) are folded while the loads above are in flight
    __shared__ float red;
    if (threadIdx.x < 64) {
        float m = 0.f;
        for (int i = threadIdx.x; i < nblk; i += 64) m = fmaxf(m, part[i]);
        m = wave_max(m);
        if (threadIdx.x == 0) red = m;
    }
    __syncthreads();
    float scale = red / 127.0f;
    if (scale == 0.0f) scale = 1.0f;
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = scale;
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            unsigned int pk = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) pk |= ((unsigned int)(quant1(a[u][j], scale, rounding) & 0xFF)) << (8 * j);
            q4[i] = (int)pk;
        }
    }
}

// The reference's quantizer as it is written (bridge/ane_bridge.m:346-365: the maximum of |x|, then the rounding) in
// ONE launch that reads x once: a workgroup keeps its share of the tensor in registers (PER groups of four per
// thread), publishes the maximum of it as absmax_scale_kernel does, gathers every workgroup's, and quantizes what
// it holds.  The maximum is exact in any order, so every workgroup computes the same scale and the bytes are those of
// the two separate steps.  A workgroup whose wait for another's maximum expires takes the maximum of the whole tensor
// itself.  (A workgroup raises its launch counter only after it has gathered everyone's maximum, that is after every
// other workgroup has started and read that counter: nobody can be taken for absent because it was too fast.)
template <int PER>
__global__ __launch_bounds__(1024) void quant_dyn_one_kernel(int *__restrict__ q4, float *__restrict__ scale_out,
                                                             const float *__restrict__ x, size_t n, size_t n4,
                                                             int rounding, Mi355Exchange ws, int spin_ticks) {
    __shared__ float red[16];
    __shared__ int failed;
    const int nblk = (int)gridDim.x, blk = (int)blockIdx.x, t = (int)threadIdx.x;
    if (t == 0) failed = 0;
    unsigned want = 0;
    if (t < nblk) want = ws.cnt[t] + 1u;
    const unsigned my_tag = ws.cnt[blk] + 1u;
    v4f a[PER];
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const size_t i = ((size_t)u * nblk + blk) * 1024 + t;
        const v4f zero = {0.f, 0.f, 0.f, 0.f};
        a[u] = i < n4 ? ld4_nt(x + 4 * i) : zero;
    }
    auto block_max = [&](float m) {          // maximum over the workgroup, in every thread
        m = wave_max(m);
        __syncthreads();
        if ((t & 63) == 0) red[t >> 6] = m;
        __syncthreads();
        float r = red[0];
#pragma unroll
        for (int k = 1; k < 16; k++) r = fmaxf(r, red[k]);
        return r;
    };
    float m = 0.f;
    if (blk == 0 && n4 * 4 + t < n) m = fabsf(x[n4 * 4 + t]);       // the few elements behind the last whole group
#pragma unroll
    for (int u = 0; u < PER; u++)
#pragma unroll
        for (int j = 0; j < 4; j++) m = fmaxf(m, fabsf(a[u][j]));
    m = block_max(m);
    if (t == 0)
        __hip_atomic_store(&ws.slots[(size_t)blk * XCH_SLOT_STRIDE], ((unsigned long long)my_tag << 32) | __float_as_uint(m),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float g = 0.f;
    if (t < nblk) {
        const unsigned long long *sp = &ws.slots[(size_t)t * XCH_SLOT_STRIDE];
        const long long t0 = wall_clock64();
        unsigned long long pk;
        bool ok = false;
        for (;;) {
            pk = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (spin_ticks < 0) break;                            // test mode: whatever the slot holds is refused
            if ((unsigned)(pk >> 32) == want) { ok = true; break; }
            if (wall_clock64() - t0 >= (long long)spin_ticks) break;
            __builtin_amdgcn_s_sleep(2);
        }
        if (!ok) failed = 1;
        g = __uint_as_float((unsigned)pk);
    }
    g = block_max(g);
    if (failed) {                                                 // (block-uniform: read after the barriers above)
        if (t == 0) atomicAdd(ws.fallbacks, 1);
        float w = 0.f;
        for (size_t i = t; i < n4; i += 1024) {
            const v4f v = ld4(x + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; j++) w = fmaxf(w, fabsf(v[j]));
        }
        for (size_t i = n4 * 4 + t; i < n; i += 1024) w = fmaxf(w, fabsf(x[i]));
        g = block_max(w);
    }
    float scale = g / 127.0f;
    if (scale == 0.0f) scale = 1.0f;
    if (blk == 0 && t == 0) *scale_out = scale;
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const size_t i = ((size_t)u * nblk + blk) * 1024 + t;
        if (i < n4) {
            unsigned int pk = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) pk |= ((unsigned int)(quant1(a[u][j], scale, rounding) & 0xFF)) << (8 * j);
            q4[i] = (int)pk;
        }
    }
    if (t == 0) ws.cnt[blk] = my_tag;
}

template <int UNROLL>
__global__ __launch_bounds__(EW_THREADS) void dequant_kernel(float *__restrict__ x, const int *__restrict__ q4,
                                                             const float *__restrict__ scale_p, size_t n4) {
    const float scale = *scale_p;
    const size_t base = (size_t)blockIdx.x * (EW_THREADS * UNROLL) + threadIdx.x;
    int a[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) a[u] = q4[i];
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * EW_THREADS;
        if (i < n4) {
            v4f o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = (float)(int)(signed char)((a[u] >> (8 * j)) & 0xFF) * scale;
            st4(x + 4 * i, o);
        }
    }
}

__global__ void dequant_scalar(float *x, const int8_t *q, const float *scale_p, size_t lo, size_t n) {
    size_t i = lo + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = (float)q[i] * *scale_p;
}

// One 128-bit access per lane and as many workgroups as that takes measured fastest on MI355X
// (75-77 % of peak for the SwiGLU streams against 68-70 % with four accesses per lane).
// ---- GQA tile / reduce (training/training_dynamic/io.h:330-351) ----
// slab = hd*S floats of one head; one lane = one 128-bit column group of one KV-head slab
template <int VEC>
__global__ __launch_bounds__(EW_THREADS) void gqa_tile_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                              int kv_heads, int ratio, size_t slabv, size_t total) {
    const size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;      // over batch*kv_heads*slabv
    if (i >= total) return;
    const size_t head = i / slabv, off = i - head * slabv;             // head = b*kv_heads + kv
    const size_t b = head / kv_heads, kv = head - b * kv_heads;
    const size_t dst0 = ((b * kv_heads + kv) * ratio) * slabv + off;
    if constexpr (VEC == 4) {
        const v4f v = ld4_nt(in + 4 * i);
        for (int r = 0; r < ratio; r++) st4_nt(out + 4 * (dst0 + (size_t)r * slabv), v);
    } else {
        const float v = in[i];
        for (int r = 0; r < ratio; r++) out[dst0 + (size_t)r * slabv] = v;
    }
}

template <int VEC>
__global__ __launch_bounds__(EW_THREADS) void gqa_reduce_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                                int kv_heads, int ratio, size_t slabv, size_t total) {
    const size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;      // over batch*kv_heads*slabv (outputs)
    if (i >= total) return;
    const size_t head = i / slabv, off = i - head * slabv;
    const size_t b = head / kv_heads, kv = head - b * kv_heads;
    const size_t src0 = ((b * kv_heads + kv) * ratio) * slabv + off;
    if constexpr (VEC == 4) {
        v4f acc = {0.f, 0.f, 0.f, 0.f};                                 // memset, then += in head order (io.h:342-350)
        for (int r = 0; r < ratio; r++) acc += ld4_nt(in + 4 * (src0 + (size_t)r * slabv));
        st4_nt(out + 4 * i, acc);
    } else {
        float acc = 0.f;
        for (int r = 0; r < ratio; r++) acc += in[src0 + (size_t)r * slabv];
        out[i] = acc;
    }
}

inline int pick_unroll(size_t n4, int deflt) {
    int u = g_ctx.ew_unroll ? g_ctx.ew_unroll : deflt;
    if (u != 1 && u != 2 && u != 4 && u != 8) u = deflt;
    // small tensors: favour more workgroups over deeper unrolling
    while (u > 1 && ceil_div(n4, (size_t)EW_THREADS * u) < 2048) u >>= 1;
    return u;
}

#define EW_LAUNCH(KERNEL_T, unroll, n4, ...)                                                               \
    do {                                                                                                   \
        const unsigned _g1 = (unsigned)ceil_div(n4, (size_t)EW_THREADS * 1);                               \
        switch (unroll) {                                                                                  \
            case 8: hipLaunchKernelGGL((KERNEL_T<8>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 8)), \
                                       dim3(EW_THREADS), 0, g_ctx.stream, __VA_ARGS__); break;             \
            case 4: hipLaunchKernelGGL((KERNEL_T<4>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 4)), \
                                       dim3(EW_THREADS), 0, g_ctx.stream, __VA_ARGS__); break;             \
            case 2: hipLaunchKernelGGL((KERNEL_T<2>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 2)), \
                                       dim3(EW_THREADS), 0, g_ctx.stream, __VA_ARGS__); break;             \
            default: hipLaunchKernelGGL((KERNEL_T<1>), dim3(_g1), dim3(EW_THREADS), 0, g_ctx.stream,       \
                                        __VA_ARGS__); break;                                               \
        }                                                                                                  \
    } while (0)

}   // namespace

// n4 vector part + scalar tail split used by every elementwise op
static inline void split_vec(size_t n, bool vec_ok, size_t &n4, size_t &tail_lo) {
    n4 = vec_ok ? n / 4 : 0;
    tail_lo = n4 * 4;
}

MI355_API int mi355_swiglu_fwd_dev(float *out, const float *h1, const float *h3, size_t n) {
    if (!mi355_ready("swiglu_fwd")) return -1;
    if (!out || !h1 || !h3) return mi355_fail("swiglu_fwd: NULL pointer");
    if (n == 0) return mi355_fail("swiglu_fwd: empty tensor");
    size_t n4, lo;
    split_vec(n, aligned16(out) && aligned16(h1) && aligned16(h3), n4, lo);
    if (n4) {
        const int u = pick_unroll(n4, 1);
        EW_LAUNCH(swiglu_fwd_kernel, u, n4, out, h1, h3, n4);
        LAUNCH_OK("swiglu_fwd");
    }
    if (lo < n) {
        hipLaunchKernelGGL(swiglu_fwd_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, out,
                           h1, h3, lo, n);
        LAUNCH_OK("swiglu_fwd tail");
    }
    return 0;
}

MI355_API int mi355_swiglu_bwd_dev(float *dh1, float *dh3, const float *dsilu, const float *h1, const float *h3,
                                   size_t n) {
    if (!mi355_ready("swiglu_bwd")) return -1;
    if (!dh1 || !dh3 || !dsilu || !h1 || !h3) return mi355_fail("swiglu_bwd: NULL pointer");
    if (n == 0) return mi355_fail("swiglu_bwd: empty tensor");
    size_t n4, lo;
    split_vec(n, aligned16(dh1) && aligned16(dh3) && aligned16(dsilu) && aligned16(h1) && aligned16(h3), n4, lo);
    if (n4) {
        const int u = pick_unroll(n4, 1);
        EW_LAUNCH(swiglu_bwd_kernel, u, n4, dh1, dh3, dsilu, h1, h3, n4);
        LAUNCH_OK("swiglu_bwd");
    }
    if (lo < n) {
        hipLaunchKernelGGL(swiglu_bwd_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, dh1,
                           dh3, dsilu, h1, h3, lo, n);
        LAUNCH_OK("swiglu_bwd tail");
    }
    return 0;
}

template <int MODE>
static int axpby_run(float *y, const float *a, const float *b, float alpha, size_t n) {
    size_t n4, lo;
    split_vec(n, aligned16(y) && aligned16(a) && (MODE == 1 || aligned16(b)), n4, lo);
    if (n4) {
        const int u = pick_unroll(n4, 1);
        switch (u) {
            case 8: hipLaunchKernelGGL((axpby_kernel<MODE, 8>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 8)), dim3(EW_THREADS), 0, g_ctx.stream, y, a, b, alpha, n4); break;
            case 4: hipLaunchKernelGGL((axpby_kernel<MODE, 4>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 4)), dim3(EW_THREADS), 0, g_ctx.stream, y, a, b, alpha, n4); break;
            case 2: hipLaunchKernelGGL((axpby_kernel<MODE, 2>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS * 2)), dim3(EW_THREADS), 0, g_ctx.stream, y, a, b, alpha, n4); break;
            default: hipLaunchKernelGGL((axpby_kernel<MODE, 1>), dim3((unsigned)ceil_div(n4, (size_t)EW_THREADS)), dim3(EW_THREADS), 0, g_ctx.stream, y, a, b, alpha, n4); break;
        }
        LAUNCH_OK("axpby");
    }
    if (lo < n) {
        hipLaunchKernelGGL((axpby_scalar<MODE>), dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, y, a,
                           b, alpha, lo, n);
        LAUNCH_OK("axpby tail");
    }
    return 0;
}

MI355_API int mi355_axpby_dev(float *y, const float *a, const float *b, float alpha, size_t n, int mode) {
    if (!mi355_ready("axpby")) return -1;
    if (!y || !a || (mode != 1 && !b)) return mi355_fail("axpby: NULL pointer");
    if (n == 0) return mi355_fail("axpby: empty tensor");
    switch (mode) {
        case 0: return axpby_run<0>(y, a, b, alpha, n);
        case 1: return axpby_run<1>(y, a, b, alpha, n);
        case 2: return axpby_run<2>(y, a, b, alpha, n);
        default: return mi355_fail("axpby: mode must be 0, 1 or 2");
    }
}

// ---- RoPE ----
MI355_API int mi355_rope_tables(float *cos_host, float *sin_host, int S, int hd, float theta) {
    if (!cos_host || !sin_host) return mi355_fail("rope_tables: NULL pointer");
    if (S <= 0 || hd <= 0 || (hd & 1) || !(theta > 0.f)) return mi355_fail("rope_tables: bad S/hd/theta");
    for (int i = 0; i < hd / 2; i++) {
        // training/training_dynamic/cpu_ops.h:172-175
        const float freq = 1.0f / powf(theta, 2.0f * i / (float)hd);
        for (int p = 0; p < S; p++) {
            const float ang = p * freq;
            cos_host[(size_t)i * S + p] = cosf(ang);
            sin_host[(size_t)i * S + p] = sinf(ang);
        }
    }
    return 0;
}

struct RopeCache {
    int S, hd;
    float theta;
    float *cos_d, *sin_d;
};
// Tables stay where they are until shutdown (callers keep the pointers), so the cache only grows: up to ROPE_MAX_TABLES
// entries and ROPE_MAX_BYTES of device memory, far beyond what a training job asks for (one or two sequence lengths).
constexpr int ROPE_MAX_TABLES = 1024;
constexpr size_t ROPE_MAX_BYTES = (size_t)256 << 20;
static RopeCache *g_rope = nullptr;
static int g_rope_n = 0, g_rope_cap = 0;
static size_t g_rope_bytes = 0;

void mi355_free_rope_cache(void) {
    for (int i = 0; i < g_rope_n; i++) (void)hipFree(g_rope[i].cos_d);   // one allocation holds both
    free(g_rope);
    g_rope = nullptr;
    g_rope_n = g_rope_cap = 0;
    g_rope_bytes = 0;
}

MI355_API int mi355_rope_tables_dev(const float **cos_dev, const float **sin_dev, int S, int hd, float theta) {
    if (!mi355_ready("rope_tables_dev")) return -1;
    if (!cos_dev || !sin_dev) return mi355_fail("rope_tables_dev: NULL pointer");
    for (int i = 0; i < g_rope_n; i++)
        if (g_rope[i].S == S && g_rope[i].hd == hd && g_rope[i].theta == theta) {
            *cos_dev = g_rope[i].cos_d;
            *sin_dev = g_rope[i].sin_d;
            return 0;
        }
    if (!mi355_outside_capture("rope_tables_dev (first use of this S, head size and theta)")) return -1;
    if (S <= 0 || hd <= 0 || (hd & 1) || !(theta > 0.f)) return mi355_fail("rope_tables_dev: bad S/hd/theta");
    const size_t n = (size_t)(hd / 2) * S;
    if (g_rope_n == ROPE_MAX_TABLES || g_rope_bytes + 2 * n * sizeof(float) > ROPE_MAX_BYTES)
        return mi355_fail("rope_tables_dev: table cache full (%d tables, %zu MiB; the limits are %d and %zu MiB until shutdown)",
                          g_rope_n, g_rope_bytes >> 20, ROPE_MAX_TABLES, ROPE_MAX_BYTES >> 20);
    if (g_rope_n == g_rope_cap) {
        const int cap = g_rope_cap ? 2 * g_rope_cap : 16;
        RopeCache *grown = (RopeCache *)realloc(g_rope, (size_t)cap * sizeof(RopeCache));
        if (!grown) return mi355_fail("rope_tables_dev: out of host memory");
        g_rope = grown;
        g_rope_cap = cap;
    }
    float *host = (float *)malloc(2 * n * sizeof(float));
    if (!host) return mi355_fail("rope_tables_dev: out of host memory");
    mi355_rope_tables(host, host + n, S, hd, theta);
    float *dev = nullptr;
    hipError_t e = hipMalloc((void **)&dev, 2 * n * sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(dev, host, 2 * n * sizeof(float), hipMemcpyHostToDevice);
    free(host);
    if (e != hipSuccess) {
        if (dev) (void)hipFree(dev);
        return mi355_fail("rope_tables_dev: %s", hipGetErrorString(e));
    }
    g_rope[g_rope_n++] = RopeCache{S, hd, theta, dev, dev + n};
    g_rope_bytes += 2 * n * sizeof(float);
    *cos_dev = dev;
    *sin_dev = dev + n;
    return 0;
}

MI355_API int mi355_rope_dev(float *q_out, float *k_out, const float *q_in, const float *k_in, int heads, int kv_heads,
                             int hd, int S, int batch, const float *cos_dev, const float *sin_dev, int dir) {
    if (!mi355_ready("rope")) return -1;
    if (!cos_dev || !sin_dev) return mi355_fail("rope: NULL table");
    if (hd <= 0 || (hd & 1) || S <= 0 || batch <= 0 || heads < 0 || kv_heads < 0 || heads + kv_heads == 0)
        return mi355_fail("rope: bad shape heads=%d kv_heads=%d hd=%d S=%d batch=%d", heads, kv_heads, hd, S, batch);
    if ((heads > 0 && (!q_out || !q_in)) || (kv_heads > 0 && (!k_out || !k_in))) return mi355_fail("rope: NULL pointer");
    if (dir != 1 && dir != -1) return mi355_fail("rope: dir must be +1 or -1");
    const bool vec_ok = (S % 4 == 0) && aligned16(cos_dev) && aligned16(sin_dev) &&
                        (heads == 0 || (aligned16(q_in) && aligned16(q_out))) &&
                        (kv_heads == 0 || (aligned16(k_in) && aligned16(k_out)));
    const size_t pair_rows = (size_t)batch * (heads + kv_heads) * (hd / 2);
    if (vec_ok) {
        const size_t total = pair_rows * (S / 4);
        hipLaunchKernelGGL((rope_kernel<4>), dim3((unsigned)ceil_div(total, EW_THREADS)), dim3(EW_THREADS), 0,
                           g_ctx.stream, q_out, k_out, q_in, k_in, heads, kv_heads, hd, S, batch, cos_dev, sin_dev,
                           (float)dir, total);
    } else {
        const size_t total = pair_rows * S;
        hipLaunchKernelGGL((rope_kernel<1>), dim3((unsigned)ceil_div(total, EW_THREADS)), dim3(EW_THREADS), 0,
                           g_ctx.stream, q_out, k_out, q_in, k_in, heads, kv_heads, hd, S, batch, cos_dev, sin_dev,
                           (float)dir, total);
    }
    LAUNCH_OK("rope");
    return 0;
}

// ---- range diagnostics ----
MI355_API int mi355_minmax_dev(float *out3_dev, const float *x, size_t n) {
    if (!mi355_ready("minmax")) return -1;
    if (!out3_dev || !x) return mi355_fail("minmax: NULL pointer");
    if (n == 0) return mi355_fail("minmax: empty tensor");
    const bool vec = aligned16(x);
    const size_t n4 = vec ? n / 4 : 0;
    size_t blocks = ceil_div(vec ? (n4 ? n4 : 1) : n, (size_t)EW_THREADS);
    if (blocks > 4096) blocks = 4096;
    float *part = (float *)mi355_ws(2 * blocks * sizeof(float));
    if (!part) return -1;
    hipLaunchKernelGGL(minmax_kernel, dim3((unsigned)blocks), dim3(EW_THREADS), 0, g_ctx.stream, part, x, n, n4, vec);
    hipLaunchKernelGGL(minmax_final_kernel, dim3(1), dim3(1024), 0, g_ctx.stream, out3_dev, part, (int)blocks);
    LAUNCH_OK("minmax");
    return 0;
}

// ---- INT8 ----
MI355_API int mi355_int8_scale_dev(float *scale_dev, const float *x, size_t n) {
    if (!mi355_ready("int8_scale")) return -1;
    if (!scale_dev || !x) return mi355_fail("int8_scale: NULL pointer");
    if (n == 0) return mi355_fail("int8_scale: empty tensor");
    const bool vec = aligned16(x);
    const size_t n4 = vec ? n / 4 : 0;
    if (g_ctx.rms_cluster < 0) {
        // the cooperating forms are switched off ("rms_cluster" = -1, by hand or by the watch in mi355_sync): per-workgroup
        // maxima, then one workgroup folds them (the maximum is exact in any order: the same bits)
        size_t nb = ceil_div(vec ? (n4 ? n4 : 1) : n, (size_t)EW_THREADS * 4);
        if (nb > 1024) nb = 1024;
        float *part = (float *)mi355_ws(nb * sizeof(float));
        if (!part) return -1;
        hipLaunchKernelGGL(absmax_kernel, dim3((unsigned)nb), dim3(EW_THREADS), 0, g_ctx.stream, part, x, n, n4, vec);
        hipLaunchKernelGGL(scale_from_partials_kernel, dim3(1), dim3(1024), 0, g_ctx.stream, scale_dev, part, (int)nb);
        LAUNCH_OK("int8_scale (two launches)");
        return 0;
    }
    // one workgroup of 1024 threads per compute unit, fewer for small tensors (at least 4 accesses per thread)
    const size_t per_block = (size_t)1024 * 4;
    size_t blocks = ceil_div(vec ? (n4 ? n4 : 1) : n, per_block);
    const size_t cus = g_ctx.num_cu > 0 ? (size_t)g_ctx.num_cu : 256;
    if (blocks > cus) blocks = cus;
    if (blocks > 1024) blocks = 1024;
    Mi355Exchange xch;
    if (!mi355_exchange(&xch)) return -1;
    hipLaunchKernelGGL(absmax_scale_kernel, dim3((unsigned)blocks), dim3(1024), 0, g_ctx.stream, scale_dev, x, n, n4, vec, xch,
                       mi355_exchange_spin_ticks());
    LAUNCH_OK("int8_scale");
    return 0;
}

MI355_API int mi355_int8_quant_dev(int8_t *q, const float *x, const float *scale_dev, size_t n, int rounding) {
    if (!mi355_ready("int8_quant")) return -1;
    if (!q || !x || !scale_dev) return mi355_fail("int8_quant: NULL pointer");
    if (n == 0) return mi355_fail("int8_quant: empty tensor");
    if (rounding != 0 && rounding != 1) return mi355_fail("int8_quant: rounding must be 0 or 1");
    size_t n4, lo;
    split_vec(n, aligned16(x) && ((uintptr_t)q & 3u) == 0, n4, lo);
    if (n4) {
        const int u = pick_unroll(n4, 1);
        EW_LAUNCH(quant_kernel, u, n4, (int *)q, x, scale_dev, n4, rounding);
        LAUNCH_OK("int8_quant");
    }
    if (lo < n) {
        hipLaunchKernelGGL(quant_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, q, x,
                           scale_dev, lo, n, rounding);
        LAUNCH_OK("int8_quant tail");
    }
    return 0;
}

MI355_API int mi355_int8_quantize_dynamic_dev(int8_t *q, float *scale_dev, const float *x, size_t n, int rounding) {
    if (!mi355_ready("int8_quantize_dynamic")) return -1;
    if (!q || !x || !scale_dev) return mi355_fail("int8_quantize_dynamic: NULL pointer");
    if (n == 0) return mi355_fail("int8_quantize_dynamic: empty tensor");
    if (rounding != 0 && rounding != 1) return mi355_fail("int8_quantize_dynamic: rounding must be 0 or 1");
    size_t n4, lo;
    split_vec(n, aligned16(x) && ((uintptr_t)q & 3u) == 0, n4, lo);
    if (n4 == 0) {      // no vector body: the two separate steps
        if (mi355_int8_scale_dev(scale_dev, x, n)) return -1;
        return mi355_int8_quant_dev(q, x, scale_dev, n, rounding);
    }
    {
        // one launch while a workgroup per compute unit can hold the tensor in registers (up to 8 groups of four per
        // thread: 8.4 M floats on 256 compute units); "rms_cluster" = -1 switches the cooperating forms off
        const size_t cus = g_ctx.num_cu > 0 ? (size_t)g_ctx.num_cu : 256;
        size_t nb = std::min(std::min(ceil_div(n4, (size_t)1024), cus), (size_t)XCH_MAX_BLOCKS);
        const size_t per = ceil_div(n4, nb * 1024);
        if (g_ctx.rms_cluster >= 0 && per <= 8) {
            Mi355Exchange xch;
            if (!mi355_exchange(&xch)) return -1;
            const int spin = mi355_exchange_spin_ticks();
#define QDYN(P)                                                                                                        \
    hipLaunchKernelGGL(quant_dyn_one_kernel<P>, dim3((unsigned)nb), dim3(1024), 0, g_ctx.stream, (int *)q, scale_dev, x, n, \
                       n4, rounding, xch, spin)
            if (per <= 1) QDYN(1); else if (per <= 2) QDYN(2); else if (per <= 4) QDYN(4); else QDYN(8);
#undef QDYN
            LAUNCH_OK("int8_quantize_dynamic");
            if (lo < n) {
                hipLaunchKernelGGL(quant_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, q, x,
                                   scale_dev, lo, n, rounding);
                LAUNCH_OK("int8_quantize_dynamic tail");
            }
            return 0;
        }
    }
    size_t blocks = ceil_div(n4, (size_t)EW_THREADS);
    if (blocks > 256) blocks = 256;         // one workgroup per compute unit; few maxima for the quantizer to fold
    float *part = (float *)mi355_ws(blocks * sizeof(float));
    if (!part) return -1;
    hipLaunchKernelGGL(absmax_kernel, dim3((unsigned)blocks), dim3(EW_THREADS), 0, g_ctx.stream, part, x, n, n / 4, true);
    const int u = pick_unroll(n4, 1);
    EW_LAUNCH(quant_dyn_kernel, u, n4, (int *)q, x, part, (int)blocks, scale_dev, n4, rounding);
    LAUNCH_OK("int8_quantize_dynamic");
    if (lo < n) {
        hipLaunchKernelGGL(quant_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, q, x,
                           scale_dev, lo, n, rounding);
        LAUNCH_OK("int8_quantize_dynamic tail");
    }
    return 0;
}

MI355_API int mi355_int8_dequant_dev(float *x, const int8_t *q, const float *scale_dev, size_t n) {
    if (!mi355_ready("int8_dequant")) return -1;
    if (!q || !x || !scale_dev) return mi355_fail("int8_dequant: NULL pointer");
    if (n == 0) return mi355_fail("int8_dequant: empty tensor");
    size_t n4, lo;
    split_vec(n, aligned16(x) && ((uintptr_t)q & 3u) == 0, n4, lo);
    if (n4) {
        const int u = pick_unroll(n4, 1);
        EW_LAUNCH(dequant_kernel, u, n4, x, (const int *)q, scale_dev, n4);
        LAUNCH_OK("int8_dequant");
    }
    if (lo < n) {
        hipLaunchKernelGGL(dequant_scalar, dim3((unsigned)ceil_div(n - lo, 256)), dim3(256), 0, g_ctx.stream, x, q,
                           scale_dev, lo, n);
        LAUNCH_OK("int8_dequant tail");
    }
    return 0;
}

// ---- GQA tile / reduce ----
static int gqa_run(bool reduce, float *out, const float *in, int kv_heads, int ratio, int hd, int S, int batch) {
    const char *who = reduce ? "gqa_reduce" : "gqa_tile";
    if (!mi355_ready(who)) return -1;
    if (!out || !in) return mi355_fail("%s: NULL pointer", who);
    if (kv_heads <= 0 || ratio <= 0 || hd <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("%s: bad shape kv_heads=%d ratio=%d hd=%d S=%d batch=%d", who, kv_heads, ratio, hd, S, batch);
    const size_t slab = (size_t)hd * S;
    const bool vec = (slab % 4 == 0) && aligned16(out) && aligned16(in);
    const size_t slabv = vec ? slab / 4 : slab;
    const size_t total = (size_t)batch * kv_heads * slabv;
    const unsigned blocks = (unsigned)ceil_div(total, EW_THREADS);
    if (reduce) {
        if (vec) hipLaunchKernelGGL((gqa_reduce_kernel<4>), dim3(blocks), dim3(EW_THREADS), 0, g_ctx.stream, out, in, kv_heads, ratio, slabv, total);
        else hipLaunchKernelGGL((gqa_reduce_kernel<1>), dim3(blocks), dim3(EW_THREADS), 0, g_ctx.stream, out, in, kv_heads, ratio, slabv, total);
    } else {
        if (vec) hipLaunchKernelGGL((gqa_tile_kernel<4>), dim3(blocks), dim3(EW_THREADS), 0, g_ctx.stream, out, in, kv_heads, ratio, slabv, total);
        else hipLaunchKernelGGL((gqa_tile_kernel<1>), dim3(blocks), dim3(EW_THREADS), 0, g_ctx.stream, out, in, kv_heads, ratio, slabv, total);
    }
    LAUNCH_OK(who);
    return 0;
}

MI355_API int mi355_gqa_tile_dev(float *out, const float *in, int kv_heads, int ratio, int hd, int S, int batch) {
    return gqa_run(false, out, in, kv_heads, ratio, hd, S, batch);
}

MI355_API int mi355_gqa_reduce_dev(float *out, const float *in, int kv_heads, int ratio, int hd, int S, int batch) {
    return gqa_run(true, out, in, kv_heads, ratio, hd, S, batch);
}
