// staging.hip — fp32 <-> fp16 staging converts and the attention-gradient finish.
//
// The dynamic loop keeps every activation as fp32 [C,S] on the host and converts to fp16 each time a tensor
// goes onto or comes off an accelerator surface (cvt_f32_f16 / cvt_f16_f32,
// training/training_dynamic/io.h:33-50, used by io_write_fp16 / io_read_fp16 / io_write_fp16_at /
// io_write_dyn / io_read_dyn, io.h:53-96, and the per-kernel packers io.h:160-310).  Every one of those is a
// rectangle copy with a conversion: `rows` runs of `cols` contiguous elements, source and destination each
// with their own row pitch.  The converts here take that rectangle.
//
// After the attention backward kernels the loop reads dQ, dK, dV (fp16, all at the query head count),
// sums the query heads of each KV group for dK and dV, copies dQ, and un-rotates dQ and dK
// (training/training_dynamic/train.m:646-660).  attn_grads_finish does that chain in one pass: each
// lane reads its fp16 (or fp32) inputs once and writes the three fp32 results once.
#include "common.h"

namespace {

constexpr int ST_THREADS = 256;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));

// ---- rectangle converts: one lane = 8 contiguous elements of one row ----
__global__ __launch_bounds__(ST_THREADS) void cvt_f32_f16_v8(_Float16 *__restrict__ dst, size_t dst_ld,
                                                             const float *__restrict__ src, size_t src_ld,
                                                             size_t colg, size_t total) {
    const size_t i = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / colg, g = i - r * colg;
    const float *s = src + r * src_ld + 8 * g;
    const v4f a = ld4_nt(s), b = ld4_nt(s + 4);
    h8 o;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        o[j] = (_Float16)a[j];       // round to nearest even, overflow to infinity, subnormals kept
        o[4 + j] = (_Float16)b[j];
    }
    __builtin_nontemporal_store(o, reinterpret_cast<h8 *>(dst + r * dst_ld + 8 * g));
}

__global__ __launch_bounds__(ST_THREADS) void cvt_f16_f32_v8(float *__restrict__ dst, size_t dst_ld,
                                                             const _Float16 *__restrict__ src, size_t src_ld,
                                                             size_t colg, size_t total) {
    const size_t i = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / colg, g = i - r * colg;
    const h8 v = __builtin_nontemporal_load(reinterpret_cast<const h8 *>(src + r * src_ld + 8 * g));
    v4f a, b;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        a[j] = (float)v[j];
        b[j] = (float)v[4 + j];
    }
    float *d = dst + r * dst_ld + 8 * g;
    st4_nt(d, a);
    st4_nt(d + 4, b);
}

__global__ __launch_bounds__(ST_THREADS) void cvt_f32_f16_v1(_Float16 *__restrict__ dst, size_t dst_ld,
                                                             const float *__restrict__ src, size_t src_ld,
                                                             size_t cols, size_t total) {
    const size_t i = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / cols, c = i - r * cols;
    dst[r * dst_ld + c] = (_Float16)src[r * src_ld + c];
}

__global__ __launch_bounds__(ST_THREADS) void cvt_f16_f32_v1(float *__restrict__ dst, size_t dst_ld,
                                                             const _Float16 *__restrict__ src, size_t src_ld,
                                                             size_t cols, size_t total) {
    const size_t i = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / cols, c = i - r * cols;
    dst[r * dst_ld + c] = (float)src[r * src_ld + c];
}

// ---- attention-gradient finish ----
template <typename T, int VEC>
__device__ __forceinline__ void load_cols(float (&o)[VEC], const T *p) {
    if constexpr (VEC == 1) {
        o[0] = (float)p[0];
    } else if constexpr (sizeof(T) == 2) {
        static_assert(VEC == 8, "fp16 rows are read 8 columns at a time");
        const h8 v = __builtin_nontemporal_load(reinterpret_cast<const h8 *>(p));
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = (float)v[j];
    } else {
        static_assert(VEC == 4, "fp32 rows are read 4 columns at a time");
        const v4f v = ld4_nt(reinterpret_cast<const float *>(p));
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = v[j];
    }
}

// table rows are shared by every head and sequence: ordinary (cached) loads
template <int VEC>
__device__ __forceinline__ void load_tab(float (&o)[VEC], const float *p) {
    if constexpr (VEC == 1) {
        o[0] = p[0];
    } else {
#pragma unroll
        for (int q = 0; q < VEC / 4; q++) {
            const v4f v = ld4(p + 4 * q);
#pragma unroll
            for (int j = 0; j < 4; j++) o[4 * q + j] = v[j];
        }
    }
}

template <int VEC>
__device__ __forceinline__ void store_cols(float *p, const float (&o)[VEC]) {
    if constexpr (VEC == 1) {
        p[0] = o[0];
    } else {
#pragma unroll
        for (int q = 0; q < VEC / 4; q++) {
            v4f v = {o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
            st4_nt(p + 4 * q, v);
        }
    }
}

// One lane = one interleaved row pair (2i, 2i+1) of one output head x VEC columns.
// Pair rows are numbered Q heads first, then K heads, then V heads.
template <typename T, int VEC>
__global__ __launch_bounds__(ST_THREADS) void attn_grads_finish_kernel(
    float *dq, float *__restrict__ dk, float *__restrict__ dv, const T *qf, const T *__restrict__ kf,
    const T *__restrict__ vf, size_t sq, size_t sk, size_t sv, int heads, int kv_heads, int ratio, int hd, int S,
    int batch, const float *__restrict__ cos_t, const float *__restrict__ sin_t, size_t total) {
    const size_t idx = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
    if (idx >= total) return;
    const int colg = S / VEC;
    const int cg = (int)(idx % colg);
    size_t pr = idx / colg;
    const int half = hd >> 1;
    const int s = cg * VEC;
    const size_t q_rows = (size_t)batch * heads * half, kv_rows = (size_t)batch * kv_heads * half;

    float r0[VEC], r1[VEC];
    float *out;
    int i;
    bool rotate;
    if (pr < q_rows) {
        i = (int)(pr % half);
        const size_t bh = pr / half;                 // b*heads + h
        const size_t b = bh / heads, h = bh - b * heads;
        const T *in = qf + b * sq + (h * hd + 2 * i) * (size_t)S + s;
        load_cols<T, VEC>(r0, in);
        load_cols<T, VEC>(r1, in + S);
        out = dq + (bh * hd + 2 * i) * (size_t)S + s;
        rotate = true;
    } else {
        pr -= q_rows;
        const bool is_k = pr < kv_rows;
        if (!is_k) pr -= kv_rows;
        i = (int)(pr % half);
        const size_t bh = pr / half;                 // b*kv_heads + kv
        const size_t b = bh / kv_heads, kv = bh - b * kv_heads;
        const T *in = (is_k ? kf + b * sk : vf + b * sv) + ((kv * ratio) * hd + 2 * i) * (size_t)S + s;
#pragma unroll
        for (int j = 0; j < VEC; j++) r0[j] = r1[j] = 0.f;
        for (int r = 0; r < ratio; r++) {            // zero, then += in query-head order (io.h:342-350)
            float a0[VEC], a1[VEC];
            load_cols<T, VEC>(a0, in + (size_t)r * hd * S);
            load_cols<T, VEC>(a1, in + (size_t)r * hd * S + S);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                r0[j] += a0[j];
                r1[j] += a1[j];
            }
        }
        out = (is_k ? dk : dv) + (bh * hd + 2 * i) * (size_t)S + s;
        rotate = is_k;
    }
    if (rotate && cos_t) {
        float c[VEC], sn[VEC];
        load_tab<VEC>(c, cos_t + (size_t)i * S + s);
        load_tab<VEC>(sn, sin_t + (size_t)i * S + s);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            // inverse rotation, written as the forward one with the sine negated
            const float ns = sn[j] * -1.0f;
            const float x0 = r0[j], x1 = r1[j];
            r0[j] = x0 * c[j] - x1 * ns;
            r1[j] = x0 * ns + x1 * c[j];
        }
    }
    store_cols<VEC>(out, r0);
    store_cols<VEC>(out + S, r1);
}

int cvt_args(const char *who, const void *dst, const void *src, size_t dst_ld, size_t src_ld, size_t rows,
             size_t cols) {
    if (!mi355_ready(who)) return -1;
    if (!dst || !src) return mi355_fail("%s: NULL pointer", who);
    if (rows == 0 || cols == 0) return mi355_fail("%s: empty rectangle rows=%zu cols=%zu", who, rows, cols);
    if (dst_ld < cols || src_ld < cols)
        return mi355_fail("%s: row pitch below the row length (cols=%zu dst_ld=%zu src_ld=%zu)", who, cols, dst_ld,
                          src_ld);
    return 0;
}

}   // namespace

MI355_API int mi355_cvt_f32_f16_dev(uint16_t *dst, size_t dst_ld, const float *src, size_t src_ld, size_t rows,
                                    size_t cols) {
    if (cvt_args("cvt_f32_f16", dst, src, dst_ld, src_ld, rows, cols)) return -1;
    _Float16 *d = reinterpret_cast<_Float16 *>(dst);
    const bool vec = cols % 8 == 0 && dst_ld % 8 == 0 && src_ld % 4 == 0 && aligned16(dst) && aligned16(src);
    if (vec) {
        const size_t colg = cols / 8, total = rows * colg;
        hipLaunchKernelGGL(cvt_f32_f16_v8, dim3((unsigned)ceil_div(total, ST_THREADS)), dim3(ST_THREADS), 0,
                           g_ctx.stream, d, dst_ld, src, src_ld, colg, total);
    } else {
        const size_t total = rows * cols;
        hipLaunchKernelGGL(cvt_f32_f16_v1, dim3((unsigned)ceil_div(total, ST_THREADS)), dim3(ST_THREADS), 0,
                           g_ctx.stream, d, dst_ld, src, src_ld, cols, total);
    }
    LAUNCH_OK("cvt_f32_f16");
    return 0;
}

MI355_API int mi355_cvt_f16_f32_dev(float *dst, size_t dst_ld, const uint16_t *src, size_t src_ld, size_t rows,
                                    size_t cols) {
    if (cvt_args("cvt_f16_f32", dst, src, dst_ld, src_ld, rows, cols)) return -1;
    const _Float16 *s = reinterpret_cast<const _Float16 *>(src);
    const bool vec = cols % 8 == 0 && dst_ld % 4 == 0 && src_ld % 8 == 0 && aligned16(dst) && aligned16(src);
    if (vec) {
        const size_t colg = cols / 8, total = rows * colg;
        hipLaunchKernelGGL(cvt_f16_f32_v8, dim3((unsigned)ceil_div(total, ST_THREADS)), dim3(ST_THREADS), 0,
                           g_ctx.stream, dst, dst_ld, s, src_ld, colg, total);
    } else {
        const size_t total = rows * cols;
        hipLaunchKernelGGL(cvt_f16_f32_v1, dim3((unsigned)ceil_div(total, ST_THREADS)), dim3(ST_THREADS), 0,
                           g_ctx.stream, dst, dst_ld, s, src_ld, cols, total);
    }
    LAUNCH_OK("cvt_f16_f32");
    return 0;
}

MI355_API int mi355_attn_grads_finish_dev(float *dq, float *dk, float *dv, const void *dq_full, const void *dk_full,
                                          const void *dv_full, int in_f16, size_t q_stride, size_t k_stride,
                                          size_t v_stride, int heads, int kv_heads, int hd, int S, int batch,
                                          const float *cos_dev, const float *sin_dev) {
    if (!mi355_ready("attn_grads_finish")) return -1;
    if (!dq || !dk || !dv || !dq_full || !dk_full || !dv_full) return mi355_fail("attn_grads_finish: NULL pointer");
    if ((cos_dev == nullptr) != (sin_dev == nullptr))
        return mi355_fail("attn_grads_finish: pass both rotation tables or neither");
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || hd <= 0 || (hd & 1) || S <= 0 || batch <= 0)
        return mi355_fail("attn_grads_finish: bad shape heads=%d kv_heads=%d hd=%d S=%d batch=%d", heads, kv_heads, hd,
                          S, batch);
    const size_t full = (size_t)heads * hd * S;
    if (!q_stride) q_stride = full;
    if (!k_stride) k_stride = full;
    if (!v_stride) v_stride = full;
    if (q_stride < full || k_stride < full || v_stride < full)
        return mi355_fail("attn_grads_finish: sequence stride below heads*hd*S = %zu", full);
    const int ratio = heads / kv_heads;
    const size_t pair_rows = (size_t)batch * (heads + 2 * kv_heads) * (hd / 2);
    const bool out_al = aligned16(dq) && aligned16(dk) && aligned16(dv);
    const bool tab_al = !cos_dev || (aligned16(cos_dev) && aligned16(sin_dev));
    const bool in_al = aligned16(dq_full) && aligned16(dk_full) && aligned16(dv_full);
#define FINISH(T, VEC)                                                                                               \
    do {                                                                                                             \
        const size_t total = pair_rows * (size_t)(S / (VEC));                                                        \
        hipLaunchKernelGGL((attn_grads_finish_kernel<T, VEC>), dim3((unsigned)ceil_div(total, ST_THREADS)),          \
                           dim3(ST_THREADS), 0, g_ctx.stream, dq, dk, dv, (const T *)dq_full, (const T *)dk_full,    \
                           (const T *)dv_full, q_stride, k_stride, v_stride, heads, kv_heads, ratio, hd, S, batch,   \
                           cos_dev, sin_dev, total);                                                                 \
    } while (0)
    if (in_f16) {
        const bool vec = S % 8 == 0 && out_al && tab_al && in_al && q_stride % 8 == 0 && k_stride % 8 == 0 &&
                         v_stride % 8 == 0;
        if (vec) FINISH(_Float16, 8);
        else FINISH(_Float16, 1);
    } else {
        const bool vec = S % 4 == 0 && out_al && tab_al && in_al && q_stride % 4 == 0 && k_stride % 4 == 0 &&
                         v_stride % 4 == 0;
        if (vec) FINISH(float, 4);
        else FINISH(float, 1);
    }
#undef FINISH
    LAUNCH_OK("attn_grads_finish");
    return 0;
}
