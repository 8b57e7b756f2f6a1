// qknorm_rope.hip — Qwen3 per-head QK-RMSNorm fused with RoPE, forward and backward, one HBM pass.
//
// Not present in the reference: forward = rmsnorm (training/stories_cpu_ops.h:6-21) on each head's
// [hd,S] slab with a [hd] weight shared by the heads, then the forward rotation of interleaved row
// pairs (training/forward.h:55-70, training/training_dynamic/mil_dynamic.h:131-168); backward = the
// inverse rotation (training/training_dynamic/cpu_ops.h:168-184) then rmsnorm_bwd per head
// (training/stories_cpu_ops.h:23-53).
//
// A workgroup owns one head slab x a strip of LPR*4 columns.  Each thread owns whole row PAIRS
// (2i, 2i+1), so the rotation needs no cross-lane traffic; the norm reduction over the hd rows
// uses the same shuffle + LDS exchange as the RMSNorm kernels.
#include "common.h"
#include "tile.h"

namespace {

template <int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void qknorm_rope_fwd_kernel(
    float *__restrict__ q_out, float *__restrict__ k_out, const float *__restrict__ q, const float *__restrict__ k,
    const float *__restrict__ wq, const float *__restrict__ wk, int hd, int S, int strips, int nq,
    const float *__restrict__ cos_t, const float *__restrict__ sin_t, float eps, float invhd) {
    constexpr int PPS = THREADS / LPR;   // row pairs per step
    constexpr int W = LPR * 4;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * LPR * 4];
    int blk = blockIdx.x;
    const float *in, *w;
    float *out;
    if (blk < nq) { in = q; out = q_out; w = wq; }
    else { blk -= nq; in = k; out = k_out; w = wk; }
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, p0 = threadIdx.x / LPR;
    const int col = strip * W + lc * 4;
    const bool col_ok = col < S;
    const int half = hd >> 1;
    const size_t base = (size_t)slab * hd * S + col;

    v4f x0[CAP], x1[CAP];
    float w0[CAP], w1[CAP];
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half && col_ok) {
            const float *px = in + base + (size_t)(2 * rp) * S;
            x0[kk] = ld4_nt(px);
            x1[kk] = ld4_nt(px + S);
            w0[kk] = w[2 * rp];
            w1[kk] = w[2 * rp + 1];
        } else {
            x0[kk] = x1[kk] = zero;
            w0[kk] = w1[kk] = 0.f;
        }
    }
    float acc[1][4] = {{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int kk = 0; kk < CAP; kk++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[0][j] += x0[kk][j] * x0[kk][j];
            acc[0][j] += x1[kk][j] * x1[kk][j];
        }
    strip_reduce<4, LPR, THREADS, 1>(acc, lds);
    v4f rr;
#pragma unroll
    for (int j = 0; j < 4; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invhd + eps);
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half && col_ok) {
            // the tables are shared by every head and sequence (cache-resident): read here, after the reduction,
            // rather than held in registers across it
            const v4f cs = ld4(cos_t + (size_t)rp * S + col), sn = ld4(sin_t + (size_t)rp * S + col);
            const v4f y0 = (x0[kk] * rr) * w0[kk];
            const v4f y1 = (x1[kk] * rr) * w1[kk];
            float *po = out + base + (size_t)(2 * rp) * S;
            st4_nt(po, y0 * cs - y1 * sn);
            st4_nt(po + S, y0 * sn + y1 * cs);
        }
    }
}

template <int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void qknorm_rope_bwd_kernel(
    float *dq, float *dk, float *__restrict__ part, const float *dq_out, const float *dk_out,
    const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ wq,
    const float *__restrict__ wk, int hd, int S, int strips, int nq, const float *__restrict__ cos_t,
    const float *__restrict__ sin_t, float eps, float invhd, int variant) {
    constexpr int PPS = THREADS / LPR;
    constexpr int W = LPR * 4;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * 2 * LPR * 4];
    int blk = blockIdx.x;
    float *prt = part + (size_t)blk * hd;
    const float *gin, *xin, *w;
    float *out;
    if (blk < nq) { gin = dq_out; xin = q; out = dq; w = wq; }
    else { blk -= nq; gin = dk_out; xin = k; out = dk; w = wk; }
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, p0 = threadIdx.x / LPR;
    const int col = strip * W + lc * 4;
    const bool col_ok = col < S;
    const int half = hd >> 1;
    const size_t base = (size_t)slab * hd * S + col;

    v4f x0[CAP], x1[CAP], d0[CAP], d1[CAP];
    float w0[CAP], w1[CAP];
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half && col_ok) {
            const size_t o = base + (size_t)(2 * rp) * S;
            x0[kk] = ld4_nt(xin + o);
            x1[kk] = ld4_nt(xin + o + S);
            const v4f g0 = ld4_nt(gin + o), g1 = ld4_nt(gin + o + S);
            const v4f c = ld4(cos_t + (size_t)rp * S + col), s = ld4(sin_t + (size_t)rp * S + col);
            d0[kk] = g0 * c + g1 * s;        // inverse rotation (cpu_ops.h:179-180)
            d1[kk] = (-g0) * s + g1 * c;
            w0[kk] = w[2 * rp];
            w1[kk] = w[2 * rp + 1];
        } else {
            x0[kk] = x1[kk] = d0[kk] = d1[kk] = zero;
            w0[kk] = w1[kk] = 0.f;
        }
    }
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int kk = 0; kk < CAP; kk++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[0][j] += x0[kk][j] * x0[kk][j];
            acc[0][j] += x1[kk][j] * x1[kk][j];
            acc[1][j] += (d0[kk][j] * x0[kk][j]) * w0[kk];
            acc[1][j] += (d1[kk][j] * x1[kk][j]) * w1[kk];
        }
    strip_reduce<4, LPR, THREADS, 2>(acc, lds);
    v4f rr, dotn;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        rr[j] = 1.0f / sqrtf(acc[0][j] * invhd + eps);
        dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invhd);
    }
#pragma unroll
    for (int kk = 0; kk < CAP; kk++) {
        const int rp = p0 + kk * PPS;
        if (rp < half) {   // uniform over each group of LPR lanes
            v4f o0, o1;
            if (variant == 0) {
                o0 = ((d0[kk] - x0[kk] * dotn) * rr) * w0[kk];
                o1 = ((d1[kk] - x1[kk] * dotn) * rr) * w1[kk];
            } else {
                o0 = (d0[kk] * w0[kk]) * rr - (x0[kk] * dotn) * rr;
                o1 = (d1[kk] * w1[kk]) * rr - (x1[kk] * dotn) * rr;
            }
            if (col_ok) {
                float *po = out + base + (size_t)(2 * rp) * S;
                st4_nt(po, o0);
                st4_nt(po + S, o1);
            }
            const v4f t0 = (d0[kk] * x0[kk]) * rr, t1 = (d1[kk] * x1[kk]) * rr;
            float s0 = ((t0[0] + t0[1]) + t0[2]) + t0[3];
            float s1 = ((t1[0] + t1[1]) + t1[2]) + t1[3];
            s0 = group_sum<LPR>(s0);
            s1 = group_sum<LPR>(s1);
            if (lc == 0) {
                prt[2 * rp] = s0;
                prt[2 * rp + 1] = s1;
            }
        }
    }
}

// measured at the Qwen3 shape: 8-wave workgroups (two pairs per lane, 5 waves per SIMD) run the backward
// 7 % faster than 4-wave ones (four pairs per lane, 2 waves per SIMD); the forward does not care
constexpr int QK_THREADS_FWD = 256, QK_THREADS_BWD = 512;

struct QkCfg {
    int lpr, threads, cap;
};

// widest strip whose row pairs fit the register tile (at most 4 pairs per lane: 8 would spill)
bool pick_qk(int hd, QkCfg &cfg, bool backward) {
    const int half = hd / 2;
    const int lprs[3] = {16, 8, 4};
    const int thr = g_ctx.qk_threads == 256 || g_ctx.qk_threads == 512 ? g_ctx.qk_threads : (backward ? QK_THREADS_BWD : QK_THREADS_FWD);
    for (int lpr : lprs) {
        if (g_ctx.qk_lpr && g_ctx.qk_lpr != lpr) continue;
        const int pps = thr / lpr;
        const int caps[3] = {1, 2, 4};
        for (int cap : caps)
            if (cap * pps >= half) { cfg = QkCfg{lpr, thr, cap}; return true; }
    }
    return false;
}

#define QK_DISPATCH(KERNEL, cfg, grid, ...)                                                                   \
    do {                                                                                                      \
        const int key = (cfg).lpr * 10000 + ((cfg).threads / 256) * 100 + (cfg).cap;                          \
        switch (key) {                                                                                        \
            case 160101: hipLaunchKernelGGL((KERNEL<16, 256, 1>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 160102: hipLaunchKernelGGL((KERNEL<16, 256, 2>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 160104: hipLaunchKernelGGL((KERNEL<16, 256, 4>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 160201: hipLaunchKernelGGL((KERNEL<16, 512, 1>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 160202: hipLaunchKernelGGL((KERNEL<16, 512, 2>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 160204: hipLaunchKernelGGL((KERNEL<16, 512, 4>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80101: hipLaunchKernelGGL((KERNEL<8, 256, 1>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80102: hipLaunchKernelGGL((KERNEL<8, 256, 2>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80104: hipLaunchKernelGGL((KERNEL<8, 256, 4>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80201: hipLaunchKernelGGL((KERNEL<8, 512, 1>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80202: hipLaunchKernelGGL((KERNEL<8, 512, 2>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 80204: hipLaunchKernelGGL((KERNEL<8, 512, 4>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40101: hipLaunchKernelGGL((KERNEL<4, 256, 1>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40102: hipLaunchKernelGGL((KERNEL<4, 256, 2>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40104: hipLaunchKernelGGL((KERNEL<4, 256, 4>), grid, dim3(256), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40201: hipLaunchKernelGGL((KERNEL<4, 512, 1>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40202: hipLaunchKernelGGL((KERNEL<4, 512, 2>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            case 40204: hipLaunchKernelGGL((KERNEL<4, 512, 4>), grid, dim3(512), 0, g_ctx.stream, __VA_ARGS__); break; \
            default: return mi355_fail("qknorm_rope: no kernel for tile key %d", key);                        \
        }                                                                                                     \
    } while (0)

int check_shape(const char *who, int heads, int kv_heads, int hd, int S, int batch) {
    if (hd <= 0 || (hd & 1) || S <= 0 || batch <= 0 || heads < 0 || kv_heads < 0 || heads + kv_heads == 0)
        return mi355_fail("%s: bad shape heads=%d kv_heads=%d hd=%d S=%d batch=%d", who, heads, kv_heads, hd, S, batch);
    return 0;
}

}   // namespace

MI355_API int mi355_qknorm_rope_fwd_dev(float *q_out, float *k_out, const float *q, const float *k, const float *wq,
                                        const float *wk, int heads, int kv_heads, int hd, int S, int batch,
                                        const float *cos_dev, const float *sin_dev, float eps) {
    if (!mi355_ready("qknorm_rope_fwd")) return -1;
    if (check_shape("qknorm_rope_fwd", heads, kv_heads, hd, S, batch)) return -1;
    if (!cos_dev || !sin_dev || (heads > 0 && (!q_out || !q || !wq)) || (kv_heads > 0 && (!k_out || !k || !wk)))
        return mi355_fail("qknorm_rope_fwd: NULL pointer");
    QkCfg cfg;
    const bool vec_ok = (S % 4 == 0) && aligned16(cos_dev) && aligned16(sin_dev) &&
                        (heads == 0 || (aligned16(q) && aligned16(q_out))) &&
                        (kv_heads == 0 || (aligned16(k) && aligned16(k_out)));
    if (!vec_ok || !pick_qk(hd, cfg, false)) {
        // unfused composition: per-head norm (heads folded into the batch), then the rotation in place
        if (heads > 0 && mi355_rmsnorm_fwd_dev(q_out, q, wq, hd, S, batch * heads, eps)) return -1;
        if (kv_heads > 0 && mi355_rmsnorm_fwd_dev(k_out, k, wk, hd, S, batch * kv_heads, eps)) return -1;
        return mi355_rope_dev(q_out, k_out, q_out, k_out, heads, kv_heads, hd, S, batch, cos_dev, sin_dev, +1);
    }
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * 4);
    const int nq = batch * heads * strips, nk = batch * kv_heads * strips;
    QK_DISPATCH(qknorm_rope_fwd_kernel, cfg, dim3(nq + nk), q_out, k_out, q, k, wq, wk, hd, S, strips, nq, cos_dev,
                sin_dev, eps, 1.0f / (float)hd);
    LAUNCH_OK("qknorm_rope_fwd");
    return 0;
}

MI355_API int mi355_qknorm_rope_bwd_dev(float *dq, float *dk, float *dwq, float *dwk, const float *dq_out,
                                        const float *dk_out, const float *q, const float *k, const float *wq,
                                        const float *wk, int heads, int kv_heads, int hd, int S, int batch,
                                        const float *cos_dev, const float *sin_dev, float eps, int variant) {
    if (!mi355_ready("qknorm_rope_bwd")) return -1;
    if (check_shape("qknorm_rope_bwd", heads, kv_heads, hd, S, batch)) return -1;
    if (variant != 0 && variant != 1) return mi355_fail("qknorm_rope_bwd: variant must be 0 or 1");
    if (!cos_dev || !sin_dev || (heads > 0 && (!dq || !dwq || !dq_out || !q || !wq)) ||
        (kv_heads > 0 && (!dk || !dwk || !dk_out || !k || !wk)))
        return mi355_fail("qknorm_rope_bwd: NULL pointer");
    QkCfg cfg;
    const bool vec_ok = (S % 4 == 0) && aligned16(cos_dev) && aligned16(sin_dev) &&
                        (heads == 0 || (aligned16(q) && aligned16(dq) && aligned16(dq_out))) &&
                        (kv_heads == 0 || (aligned16(k) && aligned16(dk) && aligned16(dk_out)));
    if (!vec_ok || !pick_qk(hd, cfg, true)) {
        // unfused composition: inverse rotation into dq/dk, then the per-head norm backward in place
        if (mi355_rope_dev(dq, dk, dq_out, dk_out, heads, kv_heads, hd, S, batch, cos_dev, sin_dev, -1)) return -1;
        if (heads > 0 && mi355_rmsnorm_bwd_dev(dq, dwq, dq, q, wq, hd, S, batch * heads, eps, variant)) return -1;
        if (kv_heads > 0 && mi355_rmsnorm_bwd_dev(dk, dwk, dk, k, wk, hd, S, batch * kv_heads, eps, variant)) return -1;
        return 0;
    }
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * 4);
    const int nq = batch * heads * strips, nk = batch * kv_heads * strips;
    float *part = mi355_dw_partials((size_t)(nq + nk) * hd, nq > 0 ? dwq : nullptr, nk > 0 ? dwk : nullptr);
    if (!part) return -1;
    QK_DISPATCH(qknorm_rope_bwd_kernel, cfg, dim3(nq + nk), dq, dk, part, dq_out, dk_out, q, k, wq, wk, hd, S, strips,
                nq, cos_dev, sin_dev, eps, 1.0f / (float)hd, variant);
    LAUNCH_OK("qknorm_rope_bwd");
    if (nq > 0 && mi355_dw_submit(dwq, part, nq, hd)) return -1;
    if (nk > 0 && mi355_dw_submit(dwk, part + (size_t)nq * hd, nk, hd)) return -1;
    return mi355_dw_op_end();
}
