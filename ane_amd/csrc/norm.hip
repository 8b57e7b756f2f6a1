// norm.hip — RMSNorm forward / backward on channel-first [batch][C][S] tensors.
//
// Reference ops: rmsnorm (training/stories_cpu_ops.h:6-21) and rmsnorm_bwd
// (training/stories_cpu_ops.h:23-53; twins in training/training_dynamic/cpu_ops.h:7-54).
//
// The reduction runs over the STRIDED axis c; columns s are contiguous.  A workgroup owns a
// strip of W = LPR*VEC columns of one slab.  LPR adjacent lanes cover the strip with one
// 128-bit load each, the remaining lane bits and the waves spread over rows, so every load
// instruction of a wave reads (64/LPR) full row segments.  Each thread keeps its rows in
// registers (one HBM pass), per-column partial sums are combined with cross-lane shuffles and a
// small LDS exchange between waves, then the strip is normalised from registers and stored.
// dw partials (one per workgroup and row) go to a workspace and are summed in a fixed order by
// a second kernel, so the result is deterministic and needs no floating-point atomics.
#include "common.h"
#include "tile.h"
#include "norm_cluster.h"

namespace {

// CAP > 0: rows are held in registers (C <= CAP * THREADS/LPR).  CAP == 0: rows are re-read
// in the second pass (they come back from L2).
template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void rms_fwd_kernel(float *__restrict__ y, const float *__restrict__ x,
                                                          const float *__restrict__ w, int C, int S, int strips,
                                                          int nblk, float eps, float invC) {
    constexpr int RPS = THREADS / LPR;
    constexpr int W = LPR * VEC;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * 1 * (LPR < 64 ? LPR : 64) * VEC];
    const int blk = xcd_remap(blockIdx.x, nblk);
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, row0 = threadIdx.x / LPR;
    const int col = strip * W + lc * VEC;
    const bool col_ok = col < S;
    const size_t base = (size_t)slab * C * S + col;
    const float *xs = x + base;
    float *ys = y + base;

    float acc[1][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = 0.f;

    if constexpr (CAP > 0) {
        float xv[CAP][VEC];
        float wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                ldv_nt<VEC>(xv[k], xs + (size_t)c * S);
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
                stv_nt<VEC>(ys + (size_t)c * S, o);
            }
        }
    } else {
        if (col_ok)
#pragma unroll 4
            for (int c = row0; c < C; c += RPS) {
                float t[VEC];
                ldv<VEC>(t, xs + (size_t)c * S);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc[0][j] += t[j] * t[j];
            }
        strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
        float rr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
        if (col_ok)
#pragma unroll 4
            for (int c = row0; c < C; c += RPS) {
                float t[VEC], o[VEC];
                ldv_nt<VEC>(t, xs + (size_t)c * S);
                const float wc = w[c];
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = (t[j] * rr[j]) * wc;
                stv_nt<VEC>(ys + (size_t)c * S, o);
            }
    }
}

// RES: the residual of the backward pass rides along (training/training_dynamic/train.m:586-595, :714-721):
// dx = rmsnorm_bwd(...) + res, and optionally dx2 = alpha2 * dx.  Its rows are loaded with x and dy, so the fused
// op has no extra latency phase; the adds are the ones the separate passes would do, in the same order.
template <int VEC, int LPR, int THREADS, int CAP, bool RES>
__device__ __forceinline__ void rms_bwd_body(float *dx, float *__restrict__ dw_part, const float *dy,
                                             const float *__restrict__ x, const float *__restrict__ w, int C, int S,
                                             int strips, int nblk, float eps, float invC, int variant,
                                             const float *res, float *dx2, float alpha2) {
    constexpr int RPS = THREADS / LPR;
    constexpr int W = LPR * VEC;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * 2 * (LPR < 64 ? LPR : 64) * VEC];
    const int blk = xcd_remap(blockIdx.x, nblk);
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, row0 = threadIdx.x / LPR;
    const int col = strip * W + lc * VEC;
    const bool col_ok = col < S;
    const size_t base = (size_t)slab * C * S + col;
    const float *xs = x + base, *dys = dy + base;
    float *dxs = dx + base;
    const float *ress = RES ? res + base : nullptr;
    float *dx2s = (RES && dx2) ? dx2 + base : nullptr;
    float *part = dw_part + (size_t)blk * C;

    float acc[2][VEC];   // [0] = sum x^2, [1] = sum (dy*x)*w
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = acc[1][j] = 0.f;

    auto finish = [&](float (&rr)[VEC], float (&dotn)[VEC]) {
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
            dotn[j] = acc[1][j] * ((rr[j] * rr[j]) * invC);
        }
    };
    auto row_out = [&](int c, const float (&xr)[VEC], const float (&dyr)[VEC], float wc, const float (&rr)[VEC],
                       const float (&dotn)[VEC], const float (&rs)[VEC]) {
        float o[VEC];
        float p = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            if (variant == 0) o[j] = ((dyr[j] - xr[j] * dotn[j]) * rr[j]) * wc;
            else o[j] = (dyr[j] * wc) * rr[j] - (xr[j] * dotn[j]) * rr[j];
            p += (dyr[j] * xr[j]) * rr[j];
            if constexpr (RES) o[j] = o[j] + rs[j];
        }
        if (col_ok) stv_nt<VEC>(dxs + (size_t)c * S, o);
        if constexpr (RES) {
            if (dx2s && col_ok) {
                float o2[VEC];
#pragma unroll
                for (int j = 0; j < VEC; j++) o2[j] = o[j] * alpha2;
                stv_nt<VEC>(dx2s + (size_t)c * S, o2);
            }
        }
        p = group_sum<(LPR < 64 ? LPR : 64)>(p);
        if (lc == 0) part[c] = p;
    };

    if constexpr (CAP > 0) {
        float xv[CAP][VEC], dv[CAP][VEC], wv[CAP], rv[RES ? CAP : 1][VEC];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                ldv_nt<VEC>(xv[k], xs + (size_t)c * S);
                ldv_nt<VEC>(dv[k], dys + (size_t)c * S);
                if constexpr (RES) ldv_nt<VEC>(rv[k], ress + (size_t)c * S);
                wv[k] = w[c];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) xv[k][j] = dv[k][j] = 0.f;
                if constexpr (RES) {
#pragma unroll
                    for (int j = 0; j < VEC; j++) rv[k][j] = 0.f;
                }
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
        finish(rr, dotn);
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C) row_out(c, xv[k], dv[k], wv[k], rr, dotn, rv[RES ? k : 0]);   // uniform per LPR lane group
        }
    } else {
        if (col_ok)
#pragma unroll 4
            for (int c = row0; c < C; c += RPS) {
                float a[VEC], b[VEC];
                ldv<VEC>(a, xs + (size_t)c * S);
                ldv<VEC>(b, dys + (size_t)c * S);
                const float wc = w[c];
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    acc[0][j] += a[j] * a[j];
                    acc[1][j] += (b[j] * a[j]) * wc;
                }
            }
        strip_reduce<VEC, LPR, THREADS, 2>(acc, lds);
        float rr[VEC], dotn[VEC];
        finish(rr, dotn);
#pragma unroll 4
        for (int c = row0; c < C; c += RPS) {
            float a[VEC], b[VEC], r[VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j] = 0.f;
            if (col_ok) {
                ldv_nt<VEC>(a, xs + (size_t)c * S);
                ldv_nt<VEC>(b, dys + (size_t)c * S);
                if constexpr (RES) ldv_nt<VEC>(r, ress + (size_t)c * S);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) a[j] = b[j] = 0.f;
            }
            row_out(c, a, b, w[c], rr, dotn, r);
        }
    }
}

template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void rms_bwd_kernel(float *dx, float *__restrict__ dw_part,
                                                          const float *dy, const float *__restrict__ x,
                                                          const float *__restrict__ w, int C, int S, int strips,
                                                          int nblk, float eps, float invC, int variant) {
    rms_bwd_body<VEC, LPR, THREADS, CAP, false>(dx, dw_part, dy, x, w, C, S, strips, nblk, eps, invC, variant, nullptr,
                                                nullptr, 0.f);
}

template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void rms_bwd_res_kernel(float *dx, float *__restrict__ dw_part,
                                                              const float *dy, const float *__restrict__ x,
                                                              const float *__restrict__ w, int C, int S, int strips,
                                                              int nblk, float eps, float invC, int variant,
                                                              const float *res, float *dx2, float alpha2) {
    rms_bwd_body<VEC, LPR, THREADS, CAP, true>(dx, dw_part, dy, x, w, C, S, strips, nblk, eps, invC, variant, res, dx2,
                                               alpha2);
}


// y = a + alpha*b ; yn = (y * rsqrt(mean_c y^2 + eps)) * w — the residual add and the RMSNorm that
// follows it (training/training_dynamic/train.m:460-461) in one launch.
template <int VEC, int LPR, int THREADS, int CAP>
__global__ __launch_bounds__(THREADS) void res_rms_fwd_kernel(float *y, float *__restrict__ yn, const float *a,
                                                              const float *b, float alpha,
                                                              const float *__restrict__ w, int C, int S, int strips,
                                                              int nblk, float eps, float invC) {
    constexpr int RPS = THREADS / LPR;
    constexpr int W = LPR * VEC;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * 1 * (LPR < 64 ? LPR : 64) * VEC];
    const int blk = xcd_remap(blockIdx.x, nblk);
    const int slab = blk / strips, strip = blk - slab * strips;
    const int lc = threadIdx.x % LPR, row0 = threadIdx.x / LPR;
    const int col = strip * W + lc * VEC;
    const bool col_ok = col < S;
    const size_t base = (size_t)slab * C * S + col;
    float acc[1][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = 0.f;
    if constexpr (CAP > 0) {
        // y stays in registers between the two stores
        float yv[CAP][VEC], wv[CAP];
#pragma unroll
        for (int k = 0; k < CAP; k++) {
            const int c = row0 + k * RPS;
            if (c < C && col_ok) {
                float bv[VEC];
                ldv_nt<VEC>(yv[k], a + base + (size_t)c * S);
                ldv_nt<VEC>(bv, b + base + (size_t)c * S);
#pragma unroll
                for (int j = 0; j < VEC; j++) yv[k][j] = bv[j] * alpha + yv[k][j];
                wv[k] = w[c];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) yv[k][j] = 0.f;
                wv[k] = 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < CAP; k++) {
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[0][j] += yv[k][j] * yv[k][j];
        }
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
                for (int j = 0; j < VEC; j++) o[j] = (yv[k][j] * rr[j]) * wv[k];
                stv_nt<VEC>(y + base + (size_t)c * S, yv[k]);
                stv_nt<VEC>(yn + base + (size_t)c * S, o);
            }
        }
    } else {
        // y is stored in the first sweep and read back by the same lane in the second
        if (col_ok)
#pragma unroll 4
            for (int c = row0; c < C; c += RPS) {
                float av[VEC], bv[VEC], t[VEC];
                ldv_nt<VEC>(av, a + base + (size_t)c * S);
                ldv_nt<VEC>(bv, b + base + (size_t)c * S);
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    t[j] = bv[j] * alpha + av[j];
                    acc[0][j] += t[j] * t[j];
                }
                stv<VEC>(y + base + (size_t)c * S, t);
            }
        strip_reduce<VEC, LPR, THREADS, 1>(acc, lds);
        float rr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(acc[0][j] * invC + eps);
        if (col_ok)
#pragma unroll 4
            for (int c = row0; c < C; c += RPS) {
                float t[VEC], o[VEC];
                ldv<VEC>(t, y + base + (size_t)c * S);
                const float wc = w[c];
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = (t[j] * rr[j]) * wc;
                stv_nt<VEC>(yn + base + (size_t)c * S, o);
            }
    }
}

struct NormCfg {
    int vec, lpr, threads, cap;
};

// The tiles that are instantiated (NORM_DISPATCH below has one case per entry): vec*1000000 + lpr*10000 + (threads/256)*100 + cap.
constexpr int NORM_KEYS[] = {1640100, 4160100, 4160108, 4160116, 4160200, 4160208, 4160216, 4160400, 4160408,
                             4080100, 4080108, 4080116, 4080200, 4080208, 4080216, 4080400, 4080408,
                             4040100, 4040108, 4040116, 4040200, 4040208, 4040216, 4040400, 4040408};
int norm_key(const NormCfg &c) { return c.vec * 1000000 + c.lpr * 10000 + (c.threads / 256) * 100 + c.cap; }
bool norm_tile_exists(const NormCfg &c) {
    for (int k : NORM_KEYS)
        if (k == norm_key(c)) return true;
    return false;
}

// Picks the tile: registers when the rows fit, and the narrowest strip needed to give every
// compute unit at least two workgroups.
NormCfg pick_cfg(int C, int S, int batch, bool vec_ok, int max_cap, int max_cap_1024, int lpr_knob, int thr_knob,
                 bool backward) {
    NormCfg best{};
    if (!vec_ok) return NormCfg{1, 64, 256, 0};
    if (!lpr_knob && !thr_knob && C >= 512) {
        // Tall tensors, measured on MI355X at C=1024 and 16x256 columns with operands cold in HBM: forward, 64-byte strips in registers of a 16-wave workgroup
        // 9.6 us; backward, the single-pass register tile with 8 waves 13.9 us, with 4 waves 16.3 us, a two-sweep
        // 16-wave variant 19.9 us.
        // With enough columns to put a 128-byte strip on every compute unit the wider strip wins (half as many
        // requests per byte): at 32 x 256 columns 12.8 / 26.4 us forward / backward against 18.8 / 31.3 us.
        const long strips8 = (long)ceil_div((size_t)S, 32) * batch;
        const int cus = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
        if (strips8 >= cus && C <= 1024) return backward ? NormCfg{4, 8, 512, 16} : NormCfg{4, 8, 1024, 8};
        if (!backward) return NormCfg{4, 4, 1024, C <= 2048 ? 8 : 0};
        if (C <= 1024) return NormCfg{4, 4, 512, 8};
        return NormCfg{4, strips8 >= 128 ? 8 : 4, 1024, 0};
    }
    const int lprs[3] = {16, 8, 4};
    const int thrs[3] = {256, 512, 1024};
    const int caps[2] = {8, 16};
    long best_score = -1;
    for (int lpr : lprs) {
        if (lpr_knob && lpr != lpr_knob) continue;
        for (int thr : thrs) {
            if (thr_knob && thr != thr_knob) continue;
            const int rps = thr / lpr;
            int cap = 0;
            for (int cp : caps)
                if (cp <= max_cap && (long)cp * rps >= C) { cap = cp; break; }
            if (thr == 1024 && cap > max_cap_1024) cap = 0;   // 16 waves per CU leave 128 VGPRs per lane
            if (!norm_tile_exists(NormCfg{4, lpr, thr, cap})) continue;
            const long strips = ceil_div((size_t)S, (size_t)lpr * 4);
            const long nblk = strips * batch;
            long score = (cap > 0 ? 1000000 : 0);
            const long want = 2L * (g_ctx.num_cu > 0 ? g_ctx.num_cu : 256);
            score += (nblk >= want ? want : nblk) * 100 / want * 1000;   // occupancy first
            score += lpr;                                                // then the widest strip
            score += (thr == 256 ? 1 : 0);
            if (score > best_score) { best_score = score; best = NormCfg{4, lpr, thr, cap}; }
        }
    }
    if (best_score < 0) best = NormCfg{4, 16, 256, 0};
    return best;
}

template <int VEC, int LPR, int THREADS, int CAP>
void launch_fwd(float *y, const float *x, const float *w, int C, int S, int batch, float eps) {
    const int strips = (int)ceil_div((size_t)S, (size_t)LPR * VEC);
    const int nblk = strips * batch;
    hipLaunchKernelGGL((rms_fwd_kernel<VEC, LPR, THREADS, CAP>), dim3(nblk), dim3(THREADS), 0, g_ctx.stream, y, x, w,
                       C, S, strips, nblk, eps, 1.0f / (float)C);
}

template <int VEC, int LPR, int THREADS, int CAP>
void launch_bwd(float *dx, float *part, const float *dy, const float *x, const float *w, int C, int S, int batch,
                float eps, int variant) {
    const int strips = (int)ceil_div((size_t)S, (size_t)LPR * VEC);
    const int nblk = strips * batch;
    hipLaunchKernelGGL((rms_bwd_kernel<VEC, LPR, THREADS, CAP>), dim3(nblk), dim3(THREADS), 0, g_ctx.stream, dx, part,
                       dy, x, w, C, S, strips, nblk, eps, 1.0f / (float)C, variant);
}

template <int VEC, int LPR, int THREADS, int CAP>
void launch_bwd_res(float *dx, float *part, const float *dy, const float *x, const float *w, int C, int S, int batch,
                    float eps, int variant, const float *res, float *dx2, float alpha2) {
    const int strips = (int)ceil_div((size_t)S, (size_t)LPR * VEC);
    const int nblk = strips * batch;
    hipLaunchKernelGGL((rms_bwd_res_kernel<VEC, LPR, THREADS, CAP>), dim3(nblk), dim3(THREADS), 0, g_ctx.stream, dx, part,
                       dy, x, w, C, S, strips, nblk, eps, 1.0f / (float)C, variant, res, dx2, alpha2);
}

// The tile each entry point uses: op 0 = forward, 1 = backward, 2 = backward with the residual.
NormCfg plan_tile(int op, int C, int S, int batch, bool vec_ok) {
    if (op == 0) return pick_cfg(C, S, batch, vec_ok, 16, 8, g_ctx.rms_lpr, g_ctx.rms_threads, false);
    if (op == 1) return pick_cfg(C, S, batch, vec_ok, 16, 0, g_ctx.rms_lpr, g_ctx.rms_threads, true);
    NormCfg cfg = pick_cfg(C, S, batch, vec_ok, 8, 0, g_ctx.rms_lpr, g_ctx.rms_threads, true);
    // three operands of 16 rows per lane do not fit the registers: the 8-row tile, or the two-sweep variant
    if (cfg.cap > 8) cfg = C <= 1024 ? NormCfg{4, 4, 512, 8} : NormCfg{cfg.vec, cfg.lpr, cfg.threads, 0};
    return cfg;
}

#define NORM_DISPATCH(FN, cfg, ...)                                                                   \
    do {                                                                                              \
        const int key = norm_key(cfg);                                                                \
        switch (key) {                                                                                \
            case 1640100: FN<1, 64, 256, 0>(__VA_ARGS__); break;                                      \
            case 4160100: FN<4, 16, 256, 0>(__VA_ARGS__); break;                                      \
            case 4160108: FN<4, 16, 256, 8>(__VA_ARGS__); break;                                      \
            case 4160116: FN<4, 16, 256, 16>(__VA_ARGS__); break;                                     \
            case 4160200: FN<4, 16, 512, 0>(__VA_ARGS__); break;                                      \
            case 4160208: FN<4, 16, 512, 8>(__VA_ARGS__); break;                                      \
            case 4160216: FN<4, 16, 512, 16>(__VA_ARGS__); break;                                     \
            case 4160400: FN<4, 16, 1024, 0>(__VA_ARGS__); break;                                     \
            case 4160408: FN<4, 16, 1024, 8>(__VA_ARGS__); break;                                     \
            case 4040208: FN<4, 4, 512, 8>(__VA_ARGS__); break;                                       \
            case 4040216: FN<4, 4, 512, 16>(__VA_ARGS__); break;                                      \
            case 4080208: FN<4, 8, 512, 8>(__VA_ARGS__); break;                                       \
            case 4080216: FN<4, 8, 512, 16>(__VA_ARGS__); break;                                      \
            case 4040200: FN<4, 4, 512, 0>(__VA_ARGS__); break;                                       \
            case 4080200: FN<4, 8, 512, 0>(__VA_ARGS__); break;                                       \
            case 4080100: FN<4, 8, 256, 0>(__VA_ARGS__); break;                                       \
            case 4080108: FN<4, 8, 256, 8>(__VA_ARGS__); break;                                       \
            case 4080116: FN<4, 8, 256, 16>(__VA_ARGS__); break;                                      \
            case 4080400: FN<4, 8, 1024, 0>(__VA_ARGS__); break;                                      \
            case 4080408: FN<4, 8, 1024, 8>(__VA_ARGS__); break;                                      \
            case 4040100: FN<4, 4, 256, 0>(__VA_ARGS__); break;                                       \
            case 4040108: FN<4, 4, 256, 8>(__VA_ARGS__); break;                                       \
            case 4040116: FN<4, 4, 256, 16>(__VA_ARGS__); break;                                      \
            case 4040400: FN<4, 4, 1024, 0>(__VA_ARGS__); break;                                      \
            case 4040408: FN<4, 4, 1024, 8>(__VA_ARGS__); break;                                      \
            default: return mi355_fail("rmsnorm: no kernel for tile key %d", key);                    \
        }                                                                                             \
    } while (0)

int cluster_spin_ticks(void) { return mi355_exchange_spin_ticks(); }
ClusterWs g_cluster_ws = {nullptr, nullptr, nullptr};
bool cluster_ws_ready(void) { return mi355_exchange(&g_cluster_ws); }

// The single-workgroup tiles are chosen by hand (knobs) or the shape does not cluster: csplit == 0.
ClusterPlan plan_cluster(int C, int S, int batch, bool vec_ok, int max_rpt, int rounds = 1) {
    if (g_ctx.rms_lpr || g_ctx.rms_threads) return NO_CLUSTER;
    return cluster_plan(C, S, batch, vec_ok, StoreF32::VEC, 4, max_rpt, rounds);
}

template <int RPT, bool FUSE, bool EXACT>
void launch_fwd_cluster_as(const ClusterPlan &cp, float *yn, float *y_res, const float *a, const float *b, float alpha,
                           const float *w, int C, int S, float eps) {
    hipLaunchKernelGGL((rms_fwd_cluster_kernel<StoreF32, RPT, 1024, FUSE, EXACT>), dim3(cp.nblk), dim3(1024), 0, g_ctx.stream, yn,
                       y_res, a, b, alpha, w, C, S, cp.strips, cp.nblk, cp.csplit, cp.rows_pm, eps, 1.0f / (float)C,
                       g_cluster_ws, cluster_spin_ticks());
}

template <bool FUSE>
void launch_fwd_cluster(const ClusterPlan &cp, float *yn, float *y_res, const float *a, const float *b, float alpha,
                        const float *w, int C, int S, float eps) {
    if (cp.rpt == 4 && cp.exact) launch_fwd_cluster_as<4, FUSE, true>(cp, yn, y_res, a, b, alpha, w, C, S, eps);
    else if (cp.rpt == 4) launch_fwd_cluster_as<4, FUSE, false>(cp, yn, y_res, a, b, alpha, w, C, S, eps);
    else if (cp.exact) launch_fwd_cluster_as<8, FUSE, true>(cp, yn, y_res, a, b, alpha, w, C, S, eps);
    else launch_fwd_cluster_as<8, FUSE, false>(cp, yn, y_res, a, b, alpha, w, C, S, eps);
}

// The backward tiles hold two (with the residual three) operands per row: four rows per lane fill the registers.
template <bool RES, bool EXACT>
void launch_bwd_cluster_as(const ClusterPlan &cp, float *dx, float *part, const float *dy, const float *x, const float *w,
                           int C, int S, float eps, int variant, const float *res, float *dx2, float alpha2) {
    hipLaunchKernelGGL((rms_bwd_cluster_kernel<StoreF32, 4, 1024, RES, EXACT>), dim3(cp.nblk), dim3(1024), 0, g_ctx.stream, dx, part,
                       dy, x, w, C, S, cp.strips, cp.nblk, cp.csplit, cp.rows_pm, eps, 1.0f / (float)C, variant, res, dx2,
                       alpha2, g_cluster_ws, cluster_spin_ticks());
}

template <bool RES>
void launch_bwd_cluster(const ClusterPlan &cp, float *dx, float *part, const float *dy, const float *x, const float *w,
                        int C, int S, float eps, int variant, const float *res, float *dx2, float alpha2) {
    // (with the residual's rows the unmasked variant would need more than the 128 registers a lane has)
    if constexpr (!RES) {
        if (cp.exact) { launch_bwd_cluster_as<false, true>(cp, dx, part, dy, x, w, C, S, eps, variant, res, dx2, alpha2); return; }
    }
    launch_bwd_cluster_as<RES, false>(cp, dx, part, dy, x, w, C, S, eps, variant, res, dx2, alpha2);
}

}   // namespace

// Host-only: which tile an entry point would run for a shape, and whether that tile exists.
MI355_API int mi355_rmsnorm_tile(int op, int C, int S, int batch, int aligned, int *tile5) {
    if (op < 0 || op > 2 || C <= 0 || S <= 0 || batch <= 0) return mi355_fail("rmsnorm_tile: bad arguments");
    const bool vec_ok = aligned && S % 4 == 0;
    // the single-workgroup tile is also what an in-place call of a clustered shape runs: it has to exist either way
    const NormCfg cfg = plan_tile(op, C, S, batch, vec_ok);
    if (!norm_tile_exists(cfg)) return mi355_fail("rmsnorm: no kernel for tile key %d", norm_key(cfg));
    const ClusterPlan cp = plan_cluster(C, S, batch, vec_ok, op == 0 ? 8 : 4, op == 2 ? 2 : 1);
    if (tile5) {
        if (cp.csplit) { tile5[0] = 4; tile5[1] = CL_LPR; tile5[2] = cp.threads; tile5[3] = cp.rpt; tile5[4] = cp.csplit; }
        else { tile5[0] = cfg.vec; tile5[1] = cfg.lpr; tile5[2] = cfg.threads; tile5[3] = cfg.cap; tile5[4] = 0; }
    }
    if (cp.csplit && (cp.nblk > CL_MAX_BLOCKS || cp.rows_pm > (cp.threads / CL_LPR) * cp.rpt || (cp.rpt != 4 && cp.rpt != 8) ||
                      (op != 0 && cp.rpt != 4)))
        return mi355_fail("rmsnorm: inconsistent cluster plan for C=%d S=%d batch=%d", C, S, batch);
    return 0;
}

MI355_API int mi355_rmsnorm_fwd_dev(float *y, const float *x, const float *w, int C, int S, int batch, float eps) {
    if (!mi355_ready("rmsnorm_fwd")) return -1;
    if (!y || !x || !w) return mi355_fail("rmsnorm_fwd: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0) return mi355_fail("rmsnorm_fwd: bad shape C=%d S=%d batch=%d", C, S, batch);
    const bool vec_ok = (S % 4 == 0) && aligned16(x) && aligned16(y);
    // in place the single-workgroup tile is used, for the reason given in mi355_rmsnorm_bwd_dev
    const ClusterPlan cp = y == x ? NO_CLUSTER : plan_cluster(C, S, batch, vec_ok, 8);
    if (cp.csplit) {
        if (!cluster_ws_ready()) return -1;
        launch_fwd_cluster<false>(cp, y, nullptr, x, nullptr, 0.f, w, C, S, eps);
        LAUNCH_OK("rmsnorm_fwd");
        return 0;
    }
    NormCfg cfg = plan_tile(0, C, S, batch, vec_ok);
    NORM_DISPATCH(launch_fwd, cfg, y, x, w, C, S, batch, eps);
    LAUNCH_OK("rmsnorm_fwd");
    return 0;
}

MI355_API int mi355_rmsnorm_bwd_dev(float *dx, float *dw, const float *dy, const float *x, const float *w, int C,
                                    int S, int batch, float eps, int variant) {
    if (!mi355_ready("rmsnorm_bwd")) return -1;
    if (!dx || !dw || !dy || !x || !w) return mi355_fail("rmsnorm_bwd: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0) return mi355_fail("rmsnorm_bwd: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (variant != 0 && variant != 1) return mi355_fail("rmsnorm_bwd: variant must be 0 or 1");
    if (dx == x) return mi355_fail("rmsnorm_bwd: dx must not alias x (dx may alias dy)");
    const bool vec_ok = (S % 4 == 0) && aligned16(x) && aligned16(dy) && aligned16(dx);
    // in place on dy the single-workgroup tile is used: a cluster member that has to recompute another member's
    // sums (its bounded wait expired) would read rows that their owner has already overwritten
    const ClusterPlan cp = dx == dy ? NO_CLUSTER : plan_cluster(C, S, batch, vec_ok, 4);
    if (cp.csplit) {
        if (!cluster_ws_ready()) return -1;
        const int nrows = cp.nblk / cp.csplit;
        float *part = mi355_dw_partials((size_t)nrows * C, dw, nullptr);
        if (!part) return -1;
        launch_bwd_cluster<false>(cp, dx, part, dy, x, w, C, S, eps, variant, nullptr, nullptr, 0.f);
        LAUNCH_OK("rmsnorm_bwd");
        if (mi355_dw_submit(dw, part, nrows, C)) return -1;
        return mi355_dw_op_end();
    }
    NormCfg cfg = plan_tile(1, C, S, batch, vec_ok);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    float *part = mi355_dw_partials((size_t)nblk * C, dw, nullptr);
    if (!part) return -1;
    NORM_DISPATCH(launch_bwd, cfg, dx, part, dy, x, w, C, S, batch, eps, variant);
    LAUNCH_OK("rmsnorm_bwd");
    if (mi355_dw_submit(dw, part, nblk, C)) return -1;
    return mi355_dw_op_end();
}

MI355_API int mi355_rmsnorm_bwd_residual_dev(float *dx, float *dx_scaled, float *dw, const float *dy, const float *x,
                                             const float *w, const float *res, float alpha, int C, int S, int batch,
                                             float eps, int variant) {
    if (!mi355_ready("rmsnorm_bwd_residual")) return -1;
    if (!dx || !dw || !dy || !x || !w || !res) return mi355_fail("rmsnorm_bwd_residual: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("rmsnorm_bwd_residual: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (variant != 0 && variant != 1) return mi355_fail("rmsnorm_bwd_residual: variant must be 0 or 1");
    if (dx_scaled && (dx_scaled == dx || dx_scaled == dy || dx_scaled == x || dx_scaled == res))
        return mi355_fail("rmsnorm_bwd_residual: dx_scaled must not alias another operand");
    if (dx == x) return mi355_fail("rmsnorm_bwd_residual: dx must not alias x (dx may alias res or dy)");
    const bool vec_ok = (S % 4 == 0) && aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(res) &&
                        (!dx_scaled || aligned16(dx_scaled));
    const ClusterPlan cp = dx == dy ? NO_CLUSTER : plan_cluster(C, S, batch, vec_ok, 4, 2);
    if (cp.csplit) {
        if (!cluster_ws_ready()) return -1;
        const int nrows = cp.nblk / cp.csplit;
        float *part = mi355_dw_partials((size_t)nrows * C, dw, nullptr);
        if (!part) return -1;
        launch_bwd_cluster<true>(cp, dx, part, dy, x, w, C, S, eps, variant, res, dx_scaled, alpha);
        LAUNCH_OK("rmsnorm_bwd_residual");
        if (mi355_dw_submit(dw, part, nrows, C)) return -1;
        return mi355_dw_op_end();
    }
    NormCfg cfg = plan_tile(2, C, S, batch, vec_ok);
    const int strips = (int)ceil_div((size_t)S, (size_t)cfg.lpr * cfg.vec);
    const int nblk = strips * batch;
    float *part = mi355_dw_partials((size_t)nblk * C, dw, nullptr);
    if (!part) return -1;
    NORM_DISPATCH(launch_bwd_res, cfg, dx, part, dy, x, w, C, S, batch, eps, variant, res, dx_scaled, alpha);
    LAUNCH_OK("rmsnorm_bwd_residual");
    if (mi355_dw_submit(dw, part, nblk, C)) return -1;
    return mi355_dw_op_end();
}

MI355_API int mi355_residual_rmsnorm_fwd_dev(float *y, float *yn, const float *a, const float *b, float alpha,
                                             const float *w, int C, int S, int batch, float eps) {
    if (!mi355_ready("residual_rmsnorm_fwd")) return -1;
    if (!y || !yn || !a || !b || !w) return mi355_fail("residual_rmsnorm_fwd: NULL pointer");
    if (C <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("residual_rmsnorm_fwd: bad shape C=%d S=%d batch=%d", C, S, batch);
    if (yn == y || yn == a || yn == b) return mi355_fail("residual_rmsnorm_fwd: yn must not alias y, a or b");
    const bool vec_ok = (S % 4 == 0) && aligned16(y) && aligned16(yn) && aligned16(a) && aligned16(b);
    const float invC = 1.0f / (float)C;
    // in place (y over a or b) the single-workgroup tile is used, for the reason given in mi355_rmsnorm_bwd_dev
    const ClusterPlan cp = (y == a || y == b) ? NO_CLUSTER : plan_cluster(C, S, batch, vec_ok, 8);
    if (cp.csplit) {
        if (!cluster_ws_ready()) return -1;
        launch_fwd_cluster<true>(cp, yn, y, a, b, alpha, w, C, S, eps);
        LAUNCH_OK("residual_rmsnorm_fwd");
        return 0;
    }
#define RES_RMS(VEC, LPR, THR, CAP)                                                                              \
    do {                                                                                                         \
        const int strips = (int)ceil_div((size_t)S, (size_t)(LPR) * (VEC));                                      \
        hipLaunchKernelGGL((res_rms_fwd_kernel<VEC, LPR, THR, CAP>), dim3(strips * batch), dim3(THR), 0,         \
                           g_ctx.stream, y, yn, a, b, alpha, w, C, S, strips, strips * batch, eps, invC);        \
    } while (0)
    const long strips8 = (long)ceil_div((size_t)S, 32) * batch;
    if (!vec_ok) RES_RMS(1, 64, 256, 0);
    else if (C > 512 && C <= 1024 && strips8 >= (g_ctx.num_cu > 0 ? g_ctx.num_cu : 256) && !g_ctx.rms_threads)
        RES_RMS(4, 8, 1024, 8);
    else if (C <= 128) RES_RMS(4, 16, 256, 8);
    else if (C <= 512 && g_ctx.rms_threads != 1024) RES_RMS(4, 4, 256, 8);
    else if (C <= 2048 && g_ctx.rms_threads != 256) RES_RMS(4, 4, 1024, 8);
    else if (C <= 1024) RES_RMS(4, 4, 256, 16);
    else RES_RMS(4, 8, 1024, 0);
#undef RES_RMS
    LAUNCH_OK("residual_rmsnorm_fwd");
    return 0;
}
