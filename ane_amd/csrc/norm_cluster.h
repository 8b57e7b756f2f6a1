// norm_cluster.h — RMSNorm forward / backward with the channel axis split over a cluster of workgroups.
//
// The register-tile kernels of norm.hip give one workgroup all C rows of a strip of columns, so a tensor of
// [16][1024][256] has work for 256 workgroups only if a strip is 16 columns: 64-byte pieces of 1 KiB rows, the
// access shape that this memory system serves worst.  Here a strip is 64 columns (256-byte pieces) and its C rows
// are shared by `csplit` workgroups (the members of a cluster).  Each member reduces its own rows to per-column
// partial sums, publishes them, reads the other members' partials, and normalises its rows from registers:
// still one pass over HBM, with 4 x the bytes per request and a workgroup on every compute unit.
//
// Exchange without fences.  A release/acquire pair at agent scope writes back and invalidates a whole L2 on
// this part; instead every partial travels as ONE 8-byte relaxed agent-scope atomic {value, tag} (such a store
// is written through to memory, such a load is served from there), and the tag says which launch wrote it:
//   * workgroup number b owns the slots [b][*] and a launch counter cnt[b], which it alone increments, once, at
//     its end.  Its partials of this launch carry the tag cnt[b] + 1.
//   * a consumer reads cnt[p] of every member p of its cluster when it starts (values of the previous launches:
//     kernel boundaries make them visible), and accepts a slot of p only when its tag is cnt[p] + 1.  A slot
//     written by an earlier launch, of this or any other shape or kernel, has a smaller tag.
//   * nothing is cleared between launches and nothing depends on the host, so a recorded graph can be replayed.
// The wait is bounded: after `spin_ticks` of the 100 MHz clock without the tag (members not resident together, a
// device shared with other work) the workgroup computes the other members' partials itself, with the same code in
// the same order, hence the same bits, and every kernel exits.  A member that publishes late, or whose counter
// was read after it finished, only ever makes a consumer fall back; it cannot make it accept a wrong value.
// The sums are combined in member order by every member, so all members of a cluster normalise with identical
// column sums and the result is run-to-run deterministic.
//
// Reference ops: rmsnorm and rmsnorm_bwd, training/stories_cpu_ops.h:6-53.
#pragma once
#include "common.h"
#include "tile.h"

namespace {

constexpr int CL_LPR = 16;                 // lanes per row piece: 16 x 16 B = 256 B
constexpr int CL_W = CL_LPR * 4;           // columns per strip
constexpr int CL_SLOT_STRIDE = XCH_SLOT_STRIDE;   // 8-byte slots per workgroup: two quantities per column
constexpr int CL_MAX_BLOCKS = XCH_MAX_BLOCKS;     // workgroups per launch that the slot area covers
constexpr int CL_MAX_SPLIT = 8;
static_assert(CL_SLOT_STRIDE >= 2 * CL_W, "two quantities per column must fit a workgroup's slots");
typedef Mi355Exchange ClusterWs;

// Per-thread partial sums acc[q][j] (q < NV quantities, j < 4 columns of this lane) -> per-column sums of the
// workgroup in wsum[q*CL_W + column], valid for all threads after the barrier.  lds: NW*NV*CL_W floats.
template <int THREADS, int NV>
__device__ __forceinline__ void member_sums(float (&acc)[NV][4], float *lds, float *wsum) {
    constexpr int NW = THREADS / 64;
#pragma unroll
    for (int q = 0; q < NV; q++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[q][j] = wave_sum_stride<CL_LPR>(acc[q][j]);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < CL_LPR) {
#pragma unroll
        for (int q = 0; q < NV; q++)
#pragma unroll
            for (int j = 0; j < 4; j++) lds[(wave * NV + q) * CL_W + lane * 4 + j] = acc[q][j];
    }
    __syncthreads();
    if (threadIdx.x < NV * CL_W) {
        const int q = threadIdx.x / CL_W, c = threadIdx.x % CL_W;
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < NW; wv++) s += lds[(wv * NV + q) * CL_W + c];
        wsum[threadIdx.x] = s;
    }
    __syncthreads();
}

// Publishes wsum (this member's column sums) and gathers every member's into tot[(m*NV+q)*CL_W + column].
// Returns false when the bounded wait expired for any slot (block-uniform).
template <int THREADS, int NV>
__device__ __forceinline__ bool cluster_exchange(const float *wsum, float *tot, int *failed, int blk, int cluster,
                                                 int csplit, const ClusterWs &ws, unsigned my_tag,
                                                 const unsigned (&want_tag)[(CL_MAX_SPLIT * NV * CL_W + THREADS - 1) / THREADS],
                                                 int spin_ticks) {
    constexpr int NF = (CL_MAX_SPLIT * NV * CL_W + THREADS - 1) / THREADS;
    if (threadIdx.x < NV * CL_W) {
        const unsigned long long pk = ((unsigned long long)my_tag << 32) | __float_as_uint(wsum[threadIdx.x]);
        __hip_atomic_store(&ws.slots[(size_t)blk * CL_SLOT_STRIDE + threadIdx.x], pk, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    const int nslots = csplit * NV * CL_W;
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int i = threadIdx.x + f * THREADS;
        if (i < nslots) {
            const int m = i / (NV * CL_W), c = i - m * (NV * CL_W);
            const unsigned long long *sp = &ws.slots[(size_t)(cluster * csplit + m) * CL_SLOT_STRIDE + c];
            const long long t0 = wall_clock64();
            unsigned long long pk;
            bool ok = false;
            for (;;) {
                pk = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((unsigned)(pk >> 32) == want_tag[f]) { ok = true; break; }
                if (wall_clock64() - t0 >= (long long)spin_ticks) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (!ok) *failed = 1;
            tot[i] = __uint_as_float((unsigned)pk);
        }
    }
    __syncthreads();
    return *failed == 0;
}

// Geometry shared by the kernels: workgroup number -> (slab, strip, member), rows of a member.
struct ClusterGeo {
    int blk, cluster, member, slab, strip;
};
__device__ __forceinline__ ClusterGeo cluster_geo(int nblk, int csplit, int strips) {
    ClusterGeo g;
    g.blk = xcd_remap(blockIdx.x, nblk);      // the members of a cluster are neighbours on one XCD
    g.cluster = g.blk / csplit;
    g.member = g.blk - g.cluster * csplit;
    g.slab = g.cluster / strips;
    g.strip = g.cluster - g.slab * strips;
    return g;
}

// FUSE: y = a + alpha*b is formed first (and stored), and the norm is taken of it — the residual add and the
// RMSNorm that follows it (training/training_dynamic/train.m:460-461).  Otherwise x = a and b, y_res are unused.
// EXACT: every member holds exactly RPS*RPT rows and every strip 64 columns.  Then no row or column needs a mask and
// the loads of the tile are issued back to back without branches, which is worth 0.45 us of the 8 us that the
// forward kernel takes on [16][1024][256]; other shapes take the masked loads.
template <int RPT, int THREADS, bool FUSE, bool EXACT>
__global__ __launch_bounds__(THREADS) void rms_fwd_cluster_kernel(float *__restrict__ yn, float *y_res, const float *a,
                                                                  const float *b, float alpha,
                                                                  const float *__restrict__ w, int C, int S,
                                                                  int strips, int nblk, int csplit, int rows_pm,
                                                                  float eps, float invC, ClusterWs ws,
                                                                  int spin_ticks) {
    constexpr int RPS = THREADS / CL_LPR;
    constexpr int NW = THREADS / 64;
    constexpr int NF = (CL_MAX_SPLIT * CL_W + THREADS - 1) / THREADS;
    __shared__ float lds[NW * CL_W];
    __shared__ float wsum[CL_W];
    __shared__ float tot[CL_MAX_SPLIT * CL_W];
    __shared__ int failed;
    const ClusterGeo g = cluster_geo(nblk, csplit, strips);
    const int lc = threadIdx.x % CL_LPR, row0 = threadIdx.x / CL_LPR;
    const int col = g.strip * CL_W + lc * 4;
    const bool col_ok = col < S;
    const size_t slab_base = (size_t)g.slab * C * S + col;
    if (threadIdx.x == 0) failed = 0;
    unsigned my_tag = 0, want_tag[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int i = threadIdx.x + f * THREADS;
        want_tag[f] = i < csplit * CL_W ? ws.cnt[g.cluster * csplit + i / CL_W] + 1u : 0u;
    }
    if (threadIdx.x < CL_W) my_tag = ws.cnt[g.blk] + 1u;

    // rows of member m held by this thread: c = m*rows_pm + row0 + k*RPS, valid while below (m+1)*rows_pm and C
    auto row_of = [&](int m, int k) { return m * rows_pm + row0 + k * RPS; };
    auto row_ok = [&](int m, int k) { return row0 + k * RPS < rows_pm && row_of(m, k) < C && col_ok; };
    auto load_row = [&](float (&v)[4], int c, bool streaming) {
        if constexpr (FUSE) {
            float av[4], bv[4];
            if (streaming) { ldv_nt<4>(av, a + slab_base + (size_t)c * S); ldv_nt<4>(bv, b + slab_base + (size_t)c * S); }
            else { ldv<4>(av, a + slab_base + (size_t)c * S); ldv<4>(bv, b + slab_base + (size_t)c * S); }
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = bv[j] * alpha + av[j];
        } else {
            if (streaming) ldv_nt<4>(v, a + slab_base + (size_t)c * S);
            else ldv<4>(v, a + slab_base + (size_t)c * S);
        }
    };

    float xv[RPT][4], wv[RPT];
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (EXACT || row_ok(g.member, k)) {
            load_row(xv[k], row_of(g.member, k), true);
            wv[k] = w[row_of(g.member, k)];
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) xv[k][j] = 0.f;
            wv[k] = 0.f;
        }
    }
    float acc[1][4] = {{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int k = 0; k < RPT; k++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[0][j] += xv[k][j] * xv[k][j];
    member_sums<THREADS, 1>(acc, lds, wsum);
    float ss[4] = {0.f, 0.f, 0.f, 0.f};
    if (cluster_exchange<THREADS, 1>(wsum, tot, &failed, g.blk, g.cluster, csplit, ws, my_tag, want_tag, spin_ticks)) {
        for (int m = 0; m < csplit; m++)
#pragma unroll
            for (int j = 0; j < 4; j++) ss[j] += tot[m * CL_W + lc * 4 + j];
    } else {
        if (threadIdx.x == 0) atomicAdd(ws.fallbacks, 1);
        for (int m = 0; m < csplit; m++) {
            float a2[1][4] = {{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k = 0; k < RPT; k++) {
                if (row_ok(m, k)) {
                    float t[4];
                    load_row(t, row_of(m, k), false);
#pragma unroll
                    for (int j = 0; j < 4; j++) a2[0][j] += t[j] * t[j];
                }
            }
            member_sums<THREADS, 1>(a2, lds, wsum);
#pragma unroll
            for (int j = 0; j < 4; j++) ss[j] += wsum[lc * 4 + j];
            __syncthreads();
        }
    }
    float rr[4];
#pragma unroll
    for (int j = 0; j < 4; j++) rr[j] = 1.0f / sqrtf(ss[j] * invC + eps);
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (row_ok(g.member, k)) {
            const size_t off = slab_base + (size_t)row_of(g.member, k) * S;
            if constexpr (FUSE) stv_nt<4>(y_res + off, xv[k]);
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = (xv[k][j] * rr[j]) * wv[k];
            stv_nt<4>(yn + off, o);
        }
    }
    if (threadIdx.x == 0) ws.cnt[g.blk] = my_tag;
}

// RES: dx = rmsnorm_bwd(dy, x, w) + res and optionally dx2 = alpha2*dx (training/training_dynamic/train.m:586-595,
// :714-721), as rms_bwd_res_kernel of norm.hip.  dw partials: part[cluster][c], one row per cluster.
template <int RPT, int THREADS, bool RES, bool EXACT>
__global__ __launch_bounds__(THREADS) void rms_bwd_cluster_kernel(float *dx, float *__restrict__ dw_part, const float *dy,
                                                                  const float *__restrict__ x,
                                                                  const float *__restrict__ w, int C, int S,
                                                                  int strips, int nblk, int csplit, int rows_pm,
                                                                  float eps, float invC, int variant, const float *res,
                                                                  float *dx2, float alpha2, ClusterWs ws,
                                                                  int spin_ticks) {
    constexpr int RPS = THREADS / CL_LPR;
    constexpr int NW = THREADS / 64;
    constexpr int NF = (CL_MAX_SPLIT * 2 * CL_W + THREADS - 1) / THREADS;
    __shared__ float lds[NW * 2 * CL_W];
    __shared__ float wsum[2 * CL_W];
    __shared__ float tot[CL_MAX_SPLIT * 2 * CL_W];
    __shared__ int failed;
    const ClusterGeo g = cluster_geo(nblk, csplit, strips);
    const int lc = threadIdx.x % CL_LPR, row0 = threadIdx.x / CL_LPR;
    const int col = g.strip * CL_W + lc * 4;
    const bool col_ok = col < S;
    const size_t slab_base = (size_t)g.slab * C * S + col;
    if (threadIdx.x == 0) failed = 0;
    unsigned my_tag = 0, want_tag[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int i = threadIdx.x + f * THREADS;
        want_tag[f] = i < csplit * 2 * CL_W ? ws.cnt[g.cluster * csplit + i / (2 * CL_W)] + 1u : 0u;
    }
    if (threadIdx.x < 2 * CL_W) my_tag = ws.cnt[g.blk] + 1u;

    auto row_of = [&](int m, int k) { return m * rows_pm + row0 + k * RPS; };
    auto row_ok = [&](int m, int k) { return row0 + k * RPS < rows_pm && row_of(m, k) < C && col_ok; };
    float xv[RPT][4], dv[RPT][4], rv[RES ? RPT : 1][4], wv[RPT];
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (EXACT || row_ok(g.member, k)) {
            const size_t off = slab_base + (size_t)row_of(g.member, k) * S;
            ldv_nt<4>(xv[k], x + off);
            ldv_nt<4>(dv[k], dy + off);
            if constexpr (RES) ldv_nt<4>(rv[k], res + off);
            wv[k] = w[row_of(g.member, k)];
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) xv[k][j] = dv[k][j] = 0.f;
            if constexpr (RES) {
#pragma unroll
                for (int j = 0; j < 4; j++) rv[k][j] = 0.f;
            }
            wv[k] = 0.f;
        }
    }
    float acc[2][4];      // [0] = sum x^2, [1] = sum (dy*x)*w
#pragma unroll
    for (int j = 0; j < 4; j++) acc[0][j] = acc[1][j] = 0.f;
#pragma unroll
    for (int k = 0; k < RPT; k++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[0][j] += xv[k][j] * xv[k][j];
            acc[1][j] += (dv[k][j] * xv[k][j]) * wv[k];
        }
    member_sums<THREADS, 2>(acc, lds, wsum);
    float ss[4] = {0.f, 0.f, 0.f, 0.f}, sd[4] = {0.f, 0.f, 0.f, 0.f};
    if (cluster_exchange<THREADS, 2>(wsum, tot, &failed, g.blk, g.cluster, csplit, ws, my_tag, want_tag, spin_ticks)) {
        for (int m = 0; m < csplit; m++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                ss[j] += tot[(m * 2 + 0) * CL_W + lc * 4 + j];
                sd[j] += tot[(m * 2 + 1) * CL_W + lc * 4 + j];
            }
    } else {
        if (threadIdx.x == 0) atomicAdd(ws.fallbacks, 1);
        for (int m = 0; m < csplit; m++) {
            float a2[2][4];
#pragma unroll
            for (int j = 0; j < 4; j++) a2[0][j] = a2[1][j] = 0.f;
#pragma unroll
            for (int k = 0; k < RPT; k++) {
                if (row_ok(m, k)) {
                    const size_t off = slab_base + (size_t)row_of(m, k) * S;
                    float tx[4], td[4];
                    ldv<4>(tx, x + off);
                    ldv<4>(td, dy + off);
                    const float wc = w[row_of(m, k)];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        a2[0][j] += tx[j] * tx[j];
                        a2[1][j] += (td[j] * tx[j]) * wc;
                    }
                }
            }
            member_sums<THREADS, 2>(a2, lds, wsum);
#pragma unroll
            for (int j = 0; j < 4; j++) { ss[j] += wsum[lc * 4 + j]; sd[j] += wsum[CL_W + lc * 4 + j]; }
            __syncthreads();
        }
    }
    float rr[4], dotn[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        rr[j] = 1.0f / sqrtf(ss[j] * invC + eps);
        dotn[j] = sd[j] * ((rr[j] * rr[j]) * invC);
    }
    float *part = dw_part + (size_t)g.cluster * C;
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        const int c = row_of(g.member, k);
        const bool live = row0 + k * RPS < rows_pm && c < C;       // uniform over the 16 lanes of a row piece
        if (live) {
            float o[4], p = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (variant == 0) o[j] = ((dv[k][j] - xv[k][j] * dotn[j]) * rr[j]) * wv[k];
                else o[j] = (dv[k][j] * wv[k]) * rr[j] - (xv[k][j] * dotn[j]) * rr[j];
                p += (dv[k][j] * xv[k][j]) * rr[j];
                if constexpr (RES) o[j] = o[j] + rv[k][j];
            }
            if (col_ok) {
                const size_t off = slab_base + (size_t)c * S;
                stv_nt<4>(dx + off, o);
                if constexpr (RES) {
                    if (dx2) {
                        float o2[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) o2[j] = o[j] * alpha2;
                        stv_nt<4>(dx2 + off, o2);
                    }
                }
            }
            p = group_sum<CL_LPR>(p);
            if (lc == 0) part[c] = p;
        }
    }
    if (threadIdx.x == 0) ws.cnt[g.blk] = my_tag;
}

// How a shape is split: csplit members of rows_pm rows each; rpt rows per lane.  csplit = 0: not clustered.
struct ClusterPlan {
    int csplit, rows_pm, rpt, threads, strips, nblk;
    bool exact;        // every member holds exactly rps*rpt rows and every strip 64 columns: the unmasked kernels
};

// Clustering pays when whole-C strips of 64 columns would leave most compute units idle: tall tensors
// (C >= 512) whose 64-column strips number fewer than the compute units.  Measured at C = 1024 with 32 x 256 and
// 64 x 256 columns: a launch of more workgroups than compute units (two rounds of 1024-thread workgroups) loses to
// the single-workgroup tiles with 128-byte strips (forward 30.0 against 29.1 us, backward 22.3 against 19.9 us),
// except for the backward with the residual, whose single-workgroup tile is the weakest (32.7 against 43.7 us).
// rounds: how many workgroups per compute unit a launch may have (1: all resident at once).
ClusterPlan cluster_plan(int C, int S, int batch, bool vec_ok, int max_rpt, int rounds) {
    ClusterPlan p = {0, 0, 0, 0, 0, 0, false};
    if (!vec_ok || C < 512 || g_ctx.rms_cluster < 0) return p;
    const long strips = (long)ceil_div((size_t)S, CL_W);
    const long clusters = strips * batch;
    const int cus = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    const int threads = 1024, rps = threads / CL_LPR;
    int split = 0;
    for (int s = 2; s <= CL_MAX_SPLIT; s *= 2) {
        if (clusters * s > CL_MAX_BLOCKS || clusters * s > (long)rounds * cus) break;
        const int rows = (int)ceil_div((size_t)C, (size_t)s);
        if (rows > rps * max_rpt) continue;                      // does not fit the registers yet: split further
        split = s;
        if (clusters * s >= cus) break;                          // a workgroup for every compute unit
    }
    if (g_ctx.rms_cluster > 0) split = g_ctx.rms_cluster;        // forced (2, 4 or 8) for experiments and tests
    if (split < 2 || split > CL_MAX_SPLIT || (split & (split - 1)) || clusters * split > CL_MAX_BLOCKS) return p;
    const int rows = (int)ceil_div((size_t)C, (size_t)split);
    if (rows > rps * max_rpt) return p;
    p.csplit = split;
    p.rows_pm = rows;
    p.rpt = rows <= rps * 4 ? 4 : 8;
    if (p.rpt > max_rpt) { p.csplit = 0; return p; }
    p.threads = threads;
    p.strips = (int)strips;
    p.nblk = (int)(clusters * split);
    p.exact = rows == rps * p.rpt && rows * split == C && S % CL_W == 0;
    return p;
}

}   // namespace
