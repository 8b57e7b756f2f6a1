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
// The kernels are written once for both storage types: fp32 (4 columns per lane, strips of 64 columns) and the
// optional bfloat16 storage (8 columns per lane, strips of 128 columns; arithmetic, sums and weights stay fp32).
//
// Reference ops: rmsnorm and rmsnorm_bwd, training/stories_cpu_ops.h:6-53.
#pragma once
#include "common.h"
#include "tile.h"

namespace {

constexpr int CL_LPR = 16;                        // lanes per row piece: 16 x 16 B = 256 B
constexpr int CL_SLOT_STRIDE = XCH_SLOT_STRIDE;   // 8-byte slots per workgroup: two quantities per column
constexpr int CL_MAX_BLOCKS = XCH_MAX_BLOCKS;     // workgroups per launch that the slot area covers
constexpr int CL_MAX_SPLIT = 8;
typedef Mi355Exchange ClusterWs;

// Storage of the activations: the element type in memory, columns per lane (one 128-bit access), the register
// form of such an access (Raw: for bfloat16 the packed words, half the registers of the widened values, widened at
// each use) and the conversions between Raw and fp32.
struct StoreF32 {
    typedef float T;
    typedef v4f Raw;
    static constexpr int VEC = 4;
    static __device__ __forceinline__ Raw load_nt(const T *p) { return ld4_nt(p); }
    static __device__ __forceinline__ Raw load(const T *p) { return ld4(p); }
    static __device__ __forceinline__ void store_nt(T *p, Raw r) { st4_nt(p, r); }
    static __device__ __forceinline__ void widen(float (&v)[VEC], const Raw &r) { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
    static __device__ __forceinline__ Raw pack(const float (&v)[VEC]) { Raw r = {v[0], v[1], v[2], v[3]}; return r; }
    static __device__ __forceinline__ Raw zero() { Raw r = {0.f, 0.f, 0.f, 0.f}; return r; }
    static __device__ __forceinline__ void forget(Raw &) {}
};
struct StoreBf16 {
    typedef bf16_t T;
    typedef v4u Raw;
    static constexpr int VEC = 8;
    static __device__ __forceinline__ Raw load_nt(const T *p) { return ld_raw<VEC, true>(p); }
    static __device__ __forceinline__ Raw load(const T *p) { return ld_raw<VEC, false>(p); }
    static __device__ __forceinline__ void store_nt(T *p, Raw r) { __builtin_nontemporal_store(r, reinterpret_cast<v4u *>(p)); }
    static __device__ __forceinline__ void widen(float (&v)[VEC], const Raw &r) { unpack<VEC>(v, r); }
    static __device__ __forceinline__ Raw pack(const float (&v)[VEC]) {
        Raw r;
#pragma unroll
        for (int j = 0; j < 4; j++) r[j] = f2_to_bf2(v[2 * j], v[2 * j + 1]);
        return r;
    }
    static __device__ __forceinline__ Raw zero() { return raw_zero<VEC>(); }
    // the widened copies made for the column sums are dropped instead of being kept alive across the exchange
    static __device__ __forceinline__ void forget(Raw &r) { ::forget<VEC>(r); }
};
static_assert(CL_SLOT_STRIDE >= 2 * CL_LPR * StoreBf16::VEC, "two quantities per column must fit a workgroup's slots");

// Per-thread partial sums acc[q][j] (q < NV quantities, j < VEC columns of this lane) -> per-column sums of the
// workgroup in wsum[q*W + column], valid for all threads after the barrier.  lds: NW*NV*W floats.
template <int THREADS, int NV, int VEC>
__device__ __forceinline__ void member_sums(float (&acc)[NV][VEC], float *lds, float *wsum) {
    constexpr int NW = THREADS / 64;
    constexpr int W = CL_LPR * VEC;
#pragma unroll
    for (int q = 0; q < NV; q++)
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[q][j] = wave_sum_stride<CL_LPR>(acc[q][j]);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < CL_LPR) {
#pragma unroll
        for (int q = 0; q < NV; q++)
#pragma unroll
            for (int j = 0; j < VEC; j++) lds[(wave * NV + q) * W + lane * VEC + j] = acc[q][j];
    }
    __syncthreads();
    if (threadIdx.x < NV * W) {
        const int q = threadIdx.x / W, c = threadIdx.x % W;
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < NW; wv++) s += lds[(wv * NV + q) * W + c];
        wsum[threadIdx.x] = s;
    }
    __syncthreads();
}

// slots fetched per thread: the members' NV*W column sums, THREADS at a time
template <int THREADS, int NV, int VEC>
constexpr int cluster_fetches() { return (CL_MAX_SPLIT * NV * CL_LPR * VEC + THREADS - 1) / THREADS; }

// Publishes wsum (this member's column sums) and gathers every member's into tot[(m*NV+q)*W + column].
// Returns false when the bounded wait expired for any slot (block-uniform).
template <int THREADS, int NV, int VEC>
__device__ __forceinline__ bool cluster_exchange(const float *wsum, float *tot, int *failed, int blk, int cluster,
                                                 int csplit, const ClusterWs &ws, unsigned my_tag,
                                                 const unsigned (&want_tag)[cluster_fetches<THREADS, NV, VEC>()],
                                                 int spin_ticks) {
    constexpr int NF = cluster_fetches<THREADS, NV, VEC>();
    constexpr int PER = NV * CL_LPR * VEC;            // slots per member
    static_assert(PER <= CL_SLOT_STRIDE && PER <= THREADS, "a member's column sums must fit its slots");
    if (threadIdx.x < PER) {
        const unsigned long long pk = ((unsigned long long)my_tag << 32) | __float_as_uint(wsum[threadIdx.x]);
        __hip_atomic_store(&ws.slots[(size_t)blk * CL_SLOT_STRIDE + threadIdx.x], pk, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    const int nslots = csplit * PER;
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int i = threadIdx.x + f * THREADS;
        if (i < nslots) {
            const int m = i / PER, c = i - m * PER;
            const unsigned long long *sp = &ws.slots[(size_t)(cluster * csplit + m) * CL_SLOT_STRIDE + c];
            const long long t0 = wall_clock64();
            unsigned long long pk;
            bool ok = false;
            for (;;) {
                pk = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (spin_ticks < 0) break;                        // test mode: whatever the slot holds is refused
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

// The launch tags: this workgroup's own, and for every slot it will fetch the one its owner will write.
template <int THREADS, int NV, int VEC>
__device__ __forceinline__ void cluster_tags(unsigned &my_tag, unsigned (&want_tag)[cluster_fetches<THREADS, NV, VEC>()],
                                             int blk, int cluster, int csplit, const ClusterWs &ws) {
    constexpr int PER = NV * CL_LPR * VEC;
#pragma unroll
    for (int f = 0; f < cluster_fetches<THREADS, NV, VEC>(); f++) {
        const int i = threadIdx.x + f * THREADS;
        want_tag[f] = i < csplit * PER ? ws.cnt[cluster * csplit + i / PER] + 1u : 0u;
    }
    my_tag = threadIdx.x < PER ? ws.cnt[blk] + 1u : 0u;     // used by the publishing threads and by thread 0
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
// EXACT: every member holds exactly RPS*RPT rows and every strip is whole.  Then no row or column needs a mask and
// the loads of the tile are issued back to back without branches, which is worth 0.45 us of the 8 us that the
// forward kernel takes on fp32 [16][1024][256]; other shapes take the masked loads.
template <typename ST, int RPT, int THREADS, bool FUSE, bool EXACT>
__global__ __launch_bounds__(THREADS) void rms_fwd_cluster_kernel(typename ST::T *__restrict__ yn, typename ST::T *y_res,
                                                                  const typename ST::T *a, const typename ST::T *b,
                                                                  float alpha, const float *__restrict__ w, int C,
                                                                  int S, int strips, int nblk, int csplit, int rows_pm,
                                                                  float eps, float invC, ClusterWs ws,
                                                                  int spin_ticks) {
    constexpr int VEC = ST::VEC;
    constexpr int W = CL_LPR * VEC;
    constexpr int RPS = THREADS / CL_LPR;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * W];
    __shared__ float wsum[W];
    __shared__ float tot[CL_MAX_SPLIT * W];
    __shared__ int failed;
    const ClusterGeo g = cluster_geo(nblk, csplit, strips);
    const int lc = threadIdx.x % CL_LPR, row0 = threadIdx.x / CL_LPR;
    const int col = g.strip * W + lc * VEC;
    const bool col_ok = col < S;
    const size_t slab_base = (size_t)g.slab * C * S + col;
    if (threadIdx.x == 0) failed = 0;
    unsigned my_tag, want_tag[cluster_fetches<THREADS, 1, VEC>()];
    cluster_tags<THREADS, 1, VEC>(my_tag, want_tag, g.blk, g.cluster, csplit, ws);

    // rows of member m held by this thread: c = m*rows_pm + row0 + k*RPS, valid while below (m+1)*rows_pm and C
    auto row_of = [&](int m, int k) { return m * rows_pm + row0 + k * RPS; };
    auto row_ok = [&](int m, int k) { return row0 + k * RPS < rows_pm && row_of(m, k) < C && col_ok; };
    // one row piece of x (FUSE: of y = a + alpha*b, rounded to the storage type as the stored y is)
    auto load_row = [&](int c, bool streaming) -> typename ST::Raw {
        const size_t off = slab_base + (size_t)c * S;
        if constexpr (FUSE) {
            float av[VEC], bv[VEC], v[VEC];
            ST::widen(av, streaming ? ST::load_nt(a + off) : ST::load(a + off));
            ST::widen(bv, streaming ? ST::load_nt(b + off) : ST::load(b + off));
#pragma unroll
            for (int j = 0; j < VEC; j++) v[j] = bv[j] * alpha + av[j];
            return ST::pack(v);
        } else {
            return streaming ? ST::load_nt(a + off) : ST::load(a + off);
        }
    };

    typename ST::Raw xr[RPT];
    float wv[RPT];
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (EXACT || row_ok(g.member, k)) {
            xr[k] = load_row(row_of(g.member, k), true);
            wv[k] = w[row_of(g.member, k)];
        } else {
            xr[k] = ST::zero();
            wv[k] = 0.f;
        }
    }
    float acc[1][VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = 0.f;
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        float xv[VEC];
        ST::widen(xv, xr[k]);
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[0][j] += xv[j] * xv[j];
    }
#pragma unroll
    for (int k = 0; k < RPT; k++) ST::forget(xr[k]);
    member_sums<THREADS, 1, VEC>(acc, lds, wsum);
    float ss[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) ss[j] = 0.f;
    if (cluster_exchange<THREADS, 1, VEC>(wsum, tot, &failed, g.blk, g.cluster, csplit, ws, my_tag, want_tag, spin_ticks)) {
        for (int m = 0; m < csplit; m++)
#pragma unroll
            for (int j = 0; j < VEC; j++) ss[j] += tot[m * W + lc * VEC + j];
    } else {
        if (threadIdx.x == 0) atomicAdd(ws.fallbacks, 1);
        for (int m = 0; m < csplit; m++) {
            float a2[1][VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++) a2[0][j] = 0.f;
#pragma unroll
            for (int k = 0; k < RPT; k++) {
                if (row_ok(m, k)) {
                    float t[VEC];
                    ST::widen(t, load_row(row_of(m, k), false));
#pragma unroll
                    for (int j = 0; j < VEC; j++) a2[0][j] += t[j] * t[j];
                }
            }
            member_sums<THREADS, 1, VEC>(a2, lds, wsum);
#pragma unroll
            for (int j = 0; j < VEC; j++) ss[j] += wsum[lc * VEC + j];
            __syncthreads();
        }
    }
    float rr[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) rr[j] = 1.0f / sqrtf(ss[j] * invC + eps);
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (EXACT || row_ok(g.member, k)) {
            const size_t off = slab_base + (size_t)row_of(g.member, k) * S;
            if constexpr (FUSE) ST::store_nt(y_res + off, xr[k]);
            float xv[VEC], o[VEC];
            ST::widen(xv, xr[k]);
#pragma unroll
            for (int j = 0; j < VEC; j++) o[j] = (xv[j] * rr[j]) * wv[k];
            ST::store_nt(yn + off, ST::pack(o));
        }
    }
    if (threadIdx.x == 0) ws.cnt[g.blk] = my_tag;
}

// RES: dx = rmsnorm_bwd(dy, x, w) + res and optionally dx2 = alpha2*dx (training/training_dynamic/train.m:586-595,
// :714-721), as rms_bwd_res_kernel of norm.hip.  dw partials: part[cluster][c], one row per cluster.
template <typename ST, int RPT, int THREADS, bool RES, bool EXACT>
__global__ __launch_bounds__(THREADS) void rms_bwd_cluster_kernel(typename ST::T *dx, float *__restrict__ dw_part,
                                                                  const typename ST::T *dy,
                                                                  const typename ST::T *__restrict__ x,
                                                                  const float *__restrict__ w, int C, int S,
                                                                  int strips, int nblk, int csplit, int rows_pm,
                                                                  float eps, float invC, int variant,
                                                                  const typename ST::T *res, typename ST::T *dx2,
                                                                  float alpha2, ClusterWs ws, int spin_ticks) {
    constexpr int VEC = ST::VEC;
    constexpr int W = CL_LPR * VEC;
    constexpr int RPS = THREADS / CL_LPR;
    constexpr int NW = THREADS / 64;
    __shared__ float lds[NW * 2 * W];
    __shared__ float wsum[2 * W];
    __shared__ float tot[CL_MAX_SPLIT * 2 * W];
    __shared__ int failed;
    const ClusterGeo g = cluster_geo(nblk, csplit, strips);
    const int lc = threadIdx.x % CL_LPR, row0 = threadIdx.x / CL_LPR;
    const int col = g.strip * W + lc * VEC;
    const bool col_ok = col < S;
    const size_t slab_base = (size_t)g.slab * C * S + col;
    if (threadIdx.x == 0) failed = 0;
    unsigned my_tag, want_tag[cluster_fetches<THREADS, 2, VEC>()];
    cluster_tags<THREADS, 2, VEC>(my_tag, want_tag, g.blk, g.cluster, csplit, ws);

    auto row_of = [&](int m, int k) { return m * rows_pm + row0 + k * RPS; };
    auto row_ok = [&](int m, int k) { return row0 + k * RPS < rows_pm && row_of(m, k) < C && col_ok; };

    typename ST::Raw xr[RPT], dr[RPT], rr_res[RES ? RPT : 1];
    float wv[RPT];
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        if (EXACT || row_ok(g.member, k)) {
            const size_t off = slab_base + (size_t)row_of(g.member, k) * S;
            xr[k] = ST::load_nt(x + off);
            dr[k] = ST::load_nt(dy + off);
            if constexpr (RES) rr_res[k] = ST::load_nt(res + off);
            wv[k] = w[row_of(g.member, k)];
        } else {
            xr[k] = dr[k] = ST::zero();
            if constexpr (RES) rr_res[k] = ST::zero();
            wv[k] = 0.f;
        }
    }
    float acc[2][VEC];      // [0] = sum x^2, [1] = sum (dy*x)*w
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[0][j] = acc[1][j] = 0.f;
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        float xv[VEC], dv[VEC];
        ST::widen(xv, xr[k]);
        ST::widen(dv, dr[k]);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            acc[0][j] += xv[j] * xv[j];
            acc[1][j] += (dv[j] * xv[j]) * wv[k];
        }
    }
#pragma unroll
    for (int k = 0; k < RPT; k++) { ST::forget(xr[k]); ST::forget(dr[k]); }
    member_sums<THREADS, 2, VEC>(acc, lds, wsum);
    float ss[VEC], sd[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) ss[j] = sd[j] = 0.f;
    if (cluster_exchange<THREADS, 2, VEC>(wsum, tot, &failed, g.blk, g.cluster, csplit, ws, my_tag, want_tag, spin_ticks)) {
        for (int m = 0; m < csplit; m++)
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                ss[j] += tot[(m * 2 + 0) * W + lc * VEC + j];
                sd[j] += tot[(m * 2 + 1) * W + lc * VEC + j];
            }
    } else {
        if (threadIdx.x == 0) atomicAdd(ws.fallbacks, 1);
        for (int m = 0; m < csplit; m++) {
            float a2[2][VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++) a2[0][j] = a2[1][j] = 0.f;
#pragma unroll
            for (int k = 0; k < RPT; k++) {
                if (row_ok(m, k)) {
                    const size_t off = slab_base + (size_t)row_of(m, k) * S;
                    float tx[VEC], td[VEC];
                    ST::widen(tx, ST::load(x + off));
                    ST::widen(td, ST::load(dy + off));
                    const float wc = w[row_of(m, k)];
#pragma unroll
                    for (int j = 0; j < VEC; j++) {
                        a2[0][j] += tx[j] * tx[j];
                        a2[1][j] += (td[j] * tx[j]) * wc;
                    }
                }
            }
            member_sums<THREADS, 2, VEC>(a2, lds, wsum);
#pragma unroll
            for (int j = 0; j < VEC; j++) { ss[j] += wsum[lc * VEC + j]; sd[j] += wsum[W + lc * VEC + j]; }
            __syncthreads();
        }
    }
    float rr[VEC], dotn[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        rr[j] = 1.0f / sqrtf(ss[j] * invC + eps);
        dotn[j] = sd[j] * ((rr[j] * rr[j]) * invC);
    }
    float *part = dw_part + (size_t)g.cluster * C;
#pragma unroll
    for (int k = 0; k < RPT; k++) {
        const int c = row_of(g.member, k);
        const bool live = EXACT || (row0 + k * RPS < rows_pm && c < C);       // uniform over the 16 lanes of a row piece
        if (live) {
            float xv[VEC], dv[VEC], o[VEC], p = 0.f;
            ST::widen(xv, xr[k]);
            ST::widen(dv, dr[k]);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                if (variant == 0) o[j] = ((dv[j] - xv[j] * dotn[j]) * rr[j]) * wv[k];
                else o[j] = (dv[j] * wv[k]) * rr[j] - (xv[j] * dotn[j]) * rr[j];
                p += (dv[j] * xv[j]) * rr[j];
            }
            if constexpr (RES) {
                float rv[VEC];
                ST::widen(rv, rr_res[k]);
#pragma unroll
                for (int j = 0; j < VEC; j++) o[j] = o[j] + rv[j];
            }
            if (EXACT || col_ok) {
                const size_t off = slab_base + (size_t)c * S;
                ST::store_nt(dx + off, ST::pack(o));
                if constexpr (RES) {
                    if (dx2) {
                        float o2[VEC];
#pragma unroll
                        for (int j = 0; j < VEC; j++) o2[j] = o[j] * alpha2;
                        ST::store_nt(dx2 + off, ST::pack(o2));
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
    bool exact;        // every member holds exactly rps*rpt rows and every strip is whole: the unmasked kernels
};
constexpr ClusterPlan NO_CLUSTER = {0, 0, 0, 0, 0, 0, false};

// Clustering pays when whole-C strips of 256 bytes would leave most compute units idle: tall tensors
// (C >= 512) whose strips number fewer than the compute units.  Measured at C = 1024, fp32, with 32 x 256 and
// 64 x 256 columns: a launch of more workgroups than compute units (two rounds of 1024-thread workgroups) loses to
// the single-workgroup tiles with 128-byte strips (forward 30.0 against 29.1 us, backward 22.3 against 19.9 us),
// except for the backward with the residual, whose single-workgroup tile is the weakest (32.7 against 43.7 us).
// vec: columns per lane of the storage type; rpt_lo..rpt_hi: rows per lane that are instantiated (powers of two);
// rounds: how many workgroups per compute unit a launch may have (1: all resident at once).
ClusterPlan cluster_plan(int C, int S, int batch, bool vec_ok, int vec, int rpt_lo, int rpt_hi, int rounds) {
    ClusterPlan p = NO_CLUSTER;
    if (!vec_ok || C < 512 || g_ctx.rms_cluster < 0) return p;
    const int w = CL_LPR * vec;
    const long strips = (long)ceil_div((size_t)S, (size_t)w);
    const long clusters = strips * batch;
    const int cus = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    const int threads = 1024, rps = threads / CL_LPR;
    int split = 0;
    for (int s = 2; s <= CL_MAX_SPLIT; s *= 2) {
        if (clusters * s > CL_MAX_BLOCKS || clusters * s > (long)rounds * cus) break;
        const int rows = (int)ceil_div((size_t)C, (size_t)s);
        if (rows > rps * rpt_hi) continue;                       // does not fit the registers yet: split further
        split = s;
        if (clusters * s >= cus) break;                          // a workgroup for every compute unit
    }
    if (g_ctx.rms_cluster > 0) split = g_ctx.rms_cluster;        // forced (2, 4 or 8) for experiments and tests
    if (split < 2 || split > CL_MAX_SPLIT || (split & (split - 1)) || clusters * split > CL_MAX_BLOCKS) return p;
    const int rows = (int)ceil_div((size_t)C, (size_t)split);
    int rpt = rpt_lo;
    while (rpt < rpt_hi && rows > rps * rpt) rpt *= 2;
    if (rows > rps * rpt) return p;
    p.csplit = split;
    p.rows_pm = rows;
    p.rpt = rpt;
    p.threads = threads;
    p.strips = (int)strips;
    p.nblk = (int)(clusters * split);
    p.exact = rows == rps * rpt && rows * split == C && S % w == 0;
    return p;
}

}   // namespace
