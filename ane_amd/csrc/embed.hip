// embed.hip — token-embedding gather and its deterministic scatter-add backward.
//
// Reference ops: embed_lookup (training/stories_cpu_ops.h:112-120; unchecked twin
// training/training_dynamic/cpu_ops.h:150-156) and embed_backward (stories_cpu_ops.h:123-131;
// cpu_ops.h:158-164).  The table E is [V][D] row-major, activations are [batch][D][S].
//
// Gather: a 64-token x 64-dim tile goes through LDS so that both sides are coalesced — table
// rows are read along d (256 B runs), the channel-first output is written along t (256 B runs).
//
// Scatter-add: the reference adds dx[:,t] into dE[tok_t] for t ascending, so each (row, d) sum has
// a fixed order.  To reproduce it bit for bit:
//   1. stable radix sort of (token, position) pairs by token (rocPRIM device primitive);
//   2. dx is transposed through LDS into token-major rows written in SORTED order, so a
//      segment (all positions of one token) is a run of consecutive rows;
//   3. each (segment, 64-float chunk) is summed sequentially starting from the value already
//      in dE — short segments by one wave straight from memory, long segments by a whole
//      workgroup that stages 240 rows at a time in LDS to keep enough loads in flight while one
//      wave performs the ordered adds; both kinds share one launch so the long chains overlap
//      the many short ones.
#include "common.h"

#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace {

constexpr int TT = 64;   // tokens per tile
constexpr int TD = 64;   // dims per tile
constexpr int LONG_SEG = 64;    // segments longer than this take the workgroup path
constexpr int STAGE_PER_WAVE = 15;
constexpr int STAGE_ROWS = 16 * STAGE_PER_WAVE;   // 240 rows x 256 B = 60 KiB of LDS, plus a 4 KiB work list

// ---------------------------------------------------------------------------------------------
// Gather
// ---------------------------------------------------------------------------------------------
template <bool VEC_D>
__global__ __launch_bounds__(256) void gather_kernel(float *__restrict__ x, const float *__restrict__ E,
                                                     const int32_t *__restrict__ ids, int V, int D, int S,
                                                     int t_tiles) {
    __shared__ float tile[TT][TD + 1];
    __shared__ int tok[TT];
    const int bt = blockIdx.x;                 // (b, t-tile)
    const int b = bt / t_tiles, t0 = (bt - b * t_tiles) * TT;
    const int d0 = blockIdx.y * TD;
    const int tid = threadIdx.x;
    if (tid < TT) {
        const int t = t0 + tid;
        int id = -1;
        if (t < S) {
            id = ids[(size_t)b * S + t];
            if (id < 0 || id >= V) id = -1;
        }
        tok[tid] = id;
    }
    __syncthreads();
    // phase 1: table rows -> LDS, lanes along d
    {
        const int dq = tid & 15, r0 = tid >> 4;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int r = r0 + 16 * k;
            const int id = tok[r];
            const int d = d0 + 4 * dq;
            if (id >= 0) {
                const float *src = E + (size_t)id * D + d;
                if (VEC_D && d + 3 < D) {
                    v4f v = ld4(src);
                    tile[r][4 * dq + 0] = v.x; tile[r][4 * dq + 1] = v.y;
                    tile[r][4 * dq + 2] = v.z; tile[r][4 * dq + 3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (d + j < D) tile[r][4 * dq + j] = src[j];
                }
            }
        }
    }
    __syncthreads();
    // phase 2: LDS -> channel-first output, lanes along t
    {
        const int tq = tid & 15, r0 = tid >> 4;
        const bool s_vec = (S & 3) == 0;
        const int t = t0 + 4 * tq;
        const int i0 = tok[4 * tq], i1 = tok[4 * tq + 1], i2 = tok[4 * tq + 2], i3 = tok[4 * tq + 3];
        const bool all = (i0 >= 0) & (i1 >= 0) & (i2 >= 0) & (i3 >= 0) & s_vec;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int dl = r0 + 16 * k;
            const int d = d0 + dl;
            if (d >= D) continue;
            float *dst = x + ((size_t)b * D + d) * S + t;
            if (all) {
                v4f v = {tile[4 * tq][dl], tile[4 * tq + 1][dl], tile[4 * tq + 2][dl], tile[4 * tq + 3][dl]};
                st4(dst, v);
            } else {
                if (i0 >= 0) dst[0] = tile[4 * tq][dl];
                if (i1 >= 0) dst[1] = tile[4 * tq + 1][dl];
                if (i2 >= 0) dst[2] = tile[4 * tq + 2][dl];
                if (i3 >= 0) dst[3] = tile[4 * tq + 3][dl];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Scatter-add
// ---------------------------------------------------------------------------------------------
// Sort key of a token id: the id itself, or V for an id outside [0,V) so that those sort last and are skipped.
// The sort reads ids through this functor and takes 0,1,2,... as the values, so no staging pass is needed.
struct ClampId {
    int V;
    __host__ __device__ int operator()(int32_t id) const { return (id < 0 || id >= V) ? V : id; }
};

// meta[0] = number of segments, meta[2] = number of valid (in-range) entries.
//
// Segment starts are found in two small launches: (1) every workgroup flags the heads among its
// 1024 sorted entries (key differs from its predecessor), counts them and writes the inverse
// permutation; (2) every workgroup adds up the counts before its own and writes the positions of its
// heads at that offset.
constexpr int PLAN_T = 1024;

__device__ __forceinline__ int block_excl_scan_1024(int v, int *lds, int &total) {
    // exclusive scan of one int per thread over 1024 threads: wave scan by shuffles, then the 16 wave totals
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int x = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int y = __shfl_up(x, off, 64);
        if (lane >= off) x += y;
    }
    if (lane == 63) lds[wave] = x;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int k = 0; k < PLAN_T / 64; k++) {
        const int t = lds[k];
        if (k < wave) base += t;
        tot += t;
    }
    total = tot;
    __syncthreads();
    return base + x - v;
}

__global__ __launch_bounds__(PLAN_T) void plan_flags_kernel(int *__restrict__ rank, int *__restrict__ blk_count,
                                                            int *__restrict__ meta, const int *__restrict__ keys,
                                                            const int *__restrict__ vals, int N, int V) {
    __shared__ int lds[PLAN_T / 64];
    const int i = blockIdx.x * PLAN_T + threadIdx.x;
    int head = 0;
    if (i < N) {
        const int k = keys[i];
        const int kp = i > 0 ? keys[i - 1] : -1;
        rank[vals[i]] = i;
        head = (k < V && k != kp) ? 1 : 0;
        // number of valid entries: the index of the first out-of-range key, or N when the last key is valid
        // (exactly one thread of the grid meets one of the two conditions)
        if (k >= V && kp < V) meta[2] = i;
        if (i == N - 1 && k < V) meta[2] = N;
    }
    int total;
    (void)block_excl_scan_1024(head, lds, total);
    if (threadIdx.x == 0) blk_count[blockIdx.x] = total;
}

// Second (and last) launch: every workgroup sums the head counts of the workgroups before it (a few reads),
// scans its own flags and writes its segment starts; the last one also writes the segment count and the end of
// the last segment.
__global__ __launch_bounds__(PLAN_T) void plan_write_kernel(int *__restrict__ seg_start, int *__restrict__ meta,
                                                            const int *__restrict__ blk_count,
                                                            const int *__restrict__ keys, int N, int V) {
    __shared__ int lds[PLAN_T / 64];
    __shared__ int before;
    int part = 0;
    for (int b = threadIdx.x; b < (int)blockIdx.x; b += PLAN_T) part += blk_count[b];
    int dummy;
    const int ex0 = block_excl_scan_1024(part, lds, dummy);     // dummy = total over the workgroup
    (void)ex0;
    if (threadIdx.x == 0) before = dummy;
    __syncthreads();
    const int off = before;
    const int i = blockIdx.x * PLAN_T + threadIdx.x;
    int head = 0;
    if (i < N) {
        const int k = keys[i];
        const int kp = i > 0 ? keys[i - 1] : -1;
        head = (k < V && k != kp) ? 1 : 0;
    }
    int total;
    const int ex = block_excl_scan_1024(head, lds, total);
    if (head) seg_start[off + ex] = i;
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
        meta[0] = off + total;
        seg_start[off + total] = meta[2];           // end of the last segment = number of valid entries
    }
}

// dx [batch][D][S] -> rows[rank[n]][D] (token-major, in sorted order), through a 64x64 LDS tile
__global__ __launch_bounds__(256) void transpose_sorted_kernel(float *__restrict__ rows, const float *__restrict__ dx,
                                                               const int *__restrict__ rank, int D, int S,
                                                               int t_tiles) {
    __shared__ float tile[TD][TT + 1];
    __shared__ int dst_row[TT];
    const int bt = blockIdx.x;
    const int b = bt / t_tiles, t0 = (bt - b * t_tiles) * TT;
    const int d0 = blockIdx.y * TD;
    const int tid = threadIdx.x;
    if (tid < TT) dst_row[tid] = (t0 + tid < S) ? rank[(size_t)b * S + t0 + tid] : -1;
    const bool s_vec = (S & 3) == 0;
    {   // lanes along t
        const int tq = tid & 15, r0 = tid >> 4;
        const int t = t0 + 4 * tq;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int dl = r0 + 16 * k, d = d0 + dl;
            if (d >= D) continue;
            const float *src = dx + ((size_t)b * D + d) * S + t;
            if (s_vec && t + 3 < S) {
                v4f v = ld4_nt(src);
                tile[dl][4 * tq + 0] = v.x; tile[dl][4 * tq + 1] = v.y;
                tile[dl][4 * tq + 2] = v.z; tile[dl][4 * tq + 3] = v.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (t + j < S) tile[dl][4 * tq + j] = src[j];
            }
        }
    }
    __syncthreads();
    {   // lanes along d
        const int dq = tid & 15, r0 = tid >> 4;
        const bool d_vec = (D & 3) == 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int tl = r0 + 16 * k;
            const int row = dst_row[tl];
            if (row < 0) continue;
            const int d = d0 + 4 * dq;
            float *dst = rows + (size_t)row * D + d;
            if (d_vec && d + 3 < D) {
                v4f v = {tile[4 * dq][tl], tile[4 * dq + 1][tl], tile[4 * dq + 2][tl], tile[4 * dq + 3][tl]};
                st4(dst, v);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (d + j < D) dst[j] = tile[4 * dq + j][tl];
            }
        }
    }
}

// Segment sums.  One launch, two kinds of workgroup (1024 threads each):
//  * the first `long_blocks` workgroups take the LONG segments (more than LONG_SEG rows): workgroup
//    (x, chunk) walks segments x, x + gridDim.x/..., and for each long one sums its 64-float chunk: 16 waves
//    stage 240 rows in LDS (15 loads in flight per lane), wave 0 adds them in order, 16 rows per batch of
//    LDS reads so the adds are not exposed to the LDS latency;
//  * the others take the short segments: one wave per (segment, 64-float chunk), rows read straight
//    from memory, eight loads in flight.
// Either way every (row of dE, d) is written by exactly one lane, sequentially in position order,
// starting from the value already in dE.
template <bool TREE>
__global__ __launch_bounds__(1024) void seg_sum_kernel(float *__restrict__ dE, const float *__restrict__ rows,
                                                       const int *__restrict__ seg_start, const int *__restrict__ keys,
                                                       const int *__restrict__ meta, int D, int nchunk,
                                                       int long_x, int short_blocks) {
    __shared__ float stage[STAGE_ROWS][64];
    __shared__ int work[1023];      // with nwork: 4 KiB, for 64 KiB of LDS in all
    __shared__ int nwork;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nseg = meta[0];
    const int long_blocks = long_x * nchunk;
    if ((int)blockIdx.x < long_blocks) {
        const int ch = blockIdx.x % nchunk, x0 = blockIdx.x / nchunk;
        const int d = ch * 64 + lane;
        const bool d_ok = d < D;
        // candidates of this workgroup column: segments x0, x0+long_x, ...; 1023 are screened at a time
        for (int j0 = 0; x0 + (long)j0 * long_x < nseg; j0 += 1023) {
            if (threadIdx.x == 0) nwork = 0;
            __syncthreads();
            {
                const long seg = x0 + (long)(j0 + (int)threadIdx.x) * long_x;
                if (threadIdx.x < 1023 && seg < nseg && seg_start[seg + 1] - seg_start[seg] > LONG_SEG)
                    work[atomicAdd(&nwork, 1)] = (int)seg;
            }
            __syncthreads();
            const int nw = nwork;
            for (int k = 0; k < nw; k++) {
                const int seg = work[k];
                const int lo = seg_start[seg], hi = seg_start[seg + 1];
                // Software pipeline: the rows of stage s+1 are already on their way into registers while wave 0
                // adds the rows of stage s out of LDS.
                float v[STAGE_PER_WAVE];
                auto fetch = [&](int base) {
                    const int nrow = min(STAGE_ROWS, hi - base);
#pragma unroll
                    for (int j = 0; j < STAGE_PER_WAVE; j++) {
                        const int rl = wave * STAGE_PER_WAVE + j;
                        v[j] = (rl < nrow && d_ok) ? __builtin_nontemporal_load(rows + (size_t)(base + rl) * D + d) : 0.f;
                    }
                };
                fetch(lo);                               // first, so that the token id and the old dE row load beside it
                const int tok = keys[lo];
                float acc = 0.f;
                if (wave == 0 && d_ok) acc = dE[(size_t)tok * D + d];
                for (int base = lo; base < hi; base += STAGE_ROWS) {
                    const int nrow = min(STAGE_ROWS, hi - base);
                    if constexpr (TREE) {
                        // fixed tree instead of the reference's chain (opt-in, "scatter_tree" knob): every wave sums
                        // its 15 rows in order, wave 0 adds the 16 partial rows in wave order.  Deterministic, 8x
                        // shorter chain, but rounded differently from the CPU loop.  Rows past the end are zeros.
                        float p = v[0];
#pragma unroll
                        for (int j = 1; j < STAGE_PER_WAVE; j++) p += v[j];
                        stage[wave][lane] = p;
                        __syncthreads();
                        if (base + STAGE_ROWS < hi) fetch(base + STAGE_ROWS);
                        if (wave == 0) {
#pragma unroll
                            for (int q = 0; q < 16; q++) acc += stage[q][lane];
                        }
                        __syncthreads();
                        continue;
                    }
#pragma unroll
                    for (int j = 0; j < STAGE_PER_WAVE; j++) stage[wave * STAGE_PER_WAVE + j][lane] = v[j];
                    __syncthreads();
                    if (base + STAGE_ROWS < hi) fetch(base + STAGE_ROWS);
                    if (wave == 0) {
                        int rl = 0;
                        for (; rl + 16 <= nrow; rl += 16) {
                            float t[16];
#pragma unroll
                            for (int j = 0; j < 16; j++) t[j] = stage[rl + j][lane];
#pragma unroll
                            for (int j = 0; j < 16; j++) acc += t[j];
                        }
                        for (; rl < nrow; rl++) acc += stage[rl][lane];
                    }
                    __syncthreads();
                }
                if (wave == 0 && d_ok) dE[(size_t)tok * D + d] = acc;
            }
            __syncthreads();
        }
        return;
    }
    // short segments
    const int gw = ((int)blockIdx.x - long_blocks) * 16 + wave;
    const int nwaves = short_blocks * 16;
    const long units = (long)nseg * nchunk;
    for (long u = gw; u < units; u += nwaves) {
        const int seg = (int)(u / nchunk), ch = (int)(u - (long)seg * nchunk);
        const int lo = seg_start[seg], hi = seg_start[seg + 1];
        if (hi - lo > LONG_SEG) continue;
        const int d = ch * 64 + lane;
        if (d >= D) continue;
        const int tok = keys[lo];
        float *dst = dE + (size_t)tok * D + d;
        float acc = *dst;
        const float *src = rows + (size_t)lo * D + d;
        int r = lo;
        for (; r + 8 <= hi; r += 8) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = __builtin_nontemporal_load(src + (size_t)j * D);
#pragma unroll
            for (int j = 0; j < 8; j++) acc += v[j];
            src += (size_t)8 * D;
        }
        for (; r < hi; r++) { acc += __builtin_nontemporal_load(src); src += D; }
        *dst = acc;
    }
}

// ---------------------------------------------------------------------------------------------
// Vocabulary compaction (training/training_dynamic/cpu_ops.h:127-148): whole-row copies by index.
// One workgroup row of 64 lanes x 128 bit covers 1 KiB of a table row.
// MODE 0: dst[i] = src[idx[i]] (vocab_compact_embed)   MODE 1: dst[idx[i]] = src[i] (vocab_update_full)
// MODE 2: dst[idx[i]] += src[i] (vocab_scatter_grads; idx holds distinct rows, so no two lanes meet)
// ---------------------------------------------------------------------------------------------
template <int MODE, int VEC>
__global__ __launch_bounds__(256) void rows_by_index_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                            const int32_t *__restrict__ idx, int n, int D, int rows_dst,
                                                            int rows_src) {
    const int dv = (D + VEC - 1) / VEC;                          // column groups per row
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (size_t)n * dv) return;
    const int i = (int)(t / dv), cg = (int)(t - (size_t)i * dv);
    const int r = idx[i];
    if (r < 0 || r >= (MODE == 0 ? rows_src : rows_dst)) return;  // an index outside the table is skipped
    const size_t a = (MODE == 0 ? (size_t)r : (size_t)i) * D + (size_t)cg * VEC;      // source offset
    const size_t b = (MODE == 0 ? (size_t)i : (size_t)r) * D + (size_t)cg * VEC;      // destination offset
    if constexpr (VEC == 4) {
        v4f v = ld4(src + a);
        if (MODE == 2) v = ld4(dst + b) + v;
        st4(dst + b, v);
    } else {
        float v = src[a];
        if (MODE == 2) v = dst[b] + v;
        dst[b] = v;
    }
}

template <int MODE>
int rows_by_index(const char *who, float *dst, const float *src, const int32_t *idx, int n, int D, int rows_dst,
                  int rows_src) {
    if (!mi355_ready(who)) return -1;
    if (!dst || !src || !idx) return mi355_fail("%s: NULL pointer", who);
    if (n <= 0 || D <= 0 || rows_dst <= 0 || rows_src <= 0) return mi355_fail("%s: bad shape n=%d D=%d", who, n, D);
    const bool vec = (D % 4 == 0) && aligned16(dst) && aligned16(src);
    const size_t work = (size_t)n * (vec ? D / 4 : D);
    const unsigned blocks = (unsigned)ceil_div(work, 256);
    if (vec) hipLaunchKernelGGL((rows_by_index_kernel<MODE, 4>), dim3(blocks), dim3(256), 0, g_ctx.stream, dst, src, idx, n, D, rows_dst, rows_src);
    else hipLaunchKernelGGL((rows_by_index_kernel<MODE, 1>), dim3(blocks), dim3(256), 0, g_ctx.stream, dst, src, idx, n, D, rows_dst, rows_src);
    LAUNCH_OK(who);
    return 0;
}

int key_bits(int V) {
    int bits = 1;
    while (bits < 31 && (1L << bits) <= (long)V) bits++;   // keys range over [0, V]
    return bits;
}

}   // namespace

MI355_API int mi355_embed_gather_dev(float *x, const float *E, const int32_t *ids, int V, int D, int S, int batch) {
    if (!mi355_ready("embed_gather")) return -1;
    if (!x || !E || !ids) return mi355_fail("embed_gather: NULL pointer");
    if (V <= 0 || D <= 0 || S <= 0 || batch <= 0) return mi355_fail("embed_gather: bad shape V=%d D=%d S=%d batch=%d", V, D, S, batch);
    const int t_tiles = (int)ceil_div((size_t)S, TT);
    const dim3 grid((unsigned)(batch * t_tiles), (unsigned)ceil_div((size_t)D, TD));
    if (grid.y > 65535) return mi355_fail("embed_gather: D too large");
    const bool vec_d = (D % 4 == 0) && aligned16(E) && aligned16(x);
    if (vec_d) hipLaunchKernelGGL((gather_kernel<true>), grid, dim3(256), 0, g_ctx.stream, x, E, ids, V, D, S, t_tiles);
    else hipLaunchKernelGGL((gather_kernel<false>), grid, dim3(256), 0, g_ctx.stream, x, E, ids, V, D, S, t_tiles);
    LAUNCH_OK("embed_gather");
    return 0;
}

MI355_API int mi355_embed_scatter_add_dev(float *dE, const float *dx, const int32_t *ids, int V, int D, int S,
                                          int batch) {
    if (!mi355_ready("embed_scatter_add")) return -1;
    if (!mi355_outside_capture("embed_scatter_add (its library sort may record memset nodes)")) return -1;
    if (!dE || !dx || !ids) return mi355_fail("embed_scatter_add: NULL pointer");
    if (V <= 0 || D <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("embed_scatter_add: bad shape V=%d D=%d S=%d batch=%d", V, D, S, batch);
    if ((size_t)batch * S > (size_t)1 << 30) return mi355_fail("embed_scatter_add: more than 2^30 positions");
    if (!aligned16(dx) || !aligned16(dE)) return mi355_fail("embed_scatter_add: pointers must be 16-byte aligned");
    const int N = batch * S;
    const int bits = key_bits(V);

    size_t temp_bytes = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, rocprim::make_transform_iterator(ids, ClampId{V}),
                                             (int *)nullptr, rocprim::counting_iterator<int>(0), (int *)nullptr,
                                             (size_t)N, 0, bits, g_ctx.stream);
    if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort sizing: %s", hipGetErrorString(e));

    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t nb = al((size_t)N * sizeof(int));
    const int nplan = (int)ceil_div((size_t)N, PLAN_T);
    const size_t off_keys = 0, off_vals = nb, off_rank = 2 * nb;
    const size_t off_seg = 3 * nb, off_cnt = off_seg + al((size_t)(N + 1) * sizeof(int));
    const size_t off_meta = off_cnt + al((size_t)nplan * sizeof(int)), off_temp = off_meta + 256;
    const size_t off_rows = off_temp + al(temp_bytes);
    const size_t total = off_rows + al((size_t)N * D * sizeof(float));
    char *ws = (char *)mi355_ws(total);
    if (!ws) return -1;
    int *keys = (int *)(ws + off_keys), *vals = (int *)(ws + off_vals), *rank = (int *)(ws + off_rank);
    int *seg_start = (int *)(ws + off_seg), *blk_count = (int *)(ws + off_cnt);
    int *meta = (int *)(ws + off_meta);
    float *rows = (float *)(ws + off_rows);

    e = rocprim::radix_sort_pairs(ws + off_temp, temp_bytes, rocprim::make_transform_iterator(ids, ClampId{V}), keys,
                                  rocprim::counting_iterator<int>(0), vals, (size_t)N, 0, bits, g_ctx.stream);
    if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(plan_flags_kernel, dim3(nplan), dim3(PLAN_T), 0, g_ctx.stream, rank, blk_count, meta, keys, vals,
                       N, V);
    hipLaunchKernelGGL(plan_write_kernel, dim3(nplan), dim3(PLAN_T), 0, g_ctx.stream, seg_start, meta, blk_count, keys, N,
                       V);
    LAUNCH_OK("embed_scatter_add plan");
    const int t_tiles = (int)ceil_div((size_t)S, TT);
    const dim3 tgrid((unsigned)(batch * t_tiles), (unsigned)ceil_div((size_t)D, TD));
    if (tgrid.y > 65535) return mi355_fail("embed_scatter_add: D too large");
    hipLaunchKernelGGL(transpose_sorted_kernel, tgrid, dim3(256), 0, g_ctx.stream, rows, dx, rank, D, S, t_tiles);
    LAUNCH_OK("embed_scatter_add transpose");
    const int nchunk = (int)ceil_div((size_t)D, 64);
    const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    // at most N/LONG_SEG segments can be long; a few dozen workgroup columns cover them
    int long_x = (int)std::min<size_t>((size_t)N / LONG_SEG + 1, (size_t)std::max(1, cu / nchunk));
    size_t short_blocks = ceil_div((size_t)N * nchunk, 16);
    if (short_blocks > (size_t)cu * 4) short_blocks = (size_t)cu * 4;
    if (g_ctx.scatter_tree)
        hipLaunchKernelGGL(seg_sum_kernel<true>, dim3((unsigned)(long_x * nchunk + short_blocks)), dim3(1024), 0,
                           g_ctx.stream, dE, rows, seg_start, keys, meta, D, nchunk, long_x, (int)short_blocks);
    else
        hipLaunchKernelGGL(seg_sum_kernel<false>, dim3((unsigned)(long_x * nchunk + short_blocks)), dim3(1024), 0,
                           g_ctx.stream, dE, rows, seg_start, keys, meta, D, nchunk, long_x, (int)short_blocks);
    LAUNCH_OK("embed_scatter_add segment sums");
    return 0;
}

MI355_API int mi355_vocab_compact_embed_dev(float *compact, const float *full, const int32_t *compact_to_full, int CV,
                                            int V, int D) {
    return rows_by_index<0>("vocab_compact_embed", compact, full, compact_to_full, CV, D, CV, V);
}

MI355_API int mi355_vocab_update_full_dev(float *full, const float *compact, const int32_t *compact_to_full, int CV,
                                          int V, int D) {
    return rows_by_index<1>("vocab_update_full", full, compact, compact_to_full, CV, D, V, CV);
}

MI355_API int mi355_vocab_scatter_grads_dev(float *full_grad, const float *compact_grad, const int32_t *compact_to_full,
                                            int CV, int V, int D) {
    return rows_by_index<2>("vocab_scatter_grads", full_grad, compact_grad, compact_to_full, CV, D, V, CV);
}
