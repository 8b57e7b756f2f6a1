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
//      workgroup that stages 256 rows at a time in LDS to keep enough loads in flight while one
//      wave performs the ordered adds.
#include "common.h"

#include <rocprim/rocprim.hpp>

namespace {

constexpr int TT = 64;   // tokens per tile
constexpr int TD = 64;   // dims per tile
constexpr int LONG_SEG = 64;    // segments longer than this take the workgroup path
constexpr int STAGE_ROWS = 256;

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
__global__ void prep_keys_kernel(int *keys, int *vals, const int32_t *ids, int N, int V) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n < N) {
        const int id = ids[n];
        keys[n] = (id < 0 || id >= V) ? V : id;   // out-of-range ids sort last and are skipped
        vals[n] = n;
    }
}

// meta[0] = number of segments, meta[1] = number of long segments, meta[2] = number of valid entries
__global__ __launch_bounds__(1024) void plan_kernel(int *rank, int *seg_start, int *long_list, int *meta,
                                                    const int *keys, const int *vals, int N, int V) {
    __shared__ int cnt[1024];
    __shared__ int s_nvalid, s_nlong;
    const int tid = threadIdx.x;
    const int per = (N + 1023) / 1024;
    const int lo = tid * per, hi = min(N, lo + per);
    if (tid == 0) { s_nvalid = N; s_nlong = 0; }
    __syncthreads();
    int c = 0;
    for (int i = lo; i < hi; i++) {
        const int k = keys[i];
        rank[vals[i]] = i;
        const int kp = i > 0 ? keys[i - 1] : -1;
        if (k < V && k != kp) c++;
        if (k >= V && kp < V) s_nvalid = i;   // at most one thread writes
    }
    cnt[tid] = c;
    __syncthreads();
    // exclusive scan of 1024 counts (Hillis-Steele, in place with double sync)
    for (int off = 1; off < 1024; off <<= 1) {
        int v = tid >= off ? cnt[tid - off] : 0;
        __syncthreads();
        cnt[tid] += v;
        __syncthreads();
    }
    int pos = cnt[tid] - c;
    const int nseg = cnt[1023];
    for (int i = lo; i < hi; i++) {
        const int k = keys[i];
        const int kp = i > 0 ? keys[i - 1] : -1;
        if (k < V && k != kp) seg_start[pos++] = i;
    }
    if (tid == 0) seg_start[nseg] = s_nvalid;
    __syncthreads();
    for (int j = tid; j < nseg; j += 1024)
        if (seg_start[j + 1] - seg_start[j] > LONG_SEG) long_list[atomicAdd(&s_nlong, 1)] = j;
    __syncthreads();
    if (tid == 0) { meta[0] = nseg; meta[1] = s_nlong; meta[2] = s_nvalid; }
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
                v4f v = ld4(src);
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

// Short segments: one wave per (segment, 64-float chunk); rows are consecutive in `rows`.
__global__ __launch_bounds__(256) void seg_sum_short_kernel(float *__restrict__ dE, const float *__restrict__ rows,
                                                            const int *__restrict__ seg_start,
                                                            const int *__restrict__ keys, const int *__restrict__ meta,
                                                            int D, int nchunk) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * 4) + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * 4;
    const long units = (long)meta[0] * nchunk;
    for (long u = wave; u < units; u += nwaves) {
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
            for (int j = 0; j < 8; j++) v[j] = src[(size_t)j * D];
#pragma unroll
            for (int j = 0; j < 8; j++) acc += v[j];
            src += (size_t)8 * D;
        }
        for (; r < hi; r++) { acc += *src; src += D; }
        *dst = acc;
    }
}

// Long segments: one workgroup per (segment, 64-float chunk); 16 waves stage 256 rows in LDS,
// wave 0 adds them in order.
__global__ __launch_bounds__(1024) void seg_sum_long_kernel(float *__restrict__ dE, const float *__restrict__ rows,
                                                            const int *__restrict__ seg_start,
                                                            const int *__restrict__ long_list,
                                                            const int *__restrict__ keys, const int *__restrict__ meta,
                                                            int D, int nchunk) {
    __shared__ float stage[STAGE_ROWS][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long units = (long)meta[1] * nchunk;
    for (long u = blockIdx.x; u < units; u += gridDim.x) {
        const int seg = long_list[u / nchunk], ch = (int)(u % nchunk);
        const int lo = seg_start[seg], hi = seg_start[seg + 1];
        const int d = ch * 64 + lane;
        const bool d_ok = d < D;
        const int tok = keys[lo];
        float acc = 0.f;
        if (wave == 0 && d_ok) acc = dE[(size_t)tok * D + d];
        for (int base = lo; base < hi; base += STAGE_ROWS) {
            const int nrow = min(STAGE_ROWS, hi - base);
            float v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int rl = wave * 16 + j;
                v[j] = (rl < nrow && d_ok) ? rows[(size_t)(base + rl) * D + d] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 16; j++) stage[wave * 16 + j][lane] = v[j];
            __syncthreads();
            if (wave == 0)
                for (int rl = 0; rl < nrow; rl++) acc += stage[rl][lane];
            __syncthreads();
        }
        if (wave == 0 && d_ok) dE[(size_t)tok * D + d] = acc;
    }
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
    if (!dE || !dx || !ids) return mi355_fail("embed_scatter_add: NULL pointer");
    if (V <= 0 || D <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("embed_scatter_add: bad shape V=%d D=%d S=%d batch=%d", V, D, S, batch);
    if ((size_t)batch * S > (size_t)1 << 30) return mi355_fail("embed_scatter_add: more than 2^30 positions");
    if (!aligned16(dx) || !aligned16(dE)) return mi355_fail("embed_scatter_add: pointers must be 16-byte aligned");
    const int N = batch * S;
    const int bits = key_bits(V);

    size_t temp_bytes = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, (int *)nullptr, (int *)nullptr, (int *)nullptr,
                                             (int *)nullptr, (size_t)N, 0, bits, g_ctx.stream);
    if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort sizing: %s", hipGetErrorString(e));

    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t nb = al((size_t)N * sizeof(int));
    const size_t off_keys_in = 0, off_vals_in = nb, off_keys = 2 * nb, off_vals = 3 * nb, off_rank = 4 * nb;
    const size_t off_seg = 5 * nb, off_long = off_seg + al((size_t)(N + 1) * sizeof(int));
    const size_t off_meta = off_long + nb, off_temp = off_meta + 256;
    const size_t off_rows = off_temp + al(temp_bytes);
    const size_t total = off_rows + al((size_t)N * D * sizeof(float));
    char *ws = (char *)mi355_ws(total);
    if (!ws) return -1;
    int *keys_in = (int *)(ws + off_keys_in), *vals_in = (int *)(ws + off_vals_in);
    int *keys = (int *)(ws + off_keys), *vals = (int *)(ws + off_vals), *rank = (int *)(ws + off_rank);
    int *seg_start = (int *)(ws + off_seg), *long_list = (int *)(ws + off_long), *meta = (int *)(ws + off_meta);
    float *rows = (float *)(ws + off_rows);

    hipLaunchKernelGGL(prep_keys_kernel, dim3((unsigned)ceil_div((size_t)N, 256)), dim3(256), 0, g_ctx.stream, keys_in,
                       vals_in, ids, N, V);
    LAUNCH_OK("embed_scatter_add prep");
    e = rocprim::radix_sort_pairs(ws + off_temp, temp_bytes, keys_in, keys, vals_in, vals, (size_t)N, 0, bits,
                                  g_ctx.stream);
    if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(1024), 0, g_ctx.stream, rank, seg_start, long_list, meta, keys, vals,
                       N, V);
    LAUNCH_OK("embed_scatter_add plan");
    const int t_tiles = (int)ceil_div((size_t)S, TT);
    const dim3 tgrid((unsigned)(batch * t_tiles), (unsigned)ceil_div((size_t)D, TD));
    if (tgrid.y > 65535) return mi355_fail("embed_scatter_add: D too large");
    hipLaunchKernelGGL(transpose_sorted_kernel, tgrid, dim3(256), 0, g_ctx.stream, rows, dx, rank, D, S, t_tiles);
    LAUNCH_OK("embed_scatter_add transpose");
    const int nchunk = (int)ceil_div((size_t)D, 64);
    const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    hipLaunchKernelGGL(seg_sum_long_kernel, dim3((unsigned)(cu)), dim3(1024), 0, g_ctx.stream, dE, rows, seg_start,
                       long_list, keys, meta, D, nchunk);
    LAUNCH_OK("embed_scatter_add long");
    size_t sblocks = ceil_div((size_t)N * nchunk, 4);
    if (sblocks > (size_t)cu * 16) sblocks = (size_t)cu * 16;
    hipLaunchKernelGGL(seg_sum_short_kernel, dim3((unsigned)sblocks), dim3(256), 0, g_ctx.stream, dE, rows, seg_start,
                       keys, meta, D, nchunk);
    LAUNCH_OK("embed_scatter_add short");
    return 0;
}
