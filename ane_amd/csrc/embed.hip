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
//   1. the (token, position) pairs are put in token order, positions ascending within a token: for up to
//      16 384 positions by counting smaller pairs (no full sort; fused with step 2), beyond that by the
//      rocPRIM stable radix sort;
//   2. dx is transposed through LDS into token-major rows written in that SORTED order, so a
//      segment (all positions of one token) is a run of consecutive rows;
//   3. each segment is summed sequentially starting from the value already in dE — short segments by one
//      wave straight from memory, long segments by a whole workgroup whose other waves stage the rows in LDS
//      while one wave performs the ordered adds; both kinds share one launch so the long chains overlap the
//      many short ones.
#include "common.h"

#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace {

constexpr int TT = 64;   // tokens per tile
constexpr int TD = 64;   // dims per tile
constexpr int LONG_SEG = 96;    // segments longer than this take the workgroup path (a wave sums 96 rows in ~14 us)
constexpr int LCH = 32;             // floats per chunk of a long segment
constexpr int MAX_ORDERED = 256;    // long segments that the segment-sum workgroups order by length
constexpr int MAX_MINE = 32;        // long segments a workgroup streams through its stages without a pause
constexpr int ROWS_PER_WAVE = 16;   // rows a staging wave brings in per stage
constexpr int STAGE_ROWS = 15 * ROWS_PER_WAVE;    // two buffers of 240 rows x 128 B = 60 KiB of LDS

// ---------------------------------------------------------------------------------------------
// Gather
// ---------------------------------------------------------------------------------------------
template <bool VEC_D>
__global__ __launch_bounds__(256) void gather_kernel(float *__restrict__ x, const float *__restrict__ E,
                                                     const int32_t *__restrict__ ids, int V, int D, int S, int N) {
    __shared__ float tile[TT][TD + 1];
    __shared__ int tok[TT];
    const int n0 = blockIdx.x * TT;            // 64 consecutive positions, of one or several sequences
    const int d0 = blockIdx.y * TD;
    const int tid = threadIdx.x;
    if (tid < TT) {
        const int n = n0 + tid;
        int id = -1;
        if (n < N) {
            id = ids[n];
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
    // phase 2: LDS -> channel-first output, lanes along positions; four consecutive positions lie in one sequence
    // when S is a multiple of 4
    {
        const int tq = tid & 15, r0 = tid >> 4;
        const int n4 = n0 + 4 * tq;
        const int i0 = tok[4 * tq], i1 = tok[4 * tq + 1], i2 = tok[4 * tq + 2], i3 = tok[4 * tq + 3];
        const bool all = (i0 >= 0) & (i1 >= 0) & (i2 >= 0) & (i3 >= 0) & ((S & 3) == 0) & (((uintptr_t)x & 15u) == 0);
        const int b4 = n4 / S, t4 = n4 - b4 * S;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int dl = r0 + 16 * k;
            const int d = d0 + dl;
            if (d >= D) continue;
            if (all) {
                v4f v = {tile[4 * tq][dl], tile[4 * tq + 1][dl], tile[4 * tq + 2][dl], tile[4 * tq + 3][dl]};
                st4(x + ((size_t)b4 * D + d) * S + t4, v);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (tok[4 * tq + j] < 0) continue;          // also: positions past the end
                    const int n = n4 + j, bb = n / S;
                    x[((size_t)bb * D + d) * S + (n - bb * S)] = tile[4 * tq + j][dl];
                }
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

// What the segment sums read: seg_list[i] = {first row, end row, token, 0} of segment i (rows = sorted
// positions), long_list = the entries of the long segments, meta[0] / meta[1] = the lengths of the two lists,
// rank[position] = its row.
//
// Large inputs (more than 16 384 positions, or a vocabulary of 2^18 and more): the library sort, then (1) every
// workgroup flags the heads among its 1024 sorted entries (key differs from its predecessor), counts them and
// writes the inverse permutation; (2) every workgroup adds up the counts before its own and writes the positions
// of its heads at that offset (meta[2] = number of in-range entries = end of the last segment); (3) one thread per
// segment writes the list entries.
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
    if (blockIdx.x == 0 && threadIdx.x == 0) meta[1] = 0;
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

// The plan for N <= 16 384 positions and a vocabulary below 2^18, in two launches and without a sort of the whole
// array.  A (token, position) pair is packed into one word, token above position; all words are distinct, and the
// sorted index of a position is the number of words smaller than its own.
//   1. chunk_sort_kernel: every 256 consecutive words are sorted by counting, within their workgroup.
//   2. rank_transpose_kernel: every workgroup (64 consecutive positions) holds all sorted chunks in LDS
//      (64 KiB); 16 lanes share one position and binary-search four chunks each for (a) the number of smaller words = the sorted index, (b) the largest
//      smaller word = the predecessor, which tells whether the position is the first of its token, and (c) the
//      number of words up to the last one of the same token = the end of the segment.  First positions append
//      their segment {first row, end row, token} to the segment list, and to the long list if it is long.  The
//      order of the lists depends on the order of the atomic appends; the sums do not, since a segment is summed
//      by whoever takes it, from its own rows only.  The same workgroup then writes its slab of dx token-major at
//      the rows just found (the transpose of the large path, fused in: the slab's loads are issued before the
//      searches and land meanwhile).
constexpr int SMALL_N = 16384, POS_BITS = 14, CHUNK = 256, CHUNK_PITCH = CHUNK + 1;

// The word the last kernel of a scatter-add leaves for the host: how many runs (form 1, columns: (token, block)
// pairs; form 2, rows: distinct tokens) the input of N positions and row width D had.
__host__ __device__ inline unsigned long long scatter_report(int runs, int N, int D, int form) {
    return ((unsigned long long)(unsigned)form << 60) | ((unsigned long long)((unsigned)D & 0xfffffu) << 40) |
           ((unsigned long long)((unsigned)N & 0xfffffu) << 20) | ((unsigned)runs & 0xfffffu);
}
typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned pack_word(const int32_t *__restrict__ ids, int i, int N, int V) {
    unsigned key = (unsigned)V;                             // padding and out-of-range ids sort last
    if (i < N) {
        const int id = ids[i];
        if (id >= 0 && id < V) key = (unsigned)id;
    }
    return (key << POS_BITS) | (unsigned)i;
}

__global__ __launch_bounds__(CHUNK) void chunk_sort_kernel(unsigned *__restrict__ sorted_chunks, int *__restrict__ meta,
                                                           const int32_t *__restrict__ ids, int N, int V) {
    __shared__ __attribute__((aligned(16))) unsigned sw[CHUNK];
    const int t = threadIdx.x;
    if (blockIdx.x == 0 && t < 2) meta[t] = 0;
    const unsigned w = pack_word(ids, blockIdx.x * CHUNK + t, N, V);
    sw[t] = w;
    __syncthreads();
    int r = 0;
#pragma unroll 8
    for (int j = 0; j < CHUNK; j += 4) {
        const v4u q = *reinterpret_cast<const v4u *>(&sw[j]);
        r += (q.x < w ? 1 : 0) + (q.y < w ? 1 : 0) + (q.z < w ? 1 : 0) + (q.w < w ? 1 : 0);
    }
    sorted_chunks[blockIdx.x * CHUNK + r] = w;
}

__global__ __launch_bounds__(1024) void rank_transpose_kernel(float *__restrict__ rows, v4i *__restrict__ seg_list,
                                                              v4i *__restrict__ long_list, int *__restrict__ meta,
                                                              const unsigned *__restrict__ sorted_chunks,
                                                              const float *__restrict__ dx,
                                                              const int32_t *__restrict__ ids, int N, int V, int nchunks,
                                                              int D, int S) {
    // the sorted chunks (pitch 257: lanes on different chunks, different banks) and, once the rows are known,
    // four 64x64 transpose tiles share the same LDS
    __shared__ union {
        unsigned sc[(SMALL_N / CHUNK) * CHUNK_PITCH];
        float tile[4][TD][TT + 1];
    } sh;
    __shared__ int dst_row[TT];
    __shared__ int nh, nl, base_h, base_l;
    const int t = threadIdx.x;
    // this workgroup: 64 consecutive positions (of one or several sequences); their columns of dx are independent of
    // the ranks, so the loads of the first three groups of four tiles (768 columns of D) go out now and land while
    // the ranks are computed.  A lane moves four consecutive positions; with S a multiple of 4 they lie in one
    // sequence and are one 128-bit load.
    const int n0 = blockIdx.x * TT;
    const int tq4 = t >> 8, ltq = t & 15, lr0 = (t & 255) >> 4;        // quarter; lane along positions; row group
    const int n4 = n0 + 4 * ltq;
    const bool vec_ld = (S & 3) == 0 && n4 + 3 < N && ((uintptr_t)dx & 15u) == 0;
    const int b4 = n4 / S, t4 = n4 - b4 * S;
    v4f pre0[4], pre1[4], pre2[4];
    {
        auto issue = [&](int g, v4f (&pre)[4]) {
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                const int d = (g * 4 + tq4) * TD + lr0 + 16 * kk;
                pre[kk] = (vec_ld && d < D) ? ld4_nt(dx + ((size_t)b4 * D + d) * S + t4) : v4f{0.f, 0.f, 0.f, 0.f};
            }
        };
        issue(0, pre0); issue(1, pre1); issue(2, pre2);
    }
    {
        v4u q[SMALL_N / 4096];                                  // all loads first, then the LDS writes
#pragma unroll
        for (int i = 0; i < SMALL_N / 4096; i++) {
            const int j = i * 4096 + t * 4;
            q[i] = j < nchunks * CHUNK ? *reinterpret_cast<const v4u *>(&sorted_chunks[j]) : v4u{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < SMALL_N / 4096; i++) {
            const int j = i * 4096 + t * 4;
            unsigned *dst = sh.sc + (j / CHUNK) * CHUNK_PITCH + (j % CHUNK);
            dst[0] = q[i].x; dst[1] = q[i].y; dst[2] = q[i].z; dst[3] = q[i].w;
        }
    }
    // 16 lanes per position
    const int k = t & 15, tl_mine = t >> 4;
    const int e = min(n0 + tl_mine, N);                         // N: packs as padding, never written
    const bool live = e < N;
    const unsigned w = pack_word(ids, e, N, V);
    const unsigned key = w >> POS_BITS;
    if (t == 0) nh = nl = 0;
    __syncthreads();
    // the four searches of a lane are independent chains of LDS reads and run interleaved; a chunk index past the
    // end is searched as chunk 0 and not counted
    constexpr int PER_LANE = SMALL_N / CHUNK / 16;
    const unsigned *chp[PER_LANE];
    bool okc[PER_LANE];
#pragma unroll
    for (int m = 0; m < PER_LANE; m++) {
        okc[m] = k + 16 * m < nchunks;
        chp[m] = sh.sc + (okc[m] ? k + 16 * m : 0) * CHUNK_PITCH;
    }
    auto count_below = [&](unsigned x, int (&p)[PER_LANE]) {      // per chunk: number of words < x
#pragma unroll
        for (int m = 0; m < PER_LANE; m++) p[m] = 0;
#pragma unroll
        for (int st = CHUNK / 2; st >= 1; st >>= 1) {
#pragma unroll
            for (int m = 0; m < PER_LANE; m++)
                if (chp[m][p[m] + st - 1] < x) p[m] += st;
        }
#pragma unroll
        for (int m = 0; m < PER_LANE; m++) p[m] += chp[m][p[m]] < x ? 1 : 0;
    };
    int p[PER_LANE];
    count_below(w, p);
    int below = 0;
    unsigned pred1 = 0;                                         // largest smaller word + 1, or 0 if there is none
#pragma unroll
    for (int m = 0; m < PER_LANE; m++)
        if (okc[m]) {
            below += p[m];
            if (p[m] > 0) pred1 = max(pred1, chp[m][p[m] - 1] + 1u);
        }
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) {
        below += __shfl_xor(below, m, 64);
        pred1 = max(pred1, (unsigned)__shfl_xor((int)pred1, m, 64));
    }
    // the 16 lanes of a position agree on whether it is the first of its token; only then is the end searched
    const bool first = e < N && key < (unsigned)V && (pred1 == 0 || ((pred1 - 1u) >> POS_BITS) != key);
    int upto = 0;
    if (first) {
        // words up to the last one of this token = words below the first word of the next token (no overflow:
        // a first position has key < V < 2^18)
        count_below(((key + 1u) << POS_BITS), p);
#pragma unroll
        for (int m = 0; m < PER_LANE; m++) upto += okc[m] ? p[m] : 0;
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) upto += __shfl_xor(upto, m, 64);
    }
    // one append per workgroup and list: the heads take their places within the workgroup through LDS, and one
    // 64-bit atomic moves both list lengths (meta[0] is its low word, meta[1] its high word).  The appends of all
    // workgroups queue up on that address, so nobody waits for the answer before the transpose is done.
    const bool mine = k == 0 && live;
    const bool head = mine && first;
    const bool is_long = head && upto - below > LONG_SEG;
    int ih = 0, il = 0;
    if (head) ih = atomicAdd(&nh, 1);
    if (is_long) il = atomicAdd(&nl, 1);
    if (k == 0) dst_row[tl_mine] = live ? below : -1;
    __syncthreads();                                            // also: the chunks in LDS are no longer needed
    unsigned long long old_len = 0;
    if (t == 0 && nh)
        old_len = atomicAdd(reinterpret_cast<unsigned long long *>(meta),
                            ((unsigned long long)(unsigned)nl << 32) | (unsigned)nh);

    // dx [b][D][t0..t0+63] -> rows[dst_row][D]: each quarter of the workgroup moves one 64x64 tile at a time
    {
        const bool d_vec = (D & 3) == 0;
        float(*tile)[TT + 1] = sh.tile[tq4];
        auto move_group = [&](int d0, const v4f *pre) {          // pre: this lane's four loads, already issued
            if (d0 < D) {   // lanes along positions
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    const int dl = lr0 + 16 * kk, d = d0 + dl;
                    if (d >= D) continue;
                    if (vec_ld) {
                        const v4f v = pre ? pre[kk] : ld4_nt(dx + ((size_t)b4 * D + d) * S + t4);
                        tile[dl][4 * ltq + 0] = v.x; tile[dl][4 * ltq + 1] = v.y;
                        tile[dl][4 * ltq + 2] = v.z; tile[dl][4 * ltq + 3] = v.w;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int n = n4 + j;
                            if (n < N) {
                                const int bb = n / S;
                                tile[dl][4 * ltq + j] = dx[((size_t)bb * D + d) * S + (n - bb * S)];
                            }
                        }
                    }
                }
            }
            __syncthreads();
            if (d0 < D) {   // lanes along d
                const int dq = ltq, r0 = lr0;
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    const int tl = r0 + 16 * kk;
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
            __syncthreads();
        };
        // the groups whose loads went out before the ranks were computed, then the rest (uniform trip counts)
        if (0 * 4 * TD < D) move_group((0 * 4 + tq4) * TD, pre0);
        if (1 * 4 * TD < D) move_group((1 * 4 + tq4) * TD, pre1);
        if (2 * 4 * TD < D) move_group((2 * 4 + tq4) * TD, pre2);
        for (int g = 3; g * 4 * TD < D; g++) move_group((g * 4 + tq4) * TD, nullptr);
    }
    if (t == 0) {
        base_h = (int)(old_len & 0xffffffffu);
        base_l = (int)(old_len >> 32);
    }
    __syncthreads();
    if (head) {
        const v4i entry = {below, upto, (int)key, 0};
        seg_list[base_h + ih] = entry;
        if (is_long) long_list[base_l + il] = entry;
    }
}

// Large plan, last launch: one thread per segment writes its list entry; the long ones also go to the long list.
__global__ __launch_bounds__(PLAN_T) void plan_list_kernel(v4i *__restrict__ seg_list, v4i *__restrict__ long_list,
                                                           int *__restrict__ meta, const int *__restrict__ seg_start,
                                                           const int *__restrict__ keys) {
    const int seg = blockIdx.x * PLAN_T + threadIdx.x;
    if (seg >= meta[0]) return;
    const int lo = seg_start[seg], hi = seg_start[seg + 1];
    const v4i entry = {lo, hi, keys[lo], 0};
    seg_list[seg] = entry;
    if (hi - lo > LONG_SEG) long_list[atomicAdd(&meta[1], 1)] = entry;
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
    const bool s_vec = (S & 3) == 0 && ((uintptr_t)dx & 15u) == 0;
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
//  * the first `long_blocks` workgroups take the LONG segments (more than LONG_SEG rows).  Every one of them
//    orders the long list by length (longest first, so that the longest chain of dependent adds starts at once);
//    workgroup (x, chunk) takes one entry per pass over the long_x columns and sums the 32-float chunk of each,
//    all of them as one stream of stages.  Waves 1-15 stage the rows, 240 per stage: two rows per load instruction, eight loads per lane, three stages in
//    flight in registers (720 rows, enough to cover the memory latency at the rate the adds consume them), and
//    write them into one of two LDS buffers.  Wave 0 adds the rows of the other buffer in order, with the LDS
//    reads of the next 16 rows issued ahead of the adds of the current 16, so the dependent adds run back to
//    back.  One barrier per stage.
//  * the others take the short segments: one wave per (segment, 256-float block), rows read straight
//    from memory, eight loads in flight.
// Either way every (row of dE, d) is written by exactly one lane, sequentially in position order,
// starting from the value already in dE.  Rows past the end of a segment are staged as -0.0f, which leaves
// every float unchanged when added (+0.0f would turn a -0.0f sum into +0.0f).
template <bool TREE>
__global__ __launch_bounds__(1024, 8) void seg_sum_kernel(float *__restrict__ dE, const float *__restrict__ rows,
                                                       const v4i *__restrict__ seg_list,
                                                       const int *__restrict__ meta, const v4i *__restrict__ long_list,
                                                       int D, int nchunk, int nchunk_long,
                                                       int long_x, int short_blocks, bool vec,
                                                       unsigned long long *report, int N) {
    __shared__ float stage[2][STAGE_ROWS][LCH];
    __shared__ v4i ent[MAX_ORDERED];
    __shared__ short order[MAX_ORDERED];
    __shared__ int it_lo[MAX_MINE], it_hi[MAX_MINE], it_tok[MAX_MINE];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nseg = meta[0];
    const int long_blocks = long_x * nchunk_long;
    // what the host looks at before it picks a form for the next call of this shape (one 8-byte store to host memory)
    if (report && blockIdx.x == 0 && threadIdx.x == 0) *report = scatter_report(nseg, N, D, 2);
    if ((int)blockIdx.x < long_blocks) {
        const int ch = blockIdx.x % nchunk_long, x0 = blockIdx.x / nchunk_long;
        const int col = lane & (LCH - 1), sub = lane / LCH;      // a load instruction covers rows r and r+1
        const int d = ch * LCH + col;
        const bool d_ok = d < D;
        // the long list in LDS, longest first (ties: smaller first row); beyond MAX_ORDERED entries, as listed.
        // The entries are fetched before their number is known (the list has room for MAX_ORDERED and more), so
        // that the two loads travel together.
        v4i mine = {0, 0, 0, 0};
        if (threadIdx.x < MAX_ORDERED) mine = long_list[threadIdx.x];
        const int nlong = meta[1];
        if (x0 >= nlong) return;
        const int nord = min(nlong, MAX_ORDERED);
        if ((int)threadIdx.x < nord) ent[threadIdx.x] = mine;
        __syncthreads();
        if ((int)threadIdx.x < nord && nlong <= MAX_ORDERED) {
            const v4i ea = ent[threadIdx.x];
            const int la = ea.y - ea.x;
            int before = 0;
            for (int b = 0; b < nord; b++) {
                const v4i eb = ent[b];
                const int lb = eb.y - eb.x;
                before += (lb > la || (lb == la && eb.x < ea.x)) ? 1 : 0;
            }
            order[before] = (short)threadIdx.x;
        }
        __syncthreads();
        // This workgroup's entries of that order: one per pass over the columns, the passes running alternately
        // up and down the columns so that the column with the longest entry gets the shortest of the next two
        // passes.  MAX_MINE of them at a time go through the stages back to back, as one stream: the staging waves
        // run ahead over the boundary between two segments, so a segment of one stage costs one stage.
        const int full_passes = nlong / long_x, rest = nlong - full_passes * long_x;
        const int my_off_last = (full_passes & 1) ? long_x - 1 - x0 : x0;
        const int n_all = full_passes + (my_off_last < rest ? 1 : 0);
        for (int first = 0; first < n_all; first += MAX_MINE) {
            const int n_my = min(MAX_MINE, n_all - first);
            if ((int)threadIdx.x < n_my) {
                const int m = first + threadIdx.x;
                const int idx = m * long_x + ((m & 1) ? long_x - 1 - x0 : x0);
                const v4i e = nlong <= MAX_ORDERED ? ent[order[idx]] : long_list[idx];
                it_lo[threadIdx.x] = e.x; it_hi[threadIdx.x] = e.y; it_tok[threadIdx.x] = e.z;
            }
            __syncthreads();
            int nstages = 0;
            for (int k = 0; k < n_my; k++) nstages += (it_hi[k] - it_lo[k] + STAGE_ROWS - 1) / STAGE_ROWS;
            nstages = __builtin_amdgcn_readfirstlane(nstages);
            // The two roles run separate loops (so that neither carries the other's registers) and meet at one
            // barrier per stage: barrier g tells wave 0 that buffer g&1 is complete, and tells the staging waves
            // that wave 0 has finished with the other buffer.
            if (wave == 0) {
                // this wave's chain of dependent adds sets the time of the launch: it goes first whenever it can issue
                __builtin_amdgcn_s_setprio(3);
                auto old_value = [&](int k) {           // what dE holds for entry k (0 beyond the last entry)
                    return (k < n_my && d_ok) ? dE[(size_t)it_tok[k] * D + d] : 0.f;
                };
                // the old value of an entry is loaded while the entry before it is summed (a short entry is over before
                // a load issued at its own start would be back)
                float acc = old_value(0), acc1 = old_value(1);
                int g = 0;                                  // stage count over all entries: selects the buffer
                for (int k = 0; k < n_my; k++) {
                    const int lo = __builtin_amdgcn_readfirstlane(it_lo[k]), hi = __builtin_amdgcn_readfirstlane(it_hi[k]);
                    for (int base = lo; base < hi; base += STAGE_ROWS, g++) {
                        float(*buf)[LCH] = stage[g & 1];
                        __syncthreads();
                        if constexpr (TREE) {
                            float t[30];
#pragma unroll
                            for (int q = 0; q < 30; q++) t[q] = buf[q][col];
#pragma unroll
                            for (int q = 0; q < 30; q++) acc += t[q];
                        } else {
                            const int nrow = min(STAGE_ROWS, hi - base);
                            if (nrow == STAGE_ROWS) {
                                float t[2][16];
#pragma unroll
                                for (int j = 0; j < 16; j++) t[0][j] = buf[j][col];
#pragma unroll
                                for (int b = 0; b < STAGE_ROWS / 16; b++) {
                                    if (b + 1 < STAGE_ROWS / 16) {
#pragma unroll
                                        for (int j = 0; j < 16; j++) t[(b + 1) & 1][j] = buf[(b + 1) * 16 + j][col];
                                    }
                                    // without the fences the compiler moves the reads down to 8 rows ahead of
                                    // their adds, which exposes part of the LDS latency (1.42 us per stage; 1.13 with)
                                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                                    for (int j = 0; j < 16; j++) acc += t[b & 1][j];
                                    __builtin_amdgcn_sched_barrier(0);
                                }
                            } else {
                                for (int rl = 0; rl < nrow; rl += 16) {      // rows past nrow hold -0.0f
                                    float t[16];
#pragma unroll
                                    for (int j = 0; j < 16; j++) t[j] = buf[rl + j][col];
#pragma unroll
                                    for (int j = 0; j < 16; j++) acc += t[j];
                                }
                            }
                        }
                    }
                    // the entry is done: store it, go on with the next one
                    if (sub == 0 && d_ok) dE[(size_t)it_tok[k] * D + d] = acc;
                    acc = acc1;
                    acc1 = old_value(k + 2);
                }
                __builtin_amdgcn_s_setprio(0);
            } else {
                float g0[8], g1[8], g2[8];
                int fk = 0, fs = 0;                         // entry and stage of the next fetch
                auto fetch_next = [&](float (&g)[8]) {
                    if (fk >= n_my) return;                 // past the last stage: the registers are not used again
                    const int lo = __builtin_amdgcn_readfirstlane(it_lo[fk]), hi = __builtin_amdgcn_readfirstlane(it_hi[fk]);
                    const int r0 = lo + fs * STAGE_ROWS + (wave - 1) * ROWS_PER_WAVE + sub;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const int r = r0 + 2 * j;
                        g[j] = (r < hi && d_ok) ? __builtin_nontemporal_load(rows + (size_t)r * D + d) : -0.0f;
                    }
                    fs++;
                    if (lo + fs * STAGE_ROWS >= hi) { fk++; fs = 0; }
                };
                auto put = [&](float (&g)[8], int gi) {
                    if (gi >= nstages) return;
                    float(*buf)[LCH] = stage[gi & 1];
                    if constexpr (TREE) {
                        // fixed tree instead of the reference's chain (opt-in, "scatter_tree" knob): every lane
                        // sums its 8 rows of the stage in order, wave 0 adds the 30 partial rows in order.
                        // Deterministic, 8x shorter chain, but rounded differently from the CPU loop.
                        float p = g[0];
#pragma unroll
                        for (int j = 1; j < 8; j++) p += g[j];
                        buf[(wave - 1) * 2 + sub][col] = p;
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; j++) buf[(wave - 1) * ROWS_PER_WAVE + sub + 2 * j][col] = g[j];
                    }
                    fetch_next(g);
                    __syncthreads();
                };
                fetch_next(g0);
                fetch_next(g1);
                fetch_next(g2);
                for (int gi = 0; gi < nstages; gi += 3) {
                    put(g0, gi);
                    put(g1, gi + 1);
                    put(g2, gi + 2);
                }
            }
            __syncthreads();             // the next round rewrites the table and reuses buffer 0
        }
        return;
    }
    // short segments: one wave per (segment, block of 256 columns), 128 bits per lane (64 columns and 32 bits
    // per lane when D is not a multiple of 4)
    const int gw = __builtin_amdgcn_readfirstlane(((int)blockIdx.x - long_blocks) * 16 + wave);
    const int nwaves = short_blocks * 16;
    const long units = (long)nseg * nchunk;
    for (long u = gw; u < units; u += nwaves) {
        const int seg = (int)(u / nchunk), ch = (int)(u - (long)seg * nchunk);
        const v4i e = seg_list[seg];
        const int lo = __builtin_amdgcn_readfirstlane(e.x), hi = __builtin_amdgcn_readfirstlane(e.y);
        if (hi - lo > LONG_SEG) continue;
        const int tok = __builtin_amdgcn_readfirstlane(e.z);
        if (vec) {
            const int d = ch * 256 + lane * 4;
            if (d >= D) continue;
            float *dst = dE + (size_t)tok * D + d;
            const float *src = rows + (size_t)lo * D + d;
            v4f acc = ld4(dst);
            int r = lo;
            for (; r + 8 <= hi; r += 8) {
                v4f v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = ld4_nt(src + (size_t)j * D);
#pragma unroll
                for (int j = 0; j < 8; j++) acc += v[j];
                src += (size_t)8 * D;
            }
            for (; r < hi; r++) { acc += ld4_nt(src); src += D; }
            st4(dst, acc);
        } else {
            const int d = ch * 64 + lane;
            if (d >= D) continue;
            float *dst = dE + (size_t)tok * D + d;
            const float *src = rows + (size_t)lo * D + d;
            float acc = *dst;
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

// Vocabulary map (training/training_dynamic/cpu_ops.h:102-126): mark the tokens that occur in the data, number
// the marked ones in ascending token order.
__global__ __launch_bounds__(256) void vocab_fill_kernel(int *__restrict__ f2c, int V) {
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v < V) f2c[v] = -1;
}
__global__ __launch_bounds__(256) void vocab_mark_kernel(int *__restrict__ f2c, const uint16_t *__restrict__ data,
                                                         size_t n, int V) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const int tok = data[i];
        if (tok < V) f2c[tok] = 0;                 // every writer stores the same value
    }
}
// one workgroup walks the vocabulary 1024 tokens at a time (a one-time step of the loops' start-up)
__global__ __launch_bounds__(PLAN_T) void vocab_number_kernel(int *__restrict__ f2c, int *__restrict__ c2f,
                                                              int *__restrict__ cv_out, int V) {
    __shared__ int lds[PLAN_T / 64];
    int base = 0;
    for (int v0 = 0; v0 < V; v0 += PLAN_T) {
        const int v = v0 + threadIdx.x;
        const int used = (v < V && f2c[v] == 0) ? 1 : 0;
        int total;
        const int ex = block_excl_scan_1024(used, lds, total);
        if (v < V) f2c[v] = used ? base + ex : -1;
        if (used) c2f[base + ex] = v;
        base += total;
    }
    if (threadIdx.x == 0) *cv_out = base;
}
// ids of the full vocabulary -> ids of the compact one (train.m:403); an id outside [0,V) or unused becomes -1
__global__ __launch_bounds__(256) void vocab_remap_kernel(int32_t *__restrict__ out, const int32_t *__restrict__ ids,
                                                          const int *__restrict__ f2c, size_t n, int V) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int id = ids[i];
    out[i] = (id >= 0 && id < V) ? f2c[id] : -1;
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

#include "embed_cols.h"

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
    if ((size_t)batch * S > (size_t)1 << 30) return mi355_fail("embed_gather: more than 2^30 positions");
    const int N = batch * S;
    const dim3 grid((unsigned)ceil_div((size_t)N, TT), (unsigned)ceil_div((size_t)D, TD));
    if (grid.y > 65535) return mi355_fail("embed_gather: D too large");
    const bool vec_d = (D % 4 == 0) && aligned16(E) && aligned16(x);
    if (vec_d) hipLaunchKernelGGL((gather_kernel<true>), grid, dim3(256), 0, g_ctx.stream, x, E, ids, V, D, S, N);
    else hipLaunchKernelGGL((gather_kernel<false>), grid, dim3(256), 0, g_ctx.stream, x, E, ids, V, D, S, N);
    LAUNCH_OK("embed_gather");
    return 0;
}

// Which form takes an input of N positions and row width D.  Both forms give the same bits, so the choice is only a
// matter of time, and what decides it is how the ids repeat: the column form pays one small access to dE per
// (token, block of 8192 positions) and workgroup, the row form a token-major copy of dx whatever the ids are.  Ids of
// text repeat (config 2: 4621 pairs in 16384 positions) and the column form is the default; for ids that hardly
// repeat (drawn uniformly from a large vocabulary) it is up to twice as slow.  The ids are on the device, so the
// library learns from the previous call: the last kernel of either form leaves its number of runs in a word of
// pinned host memory, and the next call of the same N and D compares it with the number at which the two forms
// cost the same (fitted to measurements: column form 10 + 2.5 per block + 4.9 ns per pair, row form
// 24 + 1.4e-6 N D, in us).  The row form reports distinct tokens, not pairs; how many pairs a token makes is taken
// from the last time both forms saw this shape (1.2, config 2's figure, until then), so that a steady input settles
// on one form instead of alternating.
namespace {
unsigned long long *g_report = nullptr;        // pinned, written by the device
unsigned long long *g_report_dev = nullptr;
int g_cols_runs = 0, g_cols_N = 0, g_cols_D = 0;   // the column form's last report
double g_pairs_per_token = 1.2;

unsigned long long *scatter_report_word(void) {
    if (!g_report && !g_ctx.capturing) {
        void *h = nullptr, *d = nullptr;
        if (hipHostMalloc(&h, 64, hipHostMallocMapped) == hipSuccess && hipHostGetDevicePointer(&d, h, 0) == hipSuccess) {
            g_report = (unsigned long long *)h;
            g_report_dev = (unsigned long long *)d;
            *(volatile unsigned long long *)g_report = 0ull;
        } else {
            if (h) (void)hipHostFree(h);
            (void)hipGetLastError();
        }
    }
    return g_report_dev;
}

// 1: columns of dE owned by workgroups, -1: token-major copy and row sums.  `cols_ok`: the column form can take the call.
int scatter_form(int N, int D, bool cols_ok, bool rows_recordable) {
    if (!cols_ok) return -1;
    if (g_ctx.scatter_cols > 0) return 1;
    if (g_ctx.capturing && !rows_recordable) return 1;
    const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    if (N > SMALL_N || (int)ceil_div((size_t)D, cols_per_workgroup(D)) > cu) return -1;
    if (N <= COL_SMALL || !g_report) return 1;
    const unsigned long long w = *(volatile unsigned long long *)g_report;
    const int form = (int)(w >> 60), rD = (int)((w >> 40) & 0xfffffu), rN = (int)((w >> 20) & 0xfffffu);
    const int runs = (int)(w & 0xfffffu);
    if (form == 0 || rN != N || rD != D) return 1;
    const int nblk = (int)ceil_div((size_t)N, CB);
    const double even = std::max((14.0 - 2.5 * nblk + 1.4e-6 * (double)N * D) / 4.9e-3, 0.30 * N);
    if (form == 1) {
        g_cols_runs = runs; g_cols_N = N; g_cols_D = D;
        return runs <= 1.08 * even ? 1 : -1;
    }
    if (g_cols_N == N && g_cols_D == D && runs > 0) {       // both forms have seen this shape: pairs per distinct token
        g_pairs_per_token = std::min(std::max((double)g_cols_runs / runs, 1.0), (double)nblk);
        g_cols_N = 0;                                       // (used once: the next column report refreshes it)
    }
    return runs * std::min(g_pairs_per_token, (double)nblk) <= even ? 1 : -1;
}
}   // namespace

void mi355_free_scatter_report(void) {
    if (g_report) (void)hipHostFree(g_report);
    g_report = g_report_dev = nullptr;
}

MI355_API int mi355_embed_scatter_add_form(int V, int D, int S, int batch, int aligned) {
    if (!mi355_ready("embed_scatter_add_form")) return 0;
    if (V <= 0 || D <= 0 || S <= 0 || batch <= 0 || (size_t)batch * S > (size_t)1 << 30) return 0;
    const int N = batch * S;
    const bool cols_ok = !g_ctx.scatter_tree && g_ctx.scatter_cols >= 0 && ((S % 4 == 0 && aligned) || N <= COL_SMALL) &&
                         V < (1 << (32 - CB_BITS));
    return scatter_form(N, D, cols_ok, N <= SMALL_N && key_bits(V) + POS_BITS <= 32);
}

MI355_API int mi355_embed_scatter_add_dev(float *dE, const float *dx, const int32_t *ids, int V, int D, int S,
                                          int batch) {
    if (!mi355_ready("embed_scatter_add")) return -1;
    if (!dE || !dx || !ids) return mi355_fail("embed_scatter_add: NULL pointer");
    if (V <= 0 || D <= 0 || S <= 0 || batch <= 0)
        return mi355_fail("embed_scatter_add: bad shape V=%d D=%d S=%d batch=%d", V, D, S, batch);
    if ((size_t)batch * S > (size_t)1 << 30) return mi355_fail("embed_scatter_add: more than 2^30 positions");
    // (any 4-byte alignment of dx and dE: a dx that is not 16-byte aligned is read four bytes at a time by the row form,
    // a dE that is not is read and written so)
    const int N = batch * S;
    // Two forms with the same bits (embed_cols.h says what each costs).  Columns of dE owned by workgroups: dx is
    // read where it lies, nothing is copied; chosen where one round of workgroups covers D and the positions are few
    // enough that the small accesses to dE (one per token and workgroup) do not outweigh the copy.
    const bool cols_ok = !g_ctx.scatter_tree && g_ctx.scatter_cols >= 0 &&
                         ((S % 4 == 0 && aligned16(dx)) || N <= COL_SMALL) && V < (1 << (32 - CB_BITS));
    // (the column form also while a graph is recorded, for inputs whose row form would call the library sort, which cannot be)
    unsigned long long *report = scatter_report_word();
    if (scatter_form(N, D, cols_ok, N <= SMALL_N && key_bits(V) + POS_BITS <= 32) > 0)
        return scatter_add_cols(dE, dx, ids, V, D, S, N, report);
    const int bits = key_bits(V);
    const bool small = N <= SMALL_N && bits + POS_BITS <= 32;
    if (!small &&
        !mi355_outside_capture("embed_scatter_add beyond 16384 positions or a vocabulary of 2^18 (its library sort may "
                               "record memset nodes)"))
        return -1;
    const bool vec = (D % 4 == 0) && aligned16(dE);     // the token-major copy is 16-byte aligned: every row start is too
    const int nchunk = (int)ceil_div((size_t)D, vec ? 256 : 64), nchunk_long = (int)ceil_div((size_t)D, LCH);
    const int cu = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    // Every workgroup of the segment-sum launch reserves 64 KiB of LDS, so two fit on a compute unit and the grid is
    // kept near one round of them: a larger grid is started only as fast as earlier workgroups retire.  At most
    // N/(LONG_SEG+1) segments can be long.
    const int max_long = std::max(N / (LONG_SEG + 1) + 1, MAX_ORDERED);
    const int long_x = std::min(max_long, std::max(1, cu / nchunk_long));

    size_t temp_bytes = 0;
    hipError_t e = hipSuccess;
    if (!small) {
        e = rocprim::radix_sort_pairs(nullptr, temp_bytes, rocprim::make_transform_iterator(ids, ClampId{V}),
                                      (int *)nullptr, rocprim::counting_iterator<int>(0), (int *)nullptr, (size_t)N, 0,
                                      bits, g_ctx.stream);
        if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort sizing: %s", hipGetErrorString(e));
    }

    // one workspace, carved in 256-byte steps; the sort's arrays only where the library sort runs
    const int nplan = (int)ceil_div((size_t)N, PLAN_T);
    const int nchunks = (int)ceil_div((size_t)N, CHUNK);
    size_t total = 0;
    auto take = [&total](size_t bytes) {
        const size_t off = total;
        total += (bytes + 255) & ~(size_t)255;
        return off;
    };
    const size_t big = small ? 0 : 1;
    const size_t off_keys = take(big * N * sizeof(int)), off_vals = take(big * N * sizeof(int));
    const size_t off_rank = take(big * N * sizeof(int)), off_seg = take(big * ((size_t)N + 1) * sizeof(int));
    const size_t off_cnt = take(big * nplan * sizeof(int)), off_temp = take(temp_bytes);
    const size_t off_chunks = take(small ? (size_t)nchunks * CHUNK * sizeof(unsigned) : 0);
    const size_t off_meta = take(256), off_long = take((size_t)max_long * sizeof(v4i));
    const size_t off_list = take((size_t)N * sizeof(v4i)), off_rows = take((size_t)N * D * sizeof(float));
    char *ws = (char *)mi355_ws(total);
    if (!ws) return -1;
    int *keys = (int *)(ws + off_keys), *vals = (int *)(ws + off_vals), *rank = (int *)(ws + off_rank);
    int *seg_start = (int *)(ws + off_seg), *blk_count = (int *)(ws + off_cnt);
    int *meta = (int *)(ws + off_meta);
    v4i *long_list = (v4i *)(ws + off_long), *seg_list = (v4i *)(ws + off_list);
    float *rows = (float *)(ws + off_rows);

    if (small) {
        unsigned *sorted_chunks = (unsigned *)(ws + off_chunks);
        hipLaunchKernelGGL(chunk_sort_kernel, dim3(nchunks), dim3(CHUNK), 0, g_ctx.stream, sorted_chunks, meta, ids,
                           N, V);
        hipLaunchKernelGGL(rank_transpose_kernel, dim3((unsigned)ceil_div((size_t)N, TT)), dim3(1024), 0, g_ctx.stream, rows,
                           seg_list, long_list, meta, sorted_chunks, dx, ids, N, V, nchunks, D, S);
    } else {
        e = rocprim::radix_sort_pairs(ws + off_temp, temp_bytes, rocprim::make_transform_iterator(ids, ClampId{V}), keys,
                                      rocprim::counting_iterator<int>(0), vals, (size_t)N, 0, bits, g_ctx.stream);
        if (e != hipSuccess) return mi355_fail("embed_scatter_add: sort: %s", hipGetErrorString(e));
        hipLaunchKernelGGL(plan_flags_kernel, dim3(nplan), dim3(PLAN_T), 0, g_ctx.stream, rank, blk_count, meta,
                           keys, vals, N, V);
        hipLaunchKernelGGL(plan_write_kernel, dim3(nplan), dim3(PLAN_T), 0, g_ctx.stream, seg_start, meta, blk_count,
                           keys, N, V);
        hipLaunchKernelGGL(plan_list_kernel, dim3(nplan), dim3(PLAN_T), 0, g_ctx.stream, seg_list, long_list, meta,
                           seg_start, keys);
    }
    LAUNCH_OK("embed_scatter_add plan");
    if (!small) {
        const int t_tiles = (int)ceil_div((size_t)S, TT);
        const dim3 tgrid((unsigned)(batch * t_tiles), (unsigned)ceil_div((size_t)D, TD));
        if (tgrid.y > 65535) return mi355_fail("embed_scatter_add: D too large");
        hipLaunchKernelGGL(transpose_sorted_kernel, tgrid, dim3(256), 0, g_ctx.stream, rows, dx, rank, D, S, t_tiles);
    }
    LAUNCH_OK("embed_scatter_add transpose");
    const size_t short_blocks = std::min<size_t>(ceil_div((size_t)N * nchunk, 16), (size_t)cu);
    const dim3 sgrid((unsigned)((size_t)long_x * nchunk_long + short_blocks));
    if (g_ctx.scatter_tree)
        hipLaunchKernelGGL(seg_sum_kernel<true>, sgrid, dim3(1024), 0, g_ctx.stream, dE, rows, seg_list, meta,
                           long_list, D, nchunk, nchunk_long, long_x, (int)short_blocks, vec, report, N);
    else
        hipLaunchKernelGGL(seg_sum_kernel<false>, sgrid, dim3(1024), 0, g_ctx.stream, dE, rows, seg_list, meta,
                           long_list, D, nchunk, nchunk_long, long_x, (int)short_blocks, vec, report, N);
    LAUNCH_OK("embed_scatter_add segment sums");
    return 0;
}

MI355_API int mi355_vocab_map_build_dev(int32_t *full_to_compact, int32_t *compact_to_full, int32_t *compact_vocab_dev,
                                        const uint16_t *data, size_t n_tokens, int V) {
    if (!mi355_ready("vocab_map_build")) return -1;
    if (!full_to_compact || !compact_to_full || !compact_vocab_dev || (!data && n_tokens))
        return mi355_fail("vocab_map_build: NULL pointer");
    if (V <= 0) return mi355_fail("vocab_map_build: bad vocabulary size %d", V);
    hipLaunchKernelGGL(vocab_fill_kernel, dim3((unsigned)ceil_div((size_t)V, 256)), dim3(256), 0, g_ctx.stream,
                       full_to_compact, V);
    if (n_tokens) {
        const size_t blocks = std::min<size_t>(ceil_div(n_tokens, 256), 4096);
        hipLaunchKernelGGL(vocab_mark_kernel, dim3((unsigned)blocks), dim3(256), 0, g_ctx.stream, full_to_compact, data,
                           n_tokens, V);
    }
    hipLaunchKernelGGL(vocab_number_kernel, dim3(1), dim3(PLAN_T), 0, g_ctx.stream, full_to_compact, compact_to_full,
                       compact_vocab_dev, V);
    LAUNCH_OK("vocab_map_build");
    return 0;
}

MI355_API int mi355_vocab_remap_dev(int32_t *out, const int32_t *ids, const int32_t *full_to_compact, size_t n, int V) {
    if (!mi355_ready("vocab_remap")) return -1;
    if (!out || !ids || !full_to_compact) return mi355_fail("vocab_remap: NULL pointer");
    if (n == 0 || V <= 0) return mi355_fail("vocab_remap: bad size");
    hipLaunchKernelGGL(vocab_remap_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, g_ctx.stream, out, ids,
                       full_to_compact, n, V);
    LAUNCH_OK("vocab_remap");
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
