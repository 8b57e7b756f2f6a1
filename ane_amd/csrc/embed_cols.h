// embed_cols.h — the ordered scatter-add of the embedding backward with the columns of dE dealt out to the workgroups.
// Included by embed.hip inside its unnamed namespace.
//
// embed_backward (training/stories_cpu_ops.h:123-131, training/training_dynamic/cpu_ops.h:158-164) adds dx[:,t] into
// dE[tok_t] for t ascending: every (row, d) sum has one fixed fp32 order, and the columns d are independent of one
// another.  Here a workgroup owns K adjacent columns of dE (K = 3 for D = 768, 4 for D = 1024, on 256 compute units)
// and sees every position: its part of dx is K whole rows of every sequence, contiguous in the channel-first layout,
// so dx is read once, coalesced, by exactly one workgroup, and nothing is copied token-major through memory.  The
// positions are taken in blocks of CB, in order; within a block they are ranked by (token, position), so a token's
// positions form a run of consecutive ranks, and a lane adds a run to dE[token][d] sequentially: acc = dE;
// acc += x[rank] for the ranks ascending; dE = acc.  Blocks in ascending order and ranks ascending within a run are
// the order of the reference loop, so the result is that loop's bit for bit.
//
// Three launches (one, col_sum_small_kernel, up to 512 positions):
//   1. chunk_sort_blk_kernel: every 256 consecutive (token, position-in-block) words sorted by counting.
//   2. block_rank_kernel: the sorted chunks of a block merged by rank (16 lanes per position, a binary search per
//      chunk): rk[position] = its rank within the block, and the block's runs {token, first rank, length}, long runs
//      listed from the front of the block's task array, short ones from its back.
//   3. col_sum_kernel<K>: per block, every thread writes its values of dx (fetched into registers while the previous
//      block was summed) to LDS at their ranks, so that a run is a contiguous piece of an LDS column.  Waves 0..K-1
//      take the long runs of one column each (128-bit LDS reads issued sixteen adds ahead); the other waves take the
//      short runs, K columns to a lane, the old sums of a lane's runs asked for before the block's values are put in
//      their places.  A long run's result also stays in LDS under its token, so the run of the same token in the
//      next block starts from there and not from a load of dE: the chain of the most frequent token, which bounds
//      the whole operation, goes on from block to block without a trip to memory.  The last thing the launch does is
//      to leave the number of runs it saw where the host finds it before the next call (see scatter_form in embed.hip).
#pragma once

constexpr int CB = 8192, CB_BITS = 13;      // positions per block
constexpr int CB_CHUNKS = CB / CHUNK;       // sorted chunks per block
constexpr int CB_CPL = CB_CHUNKS / 16;      // chunks searched by one lane
constexpr int COL_LONG = 16;                // runs of at least this many positions go to the long-run waves
constexpr int COL_CARRY = 256;              // entries of the token-indexed table that carries long runs' sums to the next block
constexpr int COL_PPT = CB / 1024;          // positions of a block per thread
static_assert(CB_CPL >= 1 && COL_PPT % 4 == 0, "block size");

typedef unsigned v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned pack_word_blk(const int32_t *__restrict__ ids, int i, int N, int V) {
    unsigned key = (unsigned)V;                             // padding and out-of-range ids sort last
    if (i < N) {
        const int id = ids[i];
        if (id >= 0 && id < V) key = (unsigned)id;
    }
    return (key << CB_BITS) | (unsigned)(i & (CB - 1));
}

__global__ __launch_bounds__(CHUNK) void chunk_sort_blk_kernel(unsigned *__restrict__ sorted_chunks,
                                                               unsigned long long *__restrict__ cnt, int nblk,
                                                               const int32_t *__restrict__ ids, int N, int V) {
    __shared__ __attribute__((aligned(16))) unsigned sw[CHUNK];
    const int t = threadIdx.x;
    if (blockIdx.x == 0)
        for (int i = t; i < nblk; i += CHUNK) cnt[i] = 0ull;
    const unsigned w = pack_word_blk(ids, blockIdx.x * CHUNK + t, N, V);
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

// One workgroup = 64 consecutive positions of one block, 16 lanes per position, one chunk of the block per lane.
// rk[position] = its rank within its block.
// tasks[block][...] = {token, start | length << 16}; cnt[block] = number of long runs (low word) and of short runs.
__global__ __launch_bounds__(1024) void block_rank_kernel(uint16_t *__restrict__ rk, v2u *__restrict__ tasks,
                                                          unsigned long long *__restrict__ cnt,
                                                          const unsigned *__restrict__ sorted_chunks,
                                                          const int32_t *__restrict__ ids, int N, int V, int nchunks) {
    __shared__ unsigned sc[CB_CHUNKS * CHUNK_PITCH];
    __shared__ int n_long, n_short, base_long, base_short;
    const int t = threadIdx.x;
    const int n0 = blockIdx.x * 64, blk = n0 >> CB_BITS, c0 = blk * CB_CHUNKS;
#pragma unroll
    for (int i = 0; i < CB / 4096; i++) {
        const int j = i * 4096 + 4 * t;
        const v4u q = (c0 + j / CHUNK < nchunks) ? *reinterpret_cast<const v4u *>(&sorted_chunks[(size_t)c0 * CHUNK + j])
                                                 : v4u{0, 0, 0, 0};
        unsigned *dst = sc + (j / CHUNK) * CHUNK_PITCH + (j % CHUNK);
        dst[0] = q.x; dst[1] = q.y; dst[2] = q.z; dst[3] = q.w;
    }
    const int k = t & 15, tl = t >> 4;
    const int e = n0 + tl;
    const bool live = e < N;
    const unsigned w = pack_word_blk(ids, e, N, V);
    const unsigned key = w >> CB_BITS;
    if (t == 0) n_long = n_short = 0;
    __syncthreads();
    // a lane's chunks: k, k + 16, ...; one past the end is searched as chunk 0 and not counted.  The searches of a
    // lane are independent chains of LDS reads and run interleaved.
    const unsigned *chp[CB_CPL];
    bool okc[CB_CPL];
#pragma unroll
    for (int m = 0; m < CB_CPL; m++) {
        okc[m] = c0 + k + 16 * m < nchunks;
        chp[m] = sc + (okc[m] ? k + 16 * m : 0) * CHUNK_PITCH;
    }
    auto count_below = [&](unsigned x, int (&p)[CB_CPL]) {       // per chunk: number of words < x
#pragma unroll
        for (int m = 0; m < CB_CPL; m++) p[m] = 0;
#pragma unroll
        for (int st = CHUNK / 2; st >= 1; st >>= 1) {
#pragma unroll
            for (int m = 0; m < CB_CPL; m++)
                if (chp[m][p[m] + st - 1] < x) p[m] += st;
        }
#pragma unroll
        for (int m = 0; m < CB_CPL; m++) p[m] += chp[m][p[m]] < x ? 1 : 0;
    };
    int p[CB_CPL];
    int below = 0;
    unsigned pred1 = 0;                                         // largest smaller word + 1, or 0 if there is none
    count_below(w, p);
#pragma unroll
    for (int m = 0; m < CB_CPL; m++)
        if (okc[m]) {
            below += p[m];
            if (p[m] > 0) pred1 = max(pred1, chp[m][p[m] - 1] + 1u);
        }
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) {
        below += __shfl_xor(below, m, 64);
        pred1 = max(pred1, (unsigned)__shfl_xor((int)pred1, m, 64));
    }
    const bool first = live && key < (unsigned)V && (pred1 == 0 || ((pred1 - 1u) >> CB_BITS) != key);
    int upto = 0;
    if (first) {                                                // uniform over the 16 lanes of a position
        count_below((key + 1u) << CB_BITS, p);                  // no overflow: key < V < 2^(32 - CB_BITS)
#pragma unroll
        for (int m = 0; m < CB_CPL; m++) upto += okc[m] ? p[m] : 0;
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) upto += __shfl_xor(upto, m, 64);
    }
    const bool head = k == 0 && first;
    const int len = upto - below;
    const bool is_long = head && len >= COL_LONG;
    int idx = 0;
    if (head) idx = atomicAdd(is_long ? &n_long : &n_short, 1);
    if (k == 0 && live) rk[e] = (uint16_t)below;
    __syncthreads();
    if (t == 0) {
        unsigned long long old = 0;
        if (n_long | n_short)
            old = atomicAdd(&cnt[blk], ((unsigned long long)(unsigned)n_short << 32) | (unsigned)n_long);
        base_long = (int)(old & 0xffffffffu);
        base_short = (int)(old >> 32);
    }
    __syncthreads();
    if (head) {
        const v2u entry = {key, (unsigned)below | ((unsigned)len << 16)};
        tasks[(size_t)blk * CB + (is_long ? base_long + idx : CB - 1 - (base_short + idx))] = entry;
    }
}


// acc + x[start] + x[start+1] + ... + x[start+len-1], in that order, from one LDS column.  The column is read in
// aligned groups of eight; what lies outside the run in the first and in the last groups is replaced by -0, which
// leaves every float as it is.  Runs of 32 and more go through a loop of three groups per trip whose reads are
// issued two groups (sixteen adds) ahead of their use, in three register sets that take turns, so the wave issues
// little else than the adds.
__device__ __forceinline__ float long_chain(float acc, const float *xc, int start, int len) {
    const int a0 = start & ~3, lead = start - a0, n = lead + len;       // the run is [lead, n) counted from a0
    const v4f *p = reinterpret_cast<const v4f *>(xc + a0);
    auto add8 = [&](const v4f &c0, const v4f &c1) {
        acc += c0.x; acc += c0.y; acc += c0.z; acc += c0.w;
        acc += c1.x; acc += c1.y; acc += c1.z; acc += c1.w;
    };
    auto masked = [&](const v4f &c0, const v4f &c1, int lo, int hi) {
        acc += (0 >= lo && 0 < hi) ? c0.x : -0.0f; acc += (1 >= lo && 1 < hi) ? c0.y : -0.0f;
        acc += (2 >= lo && 2 < hi) ? c0.z : -0.0f; acc += (3 >= lo && 3 < hi) ? c0.w : -0.0f;
        acc += 4 < hi ? c1.x : -0.0f; acc += 5 < hi ? c1.y : -0.0f;
        acc += 6 < hi ? c1.z : -0.0f; acc += 7 < hi ? c1.w : -0.0f;
    };
    v4f a0_ = p[0], a1_ = p[1];
    masked(a0_, a1_, lead, n);
    int pos = 8;                                                // elements before pos are added
    if (pos + 24 <= n) {
        v4f b0 = p[4], b1 = p[5];                               // group pos + 8
        a0_ = p[2]; a1_ = p[3];                                 // group pos
        v4f c0, c1;
        // at the top: a = group pos, b = group pos + 8, both on their way or here
        for (; pos + 24 <= n; pos += 24) {
            c0 = p[pos / 4 + 4]; c1 = p[pos / 4 + 5];           // group pos + 16
            __builtin_amdgcn_sched_barrier(0);
            add8(a0_, a1_);
            __builtin_amdgcn_sched_barrier(0);
            a0_ = p[pos / 4 + 6]; a1_ = p[pos / 4 + 7];         // group pos + 24
            __builtin_amdgcn_sched_barrier(0);
            add8(b0, b1);
            __builtin_amdgcn_sched_barrier(0);
            b0 = p[pos / 4 + 8]; b1 = p[pos / 4 + 9];           // group pos + 32
            __builtin_amdgcn_sched_barrier(0);
            add8(c0, c1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (; pos < n; pos += 8) {                                 // fewer than 24 are left (more for a run that never had 32)
        a0_ = p[pos / 4]; a1_ = p[pos / 4 + 1];
        masked(a0_, a1_, 0, n - pos);
    }
    return acc;
}

// K adjacent floats of a row of dE, moved as one access (4-byte aligned)
template <int K>
struct __attribute__((packed, aligned(4))) ColVec { float f[K]; };

template <int K, bool FULL>                                     // FULL: D is a multiple of K, every workgroup has K columns
__global__ __launch_bounds__(1024) void col_sum_kernel(float *dE, const float *__restrict__ dx,
                                                       const v2u *__restrict__ tasks,
                                                       const unsigned long long *__restrict__ cnt,
                                                       const uint16_t *__restrict__ rk, int N, int D, int S, int nblk,
                                                       unsigned long long *report) {
    constexpr int XP = CB + 48;                                 // a column in LDS, with room for the reads issued ahead
    constexpr int NSL = (16 - K) * 64;                          // lanes that take short runs
    constexpr int RPL = 4;                                      // runs of a block whose old sums a lane asks for in one go
    __shared__ __attribute__((aligned(16))) float xs[K][XP];
    __shared__ unsigned long long carry[2][K][COL_CARRY];       // {token, bits of the sum} of the long runs of a block
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int d0 = xcd_remap(blockIdx.x, gridDim.x) * K;        // neighbouring columns on one XCD: they share lines of dE
    const int kv = FULL ? K : min(K, D - d0);                   // columns of this workgroup that exist
    const bool hot = wave < K;                                  // wave d < K: the long runs of column d0 + d
    const int sl = (wave - K) * 64 + lane;                      // the other lanes: short runs, all K columns each

    // What a thread fetches ahead for a block: its positions' values of dx and ranks, the numbers of runs, and the
    // first runs it will take.
    struct Pre {
        v4f px[K][COL_PPT / 4];
        unsigned prk[COL_PPT / 2];
        unsigned long long pc;
        v2u pd[RPL];
    };
    Pre o;
    auto fetch_runs = [&](Pre &o, int blk) __attribute__((always_inline)) {
        const v2u *tb = tasks + (size_t)blk * CB;
        o.pc = cnt[blk];
#pragma unroll
        for (int i = 0; i < RPL; i++) o.pd[i] = tb[hot ? lane + 64 * i : CB - 1 - (sl + NSL * i)];
    };
    auto fetch_values = [&](Pre &o, int blk) __attribute__((always_inline)) {
        const int p0 = blk * CB + COL_PPT * t;
#pragma unroll
        for (int q = 0; q < COL_PPT / 4; q++) {
            const int p = p0 + 4 * q < N ? p0 + 4 * q : 0;       // (past the end: any address; the values are not used)
            const int b = p / S, s = p - b * S;
#pragma unroll
            for (int d = 0; d < K; d++)
                o.px[d][q] = ld4_nt(dx + ((size_t)b * D + d0 + (d < kv ? d : 0)) * S + s);
        }
        const unsigned *rp = reinterpret_cast<const unsigned *>(rk + (size_t)blk * CB + COL_PPT * t);
#pragma unroll
        for (int q = 0; q < COL_PPT / 2; q++) o.prk[q] = rp[q];
    };
    float *dcol = dE + d0 + (hot ? wave : 0);
    const float *xc = &xs[hot ? wave : 0][0];
    const bool col_ok = wave < kv;

    // The long runs of the first block start from dE itself, and the chain of the most frequent token is what the
    // launch waits for.  The waves that take them are the first of the workgroup to issue anything, so their piece of
    // the run list is back within half a microsecond; they ask for their old sums then, ahead of every value of dx,
    // and have them when the block is in its place (asked for with everybody else's, behind 25 MB of dx, they come
    // 2.4 us after that for the median workgroup and 4.8 us for the slowest).
    fetch_runs(o, 0);
    float h0 = 0.f;
    if (hot) {
        const bool hv = col_ok && lane < (int)(o.pc & 0xffffffffu);
        h0 = dcol[(size_t)(hv ? o.pd[0].x : 0u) * D];
    }
    fetch_values(o, 0);
    int runs = 0;
    for (int blk = 0; blk < nblk; blk++) {
        const int n_long = (int)(o.pc & 0xffffffffu), n_short = (int)(o.pc >> 32);
        runs += n_long + n_short;
        const v2u *tb = tasks + (size_t)blk * CB;
        v2u dsc_[RPL];
#pragma unroll
        for (int i = 0; i < RPL; i++) dsc_[i] = o.pd[i];
        __syncthreads();                                    // the previous block's runs are summed and stored
        // the old sums are asked for first: they travel while the block's values are put in their places
        // (every wave issues the same loads, a row that is not needed read as row 0: the wait for the values of
        // dx below then counts these loads exactly and does not include them)
        float acc[RPL][K];
        bool valid[RPL];
        unsigned row[RPL];
        bool hvalid = false, hcarried = false;
        float hacc = 0.f;
#pragma unroll
        for (int i = 0; i < RPL; i++) {
            valid[i] = !hot && sl + NSL * i < n_short;
            row[i] = valid[i] ? dsc_[i].x : 0u;
        }
        if (hot) {
            hvalid = col_ok && lane < n_long;
            const unsigned tok = hvalid ? dsc_[0].x : 0u;
            if (hvalid && blk > 0) {
                const unsigned long long e = carry[(blk - 1) & 1][wave][tok & (COL_CARRY - 1)];
                if ((unsigned)e == tok) {
                    hacc = __uint_as_float((unsigned)(e >> 32));
                    hcarried = true;
                }
            }
            if (blk == 0) {
                hacc = h0;
                hcarried = true;
            }
            row[0] = hvalid && !hcarried ? tok : 0u;
        }
#pragma unroll
        for (int i = 0; i < RPL; i++) {
            const float *src = dE + (size_t)row[i] * D + d0;
            if (FULL || kv == K) {                                  // one request for the K columns
                const ColVec<K> v = *reinterpret_cast<const ColVec<K> *>(src);
#pragma unroll
                for (int d = 0; d < K; d++) acc[i][d] = v.f[d];
            } else {
#pragma unroll
                for (int d = 0; d < K; d++) acc[i][d] = src[d < kv ? d : 0];
            }
        }
#pragma unroll
        for (int q = 0; q < COL_PPT; q++) {
            const int r = (o.prk[q / 2] >> (16 * (q & 1))) & 0xffff;
            if (blk * CB + COL_PPT * t + q < N) {
#pragma unroll
                for (int d = 0; d < K; d++) xs[d][r] = o.px[d][q / 4][q & 3];
            }
        }
        if (t < K * COL_CARRY) carry[blk & 1][t / COL_CARRY][t % COL_CARRY] = ~0ull;
        __syncthreads();
        if (blk + 1 < nblk) {                               // (behind the loads of the old sums: those arrive first)
            fetch_runs(o, blk + 1);
            fetch_values(o, blk + 1);
        }
        if (hot) {
            __builtin_amdgcn_s_setprio(3);
            if (hvalid) {
                const unsigned tok = dsc_[0].x;
                if (!hcarried) {
#pragma unroll
                    for (int d = 0; d < K; d++)
                        if (d == wave) hacc = acc[0][d];
                }
                hacc = long_chain(hacc, xc, (int)(dsc_[0].y & 0xffffu), (int)(dsc_[0].y >> 16));
                dcol[(size_t)tok * D] = hacc;
                carry[blk & 1][wave][tok & (COL_CARRY - 1)] = ((unsigned long long)__float_as_uint(hacc) << 32) | tok;
            }
            for (int r = 1; r * 64 < n_long; r++) {          // more than 64 long runs in the block
                const int a = lane + 64 * r;
                const bool val = col_ok && a < n_long;
                const v2u dsc = tb[min(a, CB - 1)];
                const unsigned tok = val ? dsc.x : 0u;
                float ac = 0.f;
                bool need = val;
                if (val && blk > 0) {
                    const unsigned long long e = carry[(blk - 1) & 1][wave][tok & (COL_CARRY - 1)];
                    if ((unsigned)e == tok) {
                        ac = __uint_as_float((unsigned)(e >> 32));
                        need = false;
                    }
                }
                if (need) ac = dcol[(size_t)tok * D];
                if (val) {
                    ac = long_chain(ac, xc, (int)(dsc.y & 0xffffu), (int)(dsc.y >> 16));
                    dcol[(size_t)tok * D] = ac;
                    carry[blk & 1][wave][tok & (COL_CARRY - 1)] = ((unsigned long long)__float_as_uint(ac) << 32) | tok;
                }
            }
            __builtin_amdgcn_s_setprio(0);
        } else {
            auto finish = [&](const v2u dsc, float (&ac)[K]) {
                const int start = (int)(dsc.y & 0xffffu), len = (int)(dsc.y >> 16);
#pragma unroll 4
                for (int jj = 0; jj < len; jj++) {
#pragma unroll
                    for (int d = 0; d < K; d++) ac[d] += xs[d][start + jj];
                }
                float *dst = dE + (size_t)dsc.x * D + d0;
                if (FULL || kv == K) {
                    ColVec<K> v;
#pragma unroll
                    for (int d = 0; d < K; d++) v.f[d] = ac[d];
                    *reinterpret_cast<ColVec<K> *>(dst) = v;
                } else {
#pragma unroll
                    for (int d = 0; d < K; d++)
                        if (d < kv) dst[d] = ac[d];
                }
            };
#pragma unroll
            for (int i = 0; i < RPL; i++)
                if (valid[i]) finish(dsc_[i], acc[i]);
            for (int r0 = RPL; r0 * NSL < n_short; r0++) {   // more short runs than RPL per lane: one at a time
                const int s = sl + r0 * NSL;
                if (s >= n_short) continue;
                const v2u dsc = tb[CB - 1 - s];
                const float *src = dE + (size_t)dsc.x * D + d0;
                float ac[K];
#pragma unroll
                for (int d = 0; d < K; d++) ac[d] = src[d < kv ? d : 0];
                finish(dsc, ac);
            }
        }
    }
    // what the host looks at before it picks a form for the next call of this shape (one 8-byte store to host memory)
    if (report && blockIdx.x == 0 && t == 0) *report = scatter_report(runs, N, D, 1);
}

// Up to COL_SMALL positions (one sequence of the reference's loops): plan and sums in ONE launch.  Every workgroup
// ranks all positions itself in LDS (two threads per position count the smaller words; 1 us, redundant but without
// a launch boundary), marks the first rank of every run in a 512-bit mask, writes its K columns of dx to LDS at their
// ranks and sums the runs, one lane per (run, column), from dE and back to it.  Any S.
constexpr int COL_SMALL = 512, COL_SMALL_BITS = 10;

template <int K>
__global__ __launch_bounds__(1024) void col_sum_small_kernel(float *dE, const float *__restrict__ dx,
                                                             const int32_t *__restrict__ ids, int N, int V, int D, int S) {
    constexpr int XP = COL_SMALL + 48;
    __shared__ __attribute__((aligned(16))) unsigned words[COL_SMALL];
    __shared__ unsigned sorted[COL_SMALL];
    __shared__ unsigned short rank_of[COL_SMALL];
    __shared__ unsigned long long heads[COL_SMALL / 64];
    __shared__ __attribute__((aligned(16))) float xs[K][XP];
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int d0 = xcd_remap(blockIdx.x, gridDim.x) * K;
    const int kv = min(K, D - d0);
    // this thread's values of dx: element i = column i / N, position i % N (coalesced along the positions)
    constexpr int XPT = (COL_SMALL * K + 1023) / 1024;
    float xv[XPT];
#pragma unroll
    for (int q = 0; q < XPT; q++) {
        const int i = t + 1024 * q, d = i / N, p = i - d * N;
        xv[q] = 0.f;
        if (d < kv) {
            const int b = p / S;
            xv[q] = dx[((size_t)b * D + d0 + d) * S + (p - b * S)];
        }
    }
    if (t < COL_SMALL) {
        unsigned key = (unsigned)V;                             // padding and out-of-range ids sort last
        if (t < N) {
            const int id = ids[t];
            if (id >= 0 && id < V) key = (unsigned)id;
        }
        words[t] = (key << COL_SMALL_BITS) | (unsigned)t;
    }
    __syncthreads();
    {
        const int p = t >> 1, h = t & 1;
        const unsigned w = words[p];
        int r = 0;
#pragma unroll 8
        for (int j = 0; j < COL_SMALL / 2; j += 4) {
            const v4u q = *reinterpret_cast<const v4u *>(&words[h * (COL_SMALL / 2) + j]);
            r += (q.x < w ? 1 : 0) + (q.y < w ? 1 : 0) + (q.z < w ? 1 : 0) + (q.w < w ? 1 : 0);
        }
        r += __shfl_xor(r, 1, 64);
        if (h == 0) {
            rank_of[p] = (unsigned short)r;
            sorted[r] = w;
        }
    }
    __syncthreads();
    if (t < COL_SMALL) {
        // a run starts where the token changes; the first padding word starts one too, so every run ends at a mark
        const bool head = t == 0 || (sorted[t - 1] >> COL_SMALL_BITS) != (sorted[t] >> COL_SMALL_BITS);
        const unsigned long long m = __builtin_amdgcn_ballot_w64(head);
        if (lane == 0) heads[wave] = m;
    }
#pragma unroll
    for (int q = 0; q < XPT; q++) {
        const int i = t + 1024 * q, d = i / N, p = i - d * N;
        if (d < K) xs[d][rank_of[p]] = xv[q];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < XPT; q++) {
        const int i = t + 1024 * q, d = i / COL_SMALL, r = i % COL_SMALL;
        const unsigned tok = sorted[r] >> COL_SMALL_BITS;
        const bool head = (heads[r >> 6] >> (r & 63)) & 1ull;
        if (d < kv && head && tok < (unsigned)V) {
            // the next mark after r
            int end = COL_SMALL;
            unsigned long long m = (r & 63) == 63 ? 0ull : (heads[r >> 6] >> ((r & 63) + 1));
            if (m) end = r + 1 + __builtin_ctzll(m);
            else
                for (int wq = (r >> 6) + 1; wq < COL_SMALL / 64; wq++)
                    if (heads[wq]) { end = wq * 64 + __builtin_ctzll(heads[wq]); break; }
            float *dst = dE + (size_t)tok * D + d0 + d;
            *dst = long_chain(*dst, &xs[d][0], r, end - r);
        }
    }
}

// Columns of dE per workgroup: three from D = 513 on (256 workgroups at D = 768), four from 769 (256 at D = 1024:
// 148 KB of LDS, the most a workgroup can hold of a block of 8192 positions).
int cols_per_workgroup(int D) { return D > 768 ? 4 : D > 512 ? 3 : D > 256 ? 2 : 1; }

// Launches the kernels of the column form.  The caller has checked: V < 2^(32 - CB_BITS) and, beyond COL_SMALL
// positions, S a multiple of 4 and dx 16-byte aligned.
int scatter_add_cols(float *dE, const float *dx, const int32_t *ids, int V, int D, int S, int N,
                     unsigned long long *report) {
    const int K = cols_per_workgroup(D);
    const dim3 grid((unsigned)ceil_div((size_t)D, K));
    if (N <= COL_SMALL) {
#define COL_LAUNCH(KK)                                                                                              \
    case KK:                                                                                                        \
        hipLaunchKernelGGL(col_sum_small_kernel<KK>, grid, dim3(1024), 0, g_ctx.stream, dE, dx, ids, N, V, D, S);   \
        break;
        switch (K) { COL_LAUNCH(1) COL_LAUNCH(2) COL_LAUNCH(3) COL_LAUNCH(4) }
#undef COL_LAUNCH
        LAUNCH_OK("embed_scatter_add column sums");
        return 0;
    }
    const int nchunks = (int)ceil_div((size_t)N, CHUNK), nblk = (int)ceil_div((size_t)N, CB);
    size_t total = 0;
    auto take = [&total](size_t bytes) {
        const size_t off = total;
        total += (bytes + 255) & ~(size_t)255;
        return off;
    };
    const size_t off_chunks = take((size_t)nchunks * CHUNK * sizeof(unsigned));
    const size_t off_cnt = take((size_t)nblk * sizeof(unsigned long long));
    const size_t off_rk = take((size_t)nblk * CB * sizeof(uint16_t));
    const size_t off_tasks = take((size_t)nblk * CB * sizeof(v2u));
    char *ws = (char *)mi355_ws(total);
    if (!ws) return -1;
    unsigned *sorted_chunks = (unsigned *)(ws + off_chunks);
    unsigned long long *cnt = (unsigned long long *)(ws + off_cnt);
    uint16_t *rk = (uint16_t *)(ws + off_rk);
    v2u *tasks = (v2u *)(ws + off_tasks);
    hipLaunchKernelGGL(chunk_sort_blk_kernel, dim3(nchunks), dim3(CHUNK), 0, g_ctx.stream, sorted_chunks, cnt, nblk, ids,
                       N, V);
    hipLaunchKernelGGL(block_rank_kernel, dim3((unsigned)ceil_div((size_t)N, 64)), dim3(1024), 0, g_ctx.stream, rk, tasks,
                       cnt, sorted_chunks, ids, N, V, nchunks);
    LAUNCH_OK("embed_scatter_add plan");
#define COL_LAUNCH(KK)                                                                                              \
    case KK:                                                                                                        \
        if (D % KK == 0)                                                                                            \
            hipLaunchKernelGGL((col_sum_kernel<KK, true>), grid, dim3(1024), 0, g_ctx.stream, dE, dx, tasks, cnt, rk, N, D, \
                               S, nblk, report);                                                                    \
        else                                                                                                        \
            hipLaunchKernelGGL((col_sum_kernel<KK, false>), grid, dim3(1024), 0, g_ctx.stream, dE, dx, tasks, cnt, rk, N, D, \
                               S, nblk, report);                                                                    \
        break;
    switch (K) {
        COL_LAUNCH(1) COL_LAUNCH(2) COL_LAUNCH(3) COL_LAUNCH(4)
    default: return mi355_fail("embed_scatter_add: no kernel for %d columns per workgroup", K);
    }
#undef COL_LAUNCH
    LAUNCH_OK("embed_scatter_add column sums");
    return 0;
}
