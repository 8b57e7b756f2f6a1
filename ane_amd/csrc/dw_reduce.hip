// dw_reduce.hip — deterministic reduction of per-workgroup weight-gradient partials.
//
// rmsnorm_bwd accumulates dw[i] += sum_s (dy*x)*rr (training/stories_cpu_ops.h:47-50).  On the GPU
// every workgroup of a backward kernel writes one partial row per channel; this file sums the rows
// in a fixed order (no floating-point atomics) and adds the total to dw.
//
// The loops consume these gradients only at the optimizer step, after the whole backward pass
// (training/training_dynamic/train.m:748-869).  mi355_dw_defer(1) uses that: reductions are queued
// and run together — 32 per launch — at mi355_dw_flush() / mi355_sync(), instead of one small
// launch behind every backward op.
#include "common.h"
#include "tile.h"

namespace {

constexpr int MAX_JOBS = 32;

struct ReduceJob {
    float *out;
    const float *part;
    int nrows, C;
};
struct JobBatch {
    ReduceJob j[MAX_JOBS];
};

// One workgroup = 32 channels of one job: 32 interleaved row groups, each summed with four
// independent accumulators (four loads in flight), then combined in a fixed order.
__global__ __launch_bounds__(1024) void reduce_jobs_kernel(JobBatch jobs) {
    __shared__ float lds[32][33];
    const ReduceJob job = jobs.j[blockIdx.y];
    const int C = job.C, nrows = job.nrows;
    if ((int)blockIdx.x * 32 >= C) return;
    const int cl = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int c = blockIdx.x * 32 + cl;
    const float *__restrict__ part = job.part;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < C) {
        int r = g;
        for (; r + 96 < nrows; r += 128) {
            s0 += part[(size_t)r * C + c];
            s1 += part[(size_t)(r + 32) * C + c];
            s2 += part[(size_t)(r + 64) * C + c];
            s3 += part[(size_t)(r + 96) * C + c];
        }
        for (; r < nrows; r += 32) s0 += part[(size_t)r * C + c];
    }
    lds[g][cl] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (g == 0 && c < C) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 32; k++) t += lds[k][cl];
        job.out[c] = job.out[c] + t;
    }
}

JobBatch g_jobs;
int g_njobs = 0, g_max_c = 0;
bool g_defer = false;
float *g_arena = nullptr;          // partial rows of queued jobs (deferred mode)
size_t g_arena_floats = 0, g_arena_used = 0;

int launch_pending(void) {
    if (g_njobs == 0) return 0;
    const dim3 grid((unsigned)ceil_div((size_t)g_max_c, 32), (unsigned)g_njobs);
    hipLaunchKernelGGL(reduce_jobs_kernel, grid, dim3(1024), 0, g_ctx.stream, g_jobs);
    g_njobs = 0;
    g_max_c = 0;
    g_arena_used = 0;       // later writers are ordered behind this launch on the stream
    LAUNCH_OK("dw reduce");
    return 0;
}

bool pending_targets(const float *out) {
    if (!out) return false;
    for (int i = 0; i < g_njobs; i++)
        if (g_jobs.j[i].out == out) return true;
    return false;
}

}   // namespace

float *mi355_dw_partials(size_t floats, const float *out0, const float *out1) {
    if (!g_defer) return (float *)mi355_ws(floats * sizeof(float));
    // two queued jobs must not add into the same dw: run what is queued first to keep the order
    if (pending_targets(out0) || pending_targets(out1) || g_njobs + 2 > MAX_JOBS ||
        g_arena_used + floats > g_arena_floats) {
        if (launch_pending()) return nullptr;
    }
    if (floats > g_arena_floats) {
        if (!mi355_outside_capture("growth of the weight-gradient arena")) return nullptr;
        size_t want = floats > ((size_t)32 << 20) ? floats : ((size_t)32 << 20);      // at least 128 MiB
        (void)hipStreamSynchronize(g_ctx.stream);
        if (g_arena) (void)hipFree(g_arena);
        g_arena = nullptr;
        g_arena_floats = 0;
        hipError_t e = hipMalloc((void **)&g_arena, want * sizeof(float));
        if (e != hipSuccess) {
            mi355_fail("dw arena hipMalloc(%zu): %s", want * sizeof(float), hipGetErrorString(e));
            return nullptr;
        }
        g_arena_floats = want;
        g_ctx.alloc_epoch++;
    }
    float *p = g_arena + g_arena_used;
    g_arena_used += (floats + 63) & ~(size_t)63;
    return p;
}

int mi355_dw_submit(float *out, const float *part, int nrows, int C) {
    if (g_njobs == MAX_JOBS && launch_pending()) return -1;
    g_jobs.j[g_njobs++] = ReduceJob{out, part, nrows, C};
    if (C > g_max_c) g_max_c = C;
    return 0;
}

int mi355_dw_op_end(void) { return g_defer ? 0 : launch_pending(); }

void mi355_dw_free(void) {
    if (g_arena) (void)hipFree(g_arena);
    g_arena = nullptr;
    g_arena_floats = g_arena_used = 0;
    g_njobs = 0;
    g_max_c = 0;
    g_defer = false;
}

MI355_API int mi355_dw_flush(void) {
    if (!g_ctx.ready) return g_njobs == 0 ? 0 : -1;
    return launch_pending();
}

MI355_API int mi355_dw_defer(int on) {
    if (!mi355_ready("dw_defer")) return -1;
    if (!mi355_outside_capture("dw_defer")) return -1;
    if (launch_pending()) return -1;
    g_defer = on != 0;
    return 0;
}
