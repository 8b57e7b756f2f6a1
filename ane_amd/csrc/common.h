// common.h — shared device helpers and the bridge context for the gfx950 op library.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/mi355_bridge.h"

#define MI355_API extern "C" __attribute__((visibility("default")))

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));

// -------------------------------------------------------------------------------------------
// Host-side context (context.hip)
// -------------------------------------------------------------------------------------------
struct Mi355Ctx {
    bool ready;
    int device;
    int num_cu;
    hipStream_t stream;
    unsigned alloc_epoch;      // bumped whenever a workspace that recorded graphs may point into is reallocated
    bool capturing;            // between mi355_graph_begin and mi355_graph_end: `stream` is the capture stream
    void *ws;          // grow-only workspace
    size_t ws_bytes;
    // tuning knobs (0 = pick per shape)
    int rms_lpr, rms_threads, ew_unroll, ce_rows, ce_rows2, qk_lpr, qk_threads, gemm_splitk, scatter_tree, buf_phase;
    int rms_cluster;           // channel split of the clustered RMSNorm: 0 = per shape, -1 = never, 2/4/8 = forced
    int rms_cluster_spin;      // its bounded wait in ticks of the 100 MHz clock: 0 = 2 ms, negative = do not wait at all
};
extern Mi355Ctx g_ctx;

// Records the message for mi355_last_error() and prints "mi355_bridge: ..." once; returns -1.
int mi355_fail(const char *fmt, ...);
// True when the context is usable; otherwise records the error.
bool mi355_ready(const char *who);
// False (with the error recorded) while a graph is being captured: for calls that allocate, free, copy to
// or from the host, or wait.
bool mi355_outside_capture(const char *who);
// Workspace of at least `bytes` (256-byte aligned), NULL on failure.
void *mi355_ws(size_t bytes);
// Runs every queued weight-gradient reduction (dw_reduce.hip).
extern "C" int mi355_dw_flush(void);

#define HIP_OK(expr)                                                                          \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess) return mi355_fail("%s: %s", #expr, hipGetErrorString(_e));      \
    } while (0)

#define LAUNCH_OK(who)                                                                        \
    do {                                                                                      \
        hipError_t _e = hipGetLastError();                                                    \
        if (_e != hipSuccess) return mi355_fail("%s launch: %s", who, hipGetErrorString(_e)); \
    } while (0)

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
static inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

// -------------------------------------------------------------------------------------------
// Device helpers
// -------------------------------------------------------------------------------------------

// MI355X has 8 XCDs, each with a private L2; consecutive workgroup ids are dealt round-robin
// to the XCDs.  This maps the hardware id to a logical id so that consecutive LOGICAL ids
// (neighbouring tiles that share cache lines) run on the same XCD.
__device__ __forceinline__ int xcd_remap(int bid, int n) {
    const int q = n >> 3, r = n & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    return xcd * q + (xcd < r ? xcd : r) + idx;
}

__device__ __forceinline__ v4f ld4(const float *p) { return *reinterpret_cast<const v4f *>(p); }
__device__ __forceinline__ void st4(float *p, v4f v) { *reinterpret_cast<v4f *>(p) = v; }
// streaming store: output is not re-read by this kernel, keep it out of the way of the inputs
__device__ __forceinline__ void st4_nt(float *p, v4f v) {
    __builtin_nontemporal_store(v, reinterpret_cast<v4f *>(p));
}
__device__ __forceinline__ v4f ld4_nt(const float *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
}

// sum over the lanes {l ^ m : m in multiples of STEP below 64}, i.e. lanes that share (l % STEP)
template <int STEP>
__device__ __forceinline__ float wave_sum_stride(float v) {
#pragma unroll
    for (int m = STEP; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}
// sum over groups of G adjacent lanes (G a power of two <= 64)
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int m = 1; m < G; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// exp(d) for d <= 0 through the hardware exp2: the product d*log2(e) is carried in two floats
// so the result keeps ~1 ulp for |d| up to ~100 (a single-float product loses |d|*2^-24).
__device__ __forceinline__ float exp_neg(float d) {
    const float L2E_HI = 1.44269502162933349609375f;      // float(log2 e)
    const float L2E_LO = 1.925963033500011e-08f;          // log2 e - L2E_HI
    d = fmaxf(d, -200.0f);                                // exp2 of the product is already 0 there; keeps -inf finite
    float hi = d * L2E_HI;
    float lo = __builtin_fmaf(d, L2E_HI, -hi) + d * L2E_LO;
    float e = __builtin_amdgcn_exp2f(hi);
    return __builtin_fmaf(e, lo * 0.693147180559945f, e);
}

// exp(d) for d <= 0 with a single-float product: relative error up to |d| * 6e-8.  Used where the
// values are only summed (terms with large |d| are negligible there).
__device__ __forceinline__ float exp_neg_fast(float d) {
    return __builtin_amdgcn_exp2f(fmaxf(d, -200.0f) * 1.44269502162933349609375f);
}
