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
    int scatter_cols;          // ordered scatter-add with the columns of dE dealt out to the workgroups: 0 = where it pays,
                               // 1 = whenever the shape allows, -1 = never
    int rms_cluster;           // channel split of the clustered RMSNorm: 0 = per shape, -1 = never, 2/4/8 = forced
    int ce_resident;           // one-launch softmax-CE: 0 = where it pays, 1 = whenever the shape allows, -1 = never
    int rms_cluster_spin;      // its bounded wait in ticks of the 100 MHz clock: 0 = 2 ms, negative = do not wait at all
    int xch_take_nothing;      // test mode of those kernels: 1 = no partner's value is taken, present or not, so every
                               // workgroup goes the way of an expired wait
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
// Exchange area for kernels whose workgroups pass values to one another inside one launch (the clustered
// RMSNorm, the single-launch INT8 scale and scale + quantize): 8-byte slots {fp32 value, tag}, XCH_SLOT_STRIDE per workgroup number, and
// one launch counter per workgroup number; norm_cluster.h describes the protocol.  Allocated and zeroed on first
// use (not possible during a graph capture); false with the error recorded on failure.
constexpr int XCH_SLOT_STRIDE = 256;
constexpr int XCH_MAX_BLOCKS = 2048;
struct Mi355Exchange {
    unsigned long long *slots;     // [XCH_MAX_BLOCKS][XCH_SLOT_STRIDE]
    unsigned *cnt;                 // [XCH_MAX_BLOCKS] launches completed by each workgroup number
    int *fallbacks;                // workgroups whose bounded wait expired, ever (diagnostic)
};
bool mi355_exchange(Mi355Exchange *out);
// Ticks of the 100 MHz clock that such a kernel waits for a partner before it does the partner's work itself;
// negative: the kernel does not even look at a partner's slot (the xch_take_nothing test mode).
int mi355_exchange_spin_ticks(void);
// Device address of the expired-wait counter of the one-launch cross-entropy (softmax_ce.hip), NULL before init.
int *mi355_ce_fallbacks_dev(void);
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

// Value of lane (l ^ M) of a wave64, through the cheapest path measured for each distance: a DPP quad permute inside
// the adder for 1 and 2, ds_bpermute for 4, 8 and 16, v_permlane32_swap for 32.  (ds_swizzle in bit-mask mode also
// reaches 4, 8 and 16, without an address register, but the 16-wave RMSNorm tile ran 0.2-0.3 us slower with it
// than with ds_bpermute: 10.4-10.7 against 10.0-10.5 us; v_permlane32_swap and ds_bpermute were equal for 32.)
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "lane distance");
    const int iv = __float_as_int(v);
    int r;
    if constexpr (M == 1) r = __builtin_amdgcn_update_dpp(0, iv, 0xB1, 0xF, 0xF, true);          // quad_perm:[1,0,3,2]
    else if constexpr (M == 2) r = __builtin_amdgcn_update_dpp(0, iv, 0x4E, 0xF, 0xF, true);     // quad_perm:[2,3,0,1]
    else if constexpr (M == 4 || M == 8 || M == 16) return __shfl_xor(v, M, 64);                 // ds_bpermute_b32
    else {
        typedef unsigned lane_pair __attribute__((ext_vector_type(2)));
        // {v with its upper half replaced by the lower half, v with its lower half replaced by the upper half}
        const lane_pair p = __builtin_amdgcn_permlane32_swap((unsigned)iv, (unsigned)iv, false, false);
        r = (int)((__lane_id() & 32) ? p[0] : p[1]);
    }
    return __int_as_float(r);
}
// DPP mirrors within half a row (lane i <-> 7-i) and a row (i <-> 15-i): in a butterfly whose earlier steps have
// made the lanes of each group of 4 (of 8) agree, the mirrored lane holds what lane i^4 (i^8) holds.
__device__ __forceinline__ float dpp_half_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_row_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
}

// sum over the lanes {l ^ m : m in multiples of STEP below 64}, i.e. lanes that share (l % STEP); every lane of a
// class adds the same pairs in the same order, so all of them end with the same bits
template <int STEP>
__device__ __forceinline__ float wave_sum_stride(float v) {
    if constexpr (STEP <= 1) v += lane_xor<1>(v);
    if constexpr (STEP <= 2) v += lane_xor<2>(v);
    if constexpr (STEP <= 4) v += lane_xor<4>(v);
    if constexpr (STEP <= 8) v += lane_xor<8>(v);
    if constexpr (STEP <= 16) v += lane_xor<16>(v);
    if constexpr (STEP <= 32) v += lane_xor<32>(v);
    return v;
}
// sum over groups of G adjacent lanes (G a power of two <= 64)
template <int G>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (G >= 2) v += lane_xor<1>(v);
    if constexpr (G >= 4) v += lane_xor<2>(v);
    if constexpr (G >= 8) v += dpp_half_mirror(v);
    if constexpr (G >= 16) v += dpp_row_mirror(v);
    if constexpr (G >= 32) v += lane_xor<16>(v);
    if constexpr (G >= 64) v += lane_xor<32>(v);
    return v;
}

// whole-wave reductions on the same lane exchanges; every lane ends with the result
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, lane_xor<1>(v)); v = fmaxf(v, lane_xor<2>(v)); v = fmaxf(v, lane_xor<4>(v));
    v = fmaxf(v, lane_xor<8>(v)); v = fmaxf(v, lane_xor<16>(v)); v = fmaxf(v, lane_xor<32>(v));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
    v = fminf(v, lane_xor<1>(v)); v = fminf(v, lane_xor<2>(v)); v = fminf(v, lane_xor<4>(v));
    v = fminf(v, lane_xor<8>(v)); v = fminf(v, lane_xor<16>(v)); v = fminf(v, lane_xor<32>(v));
    return v;
}
// sum with the far lanes first (32, 16, ... 1)
__device__ __forceinline__ float wave_sum_far_first(float v) {
    v += lane_xor<32>(v); v += lane_xor<16>(v); v += lane_xor<8>(v);
    v += lane_xor<4>(v); v += lane_xor<2>(v); v += lane_xor<1>(v);
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
