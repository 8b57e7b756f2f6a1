// tile.h — register-tile helpers shared by the strided-axis reduction kernels.
#pragma once
#include "common.h"

template <int VEC>
__device__ __forceinline__ void ldv(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        v4f t = ld4(p);
        r[0] = t.x; r[1] = t.y; r[2] = t.z; r[3] = t.w;
    } else {
        r[0] = *p;
    }
}
// streaming variants: the operand is touched once by this kernel
template <int VEC>
__device__ __forceinline__ void ldv_nt(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        v4f t = ld4_nt(p);
        r[0] = t.x; r[1] = t.y; r[2] = t.z; r[3] = t.w;
    } else {
        r[0] = __builtin_nontemporal_load(p);
    }
}
template <int VEC>
__device__ __forceinline__ void stv_nt(float *p, const float (&r)[VEC]) {
    if constexpr (VEC == 4) {
        v4f t = {r[0], r[1], r[2], r[3]};
        st4_nt(p, t);
    } else {
        __builtin_nontemporal_store(r[0], p);
    }
}
template <int VEC>
__device__ __forceinline__ void stv(float *p, const float (&r)[VEC]) {
    if constexpr (VEC == 4) {
        v4f t = {r[0], r[1], r[2], r[3]};
        st4(p, t);
    } else {
        *p = r[0];
    }
}

// Sum acc[q][j] over all threads of the block that share the same lane column (tid % LPR).
// Every thread ends with the full per-column totals.  lds: NW*NV*LPR*VEC floats.
template <int VEC, int LPR, int THREADS, int NV>
__device__ __forceinline__ void strip_reduce(float (&acc)[NV][VEC], float *lds) {
    constexpr int NW = THREADS / 64;
    constexpr int WLPR = LPR < 64 ? LPR : 64;
#pragma unroll
    for (int q = 0; q < NV; q++)
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[q][j] = wave_sum_stride<WLPR>(acc[q][j]);
    if constexpr (NW > 1) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int lc = threadIdx.x % LPR;
        if (lane < WLPR) {
#pragma unroll
            for (int q = 0; q < NV; q++)
#pragma unroll
                for (int j = 0; j < VEC; j++) lds[((wave * NV + q) * WLPR + lane) * VEC + j] = acc[q][j];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < NV; q++)
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                float s = 0.f;
#pragma unroll
                for (int wv = 0; wv < NW; wv++) s += lds[((wv * NV + q) * WLPR + (lc & (WLPR - 1))) * VEC + j];
                acc[q][j] = s;
            }
    }
}


// ---- weight-gradient reductions (dw_reduce.hip) -------------------------------------------------
// A backward op writes per-workgroup partial rows part[nrows][C] and submits "out[c] += sum_r part[r][c]".
// Immediately (default) the jobs of one op go out as one launch when the op ends; in deferred mode they
// are queued and reduced together by mi355_dw_flush().
//
// Buffer for `floats` partials of the op that will accumulate into out0 / out1 (either may be NULL).
float *mi355_dw_partials(size_t floats, const float *out0, const float *out1);
int mi355_dw_submit(float *out, const float *part, int nrows, int C);
int mi355_dw_op_end(void);
