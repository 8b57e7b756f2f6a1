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

// ---- bfloat16 storage: values travel as uint16_t bit patterns (the upper half of the fp32 pattern) and are
// widened to fp32 on load, rounded to nearest even on store ----
typedef uint16_t bf16_t;
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf_to_f(unsigned bits16) { return __uint_as_float(bits16 << 16); }
// round to nearest even; NaN stays NaN (quiet bit forced): the conversion instruction of gfx950, one for two
// values (v_cvt_pk_bf16_f32; the same bits as (u + 0x7fff + ((u >> 16) & 1)) >> 16 with NaNs kept, in a seventh
// of the instructions, which is what the bfloat16 tile kernels spend most of their time on)
__device__ __forceinline__ unsigned f2_to_bf2(float lo, float hi) {
    typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
    typedef float f2_t __attribute__((ext_vector_type(2)));
    const f2_t v = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf2_t));
}
__device__ __forceinline__ unsigned f_to_bf(float f) { return f2_to_bf2(f, 0.f) & 0xffffu; }

// VEC bf16 values -> VEC floats.  VEC = 8: one 128-bit access, element 2j in the low half of word j.
template <int VEC, bool NT>
__device__ __forceinline__ void ldb(float (&r)[VEC], const bf16_t *p) {
    if constexpr (VEC == 8) {
        const v4u *q = reinterpret_cast<const v4u *>(p);
        const v4u w = NT ? __builtin_nontemporal_load(q) : *q;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            r[2 * j] = bf_to_f(w[j] & 0xffffu);
            r[2 * j + 1] = bf_to_f(w[j] >> 16);
        }
    } else {
        static_assert(VEC == 1, "bf16 rows are read 8 columns or 1 column at a time");
        r[0] = bf_to_f(*p);
    }
}
template <int VEC>
__device__ __forceinline__ void stb(bf16_t *p, const float (&r)[VEC]) {
    if constexpr (VEC == 8) {
        v4u w;
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = f2_to_bf2(r[2 * j], r[2 * j + 1]);
        __builtin_nontemporal_store(w, reinterpret_cast<v4u *>(p));
    } else {
        *p = (bf16_t)f_to_bf(r[0]);
    }
}

// Register tiles keep the bf16 words packed (half the registers of an fp32 tile) and widen them at each use.
template <int VEC> struct RawT { typedef unsigned type; };
template <> struct RawT<8> { typedef v4u type; };
template <int VEC, bool NT>
__device__ __forceinline__ typename RawT<VEC>::type ld_raw(const bf16_t *p) {
    if constexpr (VEC == 8) {
        const v4u *q = reinterpret_cast<const v4u *>(p);
        return NT ? __builtin_nontemporal_load(q) : *q;
    } else {
        return (unsigned)*p;
    }
}
template <int VEC>
__device__ __forceinline__ void unpack(float (&r)[VEC], const typename RawT<VEC>::type &w) {
    if constexpr (VEC == 8) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            r[2 * j] = bf_to_f(w[j] & 0xffffu);
            r[2 * j + 1] = bf_to_f(w[j] >> 16);
        }
    } else {
        r[0] = bf_to_f(w);
    }
}
// Tells the compiler nothing about the words' contents from here on, so that the widened copies made before a
// reduction are dropped instead of being kept alive across it (they would double the register tile).
template <int VEC>
__device__ __forceinline__ void forget(typename RawT<VEC>::type &w) {
    if constexpr (VEC == 8) {
        unsigned a = w[0], b = w[1], c = w[2], d = w[3];
        asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
        w[0] = a; w[1] = b; w[2] = c; w[3] = d;
    } else {
        asm volatile("" : "+v"(w));
    }
}
template <int VEC>
__device__ __forceinline__ typename RawT<VEC>::type raw_zero() {
    if constexpr (VEC == 8) { v4u z = {0u, 0u, 0u, 0u}; return z; }
    else return 0u;
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
