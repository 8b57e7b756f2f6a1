// gemm.hip — the loops' cblas_sgemm(CblasRowMajor, ...) calls on device memory.
//
// The dynamic loop runs the classifier and every weight-gradient product on the CPU through cblas_sgemm:
// logits = cembed . x_final (training/training_dynamic/train.m:490-491), dy = cembed^T . dlogits (:501-502),
// gcembed += dlogits . x_final^T (:507-508), and the dW products of each layer (:577-581, :613, :681-685).
// These are plain dense fp32 products, which belong to the vendor GEMM library: rocBLAS is opened on the
// first call (dlopen, so that the op library itself carries no link-time dependency on it) and fed the
// row-major problem as the equivalent column-major one, C^T = op(B)^T . op(A)^T.
//
// A product with a small output and a long inner dimension (dy = cembed^T . dlogits: 1024 x 256 outputs, K = the
// vocabulary) leaves most of the chip idle in a single GEMM: 16 output tiles for 256 compute units.  Such
// calls are split along K into a strided-batched GEMM whose partial products are then summed in a fixed
// order by a small kernel (deterministic; no atomics), which also applies beta.
#include "common.h"

#include <dlfcn.h>
#include <rocblas/rocblas.h>

namespace {

struct Blas {
    void *dl;
    rocblas_handle handle;
    decltype(&rocblas_create_handle) create;
    decltype(&rocblas_destroy_handle) destroy;
    decltype(&rocblas_set_stream) set_stream;
    decltype(&rocblas_set_pointer_mode) set_pointer_mode;
    decltype(&rocblas_sgemm) sgemm;
    decltype(&rocblas_sgemm_strided_batched) sgemm_sb;
};
Blas g_blas{};

template <typename F>
bool sym(F &fn, const char *name) {
    fn = reinterpret_cast<F>(dlsym(g_blas.dl, name));
    return fn != nullptr;
}

int blas_open() {
    if (g_blas.handle) return 0;
    if (!g_blas.dl) {
        const char *names[] = {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"};
        for (const char *n : names)
            if ((g_blas.dl = dlopen(n, RTLD_NOW | RTLD_LOCAL))) break;
        if (!g_blas.dl) return mi355_fail("sgemm: cannot open rocBLAS: %s", dlerror());
        if (!sym(g_blas.create, "rocblas_create_handle") || !sym(g_blas.destroy, "rocblas_destroy_handle") ||
            !sym(g_blas.set_stream, "rocblas_set_stream") || !sym(g_blas.set_pointer_mode, "rocblas_set_pointer_mode") ||
            !sym(g_blas.sgemm, "rocblas_sgemm") || !sym(g_blas.sgemm_sb, "rocblas_sgemm_strided_batched")) {
            dlclose(g_blas.dl);
            g_blas = Blas{};
            return mi355_fail("sgemm: rocBLAS lacks an expected symbol");
        }
    }
    rocblas_handle h = nullptr;
    if (g_blas.create(&h) != rocblas_status_success || !h) return mi355_fail("sgemm: rocblas_create_handle failed");
    if (g_blas.set_pointer_mode(h, rocblas_pointer_mode_host) != rocblas_status_success) {
        g_blas.destroy(h);
        return mi355_fail("sgemm: rocblas_set_pointer_mode failed");
    }
    g_blas.handle = h;
    return 0;
}

// 0 / 111 (CblasNoTrans) -> false, 1 / 112 (CblasTrans) -> true, anything else -> -1
int trans_flag(int t) {
    if (t == 0 || t == 111) return 0;
    if (t == 1 || t == 112) return 1;
    return -1;
}

// C[i] = beta*C[i] + sum_s part[s][i], s ascending; beta == 0 does not read C (cblas semantics)
template <int VEC>
__global__ __launch_bounds__(256) void splitk_sum_kernel(float *__restrict__ C, const float *__restrict__ part,
                                                         int splits, size_t n, size_t nv, float beta) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nv) return;
    if constexpr (VEC == 4) {
        v4f acc = {0.f, 0.f, 0.f, 0.f};
        if (beta != 0.f) acc = ld4(C + 4 * i) * beta;
        for (int s = 0; s < splits; s++) acc += ld4_nt(part + (size_t)s * n + 4 * i);
        st4(C + 4 * i, acc);
    } else {
        float acc = beta != 0.f ? C[i] * beta : 0.f;
        for (int s = 0; s < splits; s++) acc += part[(size_t)s * n + i];
        C[i] = acc;
    }
}

// Number of K slices for a product with few output tiles and a long K; 1 = do not split.
int pick_splits(int M, int N, int K, int ldc) {
    if (ldc != N) return 1;
    if (g_ctx.gemm_splitk) return g_ctx.gemm_splitk > 1 && K >= 2 * g_ctx.gemm_splitk ? g_ctx.gemm_splitk : 1;
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    const int cus = g_ctx.num_cu > 0 ? g_ctx.num_cu : 256;
    if (tiles * 2 > cus || K < 4096) return 1;
    // Measured on MI355X for M=1024, N=256, K=32000: 0.45 ms unsplit, 0.24-0.29 ms with 2-16 slices,
    // 0.16-0.19 ms with 24-40, slower again beyond 48.
    long s = 2 * cus / tiles;                   // two slices per otherwise idle compute unit...
    if (s > K / 768) s = K / 768;               // ...but at least 768 of K per slice
    if (s > 32) s = 32;
    return s < 2 ? 1 : (int)s;
}

}   // namespace

void mi355_blas_free(void) {
    if (g_blas.handle) {
        g_blas.destroy(g_blas.handle);
        g_blas.handle = nullptr;
    }
    // the library stays mapped: unloading it while the HIP runtime still holds its code objects is not safe
}

MI355_API int mi355_sgemm_dev(int trans_a, int trans_b, int M, int N, int K, float alpha, const float *A, int lda,
                              const float *B, int ldb, float beta, float *C, int ldc) {
    if (!mi355_ready("sgemm")) return -1;
    if (!mi355_outside_capture("sgemm (the GEMM library manages its own workspace)")) return -1;
    if (!A || !B || !C) return mi355_fail("sgemm: NULL pointer");
    const int ta = trans_flag(trans_a), tb = trans_flag(trans_b);
    if (ta < 0 || tb < 0) return mi355_fail("sgemm: transpose flags must be 0/1 (or CblasNoTrans/CblasTrans)");
    if (M <= 0 || N <= 0 || K <= 0) return mi355_fail("sgemm: bad shape M=%d N=%d K=%d", M, N, K);
    // row-major leading dimensions: A is M x K (or K x M when transposed), B is K x N (or N x K), C is M x N
    if (lda < (ta ? M : K) || ldb < (tb ? K : N) || ldc < N)
        return mi355_fail("sgemm: leading dimension too small (lda=%d ldb=%d ldc=%d)", lda, ldb, ldc);
    if (blas_open()) return -1;
    if (g_blas.set_stream(g_blas.handle, g_ctx.stream) != rocblas_status_success)
        return mi355_fail("sgemm: rocblas_set_stream failed");
    const rocblas_operation op_b = tb ? rocblas_operation_transpose : rocblas_operation_none;
    const rocblas_operation op_a = ta ? rocblas_operation_transpose : rocblas_operation_none;
    const int splits = pick_splits(M, N, K, ldc);
    if (splits > 1) {
        const size_t n = (size_t)M * N;
        float *part = (float *)mi355_ws((size_t)splits * n * sizeof(float));
        if (!part) return -1;
        // slice s covers k in [s*ks, (s+1)*ks); the last slice is shorter and runs as its own call
        const int ks = (int)ceil_div((size_t)K, (size_t)splits), full = K / ks, rest = K - full * ks;
        // row-major A is M x K (stride along k: 1, or lda when transposed), B is K x N (ldb, or 1 when transposed)
        const rocblas_stride sa = ta ? (rocblas_stride)ks * lda : ks, sb = tb ? ks : (rocblas_stride)ks * ldb;
        const float zero = 0.f;
        rocblas_status st = g_blas.sgemm_sb(g_blas.handle, op_b, op_a, N, M, ks, &alpha, B, ldb, sb, A, lda, sa, &zero,
                                            part, N, (rocblas_stride)n, full);
        int used = full;
        if (st == rocblas_status_success && rest > 0) {
            st = g_blas.sgemm(g_blas.handle, op_b, op_a, N, M, rest, &alpha, B + (size_t)full * sb, ldb,
                              A + (size_t)full * sa, lda, &zero, part + (size_t)full * n, N);
            used++;
        }
        if (st != rocblas_status_success) return mi355_fail("sgemm: rocblas split-K status %d", (int)st);
        const bool vec = n % 4 == 0 && aligned16(C) && aligned16(part);
        const size_t nv = vec ? n / 4 : n;
        if (vec) hipLaunchKernelGGL(splitk_sum_kernel<4>, dim3((unsigned)ceil_div(nv, 256)), dim3(256), 0, g_ctx.stream, C, part, used, n, nv, beta);
        else hipLaunchKernelGGL(splitk_sum_kernel<1>, dim3((unsigned)ceil_div(nv, 256)), dim3(256), 0, g_ctx.stream, C, part, used, n, nv, beta);
        LAUNCH_OK("sgemm split-K sum");
        return 0;
    }
    const rocblas_status st =
        g_blas.sgemm(g_blas.handle, op_b, op_a, N, M, K, &alpha, B, ldb, A, lda, &beta,
                     C, ldc);
    if (st != rocblas_status_success) return mi355_fail("sgemm: rocblas_sgemm status %d", (int)st);
    return 0;
}
