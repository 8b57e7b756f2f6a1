// gemm.hip — the loops' cblas_sgemm(CblasRowMajor, ...) calls on device memory.
//
// The dynamic loop runs the classifier and every weight-gradient product on the CPU through cblas_sgemm:
// logits = cembed . x_final (training/training_dynamic/train.m:490-491), dy = cembed^T . dlogits (:501-502),
// gcembed += dlogits . x_final^T (:507-508), and the dW products of each layer (:577-581, :613, :681-685).
// These are plain dense fp32 products, which belong to the vendor GEMM library: rocBLAS is opened on the
// first call (dlopen, so that the op library itself carries no link-time dependency on it) and fed the
// row-major problem as the equivalent column-major one, C^T = op(B)^T . op(A)^T.
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
            !sym(g_blas.sgemm, "rocblas_sgemm")) {
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
    const rocblas_status st =
        g_blas.sgemm(g_blas.handle, tb ? rocblas_operation_transpose : rocblas_operation_none,
                     ta ? rocblas_operation_transpose : rocblas_operation_none, N, M, K, &alpha, B, ldb, A, lda, &beta,
                     C, ldc);
    if (st != rocblas_status_success) return mi355_fail("sgemm: rocblas_sgemm status %d", (int)st);
    return 0;
}
