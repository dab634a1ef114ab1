// Comparison baseline, outside the measured path: the vendor library's SGEMM (rocBLAS) for
// the dense product of a GCN layer, Z = X W with row-major operands, on the same
// device-resident arrays and timed with HIP events.  Upstream has no dense product (its
// operator takes A X's operand as given, spmm_accel.cu:16-102); this is the library a caller
// would otherwise use for it.  Lives in libaccelgcn_baselines.so: the product library
// links no BLAS.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <chrono>
#include <cstdint>
#include <cstdio>

namespace {
thread_local char g_err[256] = "";
int fail(const char *what, int code)
{
    snprintf(g_err, sizeof g_err, "%s failed with status %d", what, code);
    return -1;
}
}  // namespace

#define RB(call)                                                         \
    do {                                                                 \
        rocblas_status st_ = (call);                                     \
        if (st_ != rocblas_status_success) return fail(#call, (int)st_); \
    } while (0)
#define HIPC(call)                                                 \
    do {                                                           \
        hipError_t e_ = (call);                                    \
        if (e_ != hipSuccess) return fail(#call, (int)e_);         \
    } while (0)

extern "C" {

const char *baseline_rocblas_last_error(void) { return g_err; }

// Z (rows x N, row-major) = X (rows x K) W (K x N).  In the library's column-major terms
// that is Z^T = W^T X^T: m = N, n = rows, k = K with leading dimensions N, K, N.
// ms_each receives `iters` per-launch times (HIP events around each launch) after `warmup`
// untimed launches; *ms_queued (optional) the host-clock average of `iters` more launches
// queued back to back between two synchronisations.
int baseline_rocblas_sgemm(const float *X, const float *W, float *Z, int64_t rows, int32_t K, int32_t N,
                           int warmup, int iters, float *ms_each, float *ms_queued)
{
    if (rows <= 0 || rows > 0x7fffffffLL || K <= 0 || N <= 0) return fail("shape check", 0);
    rocblas_handle handle;
    RB(rocblas_create_handle(&handle));
    const float alpha = 1.0f, beta = 0.0f;
    hipEvent_t e0, e1;
    HIPC(hipEventCreate(&e0));
    HIPC(hipEventCreate(&e1));
    for (int i = 0; i < warmup + iters; i++) {
        if (i >= warmup) HIPC(hipEventRecord(e0, nullptr));
        RB(rocblas_sgemm(handle, rocblas_operation_none, rocblas_operation_none, N, (rocblas_int)rows, K, &alpha, W, N,
                         X, K, &beta, Z, N));
        if (i >= warmup) {
            HIPC(hipEventRecord(e1, nullptr));
            HIPC(hipEventSynchronize(e1));
            HIPC(hipEventElapsedTime(&ms_each[i - warmup], e0, e1));
        }
    }
    HIPC(hipDeviceSynchronize());
    if (ms_queued && iters > 0) {
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < iters; i++)
            RB(rocblas_sgemm(handle, rocblas_operation_none, rocblas_operation_none, N, (rocblas_int)rows, K, &alpha, W,
                             N, X, K, &beta, Z, N));
        HIPC(hipDeviceSynchronize());
        *ms_queued = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count() / iters;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    rocblas_destroy_handle(handle);
    return 0;
}

}  // extern "C"
