// Comparison baseline, outside the measured path: the vendor library's CSR SpMM
// (rocSPARSE) on the same device-resident operands, timed with HIP events.
// Upstream compares its kernel with cuSPARSE's CSR SpMM, row-major dense,
// alpha = 1, beta = 0 (spmm_cusparse.cu:6-62, 10 warm-up + 10 timed launches);
// this is the same comparison on AMD hardware.  Built into its own library
// (libaccelgcn_baselines.so) so that the product library never links rocSPARSE.
#include <hip/hip_runtime.h>
#include <rocsparse/rocsparse.h>

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

#define RS(call)                                                   \
    do {                                                           \
        rocsparse_status st_ = (call);                             \
        if (st_ != rocsparse_status_success) return fail(#call, (int)st_); \
    } while (0)
#define HIPC(call)                                                 \
    do {                                                           \
        hipError_t e_ = (call);                                    \
        if (e_ != hipSuccess) return fail(#call, (int)e_);         \
    } while (0)

extern "C" {

const char *baseline_last_error(void) { return g_err; }

// alg: 0 default, 1 csr, 4 row split, 5 nnz split, 9 merge path (rocsparse_spmm_alg values).
// Y = A X.  ms_each receives `iters` per-launch times (compute stage only; the
// library's buffer-size and preprocess stages run once before and are returned
// in *preprocess_ms).
int baseline_rocsparse_spmm(const int32_t *indptr, const int32_t *idx, const float *val, int64_t rows,
                            int64_t cols, int64_t nnz, const float *X, float *Y, int32_t N, int alg,
                            int warmup, int iters, float *ms_each, float *preprocess_ms)
{
    rocsparse_handle handle;
    RS(rocsparse_create_handle(&handle));
    rocsparse_spmat_descr A;
    rocsparse_dnmat_descr B, C;
    RS(rocsparse_create_csr_descr(&A, rows, cols, nnz, const_cast<int32_t *>(indptr),
                                  const_cast<int32_t *>(idx), const_cast<float *>(val),
                                  rocsparse_indextype_i32, rocsparse_indextype_i32,
                                  rocsparse_index_base_zero, rocsparse_datatype_f32_r));
    RS(rocsparse_create_dnmat_descr(&B, cols, N, N, const_cast<float *>(X), rocsparse_datatype_f32_r,
                                    rocsparse_order_row));
    RS(rocsparse_create_dnmat_descr(&C, rows, N, N, Y, rocsparse_datatype_f32_r, rocsparse_order_row));
    const float alpha = 1.0f, beta = 0.0f;
    const rocsparse_spmm_alg a = (rocsparse_spmm_alg)alg;
    size_t buf_size = 0;
    void *buf = nullptr;
    hipEvent_t e0, e1;
    HIPC(hipEventCreate(&e0));
    HIPC(hipEventCreate(&e1));
    HIPC(hipEventRecord(e0, nullptr));
    RS(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, C,
                      rocsparse_datatype_f32_r, a, rocsparse_spmm_stage_buffer_size, &buf_size, nullptr));
    HIPC(hipMalloc(&buf, buf_size ? buf_size : 4));
    RS(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta, C,
                      rocsparse_datatype_f32_r, a, rocsparse_spmm_stage_preprocess, &buf_size, buf));
    HIPC(hipEventRecord(e1, nullptr));
    HIPC(hipEventSynchronize(e1));
    if (preprocess_ms) HIPC(hipEventElapsedTime(preprocess_ms, e0, e1));
    for (int i = 0; i < warmup + iters; i++) {
        if (i >= warmup) HIPC(hipEventRecord(e0, nullptr));
        RS(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, B, &beta,
                          C, rocsparse_datatype_f32_r, a, rocsparse_spmm_stage_compute, &buf_size, buf));
        if (i >= warmup) {
            HIPC(hipEventRecord(e1, nullptr));
            HIPC(hipEventSynchronize(e1));
            HIPC(hipEventElapsedTime(&ms_each[i - warmup], e0, e1));
        }
    }
    HIPC(hipDeviceSynchronize());
    (void)hipFree(buf);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    rocsparse_destroy_spmat_descr(A);
    rocsparse_destroy_dnmat_descr(B);
    rocsparse_destroy_dnmat_descr(C);
    rocsparse_destroy_handle(handle);
    return 0;
}

}  // extern "C"
