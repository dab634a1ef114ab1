// operator_check: exercises the error paths of the C++ operator (SPMM_ACCEL over
// SPMM_BASE) that the command-line harness cannot reach.  Prints one "ok: ..." line per
// check and exits 0, or prints "FAIL: ..." and exits 1.  Needs a GPU (exit 3 without).
#include <cmath>
#include <cstdio>
#include <vector>

#include "accel_gcn.h"
#include "spmm_accel.h"

namespace {

struct Counting : SPMM_ACCEL {
    using SPMM_ACCEL::SPMM_ACCEL;
    int calls = 0;
    void run(int dim) override
    {
        calls++;
        SPMM_ACCEL::run(dim);
    }
};

int fail(const char *what)
{
    std::printf("FAIL: %s\n", what);
    return 1;
}

}  // namespace

int main()
{
    int n_dev = 0;
    if (accel_device_count(&n_dev) != ACCEL_OK || n_dev < 1) {
        std::fprintf(stderr, "operator_check: no GPU (%s)\n", accel_last_error());
        return 3;
    }
    // a 6-row matrix, rows already in ascending degree order: degrees 0 1 1 2 3 3
    const int v_num = 6, dim_max = 8;
    const std::vector<int> ptr_h = {0, 0, 1, 2, 4, 7, 10};
    const std::vector<int> idx_h = {3, 0, 1, 5, 0, 2, 4, 1, 3, 5};
    const int e_num = (int)idx_h.size();
    int *ptr = nullptr, *idx = nullptr;
    float *val = nullptr, *vin = nullptr, *vout = nullptr;
    if (hipMallocManaged((void **)&ptr, sizeof(int) * (v_num + 1)) != hipSuccess ||
        hipMallocManaged((void **)&idx, sizeof(int) * e_num) != hipSuccess ||
        hipMallocManaged((void **)&val, sizeof(float) * e_num) != hipSuccess ||
        hipMallocManaged((void **)&vin, sizeof(float) * v_num * dim_max) != hipSuccess ||
        hipMallocManaged((void **)&vout, sizeof(float) * v_num * dim_max) != hipSuccess)
        return fail("hipMallocManaged");
    for (int i = 0; i <= v_num; i++) ptr[i] = ptr_h[i];
    for (int i = 0; i < e_num; i++) { idx[i] = idx_h[i]; val[i] = 1.0f; }
    for (int i = 0; i < v_num * dim_max; i++) { vin[i] = (float)(i % 7) - 3.0f; vout[i] = NAN; }

    Counting op("check", ptr, idx, val, vin, vout, v_num, e_num, dim_max);
    op.set_meta_dir("/nonexistent/");
    // a launch that the library refuses: do_test reports it, and the timing protocol does not
    // keep launching (8 calls of run, of which only the first reaches the library)
    if (op.do_test(true, 0) >= 0) return fail("do_test(true, 0) did not report the refused launch");
    if (op.error().empty()) return fail("no error text after the refused launch");
    if (op.calls != 8) return fail("timing protocol did not make its 8 calls");
    for (int i = 0; i < v_num * dim_max; i++)
        if (!std::isnan(vout[i])) return fail("vout was written by a refused launch");
    std::printf("ok: refused launch reported (%s), nothing written\n", op.error().c_str());
    // the failure does not stick: the next call computes
    if (op.do_test(false, 4) != 0.0) return fail("do_test(false, 4) after a failure");
    if (!op.error().empty()) return fail("error text left over after a good run");
    for (int r = 0; r < v_num; r++)
        for (int c = 0; c < 4; c++) {
            float want = 0.0f;
            for (int p = ptr[r]; p < ptr[r + 1]; p++) want += vin[idx[p] * 4 + c];
            if (vout[r * 4 + c] != want) return fail("wrong product after recovery");
        }
    std::printf("ok: operator computes again after the failure\n");
    const double t = op.do_test(true, 8);
    if (!(t > 0.0 && t < 1.0)) return fail("timing run");
    std::printf("ok: timing %.1f us\n", t * 1e6);
    // a host address as vout: refused with an error code instead of a GPU fault
    std::vector<float> host_out((size_t)v_num * dim_max);
    SPMM_ACCEL bad("check", ptr, idx, val, vin, host_out.data(), v_num, e_num, dim_max);
    bad.set_meta_dir("/nonexistent/");
    if (bad.do_test(false, 4) >= 0) return fail("host pointer as vout was accepted");
    std::printf("ok: host pointer refused (%s)\n", bad.error().c_str());
    // values rewritten between two calls: the second call computes with the new ones, also when
    // the operator works from a degree-sorted copy (rows here are in descending degree order)
    {
        const std::vector<int> rptr_h = {0, 3, 6, 8, 9, 10, 10};
        const std::vector<int> ridx_h = {1, 3, 5, 0, 2, 4, 1, 5, 0, 3};
        for (int i = 0; i <= v_num; i++) ptr[i] = rptr_h[i];
        for (int i = 0; i < e_num; i++) { idx[i] = ridx_h[i]; val[i] = 1.0f + (float)i; }
        SPMM_ACCEL again("check", ptr, idx, val, vin, vout, v_num, e_num, dim_max);
        again.set_meta_dir("/nonexistent/");
        for (int pass = 0; pass < 2; pass++) {
            if (pass == 1)
                for (int i = 0; i < e_num; i++) val[i] = 0.5f * (float)(e_num - i);
            if (again.do_test(false, 4) != 0.0) return fail("do_test on the unsorted matrix");
            for (int r = 0; r < v_num; r++)
                for (int c = 0; c < 4; c++) {
                    float want = 0.0f;
                    for (int p = ptr[r]; p < ptr[r + 1]; p++) want += val[p] * vin[idx[p] * 4 + c];
                    if (std::fabs(vout[r * 4 + c] - want) > 1e-4f * (1.0f + std::fabs(want)))
                        return fail(pass ? "values rewritten between two calls were not picked up"
                                         : "wrong product on the unsorted matrix");
                }
        }
        std::printf("ok: values rewritten between two do_test calls are used\n");
    }
    (void)hipFree(ptr); (void)hipFree(idx); (void)hipFree(val); (void)hipFree(vin); (void)hipFree(vout);
    return 0;
}
