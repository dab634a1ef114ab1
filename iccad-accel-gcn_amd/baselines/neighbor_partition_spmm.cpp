// Comparison baseline, outside the measured path: a neighbour-partition SpMM in the
// style of GNNAdvisor, the second kernel upstream compares itself with
// (spmm_gnna.cu:20-58 builds the partitions, :60-138 is the kernel, :145-175 the
// driver).  The scheme: every row's non-zeros are cut into parts of at most
// part_size = max(1, nnz / rows) neighbours (spmm_gnna.cu:147-150), one wavefront
// aggregates one part with its lanes spread over the columns of X, and the part's
// sum is added to the output row with floating-point atomics, so the output has to
// be zero before every launch.
//
// Written for wave64: a part is owned by one 64-lane wavefront (upstream: a 32-lane
// warp with dimWorker = 32), four wavefronts per workgroup, neighbour ids and values
// staged in LDS, accumulators in registers instead of upstream's shared-memory
// array.  Unlike upstream's kernel, which sums unweighted neighbours (it never reads
// val), this one multiplies by the matrix values, so that its output is A X and can
// be checked against the operator's.
//
// Lives in libaccelgcn_baselines.so; the product library does not contain it.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <vector>

namespace {

constexpr int kWaves = 4;          // parts per workgroup
constexpr int kMaxPart = 1024;     // largest part size staged in LDS

thread_local char g_np_err[256] = "";
int np_fail(const char *what, int code)
{
    snprintf(g_np_err, sizeof g_np_err, "%s failed with status %d", what, code);
    return -1;
}

#define NP_HIP(call)                                                  \
    do {                                                              \
        hipError_t e_ = (call);                                       \
        if (e_ != hipSuccess) return np_fail(#call, (int)e_);         \
    } while (0)

__global__ __launch_bounds__(64 * kWaves) void neighbor_partition_kernel(
    const int32_t *__restrict__ part_ptr, const int32_t *__restrict__ part_row, int n_parts,
    const int32_t *__restrict__ idx, const float *__restrict__ val, const float *__restrict__ X,
    float *__restrict__ Y, int N, int part_size)
{
    extern __shared__ int2 np_stage[];                     // kWaves * part_size (column, value) pairs
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int part = blockIdx.x * kWaves + wv;
    if (part >= n_parts) return;
    const int beg = part_ptr[part], end = part_ptr[part + 1], row = part_row[part];
    int2 *st = np_stage + wv * part_size;
    for (int i = beg + lane; i < end; i += 64) st[i - beg] = make_int2(idx[i], __float_as_int(val[i]));
    __builtin_amdgcn_wave_barrier();
    for (int c = lane; c < N; c += 64) {
        float acc = 0.0f;
        for (int i = 0; i < end - beg; i++) {
            const int2 p = st[i];
            acc = fmaf(__int_as_float(p.y), X[(int64_t)p.x * N + c], acc);
        }
        unsafeAtomicAdd(Y + (int64_t)row * N + c, acc);
    }
}

}  // namespace

extern "C" {

const char *baseline_neighbor_partition_last_error(void) { return g_np_err; }

// indptr_host: the CSR row pointers on the host (the parts are built on the host, as
// upstream does); idx, val, X, Y: device pointers.  part_size 0 = nnz / rows, at least 1.
// ms_each receives `iters` per-launch kernel times; the memset that clears Y before
// each launch is outside the timed interval.  After the call Y = A X.
int baseline_neighbor_partition_spmm(const int32_t *indptr_host, const int32_t *idx, const float *val,
                                     int64_t rows, int64_t nnz, const float *X, float *Y, int32_t N,
                                     int part_size, int warmup, int iters, float *ms_each,
                                     float *preprocess_ms, int64_t *n_parts_out)
{
    if (!indptr_host || rows <= 0 || N <= 0 || iters <= 0) return np_fail("argument check", 1);
    if (part_size <= 0) part_size = (int)std::max<int64_t>(1, nnz / rows);
    part_size = std::min(part_size, kMaxPart);
    hipEvent_t e0, e1;
    NP_HIP(hipEventCreate(&e0));
    NP_HIP(hipEventCreate(&e1));
    NP_HIP(hipEventRecord(e0, nullptr));
    std::vector<int32_t> part_ptr, part_row;
    for (int64_t r = 0; r < rows; r++)
        for (int32_t b = indptr_host[r]; b < indptr_host[r + 1]; b += part_size) {
            part_ptr.push_back(b);
            part_row.push_back((int32_t)r);
        }
    part_ptr.push_back(indptr_host[rows]);
    const int64_t n_parts = (int64_t)part_row.size();
    if (n_parts_out) *n_parts_out = n_parts;
    if (n_parts / kWaves + 1 > 0x7fffffffLL) return np_fail("grid size check", 2);
    int32_t *d_ptr = nullptr, *d_row = nullptr;
    NP_HIP(hipMalloc(reinterpret_cast<void **>(&d_ptr), sizeof(int32_t) * part_ptr.size()));
    NP_HIP(hipMalloc(reinterpret_cast<void **>(&d_row), sizeof(int32_t) * std::max<size_t>(1, part_row.size())));
    NP_HIP(hipMemcpy(d_ptr, part_ptr.data(), sizeof(int32_t) * part_ptr.size(), hipMemcpyHostToDevice));
    if (n_parts > 0)
        NP_HIP(hipMemcpy(d_row, part_row.data(), sizeof(int32_t) * part_row.size(), hipMemcpyHostToDevice));
    NP_HIP(hipEventRecord(e1, nullptr));
    NP_HIP(hipEventSynchronize(e1));
    if (preprocess_ms) NP_HIP(hipEventElapsedTime(preprocess_ms, e0, e1));

    const unsigned grid = (unsigned)((n_parts + kWaves - 1) / kWaves);
    const size_t lds = sizeof(int2) * (size_t)kWaves * (size_t)part_size;
    for (int i = 0; i < warmup + iters; i++) {
        NP_HIP(hipMemsetAsync(Y, 0, sizeof(float) * (size_t)rows * (size_t)N, nullptr));
        if (i >= warmup) NP_HIP(hipEventRecord(e0, nullptr));
        if (grid > 0)
            neighbor_partition_kernel<<<dim3(grid), dim3(64 * kWaves), lds, nullptr>>>(
                d_ptr, d_row, (int)n_parts, idx, val, X, Y, N, part_size);
        if (i >= warmup) {
            NP_HIP(hipEventRecord(e1, nullptr));
            NP_HIP(hipEventSynchronize(e1));
            NP_HIP(hipEventElapsedTime(&ms_each[i - warmup], e0, e1));
        }
    }
    NP_HIP(hipGetLastError());
    NP_HIP(hipDeviceSynchronize());
    (void)hipFree(d_ptr);
    (void)hipFree(d_row);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return 0;
}

}  // extern "C"
