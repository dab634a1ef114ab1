// Measurement probe, outside the measured path: what rate of row gathers does the GPU
// sustain when a kernel does nothing else?  Every lane group of L lanes loads random
// rows of N floats (N = 4 * L, 16-byte loads, four in flight per lane) from an array of
// n_rows_x rows and adds them up; optionally it stores one result row per `row_len`
// gathers, with ordinary or with non-temporal stores.  The SpMM gather kernel is judged
// against these rates (they bound it from above for the same access pattern).
//
// Lives in libaccelgcn_baselines.so; the product library does not contain it.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

namespace {

thread_local char g_probe_err[256] = "";
int probe_fail(const char *what, int code)
{
    snprintf(g_probe_err, sizeof g_probe_err, "%s failed with status %d", what, code);
    return -1;
}

#define PROBE_HIP(call)                                                  \
    do {                                                                 \
        hipError_t e_ = (call);                                          \
        if (e_ != hipSuccess) return probe_fail(#call, (int)e_);         \
    } while (0)

constexpr int kInFlight = 4;

// stores: 0 none (the sum is kept alive by an impossible comparison), 1 ordinary, 2 non-temporal
template <int L>
__global__ __launch_bounds__(256) void gather_probe_kernel(const int32_t *__restrict__ idx,
                                                           const float *__restrict__ X,
                                                           float *__restrict__ Y, int per_group,
                                                           int row_len, int stores)
{
    constexpr int G = 64 / L, N = 4 * L;
    const int lane = threadIdx.x & 63, g = lane / L, sub = lane % L;
    const size_t group = ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * G + g;
    const int32_t *mine = idx + group * per_group;
    size_t out_row = group * (size_t)(per_group / row_len);
    for (int r0 = 0; r0 < per_group; r0 += row_len, out_row++) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int i = r0; i < r0 + row_len; i += kInFlight) {
            int32_t c[kInFlight];
            float4 x[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; u++) c[u] = mine[i + u];
#pragma unroll
            for (int u = 0; u < kInFlight; u++)
                x[u] = *reinterpret_cast<const float4 *>(X + (size_t)c[u] * N + sub * 4);
#pragma unroll
            for (int u = 0; u < kInFlight; u++) {
                acc.x += x[u].x; acc.y += x[u].y; acc.z += x[u].z; acc.w += x[u].w;
            }
        }
        float *dst = Y + out_row * N + sub * 4;
        typedef float v4f __attribute__((ext_vector_type(4)));
        if (stores == 2) {
            const v4f t = {acc.x, acc.y, acc.z, acc.w};
            __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(dst));
        } else if (stores == 1 || acc.x == 12345.678f) {
            *reinterpret_cast<float4 *>(dst) = acc;
        }
    }
}

}  // namespace

extern "C" {

const char *baseline_gather_probe_last_error(void) { return g_probe_err; }

// n_rows_x rows of N floats (N = 16, 64 or 256) are gathered `gathers_per_group` times by each
// of 65,536 * (256 / N) lane groups; row_len (a multiple of 4 that divides gathers_per_group)
// gathers form one result row.  *ms receives the best of `iters` launches after one warm-up,
// *bytes_gathered and *bytes_stored the bytes one launch moves.
int baseline_gather_probe(int64_t n_rows_x, int32_t N, int32_t gathers_per_group, int32_t row_len,
                          int32_t stores, int32_t iters, float *ms, double *bytes_gathered,
                          double *bytes_stored)
{
    if (n_rows_x <= 0 || (N != 16 && N != 64 && N != 256) || gathers_per_group <= 0 || row_len <= 0 ||
        row_len % kInFlight || gathers_per_group % row_len || stores < 0 || stores > 2 || iters <= 0 || !ms)
        return probe_fail("argument check", 1);
    const int L = N / 4, G = 64 / L;
    const int waves = 256 * 32 * 8;
    const size_t groups = (size_t)waves * G, n_idx = groups * gathers_per_group;
    const size_t y_rows = groups * (size_t)(gathers_per_group / row_len);
    std::vector<int32_t> h(n_idx);
    uint64_t state = 0x9E3779B97F4A7C15ull;
    for (auto &v : h) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        v = (int32_t)((state >> 33) % (uint64_t)n_rows_x);
    }
    int32_t *idx = nullptr;
    float *X = nullptr, *Y = nullptr;
    PROBE_HIP(hipMalloc(reinterpret_cast<void **>(&idx), n_idx * 4));
    PROBE_HIP(hipMalloc(reinterpret_cast<void **>(&X), (size_t)n_rows_x * N * 4));
    PROBE_HIP(hipMalloc(reinterpret_cast<void **>(&Y), y_rows * N * 4));
    PROBE_HIP(hipMemcpy(idx, h.data(), n_idx * 4, hipMemcpyHostToDevice));
    PROBE_HIP(hipMemset(X, 0, (size_t)n_rows_x * N * 4));
    hipEvent_t e0, e1;
    PROBE_HIP(hipEventCreate(&e0));
    PROBE_HIP(hipEventCreate(&e1));
    float best = 1e30f;
    for (int it = 0; it <= iters; it++) {
        PROBE_HIP(hipEventRecord(e0, nullptr));
        if (N == 16)
            gather_probe_kernel<4><<<dim3(waves / 4), dim3(256)>>>(idx, X, Y, gathers_per_group, row_len, stores);
        else if (N == 64)
            gather_probe_kernel<16><<<dim3(waves / 4), dim3(256)>>>(idx, X, Y, gathers_per_group, row_len, stores);
        else
            gather_probe_kernel<64><<<dim3(waves / 4), dim3(256)>>>(idx, X, Y, gathers_per_group, row_len, stores);
        PROBE_HIP(hipEventRecord(e1, nullptr));
        PROBE_HIP(hipEventSynchronize(e1));
        float t = 0.f;
        PROBE_HIP(hipEventElapsedTime(&t, e0, e1));
        if (it > 0 && t < best) best = t;
    }
    PROBE_HIP(hipGetLastError());
    (void)hipFree(idx);
    (void)hipFree(X);
    (void)hipFree(Y);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *ms = best;
    if (bytes_gathered) *bytes_gathered = (double)n_idx * N * 4.0;
    if (bytes_stored) *bytes_stored = stores ? (double)y_rows * N * 4.0 : 0.0;
    return 0;
}

}  // extern "C"
