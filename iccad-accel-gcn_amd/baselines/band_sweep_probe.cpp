// Measurement probe, outside the measured path: would it pay to walk the columns of X in
// bands, all wavefronts of a die working on the same band at the same time, so that an L2
// only has to hold one band of X?
//
// Every lane group of 16 lanes gathers `per_group` rows of 64 floats (16-byte loads, four in
// flight per lane) and adds them up, like the SpMM gather kernel does for N = 64.  The rows
// are random (uniform, or with the popularity of a power-law graph), and each group's list
// is ordered by band: the columns a die works on are cut into `intervals` consecutive
// ranges, and a group takes all its rows of range 0, then range 1, ...  With
// `die_partition` a die (workgroup i runs on die i % 8) only gets columns of its own
// eighth of X.  With `barrier` the workgroups of a die wait for each other between ranges
// (an arrival counter per die in device memory; the wait is bounded, so the kernel ends
// whatever happens).  One round: the grid is what the GPU holds at once.
//
//   band_sweep_probe <rows_of_X> <intervals> <per_group> <workgroups> <die_partition 0|1>
//                    <barrier 0|1> <popularity 0|1> [launches]
//
// Prints the best launch time and the gathered TB/s.  The reference point is
// intervals = 1 (no order at all).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                         \
    do {                                                              \
        hipError_t e_ = (x);                                          \
        if (e_ != hipSuccess) {                                       \
            std::printf("%s: %s\n", #x, hipGetErrorString(e_));       \
            return 1;                                                 \
        }                                                             \
    } while (0)

namespace {

constexpr int L = 16, G = 4, N = 64, U = 4, kDies = 8, kSpinLimit = 20000;

__global__ __launch_bounds__(256) void sweep_kernel(const int32_t *__restrict__ idx,
                                                    const int32_t *__restrict__ ends,
                                                    const float *__restrict__ X, float *__restrict__ Y,
                                                    int per_group, int intervals,
                                                    unsigned *__restrict__ arrivals, int wg_per_die,
                                                    int use_barrier, unsigned base)
{
    const int lane = threadIdx.x & 63, g = lane / L, sub = lane % L;
    const size_t group = ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * G + g;
    const int32_t *mine = idx + group * per_group;
    const int32_t *my_ends = ends + group * intervals;
    const int die = blockIdx.x % kDies;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    int i = 0;
    for (int b = 0; b < intervals; b++) {
        const int end = my_ends[b];
        for (; i + U <= end; i += U) {
            int32_t c[U];
            float4 x[U];
#pragma unroll
            for (int u = 0; u < U; u++) c[u] = mine[i + u];
#pragma unroll
            for (int u = 0; u < U; u++) x[u] = *reinterpret_cast<const float4 *>(X + (size_t)c[u] * N + sub * 4);
#pragma unroll
            for (int u = 0; u < U; u++) {
                acc.x += x[u].x; acc.y += x[u].y; acc.z += x[u].z; acc.w += x[u].w;
            }
        }
        for (; i < end; i++) {
            const float4 x = *reinterpret_cast<const float4 *>(X + (size_t)mine[i] * N + sub * 4);
            acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
        }
        if (use_barrier && b + 1 < intervals) {
            __syncthreads();
            if (threadIdx.x == 0) {
                unsigned *ctr = arrivals + die * 32;
                __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const unsigned target = base + (unsigned)(b + 1) * (unsigned)wg_per_die;
                for (int n = 0; n < kSpinLimit; n++) {       // bounded: every wavefront leaves
                    if ((int)(__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) >= 0) break;
                    __builtin_amdgcn_s_sleep(2);
                }
            }
            __syncthreads();
        }
    }
    if (acc.x == 12345.678f) *reinterpret_cast<float4 *>(Y + group * N + sub * 4) = acc;   // keeps the sums alive
}

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 8) {
        std::printf("usage: band_sweep_probe rows_of_X intervals per_group workgroups die_partition barrier "
                    "popularity [launches]\n");
        return 2;
    }
    const int64_t nx = atoll(argv[1]);
    const int intervals = atoi(argv[2]), per_group = atoi(argv[3]), wgs = atoi(argv[4]);
    const int diepart = atoi(argv[5]), barrier = atoi(argv[6]), popular = atoi(argv[7]);
    const int iters = argc > 8 ? atoi(argv[8]) : 5;
    if (nx < 64 || intervals < 1 || per_group < 1 || wgs < kDies || wgs % kDies || wgs > 4096) {
        std::printf("bad arguments (workgroups: a multiple of 8, at most 4096)\n");
        return 2;
    }
    const size_t groups = (size_t)wgs * 4 * G, n_idx = groups * per_group;
    std::vector<int32_t> h(n_idx), ends(groups * intervals);
    uint64_t state = 0x9E3779B97F4A7C15ull;
    auto rnd = [&]() {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return (double)(state >> 11) / 9007199254740992.0;
    };
    // popularity of a Chung-Lu graph with exponent 2.1 and a largest weight of 17,000 over 124 M
    // edges (rank ~ (x + i0)^(-1/1.1)); the ranks are scattered over the rows of X
    const double i0 = 584.4, ex = 1.0 - 1.0 / 1.1, pa = std::pow(i0, ex), pb = std::pow((double)nx + i0, ex);
    for (size_t gq = 0; gq < groups; gq++) {
        const int die = (int)(gq / (4 * G)) % kDies;
        const int64_t lo = diepart ? die * (nx / kDies) : 0, span = diepart ? nx / kDies : nx;
        int32_t *mine = h.data() + gq * per_group;
        for (int i = 0; i < per_group; i++) {
            int64_t c;
            if (popular) {
                for (;;) {
                    c = (int64_t)(std::pow(pa + rnd() * (pb - pa), 1.0 / ex) - i0);
                    c = (int64_t)(((uint64_t)std::max<int64_t>(c, 0) * 2654435761ull) % (uint64_t)nx);
                    if (c >= lo && c < lo + span) break;
                }
            } else {
                c = lo + (int64_t)(rnd() * span);
            }
            mine[i] = (int32_t)std::min<int64_t>(c, nx - 1);
        }
        std::sort(mine, mine + per_group);
        int s = 0;
        for (int b = 0; b < intervals; b++) {
            const int64_t hi = lo + span * (b + 1) / intervals;
            int e = b + 1 == intervals ? per_group : (int)(std::lower_bound(mine, mine + per_group, (int32_t)hi) - mine);
            ends[gq * intervals + b] = e;
            for (int j = e - 1; j > s; j--) std::swap(mine[j], mine[s + (int)(rnd() * (j - s + 1))]);   // random inside a range
            s = e;
        }
    }
    int32_t *idx = nullptr, *dends = nullptr;
    float *X = nullptr, *Y = nullptr;
    unsigned *arrivals = nullptr;
    CK(hipMalloc((void **)&idx, n_idx * 4));
    CK(hipMalloc((void **)&dends, ends.size() * 4));
    CK(hipMalloc((void **)&X, (size_t)nx * N * 4));
    CK(hipMalloc((void **)&Y, groups * N * 4));
    CK(hipMalloc((void **)&arrivals, kDies * 32 * 4));
    CK(hipMemcpy(idx, h.data(), n_idx * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(dends, ends.data(), ends.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemset(X, 0, (size_t)nx * N * 4));
    CK(hipMemset(arrivals, 0, kDies * 32 * 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float best = 1e30f;
    for (int it = 0; it <= iters; it++) {
        CK(hipEventRecord(e0, nullptr));
        sweep_kernel<<<dim3(wgs), dim3(256)>>>(idx, dends, X, Y, per_group, intervals, arrivals, wgs / kDies, barrier,
                                              (unsigned)it * (unsigned)(intervals - 1) * (unsigned)(wgs / kDies));
        CK(hipEventRecord(e1, nullptr));
        CK(hipEventSynchronize(e1));
        float t;
        CK(hipEventElapsedTime(&t, e0, e1));
        if (it > 0 && t < best) best = t;
    }
    std::printf("X: %lld rows of 64 floats, %d ranges per die, %d gathers per lane group, %d workgroups, "
                "die partition %d, barrier %d, popularity %d: %.3f ms, %.2f TB/s gathered (%.2f GB)\n",
                (long long)nx, intervals, per_group, wgs, diepart, barrier, popular, best,
                n_idx * 256.0 / best / 1e9, n_idx * 256.0 / 1e9);
    return 0;
}
