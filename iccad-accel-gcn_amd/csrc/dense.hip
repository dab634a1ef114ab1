// Z = X * W in fp32 on the matrix cores: the dense half of a GCN layer, whose result is the
// dense operand of the sparse product (upstream's operator stops at A * X, spmm_accel.cu:16-102;
// a layer around it multiplies the features by a weight matrix first).
//
// X is rows x K with rows in the millions and K, N in the tens to hundreds, so the product
// streams X once, writes Z once and keeps W on chip: 2 K N / (4 (K + N)) flops per byte, about
// the ratio of the fp32 matrix rate to the memory rate at K = 128, N = 64.  A workgroup of four
// wavefronts owns 128 rows of X and up to 128 columns of Z; each wavefront keeps a 32-row
// band of that as 32 x 32 accumulator tiles of v_mfma_f32_32x32x2_f32.  K is walked in steps
// of 32: the workgroup reads a step's 128 x 32 block of X (full 128-byte lines, eight lanes
// per row) into registers two steps ahead and its 32 x (32 NT) block of W one step ahead,
// while the matrix cores work on the steps before, then hands them over through LDS, where a
// lane finds its row's 16 values of the step as four 16-byte reads.
#include <atomic>

#include "internal.h"

namespace accel {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kDenseWaves = 4;                          // wavefronts per workgroup
constexpr int kDenseThreads = kDenseWaves * 64;
constexpr int kDenseRows = 32;                          // rows per wavefront (one MFMA tile high)
constexpr int kDenseBlockRows = kDenseWaves * kDenseRows;
constexpr int kDenseStep = 32;                          // columns of X (rows of W) per round: 16 MFMAs per tile
// Row stride of the X block in LDS, in floats: 16-byte reads of 16 lanes whose rows are 36
// floats apart fall into 16 different groups of four banks.
constexpr int kDenseXStride = kDenseStep + 4;
constexpr int kDenseXLoads = kDenseBlockRows * kDenseStep / 4 / kDenseThreads;     // 16-byte loads per thread and step: 4

// Operand layout of v_mfma_f32_32x32x2_f32 (one block): lane l holds A[l % 32][l / 32] and
// B[l / 32][l % 32]; accumulator register v of lane l is D[8 (v / 4) + 4 (l / 32) + v % 4][l % 32].
// The two k of one instruction need not be neighbours, only the same for A and B: lanes 0..31
// carry k0 + j, lanes 32..63 carry k0 + 16 + j, so that a lane's 16 values of A are 64
// consecutive bytes of its row.
//
// The grid is sized to what the GPU holds at once and every workgroup walks blocks of 128
// rows, gridDim.x apart, as one sequence of steps: the reads of a block's first step are
// issued while the matrix cores work on the last step of the block before, and that block's
// rows of Z are stored behind them, so the memory latency is paid once per workgroup, not
// once per block.  The column tiles of one block of rows (N > 128) follow each other in the
// same workgroup: the block of X they share comes from L2 for all but the first.

// A step of a workgroup's walk: rows [128 row_block, +128), columns [32 NT tile, +32 NT), k in [k0, k0 + 32).
struct DenseStepAt {
    int64_t row_block;
    int tile, k0;
    __device__ void advance(int K, int n_col_tiles, int64_t stride)
    {
        k0 += kDenseStep;
        if (k0 >= K) {
            k0 = 0;
            if (++tile == n_col_tiles) { tile = 0; row_block += stride; }
        }
    }
};

template <int NT, bool kVec>
__global__ __launch_bounds__(kDenseThreads, NT == 4 ? 2 : 3) void dense_xw_kernel(
    const float *__restrict__ X, const float *__restrict__ W, float *__restrict__ Z, int64_t rows, int K, int N,
    int64_t ldx, int64_t ldz, int64_t n_row_blocks, int n_col_tiles)
{
    constexpr int kCols = NT * 32;
    // two floats of padding put the rows k and k + 16, read together by the two halves of a
    // wavefront, 32 banks apart
    constexpr int kWStride = kCols + 2;
    constexpr int kWLoads = kDenseStep * kCols / kDenseThreads;             // 4 NT
    __shared__ __attribute__((aligned(16))) float x_lds[kDenseBlockRows * kDenseXStride];
    __shared__ float w_lds[kDenseStep * kWStride];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half = lane >> 5, l32 = lane & 31;
    const int xc = (tid & 7) * 4;              // this thread reads 16 bytes of row tid / 8 + 32 q, q = 0..3, per step

    // Registers for the blocks of X of the next two steps and the block of W of the next one:
    // a read from memory takes several steps' worth of matrix work under load, and what is in
    // flight per compute unit bounds the rate at which X streams in.
    float4 xreg[2][kDenseXLoads];
    float wreg[kWLoads];
    // Loads only, so that nothing waits for them here, and the same number of loads on every
    // path, which keeps the waits for them exact: with kVec (rows of X start on 16-byte
    // boundaries and K is a multiple of 4) four 16-byte loads, otherwise sixteen 4-byte loads,
    // from addresses clamped into the row.  What lies past K or N is replaced by zero when the
    // registers are handed to LDS.  Rows past the end of X read the last row (their results are
    // not stored), and so does a step past the end of the walk.
    // Each has a short form for the usual case, decided for the whole workgroup: a step that
    // lies inside K, rows inside X, a tile inside N need no clamping, and then the addresses
    // of a thread's loads are one base and constant strides (a few integer instructions per
    // step instead of a hundred, which would otherwise compete with the matrix instructions
    // for the issue slots of the SIMD).
    constexpr int kWRowsPerLoad = kDenseThreads / kCols;      // rows of W between a thread's loads
    auto fetch_x = [&](float4 (&dst)[kDenseXLoads], const DenseStepAt &at) {
        const int k = at.k0 + xc;
        const int64_t r0 = at.row_block * kDenseBlockRows + (tid >> 3);
        if (kVec && at.k0 + kDenseStep <= K && (at.row_block + 1) * kDenseBlockRows <= rows) {
            const float *xb = X + r0 * ldx + k;
#pragma unroll
            for (int q = 0; q < kDenseXLoads; q++)
                dst[q] = *reinterpret_cast<const float4 *>(xb + (int64_t)q * (kDenseThreads / 8) * ldx);
            return;
        }
#pragma unroll
        for (int q = 0; q < kDenseXLoads; q++) {
            const int64_t r = r0 + (kDenseThreads / 8) * q;
            const float *xr = X + (r < rows ? r : rows - 1) * ldx;
            if (kVec) {
                dst[q] = *reinterpret_cast<const float4 *>(xr + (k < K ? k : K - 4));
            } else {
                const int last = K - 1;
                dst[q].x = xr[k < last ? k : last];
                dst[q].y = xr[k + 1 < last ? k + 1 : last];
                dst[q].z = xr[k + 2 < last ? k + 2 : last];
                dst[q].w = xr[k + 3 < last ? k + 3 : last];
            }
        }
    };
    auto fetch_w = [&](const DenseStepAt &at) {
        const int k = at.k0 + tid / kCols, col = at.tile * kCols + tid % kCols;
        if (at.k0 + kDenseStep <= K && (at.tile + 1) * kCols <= N) {
            const float *wb = W + (int64_t)k * N + col;
#pragma unroll
            for (int i = 0; i < kWLoads; i++) wreg[i] = wb[(int64_t)i * kWRowsPerLoad * N];
            return;
        }
        const int cc = col < N ? col : N - 1;
#pragma unroll
        for (int i = 0; i < kWLoads; i++) {
            const int ki = k + kWRowsPerLoad * i;
            wreg[i] = W[(int64_t)(ki < K ? ki : K - 1) * N + cc];
        }
    };

    f32x16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

    const int64_t stride = gridDim.x;          // gridDim.x <= n_row_blocks: every workgroup has work
    DenseStepAt now{(int64_t)blockIdx.x, 0, 0}, next = now, after = now;
    next.advance(K, n_col_tiles, stride);
    after = next;
    after.advance(K, n_col_tiles, stride);
    fetch_x(xreg[0], now);
    fetch_w(now);
    fetch_x(xreg[1], next);

    // one step; `mine` is the half of xreg that holds its block of X
    auto step = [&](float4 (&mine)[kDenseXLoads]) {
        __syncthreads();                       // the previous step's reads of LDS are done
        float *xs = &x_lds[(tid >> 3) * kDenseXStride + xc];
        float *ws = &w_lds[(tid / kCols) * kWStride + tid % kCols];
        if (now.k0 + kDenseStep <= K && (now.tile + 1) * kCols <= N) {         // nothing to mask
#pragma unroll
            for (int q = 0; q < kDenseXLoads; q++)
                *reinterpret_cast<float4 *>(xs + q * (kDenseThreads / 8) * kDenseXStride) = mine[q];
#pragma unroll
            for (int i = 0; i < kWLoads; i++) ws[i * kWRowsPerLoad * kWStride] = wreg[i];
        } else {
            const int kx = now.k0 + xc;
            const int kw = now.k0 + tid / kCols;
            const bool col_inside = now.tile * kCols + tid % kCols < N;
#pragma unroll
            for (int q = 0; q < kDenseXLoads; q++) {
                float4 x = mine[q];
                x.x = kx < K ? x.x : 0.f; x.y = kx + 1 < K ? x.y : 0.f;
                x.z = kx + 2 < K ? x.z : 0.f; x.w = kx + 3 < K ? x.w : 0.f;
                *reinterpret_cast<float4 *>(xs + q * (kDenseThreads / 8) * kDenseXStride) = x;
            }
#pragma unroll
            for (int i = 0; i < kWLoads; i++)
                ws[i * kWRowsPerLoad * kWStride] = (col_inside && kw + kWRowsPerLoad * i < K) ? wreg[i] : 0.f;
        }
        __syncthreads();
        // in flight while the matrix cores work: W of the next step, X of the one after it
        fetch_w(next);
        fetch_x(mine, after);
        // the loads go out here, ahead of the matrix work that hides them, not behind it
        __builtin_amdgcn_sched_barrier(0);

        float a[16];
        const float4 *ap = reinterpret_cast<const float4 *>(&x_lds[(wave * kDenseRows + l32) * kDenseXStride + half * 16]);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 x = ap[q];
            a[4 * q] = x.x; a[4 * q + 1] = x.y; a[4 * q + 2] = x.z; a[4 * q + 3] = x.w;
        }
#pragma unroll
        for (int j = 0; j < 16; j++)
#pragma unroll
            for (int t = 0; t < NT; t++)
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], w_lds[(half * 16 + j) * kWStride + t * 32 + l32],
                                                              acc[t], 0, 0, 0);

        if (next.k0 == 0) {                    // that was the last step of this tile: store it, start the next at zero
            const int64_t row0 = now.row_block * kDenseBlockRows + wave * kDenseRows;
            const int col = now.tile * kCols + l32;
            float *z = Z + (row0 + 4 * half) * ldz + col;
            if (row0 + kDenseRows <= rows && now.tile * kCols + kCols <= N) {      // the usual case: nothing to mask
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < 16; v++) z[(8 * (v / 4) + v % 4) * ldz + t * 32] = acc[t][v];
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int64_t row = row0 + 8 * (v / 4) + 4 * half + (v % 4);
                        if (col + t * 32 < N && row < rows) z[(8 * (v / 4) + v % 4) * ldz + t * 32] = acc[t][v];
                    }
            }
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = 0.f;
        }
        now = next;
        next = after;
        after.advance(K, n_col_tiles, stride);
    };
    while (now.row_block < n_row_blocks) {
        step(xreg[0]);
        if (now.row_block >= n_row_blocks) break;
        step(xreg[1]);
    }
}

// The grid: as many workgroups as the GPU holds at once (asked of the runtime for the kernel
// that runs, once per device and kernel), or one per block of rows when there are fewer.
constexpr int kDenseDevices = 64;
static std::atomic<int> g_resident[kDenseDevices][6];     // [device][kernel]: workgroups the device holds, 0 = not asked yet

template <int NT, bool kVec>
static int dense_launch(hipStream_t s, const float *X, const float *W, float *Z, int64_t rows, int K, int N, int64_t ldx,
                        int64_t ldz, int64_t n_row_blocks, int n_col_tiles)
{
    constexpr int which = (NT == 1 ? 0 : NT == 2 ? 2 : 4) + (kVec ? 1 : 0);
    int dev = 0;
    ACCEL_HIP(hipGetDevice(&dev));
    int resident = dev >= 0 && dev < kDenseDevices ? g_resident[dev][which].load(std::memory_order_relaxed) : 0;
    if (resident == 0) {
        int cus = 0, per_cu = 0;
        ACCEL_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        ACCEL_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, dense_xw_kernel<NT, kVec>, kDenseThreads, 0));
        resident = (cus > 0 ? cus : 256) * (per_cu > 0 ? per_cu : 1);
        if (dev >= 0 && dev < kDenseDevices) g_resident[dev][which].store(resident, std::memory_order_relaxed);
    }
    const unsigned grid = (unsigned)(n_row_blocks < resident ? n_row_blocks : resident);
    dense_xw_kernel<NT, kVec><<<grid, kDenseThreads, 0, s>>>(X, W, Z, rows, K, N, ldx, ldz, n_row_blocks, n_col_tiles);
    return ACCEL_OK;
}

// Arguments have been checked by the caller (accel_dense_xw): rows >= 1, K, N >= 1,
// ldx >= K, ldz >= N, operands readable and large enough.
int dense_xw_launch(const float *X, const float *W, float *Z, int64_t rows, int K, int N, int64_t ldx, int64_t ldz,
                    hipStream_t stream)
{
    (void)hipGetLastError();
    const int nt = N <= 32 ? 1 : N <= 64 ? 2 : 4;
    const int n_col_tiles = (N + nt * 32 - 1) / (nt * 32);
    const int64_t n_row_blocks = (rows + kDenseBlockRows - 1) / kDenseBlockRows;
    // 16-byte reads of X need every row to start on a 16-byte boundary and to end on one
    const bool vec = (reinterpret_cast<uintptr_t>(X) % 16 == 0) && (ldx % 4 == 0) && (K % 4 == 0);
    int rc;
#define DENSE_CASE(NT_)                                                                                  \
    rc = vec ? dense_launch<NT_, true>(stream, X, W, Z, rows, K, N, ldx, ldz, n_row_blocks, n_col_tiles)  \
             : dense_launch<NT_, false>(stream, X, W, Z, rows, K, N, ldx, ldz, n_row_blocks, n_col_tiles)
    if (nt == 1) DENSE_CASE(1);
    else if (nt == 2) DENSE_CASE(2);
    else DENSE_CASE(4);
#undef DENSE_CASE
    if (rc) return rc;
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

}  // namespace accel
