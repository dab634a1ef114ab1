// GPU preprocessing for the SpMM operator: CSR validation, stable degree sort,
// permuted-CSR gather and the block4 partition metadata.  Integer, HBM-bound
// work; every kernel is a streaming pass over rows or non-zeros.
//
// The metadata rules are those of upstream's block_level_partition.py:7-21
// (tables) and :48-103 (walk); the walk is restated as a closed form per row so
// that it runs as scans + one emit kernel:
//   - a row of degree d in 1..384 that sits (r - s) rows into its maximal run of
//     equal-degree rows (run start s) opens a block iff (r - s) % rows[d] == 0;
//     the block takes up to rows[d] rows of that run;
//   - a row of degree d > 384 opens ceil(d / 384) blocks;
//   - rows of degree 0 open none.
#include <algorithm>
#include <chrono>
#include <climits>
#include <vector>

#include "internal.h"

namespace accel {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;  // elements per workgroup in scans and sort passes

struct SumOp {
    static constexpr int identity = 0;
    __device__ int operator()(int a, int b) const { return a + b; }
};
struct MaxOp {
    static constexpr int identity = INT_MIN;
    __device__ int operator()(int a, int b) const { return a > b ? a : b; }
};

// Exclusive scan of one value per thread over a 256-thread workgroup.
template <class Op>
__device__ int block_exclusive_scan(int v, Op op, int *wave_tot /* LDS, 4 ints */, int &total)
{
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(inc, off);
        if (lane >= off) inc = op(t, inc);
    }
    if (lane == 63) wave_tot[w] = inc;
    __syncthreads();
    int prefix = Op::identity, tot = Op::identity;
#pragma unroll
    for (int i = 0; i < kThreads / 64; i++) {
        const int t = wave_tot[i];
        if (i < w) prefix = op(prefix, t);
        tot = op(tot, t);
    }
    __syncthreads();
    int exc = __shfl_up(inc, 1);
    if (lane == 0) exc = Op::identity;
    total = tot;
    return op(prefix, exc);
}

template <class Op>
__global__ __launch_bounds__(kThreads) void scan_reduce(const int *__restrict__ in, int64_t n,
                                                        int *__restrict__ sums)
{
    __shared__ int wave_tot[kThreads / 64];
    Op op;
    const int64_t base = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x * kItems;
    int acc = Op::identity;
#pragma unroll
    for (int j = 0; j < kItems; j++)
        if (base + j < n) acc = op(acc, in[base + j]);
    int total;
    block_exclusive_scan(acc, op, wave_tot, total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// One workgroup turns sums[0..nb) into their exclusive scan and stores the grand
// total at sums[nb].
template <class Op>
__global__ __launch_bounds__(kThreads) void scan_spine(int *__restrict__ sums, int64_t nb)
{
    __shared__ int wave_tot[kThreads / 64];
    Op op;
    int carry = Op::identity;
    for (int64_t base = 0; base < nb; base += kThreads) {
        const int64_t i = base + threadIdx.x;
        const int v = i < nb ? sums[i] : Op::identity;
        int total;
        const int exc = block_exclusive_scan(v, op, wave_tot, total);
        if (i < nb) sums[i] = op(carry, exc);
        carry = op(carry, total);
    }
    if (threadIdx.x == 0) sums[nb] = carry;
}

template <class Op, bool kInclusive>
__global__ __launch_bounds__(kThreads) void scan_apply(const int *__restrict__ in, int64_t n,
                                                       const int *__restrict__ sums,
                                                       int *__restrict__ out,
                                                       int *__restrict__ total_out, int64_t nb)
{
    __shared__ int wave_tot[kThreads / 64];
    Op op;
    const int64_t base = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x * kItems;
    int v[kItems];
    int acc = Op::identity;
#pragma unroll
    for (int j = 0; j < kItems; j++) {
        v[j] = base + j < n ? in[base + j] : Op::identity;
        acc = op(acc, v[j]);
    }
    int total;
    int run = op(sums[blockIdx.x], block_exclusive_scan(acc, op, wave_tot, total));
#pragma unroll
    for (int j = 0; j < kItems; j++) {
        const int inc = op(run, v[j]);
        if (base + j < n) out[base + j] = kInclusive ? inc : run;
        run = inc;
    }
    if (total_out && blockIdx.x == 0 && threadIdx.x == 0) *total_out = sums[nb];
}

// out = scan(in) over n ints (in place allowed); *total_out (device, optional)
// receives the reduction of all n.  `sums` needs n/kTile + 2 ints.
template <class Op, bool kInclusive>
int device_scan(const int *in, int64_t n, int *out, int *total_out, int *sums, hipStream_t s)
{
    if (n <= 0) {
        if (total_out) return fill_u32(total_out, (uint32_t)Op::identity, 1, s);
        return ACCEL_OK;
    }
    const int64_t nb = (n + kTile - 1) / kTile;
    scan_reduce<Op><<<dim3((unsigned)nb), dim3(kThreads), 0, s>>>(in, n, sums);
    scan_spine<Op><<<dim3(1), dim3(kThreads), 0, s>>>(sums, nb);
    scan_apply<Op, kInclusive><<<dim3((unsigned)nb), dim3(kThreads), 0, s>>>(in, n, sums, out,
                                                                            total_out, nb);
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

// ---------------------------------------------------------------------------
// CSR validation + degrees
// ---------------------------------------------------------------------------
struct Stats {
    int bad_indptr;     // non-monotone / wrong ends
    int bad_index;      // column outside [0, cols)
    int unsorted;       // some row has a smaller degree than its predecessor
    int max_degree;
    int n_zero_rows;
    int n_long_rows;
    int n_long_blocks;
    int n_split_rows;   // rows with more non-zeros than the plan's split threshold
    int n_big_rows;     // rows with more than 32 times that
    int n_split_rows_alt, n_big_rows_alt;   // the same two for the alternative threshold
    int n_wide_rows;    // rows with more than kGroupWaveMax non-zeros
    int hist[kDegBound + 1];   // rows of each degree 0..384 (what sizes the partition on the host)
    int sampled_nz;     // non-zeros looked at by locality_kernel
    int local_nz;       // ... whose column lies near their row
};

// Split rows of up to this many non-zeros are regrouped by one wavefront each, longer ones
// by a workgroup each (group_long_rows_*).
constexpr int kGroupWaveMax = 1024;

__global__ __launch_bounds__(kThreads) void degree_kernel(const int32_t *__restrict__ indptr,
                                                          int64_t rows, int64_t nnz,
                                                          uint32_t *__restrict__ deg,
                                                          Stats *__restrict__ st, int split_deg,
                                                          int alt_split_deg)
{
    // grid-stride over rows; one set of atomics per workgroup
    __shared__ int part[kThreads / 64][11];
    __shared__ int hist[kDegBound + 1];
    for (int i = threadIdx.x; i <= kDegBound; i += kThreads) hist[i] = 0;
    __syncthreads();
    int bad = 0, unsorted = 0, dmax = 0, zero = 0, lrow = 0, lblk = 0, srow = 0, brow = 0, srow2 = 0, brow2 = 0;
    int wrow = 0;
    for (int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x; r < rows;
         r += (int64_t)gridDim.x * kThreads) {
        const int a = indptr[r], b = indptr[r + 1];
        int d = b - a;
        bool row_bad = b < a;
        if (row_bad) d = 0;
        if (r == 0 && a != 0) row_bad = true;
        if (r == rows - 1 && (int64_t)b != nnz) row_bad = true;
        if (r > 0 && !row_bad && d < a - indptr[r - 1]) unsorted = 1;
        bad |= row_bad;
        deg[r] = (uint32_t)d;
        dmax = max(dmax, d);
        zero += d == 0;
        if (d > kDegBound) { lrow++; lblk += (d + kDegBound - 1) / kDegBound; }
        srow += d > split_deg;
        brow += d > 32 * split_deg;
        srow2 += d > alt_split_deg;
        brow2 += d > 32 * alt_split_deg;
        wrow += d > kGroupWaveMax;
        if (!row_bad && d <= kDegBound) atomicAdd(&hist[d], 1);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        bad |= __shfl_xor(bad, off);
        unsorted |= __shfl_xor(unsorted, off);
        dmax = max(dmax, __shfl_xor(dmax, off));
        zero += __shfl_xor(zero, off);
        lrow += __shfl_xor(lrow, off);
        lblk += __shfl_xor(lblk, off);
        srow += __shfl_xor(srow, off);
        brow += __shfl_xor(brow, off);
        srow2 += __shfl_xor(srow2, off);
        brow2 += __shfl_xor(brow2, off);
        wrow += __shfl_xor(wrow, off);
    }
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        part[w][0] = bad; part[w][1] = unsorted; part[w][2] = dmax;
        part[w][3] = zero; part[w][4] = lrow; part[w][5] = lblk; part[w][6] = srow; part[w][7] = brow;
        part[w][8] = srow2; part[w][9] = brow2; part[w][10] = wrow;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int q = 1; q < kThreads / 64; q++) {
            bad |= part[q][0]; unsorted |= part[q][1]; dmax = max(dmax, part[q][2]);
            zero += part[q][3]; lrow += part[q][4]; lblk += part[q][5]; srow += part[q][6]; brow += part[q][7];
            srow2 += part[q][8]; brow2 += part[q][9]; wrow += part[q][10];
        }
        if (bad) atomicOr(&st->bad_indptr, 1);
        if (unsorted) atomicOr(&st->unsorted, 1);
        if (dmax > 0) atomicMax(&st->max_degree, dmax);
        if (zero) atomicAdd(&st->n_zero_rows, zero);
        if (lrow) atomicAdd(&st->n_long_rows, lrow);
        if (lblk) atomicAdd(&st->n_long_blocks, lblk);
        if (srow) atomicAdd(&st->n_split_rows, srow);
        if (brow) atomicAdd(&st->n_big_rows, brow);
        if (srow2) atomicAdd(&st->n_split_rows_alt, srow2);
        if (brow2) atomicAdd(&st->n_big_rows_alt, brow2);
        if (wrow) atomicAdd(&st->n_wide_rows, wrow);
    }
    for (int i = threadIdx.x; i <= kDegBound; i += kThreads)      // after the barrier above: hist is complete
        if (hist[i]) atomicAdd(&st->hist[i], hist[i]);
}

// Does the matrix have its non-zeros near the diagonal (of the rows x cols rectangle)?
// Every kLocalityStride-th row contributes up to kLocalitySample of its non-zeros, evenly spaced; one counts
// as local when its column is within `band` columns of the row's place.  Rows whose indptr
// entries point outside [0, nnz) are skipped (degree_kernel reports them).
constexpr int kLocalityStride = 16, kLocalitySample = 16;
__global__ __launch_bounds__(kThreads) void locality_kernel(const int32_t *__restrict__ indptr,
                                                            const int32_t *__restrict__ idx, int64_t rows,
                                                            int64_t cols, int64_t nnz, int band,
                                                            Stats *__restrict__ st)
{
    const int64_t r = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * kLocalityStride;
    int seen = 0, local = 0;
    if (r < rows) {
        int a = indptr[r], d = indptr[r + 1] - a;
        if (a < 0 || d < 0 || (int64_t)a + d > nnz) d = 0;     // invalid indptr: reported by degree_kernel
        const int n = min(d, kLocalitySample);
        const int64_t place = rows > 1 ? r * (cols - 1) / (rows - 1) : 0;
        for (int i = 0; i < n; i++) {                    // spread over the row, whatever its order
            const int64_t off = (int64_t)idx[a + (int)((int64_t)i * d / n)] - place;
            local += (off < 0 ? -off : off) <= band;
        }
        seen = n;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        seen += __shfl_xor(seen, off);
        local += __shfl_xor(local, off);
    }
    if ((threadIdx.x & 63) == 0 && seen) {
        atomicAdd(&st->sampled_nz, seen);
        atomicAdd(&st->local_nz, local);
    }
}

__global__ __launch_bounds__(kThreads) void index_check_kernel(const int32_t *__restrict__ idx,
                                                               int64_t nnz, int64_t cols,
                                                               Stats *__restrict__ st)
{
    // 16-byte loads over the aligned middle of the array, single words at its two ends
    int bad = 0;
    auto look = [&](int c) { bad |= (c < 0) | ((int64_t)c >= cols); };
    const int64_t tid = (int64_t)blockIdx.x * kThreads + threadIdx.x, step = (int64_t)gridDim.x * kThreads;
    int64_t head = (int64_t)((16 - (reinterpret_cast<uintptr_t>(idx) & 15)) & 15) / 4;
    if (head > nnz) head = nnz;
    const int64_t n4 = (nnz - head) / 4;
    const int4 *v = reinterpret_cast<const int4 *>(idx + head);
    for (int64_t i = tid; i < n4; i += step) {
        const int4 c = v[i];
        look(c.x); look(c.y); look(c.z); look(c.w);
    }
    for (int64_t p = tid; p < head; p += step) look(idx[p]);
    for (int64_t p = head + 4 * n4 + tid; p < nnz; p += step) look(idx[p]);
    if (__ballot(bad) && (threadIdx.x & 63) == 0) atomicOr(&st->bad_index, 1);
}

// ---------------------------------------------------------------------------
// Stable LSD radix sort of (degree, row) pairs, 8 bits per pass.  Stability is
// what makes ties keep the caller's row order.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void radix_hist(const uint32_t *__restrict__ keys,
                                                       int64_t n, int shift,
                                                       int *__restrict__ hist, int64_t tiles)
{
    __shared__ int h[256];
    h[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kTile;
#pragma unroll
    for (int j = 0; j < kItems; j++) {
        const int64_t i = base + j * kThreads + threadIdx.x;
        if (i < n) atomicAdd(&h[(keys[i] >> shift) & 255u], 1);
    }
    __syncthreads();
    hist[(int64_t)threadIdx.x * tiles + blockIdx.x] = h[threadIdx.x];  // digit-major
}

__global__ __launch_bounds__(kThreads) void radix_scatter(
    const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
    uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out, int64_t n, int shift,
    const int *__restrict__ hist_scanned, int64_t tiles)
{
    __shared__ int running[256];               // next output slot of each digit for this tile
    __shared__ int wave_cnt[kThreads / 64][256];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    running[threadIdx.x] = hist_scanned[(int64_t)threadIdx.x * tiles + blockIdx.x];
    const int64_t base = (int64_t)blockIdx.x * kTile;
    for (int j = 0; j < kItems; j++) {
        const int64_t i = base + j * kThreads + threadIdx.x;
        const bool valid = i < n;
        const uint32_t key = valid ? keys_in[i] : 0u;
        const uint32_t val = valid ? (vals_in ? vals_in[i] : (uint32_t)i) : 0u;
        const uint32_t dg = (key >> shift) & 255u;
#pragma unroll
        for (int q = 0; q < kThreads / 64; q++) wave_cnt[q][threadIdx.x] = 0;
        __syncthreads();
        // lanes of this wave that hold the same digit
        unsigned long long peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const bool bit = (dg >> b) & 1u;
            const unsigned long long bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        const int rank = __popcll(peers & ((1ull << lane) - 1ull));
        if (valid && rank == 0) wave_cnt[w][dg] = __popcll(peers);
        __syncthreads();
        if (valid) {
            int pos = running[dg] + rank;
            for (int q = 0; q < w; q++) pos += wave_cnt[q][dg];
            keys_out[pos] = key;
            vals_out[pos] = val;
        }
        __syncthreads();
        int add = 0;
#pragma unroll
        for (int q = 0; q < kThreads / 64; q++) add += wave_cnt[q][threadIdx.x];
        running[threadIdx.x] += add;
    }
}

__global__ __launch_bounds__(kThreads) void iota_kernel(uint32_t *out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) out[i] = (uint32_t)i;
}

// Temporaries of one preprocessing call come out of a few large device allocations
// instead of one hipMalloc / hipFree each (a pair costs about 0.2 ms, and there are
// some twenty temporaries).  Chunks are freed when the arena goes out of scope.
struct Arena {
    static constexpr int kMaxChunks = 32;
    char *chunk[kMaxChunks] = {};
    size_t cap = 0, used = 0;      // of the newest chunk
    int n_chunks = 0;
    size_t next_chunk = 0;         // size hint for the next chunk
    ~Arena()
    {
        for (int i = 0; i < n_chunks; i++) (void)hipFree(chunk[i]);
    }
    void *take(size_t bytes)
    {
        bytes = (std::max<size_t>(bytes, 4) + 255) & ~(size_t)255;
        if (n_chunks == 0 || used + bytes > cap) {
            if (n_chunks == kMaxChunks) return nullptr;
            const size_t want = std::max(bytes, next_chunk);
            void *p = nullptr;
            if (hipMalloc(&p, want) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
            chunk[n_chunks++] = static_cast<char *>(p);
            cap = want;
            used = 0;
            next_chunk = std::max<size_t>(next_chunk / 4, (size_t)1 << 20);   // later chunks: leftovers only
        }
        void *p = chunk[n_chunks - 1] + used;
        used += bytes;
        return p;
    }
};

struct DevBuf {  // frees on scope exit; with an arena, the arena owns the memory
    void *p = nullptr;
    Arena *arena = nullptr;
    DevBuf() = default;
    explicit DevBuf(Arena *a) : arena(a) {}
    DevBuf(const DevBuf &) = delete;
    DevBuf &operator=(const DevBuf &) = delete;
    ~DevBuf() { if (p && !arena) (void)hipFree(p); }
    int alloc(size_t bytes)
    {
        if (arena) {
            p = arena->take(bytes);
        } else if (hipMalloc(&p, bytes ? bytes : 4) != hipSuccess) {
            p = nullptr;
            (void)hipGetLastError();
        }
        if (!p) {
            set_error("device allocation of %zu bytes failed", bytes);
            return ACCEL_ERR_ALLOC;
        }
        return ACCEL_OK;
    }
    template <class T> T *as() { return static_cast<T *>(p); }
    void *release() { void *q = p; p = nullptr; return q; }   // only for buffers without an arena
};

struct DevView {  // a part of a larger allocation, with DevBuf's accessors
    void *p = nullptr;
    template <class T> T *as() { return static_cast<T *>(p); }
};

inline unsigned grid_for(int64_t n) { return (unsigned)((n + kThreads - 1) / kThreads); }
// Workgroups of degree_kernel: each ends with a dozen atomics on the same few words, which
// the memory system applies one after the other (2,048 workgroups: 160 us on 2.45 M rows,
// almost all of it those atomics).
constexpr unsigned kDegreeGroups = 256;

// Sorts n (key, position) pairs by key, stably, in as many 8-bit passes as max_key needs.
// keys is used as one of the two key buffers; *sorted_keys / *sorted_vals point at the
// results (vals = original positions).  With max_key == 0 nothing moves.
int radix_sort_pairs(Arena *tmp, uint32_t *keys, int64_t n, uint32_t max_key, hipStream_t s,
                     uint32_t **sorted_keys, uint32_t **sorted_vals)
{
    DevBuf keys_b(tmp), vals_a(tmp), vals_b(tmp), hist(tmp), sums(tmp);
    const int64_t tiles = (n + kTile - 1) / kTile;
    int rc;
    if ((rc = keys_b.alloc(sizeof(uint32_t) * (size_t)n))) return rc;
    if ((rc = vals_a.alloc(sizeof(uint32_t) * (size_t)n))) return rc;
    if ((rc = vals_b.alloc(sizeof(uint32_t) * (size_t)n))) return rc;
    if ((rc = hist.alloc(sizeof(int) * (size_t)(256 * tiles)))) return rc;
    if ((rc = sums.alloc(sizeof(int) * (size_t)(256 * tiles / kTile + 4)))) return rc;
    int bits = 0;
    while (bits < 32 && (max_key >> bits) != 0) bits++;
    uint32_t *kin = keys, *kout = keys_b.as<uint32_t>();
    uint32_t *vin = nullptr, *vout = vals_a.as<uint32_t>();
    for (int shift = 0; shift < bits; shift += 8) {
        radix_hist<<<dim3((unsigned)tiles), dim3(kThreads), 0, s>>>(kin, n, shift, hist.as<int>(), tiles);
        if ((rc = device_scan<SumOp, false>(hist.as<int>(), 256 * tiles, hist.as<int>(), nullptr,
                                            sums.as<int>(), s)))
            return rc;
        radix_scatter<<<dim3((unsigned)tiles), dim3(kThreads), 0, s>>>(kin, vin, kout, vout, n, shift,
                                                                     hist.as<int>(), tiles);
        std::swap(kin, kout);
        vin = vout;
        vout = (vout == vals_a.as<uint32_t>()) ? vals_b.as<uint32_t>() : vals_a.as<uint32_t>();
    }
    if (!vin) {                                        // no pass ran: positions in order
        iota_kernel<<<dim3((unsigned)((n + kThreads - 1) / kThreads)), dim3(kThreads), 0, s>>>(
            vals_a.as<uint32_t>(), n);
        vin = vals_a.as<uint32_t>();
    }
    ACCEL_HIP(hipGetLastError());
    *sorted_keys = kin;
    *sorted_vals = vin;
    return ACCEL_OK;
}

// ---------------------------------------------------------------------------
// Permuted CSR: non-zero p of the sorted matrix comes from the caller's row
// perm[r], where r is the sorted row that contains p.
// ---------------------------------------------------------------------------
constexpr int kPermuteNz = 4;                        // non-zeros per thread
constexpr int kPermuteTile = kThreads * kPermuteNz;  // non-zeros per workgroup

// tile_first[t] = the sorted row that holds non-zero t * kPermuteTile of the sorted matrix,
// for every tile that starts before n_take.  One thread per row: a row writes the entry of
// every tile boundary that falls inside it (rows without non-zeros write none).
__global__ __launch_bounds__(kThreads) void tile_first_kernel(const int32_t *__restrict__ s_indptr,
                                                              int64_t rows, int64_t n_take,
                                                              int *__restrict__ tile_first)
{
    const int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (r >= rows) return;
    const int64_t a = s_indptr[r], b = min((int64_t)s_indptr[r + 1], n_take);
    for (int64_t t = (a + kPermuteTile - 1) / kPermuteTile; t * kPermuteTile < b; t++) tile_first[t] = (int)r;
}

// A workgroup copies kPermuteTile consecutive non-zeros of the sorted matrix.  They belong
// to consecutive sorted rows, from tile_first[this tile] to tile_first[next tile] (at most
// kPermuteTile + 1 rows, each but the first starting inside the tile), whose boundaries and
// source offsets are put in LDS once; each thread then finds the row of its non-zeros by a
// search in LDS.  last_row = the row that holds non-zero n_take - 1.
__global__ __launch_bounds__(kThreads) void permute_csr_kernel(
    const int32_t *__restrict__ indptr, const int32_t *__restrict__ idx,
    const float *__restrict__ val, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ s_indptr, const int *__restrict__ tile_first, int64_t last_row,
    int64_t n_take, int32_t *__restrict__ s_idx, float *__restrict__ s_val, int32_t *__restrict__ src_pos)
{
    __shared__ int row_end[kPermuteTile + 1];        // s_indptr[first + j + 1]
    __shared__ int64_t shift[kPermuteTile + 1];      // source position minus sorted position, per row
    const int64_t p0 = (int64_t)blockIdx.x * kPermuteTile;
    const int64_t p1 = min(p0 + kPermuteTile, n_take);   // this workgroup copies [p0, p1)
    const int64_t first_row = tile_first[blockIdx.x];
    const int64_t end_row = blockIdx.x + 1 < gridDim.x ? (int64_t)tile_first[blockIdx.x + 1] : last_row;
    const int n_here = (int)min((int64_t)kPermuteTile + 1, end_row - first_row + 1);
    for (int j = threadIdx.x; j < n_here; j += kThreads) {
        const int64_t r = first_row + j;
        row_end[j] = s_indptr[r + 1];
        shift[j] = (int64_t)indptr[perm ? perm[r] : r] - (int64_t)s_indptr[r];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kPermuteNz; q++) {
        const int64_t p = p0 + (int64_t)q * kThreads + threadIdx.x;
        if (p >= p1) break;
        int lo = 0, hi = n_here - 1;                 // first j with row_end[j] > p
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if ((int64_t)row_end[mid] > p) hi = mid; else lo = mid + 1;
        }
        const int64_t src = p + shift[lo];
        if (s_idx) s_idx[p] = idx[src];
        if (s_val) s_val[p] = val[src];
        if (src_pos) src_pos[p] = (int32_t)src;      // where the non-zero sits in the caller's arrays
    }
}

// ---------------------------------------------------------------------------
// Split rows: the row's non-zeros are written to the sorted CSR grouped by
// col_group(column, row_groups(degree)), stably inside each group, so that a
// work unit of such a row touches rows of X that belong to one column group.
// One workgroup per split row; counts[lr*64 + g] receives the size of each group
// (counts may be null).  Each of the three outputs may be null: the columns, the values,
// and src_pos, the position of each non-zero in the caller's arrays (what a later value
// update gathers through).
// ---------------------------------------------------------------------------
constexpr int kGroupRound = 4;   // elements per thread between two barriers of group_long_rows_kernel

__global__ __launch_bounds__(kThreads) void group_long_rows_kernel(
    const int32_t *__restrict__ indptr, const int32_t *__restrict__ idx,
    const float *__restrict__ val, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ s_indptr, int64_t first_long_row, int forced_groups,
    int32_t *__restrict__ s_idx, float *__restrict__ s_val, int *__restrict__ counts,
    int32_t *__restrict__ src_pos)
{
    __shared__ int cnt[kMaxGroups];
    __shared__ int base[kMaxGroups];
    // members of each group per (sub-round, wavefront); two copies used in turn
    __shared__ int wave_cnt[2][kGroupRound][kThreads / 64][kMaxGroups];
    const int64_t r = first_long_row + blockIdx.x;
    const int64_t src0 = indptr[perm ? perm[r] : r];
    const int64_t dst0 = s_indptr[r];
    const int d = s_indptr[r + 1] - s_indptr[r];
    const int ng = row_groups(d, forced_groups);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if ((int)threadIdx.x < kMaxGroups) cnt[threadIdx.x] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < d; i += kThreads) atomicAdd(&cnt[col_group(idx[src0 + i], ng)], 1);
    __syncthreads();
    if ((int)threadIdx.x < kMaxGroups) {              // groups beyond ng stay empty
        int b = 0;
        for (int g = 0; g < (int)threadIdx.x; g++) b += cnt[g];
        base[threadIdx.x] = b;
        if (counts) counts[(int64_t)blockIdx.x * kMaxGroups + threadIdx.x] = cnt[threadIdx.x];
    }
    __syncthreads();
    // A round places kGroupRound * 256 consecutive non-zeros; inside a round the order is
    // sub-round, then wavefront, then lane, which is the order of the row (the result is the
    // stable partition by group).  Long rows are a chain of rounds, so a round does as much
    // as fits between its two barriers.
    int flip = 0;
    for (int c0 = 0; c0 < d; c0 += kGroupRound * kThreads, flip ^= 1) {
        int col[kGroupRound], g[kGroupRound], rank[kGroupRound];
        float v[kGroupRound];
        bool valid[kGroupRound];
#pragma unroll
        for (int e = 0; e < kGroupRound; e++) {
            const int i = c0 + e * kThreads + (int)threadIdx.x;
            valid[e] = i < d;
            col[e] = valid[e] ? idx[src0 + i] : 0;
            v[e] = valid[e] && s_val ? val[src0 + i] : 0.0f;
            g[e] = col_group(col[e], ng);
            wave_cnt[flip][e][w][lane] = 0;             // each wavefront clears its own rows
        }
#pragma unroll
        for (int e = 0; e < kGroupRound; e++) {
            unsigned long long peers = __ballot(valid[e]);   // lanes of this wavefront with the same group
#pragma unroll
            for (int b = 0; b < 6; b++) {
                const bool bit = (g[e] >> b) & 1;
                const unsigned long long bal = __ballot(bit);
                peers &= bit ? bal : ~bal;
            }
            rank[e] = __popcll(peers & ((1ull << lane) - 1ull));
            if (valid[e] && rank[e] == 0) wave_cnt[flip][e][w][g[e]] = __popcll(peers);
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kGroupRound; e++) {
            if (!valid[e]) continue;
            int pos = base[g[e]] + rank[e];
            for (int e2 = 0; e2 < e; e2++)
#pragma unroll
                for (int q = 0; q < kThreads / 64; q++) pos += wave_cnt[flip][e2][q][g[e]];
            for (int q = 0; q < w; q++) pos += wave_cnt[flip][e][q][g[e]];
            if (s_idx) s_idx[dst0 + pos] = col[e];
            if (s_val) s_val[dst0 + pos] = v[e];
            if (src_pos) src_pos[dst0 + pos] = (int32_t)(src0 + c0 + e * kThreads + (int)threadIdx.x);
        }
        __syncthreads();
        if ((int)threadIdx.x < kMaxGroups) {
            int add = 0;
#pragma unroll
            for (int e = 0; e < kGroupRound; e++)
#pragma unroll
                for (int q = 0; q < kThreads / 64; q++) add += wave_cnt[flip][e][q][threadIdx.x];
            base[threadIdx.x] += add;
        }
        // the next round uses the other copy of wave_cnt and reads base only after
        // its own barrier, so no third barrier is needed here
    }
}

// The same regrouping with one wavefront per row, four rows per workgroup: for the many
// split rows of a few hundred non-zeros a workgroup per row is mostly barriers and idle
// lanes, and four times as many rows are in flight this way.  No workgroup barrier: a
// wavefront only touches its own part of LDS, whose accesses execute in program order.
__global__ __launch_bounds__(kThreads) void group_long_rows_wave_kernel(
    const int32_t *__restrict__ indptr, const int32_t *__restrict__ idx,
    const float *__restrict__ val, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ s_indptr, int64_t first_long_row, int n_rows, int forced_groups,
    int32_t *__restrict__ s_idx, float *__restrict__ s_val, int *__restrict__ counts,
    int32_t *__restrict__ src_pos)
{
    static_assert(kMaxGroups == 64, "one lane per column group");
    __shared__ int cnt[kThreads / 64][kMaxGroups];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int lr = (int)blockIdx.x * (kThreads / 64) + w;
    if (lr >= n_rows) return;                            // the whole wavefront leaves
    const int64_t r = first_long_row + lr;
    const int64_t src0 = indptr[perm ? perm[r] : r];
    const int64_t dst0 = s_indptr[r];
    const int d = s_indptr[r + 1] - s_indptr[r];
    const int ng = row_groups(d, forced_groups);
    int *my = cnt[w];
    my[lane] = 0;
    __builtin_amdgcn_wave_barrier();
    for (int i = lane; i < d; i += 64) atomicAdd(&my[col_group(idx[src0 + i], ng)], 1);
    __builtin_amdgcn_wave_barrier();
    const int c = my[lane];                              // lane g holds the size of group g
    if (counts) counts[(int64_t)lr * kMaxGroups + lane] = c;
    int inc = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(inc, off);
        if (lane >= off) inc += t;
    }
    __builtin_amdgcn_wave_barrier();
    my[lane] = inc - c;                                  // where group g starts; moves on as it fills
    __builtin_amdgcn_wave_barrier();
    for (int c0 = 0; c0 < d; c0 += 64) {
        const int i = c0 + lane;
        const bool valid = i < d;
        const int col = valid ? idx[src0 + i] : 0;
        const float v = valid && s_val ? val[src0 + i] : 0.0f;
        const int g = col_group(col, ng);
        unsigned long long peers = __ballot(valid);      // lanes with the same group
#pragma unroll
        for (int b = 0; b < 6; b++) {
            const bool bit = (g >> b) & 1;
            const unsigned long long bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        const int rank = __popcll(peers & ((1ull << lane) - 1ull));
        int pos = 0;
        if (valid) pos = my[g] + rank;
        __builtin_amdgcn_wave_barrier();
        if (valid) {
            if (s_idx) s_idx[dst0 + pos] = col;
            if (s_val) s_val[dst0 + pos] = v;
            if (src_pos) src_pos[dst0 + pos] = (int32_t)(src0 + i);
            if (rank == 0) my[g] += __popcll(peers);     // one lane per group present
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// Gathers the first n_take non-zeros of the sorted matrix (the rows before first_long)
// from the caller's arrays through perm.  tile_first: n_take / kPermuteTile + 2 ints.
static void launch_permute_csr(const int32_t *indptr, const int32_t *idx, const float *val,
                               const int32_t *perm, const int32_t *s_indptr, int64_t rows,
                               int64_t first_long, int64_t n_take, int *tile_first, int32_t *s_idx,
                               float *s_val, int32_t *src_pos, hipStream_t s)
{
    if (n_take <= 0) return;
    tile_first_kernel<<<dim3(grid_for(rows)), dim3(kThreads), 0, s>>>(s_indptr, rows, n_take, tile_first);
    permute_csr_kernel<<<dim3((unsigned)((n_take + kPermuteTile - 1) / kPermuteTile)), dim3(kThreads), 0, s>>>(
        indptr, idx, val, perm, s_indptr, tile_first, first_long - 1, n_take, s_idx, s_val, src_pos);
}

// Regroups the n_long split rows (the last rows of the sorted order, ascending by
// length, n_wide of them longer than kGroupWaveMax).
static void launch_group_long_rows(const int32_t *indptr, const int32_t *idx, const float *val,
                                   const int32_t *perm, const int32_t *s_indptr, int64_t first_long,
                                   int64_t n_long, int64_t n_wide, int forced_groups, int32_t *s_idx,
                                   float *s_val, int *counts, int32_t *src_pos, hipStream_t s)
{
    const int64_t n_narrow = n_long - n_wide;
    if (n_narrow > 0)
        group_long_rows_wave_kernel<<<dim3((unsigned)((n_narrow + kThreads / 64 - 1) / (kThreads / 64))),
                                      dim3(kThreads), 0, s>>>(
            indptr, idx, val, perm, s_indptr, first_long, (int)n_narrow, forced_groups, s_idx, s_val, counts,
            src_pos);
    if (n_wide > 0)
        group_long_rows_kernel<<<dim3((unsigned)n_wide), dim3(kThreads), 0, s>>>(
            indptr, idx, val, perm, s_indptr, first_long + n_narrow, forced_groups, s_idx, s_val,
            counts ? counts + n_narrow * kMaxGroups : nullptr, src_pos);
}

// ---------------------------------------------------------------------------
// Partition
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void run_head_kernel(const uint32_t *__restrict__ deg,
                                                            int64_t rows, int *__restrict__ head)
{
    const int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (r < rows) head[r] = (r == 0 || deg[r] != deg[r - 1]) ? (int)r : 0;
}

__global__ __launch_bounds__(kThreads) void block_count_kernel(
    const uint32_t *__restrict__ deg, const int *__restrict__ run_start, int64_t rows,
    int *__restrict__ count)
{
    const int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (r >= rows) return;
    const int d = (int)deg[r];
    int c = 0;
    if (d > kDegBound) {
        c = (d + kDegBound - 1) / kDegBound;
    } else if (d > 0) {
        int w, rpb;
        slice_rule(d, w, rpb);
        c = ((int)r - run_start[r]) % rpb == 0;
    }
    count[r] = c;
}

__global__ __launch_bounds__(kThreads) void emit_block4_kernel(
    const uint32_t *__restrict__ deg, const int32_t *__restrict__ s_indptr,
    const int *__restrict__ run_start, const int *__restrict__ row_block, int64_t rows, int n_blocks,
    int4 *__restrict__ block4)
{
    // n_blocks = entries allocated; a row whose blocks would not fit writes nothing (the host
    // compares the device's total with its own afterwards)
    const int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (r >= rows) return;
    const int d = (int)deg[r];
    if (d == 0) return;
    const int at = row_block[r];
    const int loc = s_indptr[r];
    if (d > kDegBound) {
        const int nseg = (d + kDegBound - 1) / kDegBound;
        if (at + nseg > n_blocks) return;
        for (int k = 0; k < nseg; k++)
            block4[at + k] = make_int4(d, (int)r, loc + k * kDegBound,
                                       min(kDegBound, d - k * kDegBound));
        return;
    }
    int w, rpb;
    slice_rule(d, w, rpb);
    if (((int)r - run_start[r]) % rpb != 0) return;
    int n = 1;
    while (n < rpb && r + n < rows && (int)deg[r + n] == d) n++;
    if (at < n_blocks) block4[at] = make_int4(d, (int)r, loc, (w << 16) + n);
}

// ---------------------------------------------------------------------------
// Launch plan (work list), built on the GPU.  See build_work_list below.
// ---------------------------------------------------------------------------
struct PlanParams {
    int queue_long[kXcds];   // long-row units already in each queue
};
struct BinOffsets {
    int off[kPlanBins];      // where the pieces of a (row class, column group) bin start in their queue
};

__device__ __forceinline__ int64_t plan_index(int queue, int pos, int n_queues)
{
    // queue q, position p  ->  slot of wavefront (p % 4) in workgroup (p / 4) * n_queues + q
    return ((int64_t)(pos / kWavesPerGroup) * n_queues + queue) * kWavesPerGroup + pos % kWavesPerGroup;
}

// The order of the split rows inside their (class, group) bins: key[lr] = the caller's row id
// (or, for the longest rows, a key that puts the largest first), and, after the sort,
// rank[order[i]] = i.  Only the order among rows of one class matters.
// Rows stored in up to this many column groups follow the caller's row ids inside their
// bins; the longer ones keep "largest first" (they touch all of X whatever their id, and the
// hub workload measured 2 % faster that way: 2.31 against 2.36 ms at N = 256).
constexpr int kIdOrderMaxGroups = 8;
__global__ __launch_bounds__(kThreads) void long_row_key_kernel(const uint32_t *__restrict__ perm,
                                                                const int32_t *__restrict__ s_indptr,
                                                                int forced_groups, int key_shift,
                                                                int64_t first_long, int n_long,
                                                                uint32_t *__restrict__ key)
{
    const int lr = blockIdx.x * kThreads + threadIdx.x;
    if (lr >= n_long) return;
    const int64_t row = first_long + lr;
    const int ng = row_groups(s_indptr[row + 1] - s_indptr[row], forced_groups);
    if (ng <= kIdOrderMaxGroups)
        key[lr] = (perm ? perm[row] : (uint32_t)row) >> key_shift;
    else
        key[lr] = (uint32_t)(n_long - 1 - lr) >> key_shift;   // largest rows first
}

__global__ __launch_bounds__(kThreads) void invert_order_kernel(const uint32_t *__restrict__ order, int n,
                                                                int *__restrict__ rank)
{
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i < n) rank[order[i]] = i;
}

// grp_units is laid out [bin][split row, by rank] and must be zero on entry.
__global__ __launch_bounds__(kThreads) void long_unit_count_kernel(
    const int *__restrict__ gcount, const int32_t *__restrict__ s_indptr, int64_t first_long,
    int n_long, int forced_groups, int piece, const int *__restrict__ rank,
    int *__restrict__ row_units, int *__restrict__ grp_units)
{
    const int lr = blockIdx.x * kThreads + threadIdx.x;
    if (lr >= n_long) return;
    const int ng = row_groups(s_indptr[first_long + lr + 1] - s_indptr[first_long + lr], forced_groups);
    int tot = 0;
    for (int g = 0; g < ng; g++) {
        const int u = (gcount[(int64_t)lr * kMaxGroups + g] + piece - 1) / piece;
        grp_units[(int64_t)plan_bin(ng, g) * n_long + rank[lr]] = u;
        tot += u;
    }
    row_units[lr] = tot;
}

__global__ void plan_totals_kernel(const int *__restrict__ grp_pos, int n_long, int *__restrict__ out)
{
    const int b = threadIdx.x;
    if (b <= kPlanBins) out[b] = grp_pos[(int64_t)b * n_long];   // b == kPlanBins: grand total
}

__global__ __launch_bounds__(kThreads) void emit_long_units_kernel(
    const int *__restrict__ gcount, const int32_t *__restrict__ s_indptr, int64_t first_long,
    const int *__restrict__ slot, const int *__restrict__ grp_pos, int n_long, int forced_groups,
    int piece, const int *__restrict__ rank, BinOffsets bo, int n_queues, int4 *__restrict__ work)
{
    const int t = blockIdx.x * kThreads + threadIdx.x;
    if (t >= n_long * kMaxGroups) return;
    const int lr = t / kMaxGroups, g = t % kMaxGroups;
    const int row = (int)(first_long + lr);
    const int ng = row_groups(s_indptr[row + 1] - s_indptr[row], forced_groups);
    if (g >= ng) return;
    const int c = gcount[(int64_t)lr * kMaxGroups + g];
    if (c == 0) return;
    int c_before = 0, u_before = 0;
    for (int q = 0; q < g; q++) {
        const int cq = gcount[(int64_t)lr * kMaxGroups + q];
        c_before += cq;
        u_before += (cq + piece - 1) / piece;
    }
    const int loc = s_indptr[row] + c_before;
    const int bin = plan_bin(ng, g);
    const int pos0 = bo.off[bin] + grp_pos[(int64_t)bin * n_long + rank[lr]] -
                     grp_pos[(int64_t)bin * n_long];
    const int sl = slot[lr] + u_before;
    for (int k = 0, off = 0; off < c; k++, off += piece)
        work[plan_index(g % n_queues, pos0 + k, n_queues)] =
            make_int4(kDegBound + 1 + sl + k, row, loc + off, min(piece, c - off));
}

// Rows a unit of whole rows may hold: as many as fit plan_unit non-zeros, at least one.
__device__ __forceinline__ int rows_per_unit(int d, int unit_nz) { return max(1, unit_nz / d); }

// cnt[j] = number of units block4 entry j (of the rows that are not split) is cut into.
__global__ __launch_bounds__(kThreads) void short_unit_count_kernel(
    const int4 *__restrict__ block4, int n_short, int unit_nz, int *__restrict__ cnt)
{
    const int j = blockIdx.x * kThreads + threadIdx.x;
    if (j >= n_short) return;
    const int4 b = block4[j];
    const int n_rows = b.w & 0xFFFF, rpu = rows_per_unit(b.x, unit_nz);
    cnt[j] = (n_rows + rpu - 1) / rpu;
}

// What a unit costs, for levelling the queues: a gathered row of X per non-zero, a
// written row of Y per row, a fixed part; scaled down (shift >= 2) so that the sum over
// the matrix stays below 2^31.  (Counting units, or fixed parts of 64 or 200, measured the
// same within noise.)
__device__ __forceinline__ int unit_cost(int nz, int n_rows, int shift)
{
    return ((nz + n_rows + 8) >> shift) + 1;
}

// Writes the units of whole rows in row order, and for each the caller's row id of its
// first row: the key the units are queued by.
__global__ __launch_bounds__(kThreads) void list_short_units_kernel(
    const int4 *__restrict__ block4, int n_short, int unit_nz, const int *__restrict__ first_unit,
    const uint32_t *__restrict__ perm, int key_shift, int4 *__restrict__ units,
    uint32_t *__restrict__ key)
{
    const int j = blockIdx.x * kThreads + threadIdx.x;
    if (j >= n_short) return;
    const int4 b = block4[j];
    const int d = b.x, n_rows = b.w & 0xFFFF, w_nz = b.w >> 16, rpu = rows_per_unit(d, unit_nz);
    int i = first_unit[j];
    for (int r = 0; r < n_rows; r += rpu, i++) {
        units[i] = make_int4(d, b.y + r, b.z + r * d, (w_nz << 16) + min(rpu, n_rows - r));
        key[i] = (perm ? perm[b.y + r] : (uint32_t)(b.y + r)) >> key_shift;
    }
}

__global__ __launch_bounds__(kThreads) void short_unit_cost_kernel(
    const int4 *__restrict__ units, const uint32_t *__restrict__ order, int n, int shift,
    int light_nz, int *__restrict__ cost, int *__restrict__ heavy)
{
    const int sidx = blockIdx.x * kThreads + threadIdx.x;
    if (sidx >= n) return;
    const int4 u = units[order[sidx]];
    const int n_rows = u.w & 0xFFFF;
    cost[sidx] = unit_cost(u.x * n_rows, n_rows, shift);
    heavy[sidx] = u.x * n_rows > light_nz;
}

// Non-zeros and pieces of the split rows per queue (column group g belongs to queue
// g % n_queues, n_queues = 8 or 1).  Thread t looks at (row t / 64, group t % 64), so lane l
// of a wavefront always holds a group with g % 8 == l % 8: the wavefront's eight sums are
// formed with shuffles.
__global__ __launch_bounds__(kThreads) void long_queue_load_kernel(
    const int *__restrict__ gcount, int n_long, int piece, int shift, int n_queues,
    int *__restrict__ queue_cost)
{
    static_assert(kMaxGroups == 64, "one wavefront per split row");
    const int64_t n = (int64_t)n_long * kMaxGroups;
    int v = 0;                                           // the stride keeps t % 64 == lane
    for (int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x; t < n; t += (int64_t)gridDim.x * kThreads) {
        const int c = gcount[t];
        if (c > 0) {
            const int pieces = (c + piece - 1) / piece;
            v += ((c + 9 * pieces) >> shift) + pieces;
        }
    }
    v += __shfl_xor(v, 8);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    const int lane = threadIdx.x & 63;
    if (lane < kXcds && v) atomicAdd(&queue_cost[lane % n_queues], v);
}

struct QueueCuts {
    int cut[kXcds + 1];      // queue q takes the units whose running cost lies in [cut[q], cut[q + 1])
};

__device__ __forceinline__ int queue_of(int running_cost, const QueueCuts &qc)
{
    int q = 0;
#pragma unroll
    for (int i = 1; i < kXcds; i++) q += running_cost >= qc.cut[i];
    return q;
}

// The share boundaries, computed where the numbers are: queue q takes max(0, level - long_cost[q])
// of the whole-row units' cost, level being the smallest common level that takes all of it.
// One thread; total_cost points at the sum of the units' costs.
__global__ void queue_cuts_kernel(const int *__restrict__ long_cost, const int *__restrict__ total_cost,
                                  int n_queues, QueueCuts *__restrict__ out)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const long long short_cost = *total_cost;
    long long lc[kXcds], lo = 0, hi = short_cost;
    for (int q = 0; q < n_queues; q++) {
        lc[q] = long_cost ? long_cost[q] : 0;
        if (lc[q] + short_cost > hi) hi = lc[q] + short_cost;
    }
    while (lo < hi) {                                  // smallest level that takes all of it
        const long long mid = (lo + hi) / 2;
        long long taken = 0;
        for (int q = 0; q < n_queues; q++) taken += mid > lc[q] ? mid - lc[q] : 0;
        if (taken >= short_cost) hi = mid; else lo = mid + 1;
    }
    long long run = 0;
    for (int q = 0; q < n_queues; q++) {
        out->cut[q] = (int)(run < short_cost ? run : short_cost);
        run += lo > lc[q] ? lo - lc[q] : 0;
    }
    for (int q = n_queues; q <= kXcds; q++) out->cut[q] = INT_MAX;   // queues that do not exist take nothing
}

// first[q] = rank of the first unit of queue q (n for queues that get none); first must hold n on entry.
__global__ __launch_bounds__(kThreads) void queue_first_kernel(const int *__restrict__ running, int n,
                                                               const QueueCuts *__restrict__ cuts,
                                                               int *__restrict__ first)
{
    const int sidx = blockIdx.x * kThreads + threadIdx.x;
    if (sidx >= n) return;
    const QueueCuts qc = *cuts;
    const int q = queue_of(running[sidx], qc);
    const int q_prev = sidx == 0 ? -1 : queue_of(running[sidx - 1], qc);
    for (int i = q_prev + 1; i <= q; i++) first[i] = sidx;
}

// Inside its queue a unit goes behind the pieces, in the order of the caller's row ids,
// except that the queue's last kTailLight light units (few non-zeros: short chains of
// gathers) are held back and placed at the very end, so that a queue does not end on a
// long chain.  They are the light units with the highest ids of the queue's share, i.e.
// they lie in the band of rows the die is working on at that time anyway.
// heavy_before[s] = heavy units among the first s, [n] = all.
constexpr int kTailLight = 2048;             // two rounds of the 1,024 wavefronts a die holds
__global__ __launch_bounds__(kThreads) void place_short_units_kernel(
    const int4 *__restrict__ units, const uint32_t *__restrict__ order, const int *__restrict__ running,
    const int *__restrict__ heavy_before, int n, const QueueCuts *__restrict__ cuts,
    const int *__restrict__ first, PlanParams pp, int n_queues, int4 *__restrict__ work)
{
    const int sidx = blockIdx.x * kThreads + threadIdx.x;
    if (sidx >= n) return;
    const QueueCuts qc = *cuts;
    const int q = queue_of(running[sidx], qc);
    const int f = first[q], n_q = first[q + 1] - f;
    const int h0 = heavy_before[f];
    const int light_all = n_q - (heavy_before[f + n_q] - h0);              // light units of this queue
    const int light_me = (sidx - f) - (heavy_before[sidx] - h0);           // ... before this unit
    const bool is_light = heavy_before[sidx + 1] == heavy_before[sidx];
    const int kept = max(0, light_all - kTailLight);                 // light units that stay in line
    int pos;
    if (is_light && light_me >= kept)
        pos = n_q - (light_all - light_me);                                // held back: the last ones
    else
        pos = (sidx - f) - max(0, light_me - kept);                        // in line, minus those held back before it
    work[plan_index(q, pp.queue_long[q] + pos, n_queues)] = units[order[sidx]];
}

}  // namespace

// Builds block4 from degrees given in partition order.  The output is a freshly
// allocated device array (caller frees); *n_blocks is returned on the host.
// The one synchronisation in here (the host has to know the number of blocks to allocate
// them) also brings back, if asked, the blocks that precede row probe_row and the sorted
// indptr at that row.  The emit kernel is left running on the stream.
static int partition_device(Arena *tmp, const uint32_t *deg, const int32_t *s_indptr, int64_t rows,
                            int32_t **block4_out, int64_t *n_blocks, hipStream_t s,
                            int64_t probe_row = -1, int64_t *blocks_before_probe = nullptr,
                            int64_t *nnz_before_probe = nullptr, int64_t known_blocks = -1,
                            const int **total_blocks_dev = nullptr)
{
    // known_blocks >= 0: the host already knows the number of blocks (rows in ascending degree
    // order: one run per degree, so the count follows from the degree histogram) and nothing
    // is read back here; *total_blocks_dev then points at the device's own total for a later check
    DevBuf head(tmp), cnt(tmp), sums(tmp), rb(tmp), b4;
    int rc;
    if ((rc = head.alloc(sizeof(int) * (size_t)rows))) return rc;
    if ((rc = cnt.alloc(sizeof(int) * (size_t)rows))) return rc;
    if ((rc = sums.alloc(sizeof(int) * (size_t)(rows / kTile + 4)))) return rc;
    if ((rc = rb.alloc(sizeof(int) * (size_t)(rows + 1)))) return rc;
    run_head_kernel<<<dim3(grid_for(rows)), dim3(kThreads), 0, s>>>(deg, rows, head.as<int>());
    if ((rc = device_scan<MaxOp, true>(head.as<int>(), rows, head.as<int>(), nullptr,
                                       sums.as<int>(), s)))
        return rc;
    block_count_kernel<<<dim3(grid_for(rows)), dim3(kThreads), 0, s>>>(deg, head.as<int>(), rows,
                                                                      cnt.as<int>());
    if ((rc = device_scan<SumOp, false>(cnt.as<int>(), rows, rb.as<int>(), rb.as<int>() + rows,
                                        sums.as<int>(), s)))
        return rc;
    int nb = (int)known_blocks, before = 0, nnz_before = 0;
    if (known_blocks < 0) {
        ACCEL_HIP(hipMemcpyAsync(&nb, rb.as<int>() + rows, sizeof(int), hipMemcpyDeviceToHost, s));
        if (blocks_before_probe && probe_row >= 0 && probe_row <= rows)   // rb[rows] is the total
            ACCEL_HIP(hipMemcpyAsync(&before, rb.as<int>() + probe_row, sizeof(int), hipMemcpyDeviceToHost, s));
        if (nnz_before_probe && probe_row >= 0 && probe_row <= rows)
            ACCEL_HIP(hipMemcpyAsync(&nnz_before, s_indptr + probe_row, sizeof(int), hipMemcpyDeviceToHost, s));
        ACCEL_HIP(hipStreamSynchronize(s));
        if (blocks_before_probe) *blocks_before_probe = before;
        if (nnz_before_probe) *nnz_before_probe = nnz_before;
    }
    if (total_blocks_dev) *total_blocks_dev = rb.as<int>() + rows;
    if ((rc = b4.alloc(sizeof(int4) * (size_t)nb))) return rc;
    emit_block4_kernel<<<dim3(grid_for(rows)), dim3(kThreads), 0, s>>>(
        deg, s_indptr, head.as<int>(), rb.as<int>(), rows, nb, b4.as<int4>());
    ACCEL_HIP(hipGetLastError());
    *n_blocks = nb;
    *block4_out = static_cast<int32_t *>(b4.release());
    return ACCEL_OK;
}

// Partition a row order as given (no sort): the GPU counterpart of running
// block_level_partition.py on one *.new_indptr file.
int partition_only_device(const int32_t *indptr_dev, int64_t rows, int64_t nnz,
                          int32_t **block4_dev, int64_t *n_blocks)
{
    hipStream_t s = nullptr;
    Arena tmp;
    tmp.next_chunk = (size_t)rows * 24 + (1 << 16);
    DevBuf deg(&tmp), st(&tmp);
    int rc;
    if ((rc = deg.alloc(sizeof(uint32_t) * (size_t)rows))) return rc;
    if ((rc = st.alloc(sizeof(Stats)))) return rc;
    ACCEL_HIP(hipMemsetAsync(st.p, 0, sizeof(Stats), s));
    degree_kernel<<<dim3(std::min(grid_for(rows), kDegreeGroups)), dim3(kThreads), 0, s>>>(
        indptr_dev, rows, nnz, deg.as<uint32_t>(), st.as<Stats>(), kDegBound, kDegBound);
    Stats hs;
    ACCEL_HIP(hipMemcpyAsync(&hs, st.p, sizeof(Stats), hipMemcpyDeviceToHost, s));
    ACCEL_HIP(hipStreamSynchronize(s));
    if (hs.bad_indptr) {
        set_error("indptr must start at 0, be non-decreasing and end at nnz");
        return ACCEL_ERR_CSR;
    }
    if ((rc = partition_device(&tmp, deg.as<uint32_t>(), indptr_dev, rows, block4_dev, n_blocks, s))) return rc;
    ACCEL_HIP(hipStreamSynchronize(s));               // the temporaries go away with this scope
    return ACCEL_OK;
}

// Split rows are added up by the gather kernel itself (the wavefront that stores a row's last
// piece does it: one launch) when the plan holds at most this many pieces, by a second kernel
// otherwise.  In the kernel every piece ends on a wait for its stores and one atomic, some
// microseconds of latency that nothing hides on a launch-bound matrix but that is still less
// than a second launch costs; with many pieces it adds up to more.  Measured, runs queued
// back to back, in-kernel against second kernel at N = 16 / 64 / 128: 96 pieces (1.9 M
// non-zeros) 0.88 / 0.94 / 0.96; 5,160 (1.2 M) 0.88 / 0.90 / 0.96; 8,848 (1.6 M) 0.82 / 0.94 /
// 0.98; 7,760 (2.4 M) 0.99 / 0.96 / 0.98; 68,608 (14 M) 1.01 / 1.02 / 1.02; 144,561 (27 M)
// 1.24 / 1.08 / 1.09; 0.5 M pieces (115 M non-zeros, nearly every row split) 1.30 at N = 64.
constexpr int64_t kFusedReduceMaxPieces = 16384;

// The launch plan.  One work unit per wavefront, kWavesPerGroup units per
// workgroup, as int4 (x, y, z, w):
//   x <= 384 : whole rows of one block4 entry (degree, first row, first non-zero,
//              (w_nz << 16) + n_rows): the entry itself, or a run of its rows when
//              the plan's unit is smaller than the entry;
//   x  > 384 : a piece of a split row: partial-sum slot x - 385, row y, first
//              non-zero z, length w <= plan_unit, all of one column group;
//   w == 0   : padding, nothing to do.
// Workgroups are dispatched to the eight dies round-robin (workgroup i runs on
// die i % 8), so the list is laid out as eight interleaved queues.  Column group
// g belongs to die g % 8.  A queue holds, in this order: the pieces of the rows
// stored in 64 groups (the longest rows), one group after the other, largest
// rows first; then the same for the rows with 32, 16 and 8 groups (the rows of
// an 8-group bin in the order of the caller's row ids); then the
// queue's share of the whole-row units.  While a die works through one group its
// L2 only has to hold that group's share of X.
// The whole-row units are put in the order of the caller's row ids (of each unit's
// first row) and that sequence is cut into eight consecutive shares, one per queue,
// sized so that all queues carry about the same load.  Graphs whose neighbouring
// row ids have neighbouring columns (most graphs with a meaningful vertex order)
// lose that locality to the degree sort; this gives it back: at any time a die
// works on a narrow band of the caller's rows.
// The host sees 121 bin totals and nine share boundaries, in one synchronisation, to size
// the queues (plus the number of whole-row units when entries are cut into smaller units).
static int build_work_list(Arena *tmp, accel_handle *h, const int *gcount, const int32_t *s_indptr,
                           int64_t first_long, int64_t n_short, const uint32_t *perm,
                           const int *total_blocks_dev, hipStream_t s)
{
    // "long" here = rows cut into pieces (more than plan_split non-zeros); n_short = block4
    // entries of all other rows (they precede the rest in block4)
    const int64_t n_long = h->n_split_rows;
    // pieces of split rows hold up to piece_nz non-zeros, units of several whole rows up to unit_nz
    const int unit_nz = h->plan_unit, piece_nz = std::max(h->plan_unit, h->plan_split), forced = h->plan_groups;
    const int nq = h->plan_queues;                     // 8 interleaved queues, or 1 (plain order)
    DevBuf row_units(tmp), grp_units(tmp), sums(tmp), totals(tmp), dslot, scnt(tmp), qload(tmp), lkey(tmp),
        lrank(tmp);
    int rc;
    int tot[kPlanBins + 1] = {0};
    // the order by row id is kept to 16 bits (two passes of the sort): bands of rows, not single
    // rows, are what the caches see; equal keys stay in row order (the sort is stable)
    int key_shift = 0;
    while ((std::max<int64_t>(h->rows, 1) - 1) >> key_shift >= 65536) key_shift++;
    const uint32_t max_key = (uint32_t)((std::max<int64_t>(h->rows, 1) - 1) >> key_shift);
    int cost_shift = 2;                                // total cost = about (nnz + 10 rows) >> shift + units < 2^31
    while ((((int64_t)h->nnz + 10 * h->rows) >> cost_shift) + h->rows >= ((int64_t)1 << 30)) cost_shift++;
    // the slots of each split row, and behind them one counter per split row (zero between launches)
    if ((rc = dslot.alloc(sizeof(int) * (size_t)(2 * n_long + 1)))) return rc;
    if ((rc = fill_u32(dslot.as<int>() + n_long + 1, 0u, (size_t)n_long, s))) return rc;
    if (n_long > 0) {
        if ((rc = row_units.alloc(sizeof(int) * (size_t)n_long))) return rc;
        const int64_t n_bins = (int64_t)kPlanBins * n_long;
        if ((rc = grp_units.alloc(sizeof(int) * (size_t)(n_bins + 1)))) return rc;
        if ((rc = sums.alloc(sizeof(int) * (size_t)(n_bins / kTile + 4)))) return rc;
        if ((rc = totals.alloc(sizeof(int) * (kPlanBins + 1)))) return rc;
        if ((rc = qload.alloc(sizeof(int) * kXcds))) return rc;
        if ((rc = fill_u32(grp_units.p, 0u, (size_t)n_bins + 1, s))) return rc;
        if ((rc = fill_u32(qload.p, 0u, kXcds, s))) return rc;
        // inside an 8-group bin the rows follow the caller's row ids, like the whole-row units
        // further down
        uint32_t *lkey_sorted = nullptr, *lorder = nullptr;
        if ((rc = lkey.alloc(sizeof(uint32_t) * (size_t)n_long))) return rc;
        if ((rc = lrank.alloc(sizeof(int) * (size_t)n_long))) return rc;
        long_row_key_kernel<<<dim3(grid_for(n_long)), dim3(kThreads), 0, s>>>(
            perm, s_indptr, forced, key_shift, first_long, (int)n_long, lkey.as<uint32_t>());
        if ((rc = radix_sort_pairs(tmp, lkey.as<uint32_t>(), n_long, max_key, s, &lkey_sorted, &lorder)))
            return rc;
        invert_order_kernel<<<dim3(grid_for(n_long)), dim3(kThreads), 0, s>>>(lorder, (int)n_long,
                                                                             lrank.as<int>());
        long_unit_count_kernel<<<dim3(grid_for(n_long)), dim3(kThreads), 0, s>>>(
            gcount, s_indptr, first_long, (int)n_long, forced, piece_nz, lrank.as<int>(),
            row_units.as<int>(), grp_units.as<int>());
        long_queue_load_kernel<<<dim3(std::min(grid_for(n_long * kMaxGroups), 1024u)), dim3(kThreads), 0, s>>>(
            gcount, (int)n_long, piece_nz, cost_shift, nq, qload.as<int>());
        if ((rc = device_scan<SumOp, false>(row_units.as<int>(), n_long, dslot.as<int>(),
                                            dslot.as<int>() + n_long, sums.as<int>(), s)))
            return rc;
        if ((rc = device_scan<SumOp, false>(grp_units.as<int>(), n_bins, grp_units.as<int>(),
                                            grp_units.as<int>() + n_bins, sums.as<int>(), s)))
            return rc;
        plan_totals_kernel<<<dim3(1), dim3(128), 0, s>>>(grp_units.as<int>(), (int)n_long,
                                                       totals.as<int>());
        ACCEL_HIP(hipMemcpyAsync(tot, totals.p, sizeof(tot), hipMemcpyDeviceToHost, s));
    } else {
        ACCEL_HIP(hipMemsetAsync(dslot.p, 0, sizeof(int), s));
    }
    // units of whole rows: how many each block4 entry is cut into, and where they start
    int n_short_units32 = 0;
    if ((rc = scnt.alloc(sizeof(int) * (size_t)(n_short + 1)))) return rc;
    if (n_short > 0) {
        DevBuf ssums(tmp);
        if ((rc = ssums.alloc(sizeof(int) * (size_t)(n_short / kTile + 4)))) return rc;
        short_unit_count_kernel<<<dim3(grid_for(n_short)), dim3(kThreads), 0, s>>>(
            reinterpret_cast<const int4 *>(h->block4), (int)n_short, unit_nz, scnt.as<int>());
        if ((rc = device_scan<SumOp, false>(scnt.as<int>(), n_short, scnt.as<int>(),
                                            scnt.as<int>() + n_short, ssums.as<int>(), s)))
            return rc;
        // with units of a whole block4 entry (large matrices) there is one unit per entry and
        // nothing to wait for; smaller units are counted on the device
        n_short_units32 = (int)n_short;
        if (unit_nz < kDegBound) {
            ACCEL_HIP(hipMemcpyAsync(&n_short_units32, scnt.as<int>() + n_short, sizeof(int),
                                     hipMemcpyDeviceToHost, s));
            ACCEL_HIP(hipStreamSynchronize(s));
        }
    }
    const int64_t n_short_units = n_short_units32;

    // whole-row units: list them, order them by the caller's row id, cut the sequence into
    // one share per queue so that long pieces + share cost about the same everywhere
    DevBuf units(tmp), key(tmp), cost(tmp), heavy(tmp), csums(tmp), first(tmp), cuts(tmp);
    uint32_t *order = nullptr;
    int first_h[kXcds + 1];
    for (int q = 0; q <= kXcds; q++) first_h[q] = 0;
    if (n_short_units > 0) {
        const int n = (int)n_short_units;
        uint32_t *sorted_key = nullptr;
        if ((rc = units.alloc(sizeof(int4) * (size_t)n))) return rc;
        if ((rc = key.alloc(sizeof(uint32_t) * (size_t)n))) return rc;
        if ((rc = cost.alloc(sizeof(int) * (size_t)(n + 1)))) return rc;
        if ((rc = heavy.alloc(sizeof(int) * (size_t)(n + 1)))) return rc;
        if ((rc = csums.alloc(sizeof(int) * (size_t)(n / kTile + 4)))) return rc;
        if ((rc = first.alloc(sizeof(int) * (kXcds + 1)))) return rc;
        if ((rc = cuts.alloc(sizeof(QueueCuts)))) return rc;
        list_short_units_kernel<<<dim3(grid_for(n_short)), dim3(kThreads), 0, s>>>(
            reinterpret_cast<const int4 *>(h->block4), (int)n_short, unit_nz, scnt.as<int>(), perm,
            key_shift, units.as<int4>(), key.as<uint32_t>());
        if ((rc = radix_sort_pairs(tmp, key.as<uint32_t>(), n, max_key, s, &sorted_key, &order)))
            return rc;
        const int light_nz = std::max(24, unit_nz / 4);        // a unit up to this size is a light one
        short_unit_cost_kernel<<<dim3(grid_for(n)), dim3(kThreads), 0, s>>>(
            units.as<int4>(), order, n, cost_shift, light_nz, cost.as<int>(), heavy.as<int>());
        if ((rc = device_scan<SumOp, false>(cost.as<int>(), n, cost.as<int>(), cost.as<int>() + n,
                                            csums.as<int>(), s)))
            return rc;
        if ((rc = device_scan<SumOp, false>(heavy.as<int>(), n, heavy.as<int>(), heavy.as<int>() + n,
                                            csums.as<int>(), s)))
            return rc;
        queue_cuts_kernel<<<dim3(1), dim3(1), 0, s>>>(n_long > 0 ? qload.as<int>() : nullptr, cost.as<int>() + n,
                                                      nq, cuts.as<QueueCuts>());
        if ((rc = fill_u32(first.p, (uint32_t)n, kXcds + 1, s))) return rc;
        queue_first_kernel<<<dim3(grid_for(n)), dim3(kThreads), 0, s>>>(cost.as<int>(), n, cuts.as<QueueCuts>(),
                                                                       first.as<int>());
        ACCEL_HIP(hipMemcpyAsync(first_h, first.p, sizeof(first_h), hipMemcpyDeviceToHost, s));
    }
    // the one synchronisation of the plan: bin totals, share boundaries, and the device's own
    // count of block4 entries (the host sized them from the degree histogram)
    int device_blocks = (int)h->n_blocks;
    if (total_blocks_dev)
        ACCEL_HIP(hipMemcpyAsync(&device_blocks, total_blocks_dev, sizeof(int), hipMemcpyDeviceToHost, s));
    ACCEL_HIP(hipStreamSynchronize(s));
    if (device_blocks != (int)h->n_blocks) {
        set_error("internal: the partition has %d blocks, %lld were expected from the degree histogram",
                  device_blocks, (long long)h->n_blocks);
        return ACCEL_ERR_STATE;
    }
    PlanParams pp;
    BinOffsets bo;
    for (int q = 0; q < kXcds; q++) pp.queue_long[q] = 0;
    for (int b = 0; b < kPlanBins; b++) bo.off[b] = 0;
    if (n_long > 0)
        // a die first takes the pieces of the rows with the most groups (the longest
        // rows), one group after the other, then those of the next class, ...
        for (int ng = kMaxGroups; ng >= kXcds; ng /= 2)
            for (int g = 0; g < ng; g++) {
                const int b = plan_bin(ng, g);
                bo.off[b] = pp.queue_long[g % nq];
                pp.queue_long[g % nq] += tot[b + 1] - tot[b];
            }
    const int64_t n_long_units = n_long > 0 ? tot[kPlanBins] : 0;
    int64_t per_queue = 0;
    for (int q = 0; q < nq; q++)
        per_queue = std::max<int64_t>(per_queue, (int64_t)pp.queue_long[q] + (first_h[q + 1] - first_h[q]));
    per_queue = (per_queue + kWavesPerGroup - 1) / kWavesPerGroup * kWavesPerGroup;
    const int64_t n_units = per_queue * nq;
    if (n_units > (int64_t)INT_MAX) {
        set_error("the launch plan would exceed 2^31 work units");
        return ACCEL_ERR_ARG;
    }
    DevBuf dwork;
    if ((rc = dwork.alloc(sizeof(int4) * (size_t)n_units))) return rc;
    if (n_units > 0 && (rc = fill_u32(dwork.p, 0u, (size_t)n_units * 4, s))) return rc;
    if (n_long > 0)
        emit_long_units_kernel<<<dim3(grid_for(n_long * kMaxGroups)), dim3(kThreads), 0, s>>>(
            gcount, s_indptr, first_long, dslot.as<int>(), grp_units.as<int>(), (int)n_long, forced,
            piece_nz, lrank.as<int>(), bo, nq, dwork.as<int4>());
    if (n_short_units > 0)
        place_short_units_kernel<<<dim3(grid_for(n_short_units)), dim3(kThreads), 0, s>>>(
            units.as<int4>(), order, cost.as<int>(), heavy.as<int>(), (int)n_short_units, cuts.as<QueueCuts>(),
            first.as<int>(), pp, nq, dwork.as<int4>());
    ACCEL_HIP(hipGetLastError());
    ACCEL_HIP(hipStreamSynchronize(s));
    h->n_units = n_units;
    h->n_long_units = n_long_units;
    h->work = static_cast<int32_t *>(dwork.release());
    h->long_slot = static_cast<int32_t *>(dslot.release());
    h->row_done = h->long_slot + n_long + 1;
    h->fused_reduce = h->plan_reduce_option == 1 || (h->plan_reduce_option == 0 && n_long_units <= kFusedReduceMaxPieces);
    return ACCEL_OK;
}

// Small matrices are latency-bound: the time of a launch is the longest chain of
// dependent memory round trips in one wavefront, not the traffic.  For them a unit is
// given to a whole workgroup (four wavefronts share its rows, or its row's non-zeros),
// which shortens that chain, and rows of up to 384 non-zeros stay whole, so that most
// such matrices need no partial sums and no second launch.
// Measured (everything one call launches, N = 16 / 64 / 128, wavefront units with their
// best unit size against workgroup units of 96 with whole rows up to 384):
//   99 k non-zeros, longest row 171:   10.1 / 11.2 / 16.3 us  ->  7.3 /  9.4 / 11.4 us
//   208 k non-zeros, power law:        11.8 / 12.4 / 19.8 us  ->  7.9 / 10.5 / 12.6 us
//   1.2 M, 1.6 M and 2.4 M non-zeros:  wavefront units are faster (26 / 53 / 99 us against
//                                      34 / 55 / 102 us on the 1.2 M one).
constexpr int64_t kTeamMaxNnz = 512 * 1024;
static bool choose_plan_team(int64_t rows, int64_t nnz)
{
    (void)rows;
    return nnz < kTeamMaxNnz;
}

// Unit size of the launch plan: the most non-zeros of a unit of several whole rows (and,
// with wavefront units, of a piece of a split row).  Large matrices keep the block4
// granularity (384: fewest descriptors and partial sums, and the launch is bandwidth-bound
// anyway).  Small ones want short chains: workgroup units of 96 non-zeros (48 below 64 k
// non-zeros: 10.0 against 11.2 us at N = 64 on a 35 k one).  With wavefront units on a
// small matrix (only when asked for) 48 / 96 are best too: a 99 k-non-zero matrix 11 us
// with units of 48 against 17 us with 384; from about 1 M non-zeros on 384 is best or within 2 %.
static int choose_plan_unit(int64_t rows, int64_t nnz, bool team)
{
    (void)rows;
    if (team) return nnz < (int64_t)64 * 1024 ? 48 : 96;
    if (nnz < (int64_t)128 * 1024) return 48;
    if (nnz < (int64_t)512 * 1024) return 96;
    return kDegBound;
}

// Rows above this many non-zeros are stored by column group and cut into pieces.
// Measured with 384, 256, 192, 128 and 96 (N = 64): 192 is 8 % faster than 384 on the
// dense 115 M-non-zero matrix, 2 % on the 125 M power-law one, neutral elsewhere;
// below 192 the extra partial sums start to cost at N = 16.
constexpr int kPlanSplit = 192;
// Columns within this distance of a row's place on the diagonal count as near: 8,192 rows of
// X of 64 floats are half of one L2.
constexpr int kLocalityBand = 4096;

static int choose_plan_split(int64_t rows, int64_t nnz, bool team)
{
    (void)rows;
    (void)nnz;
    return team ? kDegBound : kPlanSplit;        // workgroup units: rows up to one unit stay whole
}

// New values on an unchanged structure reach the sorted copy through a map from sorted
// position to the position in the caller's arrays.  The map is what the regathering kernels
// of the preprocessing compute anyway (where each non-zero comes from); it is built here, by
// those kernels with only that output switched on, the first time a handle's values are
// replaced, and kept.  Needs perm (or identity_perm), s_indptr, nnz_short, n_split_rows,
// n_wide_rows and plan_groups as the preprocessing left them.  Allocates; synchronises s.
int build_source_positions(accel_handle *h, hipStream_t s)
{
    if (h->src_pos || !h->owns_sorted || h->nnz == 0) return ACCEL_OK;
    const int64_t rows = h->rows, n_long = h->n_split_rows, first_long = rows - n_long;
    const int64_t nnz_short = h->nnz_short;
    DevBuf map, tiles;
    if (int rc = map.alloc(sizeof(int32_t) * (size_t)h->nnz)) return rc;
    if (nnz_short > 0) {
        if (int rc = tiles.alloc(sizeof(int) * (size_t)(nnz_short / kPermuteTile + 2))) return rc;
        launch_permute_csr(h->indptr, h->idx, h->val, h->perm, h->s_indptr, rows, first_long, nnz_short,
                           tiles.as<int>(), nullptr, nullptr, map.as<int32_t>(), s);
    }
    if (n_long > 0)
        launch_group_long_rows(h->indptr, h->idx, h->val, h->perm, h->s_indptr, first_long, n_long,
                               std::min<int64_t>(h->n_wide_rows, n_long), h->plan_groups, nullptr, nullptr,
                               nullptr, map.as<int32_t>(), s);
    ACCEL_HIP(hipGetLastError());
    ACCEL_HIP(hipStreamSynchronize(s));     // `tiles` is released on return
    h->src_pos = static_cast<int32_t *>(map.release());
    return ACCEL_OK;
}

// s_val[p] = val[src_pos[p]]: four non-zeros per thread, the map read and the values written
// as 16-byte vectors (both arrays come from hipMalloc and start 256-byte aligned).
__global__ __launch_bounds__(kThreads) void gather_values_kernel(const float *__restrict__ val,
                                                                 const int32_t *__restrict__ src_pos,
                                                                 float *__restrict__ s_val, int64_t nnz)
{
    const int64_t p = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
    if (p + 4 <= nnz) {
        const int4 q = *reinterpret_cast<const int4 *>(src_pos + p);
        const float4 v = make_float4(val[q.x], val[q.y], val[q.z], val[q.w]);
        *reinterpret_cast<float4 *>(s_val + p) = v;
    } else {
        for (int64_t i = p; i < nnz; i++) s_val[i] = val[src_pos[i]];
    }
}

// One launch on s, no allocation, no wait: the sorted copy of the values from `val` (nnz
// floats in the caller's order).  The map must exist.
int gather_values(accel_handle *h, const float *val, hipStream_t s)
{
    if (!h->owns_sorted || h->nnz == 0) return ACCEL_OK;
    if (!h->src_pos) {
        set_error("internal: the position map of the value update is missing");
        return ACCEL_ERR_STATE;
    }
    const int64_t threads = (h->nnz + 3) / 4;
    gather_values_kernel<<<dim3(grid_for(threads)), dim3(kThreads), 0, s>>>(
        val, h->src_pos, const_cast<float *>(h->s_val), h->nnz);
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

// The other direction: val[src_pos[p]] = s_val[p].  A handle that owns a copy of the caller's
// values lets that copy go stale when the values are updated from a device array (the update
// then is the one gather above); the copy is only read again by a new preprocessing of the
// same handle, which calls this first.  Synchronises s.
__global__ __launch_bounds__(kThreads) void scatter_values_kernel(const float *__restrict__ s_val,
                                                                  const int32_t *__restrict__ src_pos,
                                                                  float *__restrict__ val, int64_t nnz)
{
    const int64_t p = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
    if (p + 4 <= nnz) {
        const int4 q = *reinterpret_cast<const int4 *>(src_pos + p);
        const float4 v = *reinterpret_cast<const float4 *>(s_val + p);
        val[q.x] = v.x; val[q.y] = v.y; val[q.z] = v.z; val[q.w] = v.w;
    } else {
        for (int64_t i = p; i < nnz; i++) val[src_pos[i]] = s_val[i];
    }
}

int restore_own_values(accel_handle *h, hipStream_t s)
{
    if (!h->val_stale) return ACCEL_OK;
    if (!h->owns_input || !h->owns_sorted || !h->src_pos || !h->s_val) {
        set_error("internal: the handle's copy of the values is stale and cannot be restored");
        return ACCEL_ERR_STATE;
    }
    const int64_t threads = (h->nnz + 3) / 4;
    scatter_values_kernel<<<dim3(grid_for(threads)), dim3(kThreads), 0, s>>>(
        h->s_val, h->src_pos, const_cast<float *>(h->val), h->nnz);
    ACCEL_HIP(hipGetLastError());
    ACCEL_HIP(hipStreamSynchronize(s));
    h->val_stale = false;
    return ACCEL_OK;
}

// A row order that comes from a saved state is taken only if it is the order the sort would
// produce: ascending degree, ties by ascending row id.  That order is unique, so checking
// that the pairs (degree, row) strictly increase along it and that every entry is a row
// index proves it (strictly increasing pairs cannot repeat a row, and rows of them are then
// all the rows).  Also writes the degrees in that order.
__global__ __launch_bounds__(kThreads) void check_given_order_kernel(const uint32_t *__restrict__ deg,
                                                                     const uint32_t *__restrict__ perm,
                                                                     int64_t rows, uint32_t *__restrict__ sdeg,
                                                                     int *__restrict__ bad)
{
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= rows) return;
    const uint32_t p = perm[i];
    if (p >= (uint64_t)rows) { *bad = 1; sdeg[i] = 0; return; }
    const uint32_t d = deg[p];
    sdeg[i] = d;
    if (i > 0) {
        const uint32_t q = perm[i - 1];
        if (q >= (uint64_t)rows) { *bad = 1; return; }
        const uint32_t dq = deg[q];
        if (dq > d || (dq == d && q >= p)) *bad = 1;
    }
}

// given: a row order from a saved state (checked before it is used), or null to sort.
int preprocess_device(accel_handle *h, const SavedOrder *given)
{
    const auto t0 = std::chrono::steady_clock::now();
    hipStream_t s = nullptr;
    const int64_t rows = h->rows, nnz = h->nnz;
    int rc;

    h->ready = false;
    h->n_blocks = h->n_long_blocks = h->n_long_rows = h->n_zero_rows = 0;
    h->max_degree = 0;
    h->n_units = h->n_long_units = 0;
    h->n_split_rows = h->n_big_rows = 0;
    h->plan_team = h->plan_team_option == 2 || (h->plan_team_option == 0 && choose_plan_team(rows, nnz));
    h->plan_unit = h->plan_unit_option > 0 ? h->plan_unit_option : choose_plan_unit(rows, nnz, h->plan_team);
    h->plan_split = h->plan_split_option > 0 ? h->plan_split_option : choose_plan_split(rows, nnz, h->plan_team);
    // a wavefront never takes more than plan_unit non-zeros; a workgroup takes a whole row of
    // up to plan_split even when units of several rows are kept smaller
    if (!h->plan_team) h->plan_split = std::min(h->plan_split, h->plan_unit);
    // Eight interleaved queues when the device is the whole MI355X (8 dies of 32 compute
    // units, workgroup i on die i % 8); any other shape (a partition of the GPU) gets the
    // plan in plain order, one queue, whose column groups are still worked on one by one.
    h->plan_queues = h->plan_queues_option > 0 ? h->plan_queues_option
                                               : (h->device_cus == kXcds * kCusPerDie ? kXcds : 1);
    if (rows == 0) {
        h->identity_perm = true;
        h->ready = true;
        return ACCEL_OK;
    }

    // temporaries: a small first chunk for the degrees and the statistics; once those are
    // known, one chunk sized for everything that follows (see below)
    Arena tmp;
    tmp.next_chunk = (size_t)rows * 4 + 4096;
    DevBuf deg(&tmp), st(&tmp);
    if ((rc = deg.alloc(sizeof(uint32_t) * (size_t)rows))) return rc;
    if ((rc = st.alloc(sizeof(Stats)))) return rc;
    ACCEL_HIP(hipMemsetAsync(st.p, 0, sizeof(Stats), s));
    degree_kernel<<<dim3(std::min(grid_for(rows), kDegreeGroups)), dim3(kThreads), 0, s>>>(
        h->indptr, rows, nnz, deg.as<uint32_t>(), st.as<Stats>(), h->plan_split, h->plan_unit);
    // validation of the columns and the locality sample run in the same batch: both only read
    // idx inside [0, nnz), whatever indptr holds
    if (nnz > 0) {
        const unsigned g = (unsigned)std::min<int64_t>((nnz / 4 + kThreads - 1) / kThreads + 1, 16384);
        index_check_kernel<<<dim3(g), dim3(kThreads), 0, s>>>(h->idx, nnz, h->cols, st.as<Stats>());
        locality_kernel<<<dim3(grid_for((rows + kLocalityStride - 1) / kLocalityStride)), dim3(kThreads), 0, s>>>(
            h->indptr, h->idx, rows, h->cols, nnz, kLocalityBand, st.as<Stats>());
    }
    Stats hs;
    ACCEL_HIP(hipMemcpyAsync(&hs, st.p, sizeof(Stats), hipMemcpyDeviceToHost, s));
    ACCEL_HIP(hipStreamSynchronize(s));
    if (hs.bad_indptr) {
        set_error("indptr must start at 0, be non-decreasing and end at nnz");
        return ACCEL_ERR_CSR;
    }
    if (hs.bad_index) {
        set_error("a column index lies outside [0, cols)");
        return ACCEL_ERR_CSR;
    }
    // A matrix whose non-zeros lie near the diagonal keeps its locality only in rows that stay
    // whole (their neighbourhood of X is what a die has in its L2 while it works through a band
    // of rows); storing such rows by column group trades that for nothing.  Measured at N = 64
    // with columns within N(0, 2000) of the row id: threshold 384 against 192: 593 against 651 us
    // (42 M non-zeros), 31 against 35 us (1.6 M); with N(0, 50000), which no L2 holds, 192 stays
    // better (1.14 against 1.24 ms).
    h->local = hs.sampled_nz > 0 && 2 * (int64_t)hs.local_nz >= hs.sampled_nz;
    if (h->local && h->plan_split_option == 0 && h->plan_split < h->plan_unit) {
        h->plan_split = h->plan_unit;
        hs.n_split_rows = hs.n_split_rows_alt;
        hs.n_big_rows = hs.n_big_rows_alt;
    }
    h->max_degree = hs.max_degree;
    h->n_zero_rows = hs.n_zero_rows;
    h->n_long_rows = hs.n_long_rows;
    h->n_long_blocks = hs.n_long_blocks;
    h->n_split_rows = hs.n_split_rows;
    h->n_big_rows = hs.n_big_rows;
    h->n_wide_rows = hs.n_wide_rows;
    h->identity_perm = !hs.unsorted;
    // Everything else comes out of one more chunk: 12.5 bytes per row for the sort, 16 for
    // the scans of the partition, up to 45 per whole-row unit of the plan (at most one per
    // row), about 800 per split row (its 64 group counts and 120 bin slots).  A device
    // allocation costs some 50 us whatever its size; a dozen of them were a sixth of the
    // preprocessing time.
    tmp.next_chunk = (size_t)rows * 76 + (size_t)hs.n_split_rows * 832 + (size_t)nnz / 256 + ((size_t)2 << 20);

    // ---- degree sort ------------------------------------------------------
    uint32_t *sdeg = deg.as<uint32_t>();
    uint32_t *perm = nullptr;
    DevBuf given_deg(&tmp), given_bad(&tmp);
    if (given && given->identity != h->identity_perm) {
        set_error("the saved state was made for rows in another order (it says the rows are %s sorted by "
                  "degree, this CSR's are%s)", given->identity ? "already" : "not", h->identity_perm ? "" : " not");
        return ACCEL_ERR_META;
    }
    if (!h->identity_perm && given) {
        if ((rc = given_deg.alloc(sizeof(uint32_t) * (size_t)rows))) return rc;
        if ((rc = given_bad.alloc(sizeof(int)))) return rc;
        ACCEL_HIP(hipMemsetAsync(given_bad.p, 0, sizeof(int), s));
        check_given_order_kernel<<<dim3(grid_for(rows)), dim3(kThreads), 0, s>>>(
            deg.as<uint32_t>(), given->perm_dev, rows, given_deg.as<uint32_t>(), given_bad.as<int>());
        int bad = 0;
        ACCEL_HIP(hipMemcpyAsync(&bad, given_bad.p, sizeof(int), hipMemcpyDeviceToHost, s));
        ACCEL_HIP(hipStreamSynchronize(s));
        if (bad) {
            set_error("the saved row order is not the degree order of this CSR (state of another matrix, or damaged)");
            return ACCEL_ERR_META;
        }
        sdeg = given_deg.as<uint32_t>();
        perm = const_cast<uint32_t *>(given->perm_dev);
    } else if (!h->identity_perm) {
        // unsorted input has max_degree >= 1, so at least one pass runs
        if ((rc = radix_sort_pairs(&tmp, deg.as<uint32_t>(), rows, (uint32_t)hs.max_degree, s, &sdeg, &perm)))
            return rc;
    }

    // ---- the products that stay: one allocation for the sorted indptr, the permutation
    // and the sorted copy of the non-zeros (a device allocation costs some 50 us)
    const int64_t n_long = hs.n_split_rows, first_long = rows - n_long;
    const bool own_copy = !h->identity_perm || n_long > 0;
    auto pad = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t b_sip = pad(sizeof(int32_t) * (size_t)(rows + 1));
    const size_t b_perm = h->identity_perm ? 0 : pad(sizeof(int32_t) * (size_t)rows);
    const size_t b_nz = own_copy ? pad(sizeof(int32_t) * (size_t)nnz) : 0;
    DevBuf slab;
    if ((rc = slab.alloc(b_sip + b_perm + 2 * b_nz))) return rc;
    DevView sip, permbuf, sidx, sval;                // parts of the slab
    sip.p = slab.p;
    if (b_perm) permbuf.p = slab.as<char>() + b_sip;
    if (b_nz) {
        sidx.p = slab.as<char>() + b_sip + b_perm;
        sval.p = slab.as<char>() + b_sip + b_perm + b_nz;
    }

    // ---- sorted indptr ------------------------------------------------------
    DevBuf ssums(&tmp);
    if ((rc = ssums.alloc(sizeof(int) * (size_t)(rows / kTile + 4)))) return rc;
    if ((rc = device_scan<SumOp, false>(reinterpret_cast<const int *>(sdeg), rows, sip.as<int>(),
                                        sip.as<int>() + rows, ssums.as<int>(), s)))
        return rc;

    // ---- partition ----------------------------------------------------------
    // (before the sorted CSR: its one synchronisation also tells how many non-zeros the rows
    // that are not split hold, which sizes the gather below)
    // Sizes from the degree histogram: the rows are in ascending degree order, so every degree
    // d <= 384 forms one run, cut into ceil(count / rows per block) blocks.
    int32_t *b4 = nullptr;
    int64_t nb = hs.n_long_blocks;
    int64_t n_short_entries = 0;   // block4 entries of the rows that are not cut into pieces
    int64_t nnz_short = 0;         // their non-zeros
    for (int d = 1; d <= kDegBound; d++) {
        int w, rpb;
        slice_rule(d, w, rpb);
        const int64_t blocks = ((int64_t)hs.hist[d] + rpb - 1) / rpb;
        nb += blocks;
        if (d <= h->plan_split) {
            n_short_entries += blocks;
            nnz_short += (int64_t)d * hs.hist[d];
        }
    }
    const int *total_blocks_dev = nullptr;
    if ((rc = partition_device(&tmp, sdeg, sip.as<int32_t>(), rows, &b4, &nb, s, -1, nullptr, nullptr, nb,
                               &total_blocks_dev)))
        return rc;
    h->block4 = b4;
    h->n_blocks = nb;
    if (nb + (int64_t)kMaxGroups * n_long + kXcds * kWavesPerGroup > (int64_t)INT_MAX) {
        set_error("the launch plan would exceed 2^31 work units (%lld block4 entries)", (long long)nb);
        return ACCEL_ERR_ARG;
    }

    // ---- sorted CSR ---------------------------------------------------------
    // Split rows (more than plan_split non-zeros: the last n_long rows of the sorted
    // order) are stored grouped by column group; all other rows keep their non-zero
    // order.  The caller's arrays are used in place only when the input was already
    // sorted and has no split row.
    DevBuf gcount(&tmp), tiles(&tmp);
    if (own_copy) {
        const int32_t *pm = reinterpret_cast<const int32_t *>(perm);
        if (h->identity_perm) {
            if (nnz_short > 0) {
                ACCEL_HIP(hipMemcpyAsync(sidx.p, h->idx, sizeof(int32_t) * (size_t)nnz_short,
                                         hipMemcpyDeviceToDevice, s));
                ACCEL_HIP(hipMemcpyAsync(sval.p, h->val, sizeof(float) * (size_t)nnz_short,
                                         hipMemcpyDeviceToDevice, s));
            }
        } else {
            if (nnz_short > 0) {
                if ((rc = tiles.alloc(sizeof(int) * (size_t)(nnz_short / kPermuteTile + 2)))) return rc;
                launch_permute_csr(h->indptr, h->idx, h->val, pm, sip.as<int32_t>(), rows, first_long, nnz_short,
                                   tiles.as<int>(), sidx.as<int32_t>(), sval.as<float>(), nullptr, s);
            }
            ACCEL_HIP(hipMemcpyAsync(permbuf.p, perm, sizeof(int32_t) * (size_t)rows,
                                     hipMemcpyDeviceToDevice, s));
        }
        if (n_long > 0) {
            if ((rc = gcount.alloc(sizeof(int) * (size_t)n_long * kMaxGroups))) return rc;
            launch_group_long_rows(h->indptr, h->idx, h->val, pm, sip.as<int32_t>(), first_long, n_long,
                                   std::min<int64_t>(hs.n_wide_rows, n_long), h->plan_groups,
                                   sidx.as<int32_t>(), sval.as<float>(), gcount.as<int>(), nullptr, s);
        }
        ACCEL_HIP(hipGetLastError());
    }

    // ---- work list ------------------------------------------------------------
    if ((rc = build_work_list(&tmp, h, gcount.as<int>(), sip.as<int32_t>(), first_long, n_short_entries, perm,
                              total_blocks_dev, s)))
        return rc;

    h->slab = slab.release();
    h->nnz_short = nnz_short;
    h->s_indptr = sip.as<int32_t>();
    h->perm = permbuf.as<int32_t>();                 // null for sorted input
    if (!own_copy) {
        h->s_idx = h->idx;
        h->s_val = h->val;
        h->owns_sorted = false;
    } else {
        h->s_idx = sidx.as<int32_t>();
        h->s_val = sval.as<float>();
        h->owns_sorted = true;
    }
    h->ready = true;
    h->preprocess_ms =
        std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return ACCEL_OK;
}

}  // namespace accel
