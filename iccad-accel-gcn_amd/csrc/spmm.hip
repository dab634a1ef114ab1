// The SpMM gather kernels for gfx950 (wave64), the partial-sum reduction and two helpers.
//
// Work decomposition.  Upstream gives one CUDA thread block of 12 32-lane warps
// to each block4 entry (spmm_accel.cu:18-28).  Here one 64-lane wavefront takes
// one work unit and a 256-thread workgroup takes four.  A unit is either whole
// rows of one block4 entry (up to 12 rows of one degree, <= 384 non-zeros in
// total) or a piece of <= 384 non-zeros of a split row (every row with more than
// 384 non-zeros is split; the plan also splits somewhat shorter ones).  The units
// come from a launch plan built by the preprocessing step; it orders them so that
// workgroup i, which the hardware places on die i % 8, works on a share of X that
// die keeps in its own L2: a column group for the pieces of split rows, a band of
// the caller's rows for the whole-row units.  Small matrices use the same list
// with one unit per workgroup instead (spmm_team_kernel below).
//
// Inside the wavefront the lanes form G = 64 / L groups of L lanes; a group owns
// L * VEC consecutive columns of X/Y (VEC = 4 floats = one 16-byte load per lane
// when N allows), so one vector-memory instruction gathers G different rows of X.
// This replaces upstream's "combined warp" of ceil32(N) lanes that walks one
// non-zero at a time with 4-byte loads (spmm_accel.cu:37-48,56-78).  G groups are
// split over the unit's rows as gp groups per row (gp a power of two chosen per
// unit to minimise the step count); the gp partial sums of a row are combined by
// a cross-lane butterfly, so short rows need no atomics (upstream: atomicAdd for
// every row that spans more than one warp, spmm_accel.cu:82-99).
//
// The (column index, value) pairs of the unit are first staged in LDS with
// coalesced loads, one pair per lane; each group then reads its pairs back with
// broadcast LDS reads.  Pieces of split rows write their partial sums to a
// scratch buffer and a second small kernel adds them up in a fixed order, so the
// result is run-to-run deterministic.  Rows of degree 0 are zero-filled by extra
// workgroups of the same launch: Y = A X holds after every run with no memset.
#include <mutex>

#include <hip/hip_ext.h>

#include "internal.h"

// Partial sums for accel_run_static, the entry point that allocates nothing: one copy of
// this array per GPU, held from the moment the library's code is loaded on that GPU until
// the process ends.  In host code the name is only a handle for the runtime, not a device
// address: static_scratch_address() asks for the address once per GPU and everything else
// (kernel arguments included) uses that pointer.
static constexpr size_t kStaticScratchFloats = (size_t)ACCEL_STATIC_SCRATCH_BYTES / sizeof(float);
static constexpr int kMaxScratchDevices = 64;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

namespace accel {
namespace {

constexpr int kWaves = kWavesPerGroup;    // wavefronts (= work units) per workgroup
constexpr int kWgThreads = 64 * kWaves;
constexpr int kZeroFloats = 8192;         // floats zero-filled per extra workgroup
constexpr int kReduceThreads = 256;       // workgroup of the partial-sum reduction

// zero-degree rows handled by one zero-fill workgroup (N is a multiple of VEC, so
// a workgroup's share is a whole number of vectors)
__host__ __device__ inline int zero_rows_per_group(int N) { return N >= kZeroFloats ? 1 : kZeroFloats / N; }

constexpr int kUnroll = 4;                // gathers in flight per lane in the main loop (2 and 8 measured within 2 %)
constexpr int kTeamUnroll = 4;            // the same with workgroup units (8: 5-10 % slower)
constexpr int kPanel = 64;                // column-panel width for wide operands on large matrices
constexpr int kPanelMinNnz = 4000000;     // smaller matrices are not worth several launches
constexpr int kStreamingMinBytes = 64;    // rows of Y of at least this many bytes are stored streaming
                                          // (64-byte rows: L2-resident X -18 %, elsewhere within 1 %)

// A vector of four floats that is only 4-byte aligned: rows of X and Y start at any
// multiple of 4 bytes when N is not a multiple of 4.  The hardware takes 16-byte
// accesses at such addresses; the type keeps the compiler from assuming more.
typedef float v4f __attribute__((ext_vector_type(4)));
typedef v4f v4f_unaligned __attribute__((aligned(4)));

template <int VEC, bool kShift>
__device__ __forceinline__ void load_vec(const float *__restrict__ p, float (&v)[VEC])
{
    if constexpr (VEC == 4 && kShift) {
        const v4f t = *reinterpret_cast<const v4f_unaligned *>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else if constexpr (VEC == 4) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else {
        static_assert(VEC == 1, "vector widths: 4 or 1");
        v[0] = *p;
    }
}

// Rows of Y are written once and not read again by this launch: a streaming
// (non-temporal) store when `streaming`.  Measured on this GPU with gathers that hit L2:
// one ordinary 256-byte store per 32 gathers lowers the gather rate from 27 to 20 TB/s, a
// non-temporal one to 26 TB/s.
template <int VEC, bool kShift>
__device__ __forceinline__ void store_vec(float *__restrict__ p, const float (&v)[VEC], bool streaming)
{
    if constexpr (VEC == 4) {
        const v4f t = {v[0], v[1], v[2], v[3]};
        if constexpr (kShift) {
            if (streaming) __builtin_nontemporal_store(t, reinterpret_cast<v4f_unaligned *>(p));
            else *reinterpret_cast<v4f_unaligned *>(p) = t;
        } else {
            if (streaming) __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
            else *reinterpret_cast<v4f *>(p) = t;
        }
    } else {
        if (streaming) __builtin_nontemporal_store(v[0], p);
        else *p = v[0];
    }
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Partial sums that another wavefront of the same launch, possibly on another die, adds up
// (the row's last piece does, see finish_split_row): stored and loaded as relaxed atomics of
// device scope.  Such a store goes through to memory instead of staying in the die's L2, and
// such a load does not take a line the die's L2 may hold from before; no cache is written
// back or invalidated as a whole, which is what a device-scope fence would do on every piece.
template <int VEC>
__device__ __forceinline__ void store_partial(float *__restrict__ p, const float (&v)[VEC])
{
#pragma unroll
    for (int i = 0; i < VEC; i++) __hip_atomic_store(p + i, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_partial(const float *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A piece of a split row has stored its partial sums (this thread's stores included).  Counts
// the piece in; returns true to all T threads of the team (one wavefront, or the workgroup)
// if it was the row's last one, after which every piece's sums are in memory: each piece
// waits for its own stores before it counts itself in, and the counter is one memory location.
// `flag` is a word of LDS of the team's own.  The counter is left at zero for the next launch.
template <int T>
__device__ __forceinline__ bool last_piece_of_row(int *__restrict__ counter, int n_pieces, int tid, int *flag)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // this thread's partial sums have arrived
    if constexpr (T > 64) __syncthreads();                    // ... and those of the other wavefronts
    if (tid == 0) {
        const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = before == n_pieces - 1;
        if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last;
    }
    if constexpr (T > 64) __syncthreads(); else __builtin_amdgcn_wave_barrier();
    return *flag != 0;
}

// Adds the nseg partial sums of a split row in slot order and writes the row: T threads
// (a wavefront or a workgroup), `red` = T floats of LDS of their own.  The columns are
// covered cw at a time (cw = the power of two <= T that covers N, or T); the T / cw slot
// groups take every (T / cw)-th slot and their sums are added in group order, so the result
// does not depend on which piece finished last.
template <int T>
__device__ __forceinline__ void finish_split_row(const float *__restrict__ src, int nseg, float *__restrict__ y,
                                                 int N, int ld, const float *__restrict__ bias, int relu,
                                                 int tid, float *red)
{
    int cw = 1;
    while (cw < N && cw < T) cw <<= 1;
    const int sg = T / cw;
    const int c_in = tid % cw, my_sg = tid / cw;
    for (int c0 = 0; c0 < N; c0 += cw) {
        const int c = c0 + c_in;
        float acc = 0.0f;
        if (c < N) {
            int s = my_sg;
            for (; s + 7 * sg < nseg; s += 8 * sg) {          // eight loads in flight, added in order
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = load_partial(src + (int64_t)(s + u * sg) * ld + c);
#pragma unroll
                for (int u = 0; u < 8; u++) acc += v[u];
            }
            for (; s < nseg; s += sg) acc += load_partial(src + (int64_t)s * ld + c);
        }
        if (sg > 1) {
            red[tid] = acc;
            if constexpr (T > 64) __syncthreads(); else __builtin_amdgcn_wave_barrier();
            if (my_sg == 0)
                for (int q = 1; q < sg; q++) acc += red[q * cw + c_in];
            if constexpr (T > 64) __syncthreads(); else __builtin_amdgcn_wave_barrier();
        }
        if (my_sg == 0 && c < N) {
            if (bias) acc += bias[c];
            if (relu) acc = fmaxf(acc, 0.0f);
            y[c] = acc;
        }
    }
}

// One lane group's share of one row: non-zeros k, k + gp, ... of the d pairs at row_st are
// multiplied with their rows of X and added into acc.  U gathers are issued back to back;
// full batches carry no masks, only the last batch of a row is predicated.
// The staged pair holds the value and, when the operand is smaller than 4 GiB (kWide ==
// false), the byte offset of the row of X, so that the address is one 32-bit add to a
// uniform base; otherwise the column, and the address is formed with 64-bit arithmetic.
template <int VEC, int U, bool kWide, bool kShift>
__device__ __forceinline__ void gather_row(const int2 *__restrict__ row_st, int d, int k, int gp,
                                           const float *__restrict__ X, int col, int ld,
                                           float (&acc)[VEC])
{
    const char *xb = reinterpret_cast<const char *>(X);
    const uint32_t lane_off = (uint32_t)col * 4u;
    auto fetch = [&](int where, float (&x)[VEC]) {
        if constexpr (kWide)
            load_vec<VEC, kShift>(X + col + (int64_t)where * ld, x);
        else
            load_vec<VEC, kShift>(reinterpret_cast<const float *>(xb + ((uint32_t)where + lane_off)), x);
    };
    int o = k;
    for (; o + (U - 1) * gp < d; o += U * gp) {          // full batches
        int2 p[U];
        float x[U][VEC];
#pragma unroll
        for (int u = 0; u < U; u++) p[u] = row_st[o + u * gp];
#pragma unroll
        for (int u = 0; u < U; u++) fetch(p[u].x, x[u]);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float a = __int_as_float(p[u].y);
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] = fmaf(a, x[u][v], acc[v]);
        }
    }
    if (o < d) {                                         // the row's last, partial batch
        int2 p[U];
        float x[U][VEC];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ou = o + u * gp;
            ok[u] = ou < d;
            p[u] = row_st[ok[u] ? ou : k];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int v = 0; v < VEC; v++) x[u][v] = 0.0f;
            if (ok[u]) fetch(p[u].x, x[u]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float a = ok[u] ? __int_as_float(p[u].y) : 0.0f;
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] = fmaf(a, x[u][v], acc[v]);
        }
    }
}

// Zero-degree rows are the first n_zero_rows rows of the sorted order; the workgroups at
// the head of the grid write them (act(bias) with an epilogue).  They come first so that
// they do not form a tail.
template <int VEC>
__device__ __forceinline__ void zero_fill_rows(const int32_t *__restrict__ perm, float *__restrict__ Y,
                                               int N, int ld, int n_zero_rows,
                                               const float *__restrict__ bias, int relu)
{
    const int rows_here = zero_rows_per_group(N);
    const int r0 = (int)blockIdx.x * rows_here;
    const int n = min(rows_here, n_zero_rows - r0) * N;        // floats of this workgroup
    float fill[VEC];
    for (int i = (int)threadIdx.x * VEC; i < n; i += kWgThreads * VEC) {
        const int r = i / N, c = i - r * N;
        const int64_t out_row = perm ? perm[r0 + r] : r0 + r;
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            float t = bias ? bias[c + v] : 0.0f;                // A X is 0 for this row
            fill[v] = relu ? fmaxf(t, 0.0f) : t;
        }
        store_vec<VEC, false>(Y + out_row * ld + c, fill, N * 4 >= kStreamingMinBytes);
    }
}

template <int L, int VEC, bool kWide, bool kShift>
__global__ __launch_bounds__(kWgThreads) void spmm_gather_kernel(
    const int4 *__restrict__ work, int n_units,
    const int32_t *__restrict__ s_idx, const float *__restrict__ s_val,
    const int32_t *__restrict__ perm, const float *__restrict__ X, float *__restrict__ Y,
    float *__restrict__ partial, int N, int ld, int n_zero_rows, int n_zero_groups,
    const float *__restrict__ bias, int relu, const int32_t *__restrict__ long_slot, int first_split_row,
    int *__restrict__ row_done)
{
    // N columns are computed; rows of X, Y and the partial sums are ld floats apart
    // (ld > N when the launch covers one column panel of a wider operand)
    constexpr int G = 64 / L;        // lane groups per wavefront
    constexpr int CW = L * VEC;      // columns covered per pass
    __shared__ int2 stage[kWaves][kDegBound];

    if ((int)blockIdx.x < n_zero_groups) {
        zero_fill_rows<kShift ? 1 : VEC>(perm, Y, N, ld, n_zero_rows, bias, relu);
        return;
    }

    const int lane = threadIdx.x & 63;
    const int wv = uniform(threadIdx.x >> 6);
    const int e = ((int)blockIdx.x - n_zero_groups) * kWaves + wv;
    if (e >= n_units) return;

    const int4 b = work[e];
    const int deg = uniform(b.x), row0 = uniform(b.y), loc = uniform(b.z), info = uniform(b.w);
    if (info == 0) return;                              // padding unit
    const bool is_long = deg > kDegBound;
    const int n_rows = is_long ? 1 : (info & 0xFFFF);   // spmm_accel.cu:26
    const int d = is_long ? info : deg;                 // spmm_accel.cu:28: non-zeros per row here
    const int total_nz = n_rows * d;

    // output row of each of the unit's rows, fetched up front (lane r holds row r)
    int my_out = row0 + lane;
    if (!is_long && perm && lane < n_rows) my_out = perm[row0 + lane];

    // stage the entry's (column, value) pairs: all loads are issued before the first LDS write
    int2 *st = stage[wv];
    {
        constexpr int kRounds = kDegBound / 64;
        int ci[kRounds];
        float cv[kRounds];
#pragma unroll
        for (int j = 0; j < kRounds; j++) {
            const int i = lane + 64 * j;
            if (i < total_nz) {
                ci[j] = s_idx[loc + i];
                cv[j] = s_val[loc + i];
            }
        }
#pragma unroll
        for (int j = 0; j < kRounds; j++) {
            const int i = lane + 64 * j;
            if (i < total_nz) st[i] = make_int2(kWide ? ci[j] : (int)((uint32_t)ci[j] * ((uint32_t)ld * 4u)), __float_as_int(cv[j]));
        }
    }
    __builtin_amdgcn_wave_barrier();

    // groups per row: power of two that minimises ceil(n_rows / (G/gp)) * ceil(d / gp)
    int lg = 0;
    if constexpr (G > 1) {
        int best = 0x7fffffff;
#pragma unroll
        for (int q = 0; (1 << q) <= G; q++) {
            const int rows_at_once = G >> q;
            const int steps = ((n_rows + rows_at_once - 1) / rows_at_once) * ((d + (1 << q) - 1) >> q);
            if (steps < best) { best = steps; lg = q; }
        }
    }
    const int gp = 1 << lg;
    const int rows_at_once = G >> lg;
    const int g = lane / L, sub = lane % L;
    const int k = g & (gp - 1);          // which of the row's gp groups this is
    const int rloc = g >> lg;            // which of the rows in flight

    const bool streaming = N * 4 >= kStreamingMinBytes;
    for (int c0 = 0; c0 < N; c0 += CW) {
        int col = c0 + sub * VEC;
        const bool col_ok = col < N;
        if (kShift && col + VEC > N) col = N - VEC;   // the row's last vector ends with the row
        for (int r_it = 0; r_it < n_rows; r_it += rows_at_once) {
            const int r = r_it + rloc;
            const bool live = col_ok && r < n_rows;
            float acc[VEC];
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] = 0.0f;
            if (live) gather_row<VEC, kUnroll, kWide, kShift>(st + r * d, d, k, gp, X, col, ld, acc);
            // add the gp partial sums of each row (all lanes take part)
            for (int m = L; m < (L << lg); m <<= 1) {
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += __shfl_xor(acc[v], m);
            }
            const int64_t out_row = __shfl(my_out, r < n_rows ? r : 0);
            if (live && k == 0) {
                if (is_long) {
                    float *p = partial + (int64_t)(deg - (kDegBound + 1)) * ld + col;
                    if (row_done) store_partial<VEC>(p, acc);
                    else store_vec<VEC, kShift>(p, acc, streaming);
                } else {
                    if (bias) {
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[v] += bias[col + v];
                    }
                    if (relu) {
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[v] = fmaxf(acc[v], 0.0f);
                    }
                    store_vec<VEC, kShift>(Y + out_row * ld + col, acc, streaming);
                }
            }
        }
    }
    // The wavefront that stores a split row's last piece adds the row up, in this launch
    // (row_done: one counter per split row; null: a second kernel does it).
    if (is_long && row_done) {
        const int lr = row0 - first_split_row;
        const int first = long_slot[lr], nseg = long_slot[lr + 1] - first;
        int *flag = reinterpret_cast<int *>(st);             // the staged pairs are no longer needed
        if (last_piece_of_row<64>(row_done + lr, nseg, lane, flag)) {
            const int64_t out_row = perm ? perm[row0] : row0;
            finish_split_row<64>(partial + (int64_t)first * ld, nseg, Y + out_row * ld, N, ld, bias, relu, lane,
                                 reinterpret_cast<float *>(st) + 64);
        }
    }
}

// The same computation with one unit per workgroup: the four wavefronts form 4 * G lane
// groups that share the unit's rows, or its row's non-zeros.  When a row's groups span
// several wavefronts their sums meet in LDS.  Used for small matrices, where the time of
// a launch is the longest chain of dependent gathers in one wavefront: the chain is four
// times shorter and rows of up to one unit need no partial sums.
template <int L, int VEC, bool kWide, bool kShift>
__global__ __launch_bounds__(kWgThreads) void spmm_team_kernel(
    const int4 *__restrict__ work, int n_units,
    const int32_t *__restrict__ s_idx, const float *__restrict__ s_val,
    const int32_t *__restrict__ perm, const float *__restrict__ X, float *__restrict__ Y,
    float *__restrict__ partial, int N, int ld, int n_zero_rows, int n_zero_groups,
    const float *__restrict__ bias, int relu, const int32_t *__restrict__ long_slot, int first_split_row,
    int *__restrict__ row_done)
{
    constexpr int G = 64 / L;        // lane groups per wavefront
    constexpr int TG = G * kWaves;   // lane groups per workgroup
    constexpr int CW = L * VEC;      // columns covered per pass
    __shared__ int2 stage[kDegBound];
    __shared__ float meet[kWaves][CW];

    if ((int)blockIdx.x < n_zero_groups) {
        zero_fill_rows<kShift ? 1 : VEC>(perm, Y, N, ld, n_zero_rows, bias, relu);
        return;
    }
    const int lane = threadIdx.x & 63;
    const int wv = uniform(threadIdx.x >> 6);
    const int e = (int)blockIdx.x - n_zero_groups;
    if (e >= n_units) return;
    const int4 b = work[e];
    const int deg = uniform(b.x), row0 = uniform(b.y), loc = uniform(b.z), info = uniform(b.w);
    if (info == 0) return;                              // padding unit (the whole workgroup leaves)
    const bool is_long = deg > kDegBound;
    const int n_rows = is_long ? 1 : (info & 0xFFFF);
    const int d = is_long ? info : deg;
    const int total_nz = n_rows * d;

    int my_out = row0 + lane;
    if (!is_long && perm && lane < n_rows) my_out = perm[row0 + lane];

    {   // stage the unit's (column, value) pairs: 256 threads, at most two rounds
        constexpr int kRounds = (kDegBound + kWgThreads - 1) / kWgThreads;
        int ci[kRounds];
        float cv[kRounds];
#pragma unroll
        for (int j = 0; j < kRounds; j++) {
            const int i = (int)threadIdx.x + kWgThreads * j;
            if (i < total_nz) {
                ci[j] = s_idx[loc + i];
                cv[j] = s_val[loc + i];
            }
        }
#pragma unroll
        for (int j = 0; j < kRounds; j++) {
            const int i = (int)threadIdx.x + kWgThreads * j;
            if (i < total_nz) stage[i] = make_int2(kWide ? ci[j] : (int)((uint32_t)ci[j] * ((uint32_t)ld * 4u)), __float_as_int(cv[j]));
        }
    }
    __syncthreads();

    // groups per row: power of two that minimises ceil(n_rows / (TG/gp)) * ceil(d / gp)
    int lg = 0;
    {
        int best = 0x7fffffff;
#pragma unroll
        for (int q = 0; (1 << q) <= TG; q++) {
            const int rows_at_once = TG >> q;
            const int steps = ((n_rows + rows_at_once - 1) / rows_at_once) * ((d + (1 << q) - 1) >> q);
            if (steps < best) { best = steps; lg = q; }
        }
    }
    const int gp = 1 << lg;
    const int rows_at_once = TG >> lg;
    const int g = lane / L, sub = lane % L;
    const int vg = wv * G + g;           // this lane group among the workgroup's
    const int k = vg & (gp - 1);         // which of the row's gp groups this is
    const int rloc = vg >> lg;           // which of the rows in flight
    const int in_wave = gp < G ? gp : G;             // groups of one row inside a wavefront
    const int waves_per_row = gp > G ? gp / G : 1;   // > 1: the row's sums meet in LDS

    for (int c0 = 0; c0 < N; c0 += CW) {
        int col = c0 + sub * VEC;
        const bool col_ok = col < N;
        if (kShift && col + VEC > N) col = N - VEC;   // the row's last vector ends with the row
        for (int r_it = 0; r_it < n_rows; r_it += rows_at_once) {
            const int r = r_it + rloc;
            const bool live = col_ok && r < n_rows;
            float acc[VEC];
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] = 0.0f;
            if (live) gather_row<VEC, kTeamUnroll, kWide, kShift>(stage + r * d, d, k, gp, X, col, ld, acc);
            // the row's groups inside this wavefront (all lanes take part)
            for (int m = L; m < L * in_wave; m <<= 1) {
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += __shfl_xor(acc[v], m);
            }
            if (waves_per_row > 1) {                 // workgroup-uniform
                if (g == 0) {
#pragma unroll
                    for (int v = 0; v < VEC; v++) meet[wv][sub * VEC + v] = acc[v];
                }
                __syncthreads();
                if (wv % waves_per_row == 0 && g == 0) {
                    for (int q = 1; q < waves_per_row; q++) {
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[v] += meet[wv + q][sub * VEC + v];
                    }
                }
                __syncthreads();
            }
            const int64_t out_row = __shfl(my_out, r < n_rows ? r : 0);
            if (live && k == 0) {
                if (is_long) {
                    float *p = partial + (int64_t)(deg - (kDegBound + 1)) * ld + col;
                    if (row_done) store_partial<VEC>(p, acc);
                    else store_vec<VEC, kShift>(p, acc, false);
                } else {
                    if (bias) {
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[v] += bias[col + v];
                    }
                    if (relu) {
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[v] = fmaxf(acc[v], 0.0f);
                    }
                    store_vec<VEC, kShift>(Y + out_row * ld + col, acc, N * 4 >= kStreamingMinBytes);
                }
            }
        }
    }
    // the workgroup that stores a split row's last piece adds the row up (see the gather kernel)
    if (is_long && row_done) {                       // workgroup-uniform
        const int lr = row0 - first_split_row;
        const int first = long_slot[lr], nseg = long_slot[lr + 1] - first;
        __syncthreads();                             // every wavefront is done with the staged pairs
        int *flag = reinterpret_cast<int *>(stage);
        if (last_piece_of_row<kWgThreads>(row_done + lr, nseg, (int)threadIdx.x, flag)) {
            const int64_t out_row = perm ? perm[row0] : row0;
            finish_split_row<kWgThreads>(partial + (int64_t)first * ld, nseg, Y + out_row * ld, N, ld, bias, relu,
                                         (int)threadIdx.x, reinterpret_cast<float *>(stage) + 64);
        }
    }
}

// Adds the partial sums of each split row in slot order and writes the row.
// The first n_shared_groups workgroups take rpw rows each (256 / rpw threads per
// row): rows with few slots and few columns do not need a whole workgroup.  The
// remaining workgroups take one row each: the rows with very many slots.
// A thread covers VEC consecutive columns (VEC = 4: one 16-byte load per slot, when N and
// the row stride are multiples of 4 and the operands 16-byte aligned; else VEC = 1); NV = the
// row's columns counted in such vectors.
template <int VEC>
__global__ __launch_bounds__(kReduceThreads) void long_row_reduce_kernel(
    const float *__restrict__ partial, const int32_t *__restrict__ long_slot,
    const int32_t *__restrict__ perm, int64_t first_split_row, int n_shared_rows, int n_shared_groups,
    int rpw, int n_rows, float *__restrict__ Y, int NV, int ld, const float *__restrict__ bias, int relu)
{
    // rows of Y and of the partial sums are ld floats apart
    __shared__ float red[kReduceThreads][VEC];
    const bool shared_group = (int)blockIdx.x < n_shared_groups;
    const int T = shared_group ? kReduceThreads / rpw : kReduceThreads;   // threads per row
    const int sub_row = threadIdx.x / T, t = threadIdx.x % T;
    const int lr = shared_group ? (int)blockIdx.x * rpw + sub_row
                                : n_shared_rows + ((int)blockIdx.x - n_shared_groups);
    const bool row_ok = lr < (shared_group ? n_shared_rows : n_rows);
    const int first = row_ok ? long_slot[lr] : 0;
    const int nseg = row_ok ? long_slot[lr + 1] - first : 0;
    const float *src = partial + (int64_t)first * ld;
    const int64_t r = first_split_row + lr;
    const int64_t out_row = row_ok ? (perm ? perm[r] : r) : 0;
    int cw = 1;                                    // vectors per pass: power of two <= T
    while (cw < NV && cw < T) cw <<= 1;
    const int sg = T / cw;                         // slot groups
    const int c_in = t % cw, my_sg = t / cw;
    for (int c0 = 0; c0 < NV; c0 += cw) {
        const int c = (c0 + c_in) * VEC;           // first column of this thread's vector
        const bool col_ok = c0 + c_in < NV;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[v] = 0.0f;
        if (col_ok) {
            int sgm = my_sg;
            for (; sgm + 7 * sg < nseg; sgm += 8 * sg) {       // eight loads in flight, added in order
                float x[8][VEC];
#pragma unroll
                for (int u = 0; u < 8; u++) load_vec<VEC, false>(src + (int64_t)(sgm + u * sg) * ld + c, x[u]);
#pragma unroll
                for (int u = 0; u < 8; u++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[v] += x[u][v];
            }
            for (; sgm < nseg; sgm += sg) {
                float x[VEC];
                load_vec<VEC, false>(src + (int64_t)sgm * ld + c, x);
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += x[v];
            }
        }
        if (sg > 1) {                              // uniform over the workgroup's rows of one kind
#pragma unroll
            for (int v = 0; v < VEC; v++) red[threadIdx.x][v] = acc[v];
            __syncthreads();
            if (my_sg == 0)
                for (int q = 1; q < sg; q++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[v] += red[sub_row * T + q * cw + c_in][v];
            __syncthreads();
        }
        if (row_ok && my_sg == 0 && col_ok) {
            if (bias) {
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += bias[c + v];
            }
            if (relu) {
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] = fmaxf(acc[v], 0.0f);
            }
            store_vec<VEC, false>(Y + out_row * ld + c, acc, false);
        }
    }
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *dst, uint32_t v, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        dst[i] = v;
}

__global__ __launch_bounds__(256) void copy_u32_kernel(uint32_t *__restrict__ dst,
                                                       const uint32_t *__restrict__ src, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        dst[i] = src[i];
}

struct LaunchArgs {
    bool team;
    dim3 grid;
    hipStream_t stream;
    const int4 *work;
    int n_units;
    const int32_t *s_idx;
    const float *s_val;
    const int32_t *perm;
    const float *X;
    float *Y;
    float *partial;
    int N, ld, n_zero_rows, n_zero_groups;
    const float *bias;
    int relu;
    const int32_t *long_slot;
    int first_split_row;
    int *row_done;
    // events bound to this launch itself (its start and its end), or null: unlike an event
    // recorded behind the launch they put no packet of their own into the queue
    hipEvent_t start_ev, stop_ev;
};

template <int L, int VEC, bool kWide, bool kShift>
void launch_one(const LaunchArgs &a)
{
    if (a.start_ev || a.stop_ev) {
        if (a.team)
            hipExtLaunchKernelGGL((spmm_team_kernel<L, VEC, kWide, kShift>), a.grid, dim3(kWgThreads), 0, a.stream,
                                  a.start_ev, a.stop_ev, 0, a.work, a.n_units, a.s_idx, a.s_val, a.perm, a.X, a.Y,
                                  a.partial, a.N, a.ld, a.n_zero_rows, a.n_zero_groups, a.bias, a.relu, a.long_slot,
                                  a.first_split_row, a.row_done);
        else
            hipExtLaunchKernelGGL((spmm_gather_kernel<L, VEC, kWide, kShift>), a.grid, dim3(kWgThreads), 0, a.stream,
                                  a.start_ev, a.stop_ev, 0, a.work, a.n_units, a.s_idx, a.s_val, a.perm, a.X, a.Y,
                                  a.partial, a.N, a.ld, a.n_zero_rows, a.n_zero_groups, a.bias, a.relu, a.long_slot,
                                  a.first_split_row, a.row_done);
        return;
    }
    if (a.team)
        spmm_team_kernel<L, VEC, kWide, kShift><<<a.grid, dim3(kWgThreads), 0, a.stream>>>(
            a.work, a.n_units, a.s_idx, a.s_val, a.perm, a.X, a.Y, a.partial, a.N, a.ld, a.n_zero_rows,
            a.n_zero_groups, a.bias, a.relu, a.long_slot, a.first_split_row, a.row_done);
    else
        spmm_gather_kernel<L, VEC, kWide, kShift><<<a.grid, dim3(kWgThreads), 0, a.stream>>>(
            a.work, a.n_units, a.s_idx, a.s_val, a.perm, a.X, a.Y, a.partial, a.N, a.ld, a.n_zero_rows,
            a.n_zero_groups, a.bias, a.relu, a.long_slot, a.first_split_row, a.row_done);
}

// Lane-group widths: 1..64 lanes of one 16-byte vector each; scalar lanes only serve N < 4.
template <int VEC, bool kWide, bool kShift>
int launch_for_width(int L, const LaunchArgs &a)
{
    switch (L) {
    case 1: launch_one<1, VEC, kWide, kShift>(a); break;
    case 2: launch_one<2, VEC, kWide, kShift>(a); break;
    case 4: launch_one<4, VEC, kWide, kShift>(a); break;
    default:
        if constexpr (VEC == 4) {
            switch (L) {
            case 8: launch_one<8, VEC, kWide, kShift>(a); return ACCEL_OK;
            case 16: launch_one<16, VEC, kWide, kShift>(a); return ACCEL_OK;
            case 32: launch_one<32, VEC, kWide, kShift>(a); return ACCEL_OK;
            case 64: launch_one<64, VEC, kWide, kShift>(a); return ACCEL_OK;
            }
        }
        set_error("internal: unsupported group width %d", L);
        return ACCEL_ERR_ARG;
    }
    return ACCEL_OK;
}

// mode: 0 = 16-byte vectors at 16-byte aligned addresses, 1 = 16-byte vectors at any
// 4-byte aligned address with the row's last vector shifted to end with the row,
// 2 = scalar lanes
int launch_for_mode(int mode, bool wide, int L, const LaunchArgs &a)
{
    if (mode == 0) return wide ? launch_for_width<4, true, false>(L, a) : launch_for_width<4, false, false>(L, a);
    if (mode == 1) return wide ? launch_for_width<4, true, true>(L, a) : launch_for_width<4, false, true>(L, a);
    return wide ? launch_for_width<1, true, false>(L, a) : launch_for_width<1, false, false>(L, a);
}

}  // namespace

int fill_u32(void *dst, uint32_t v, size_t n, hipStream_t s)
{
    if (n == 0) return ACCEL_OK;
    const unsigned g = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
    fill_u32_kernel<<<dim3(g), dim3(256), 0, s>>>(static_cast<uint32_t *>(dst), v, n);
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

int copy_u32(void *dst, const void *src, size_t n, hipStream_t s)
{
    if (n == 0) return ACCEL_OK;
    const unsigned g = (unsigned)std::min<size_t>((n + 255) / 256, 65536);
    copy_u32_kernel<<<dim3(g), dim3(256), 0, s>>>(static_cast<uint32_t *>(dst),
                                                  static_cast<const uint32_t *>(src), n);
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

// Device address of this GPU's copy of `scratch`, looked up once per device (with that
// device current) and kept.
static int static_scratch_address(float **out)
{
    static std::mutex mu;
    static float *addr[kMaxScratchDevices] = {};
    int dev = 0;
    ACCEL_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxScratchDevices) {
        set_error("device ordinal %d is beyond the %d devices the static scratch is tracked for", dev,
                  kMaxScratchDevices);
        return ACCEL_ERR_ARG;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        float *p = nullptr;
        ACCEL_HIP(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
        addr[dev] = p;
    }
    *out = addr[dev];
    return ACCEL_OK;
}

// Grows the handle's partial-sum buffer to `floats` (never shrinks).  The old buffer is
// freed: graphs captured with it must be captured again.
int reserve_partial(accel_handle *h, size_t floats)
{
    if (h->partial_floats >= floats) return ACCEL_OK;
    if (h->partial_slot >= 0 && hipEventSynchronize(h->slot[h->partial_slot].done) != hipSuccess)
        (void)hipGetLastError();                       // nobody reads the old one (hipFree waits for the device as well)
    if (h->partial) (void)hipFree(h->partial);
    h->partial = nullptr;
    h->partial_floats = 0;
    if (hipMalloc(reinterpret_cast<void **>(&h->partial), floats * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        set_error("device allocation of %zu bytes for long-row partial sums failed", floats * sizeof(float));
        return ACCEL_ERR_ALLOC;
    }
    h->partial_floats = floats;
    return ACCEL_OK;
}

// main_start / main_stop: events bound to the gather kernel (to the first and the last launch
// when the run is done in column panels), for timing it alone.
int spmm_launch(accel_handle *h, const float *X, float *Y, int N, hipStream_t stream,
                hipEvent_t main_start, hipEvent_t main_stop, const float *bias, int relu, bool static_partial,
                int ld)
{
    if (h->rows == 0) return ACCEL_OK;
    (void)hipGetLastError();                         // launch errors are read back below: start from a clean slate
    if (ld <= 0) ld = N;                             // rows of X and Y are ld floats apart
    // 16-byte vectors whenever a row holds one.  When N is not a multiple of 4, or X or Y
    // is not 16-byte aligned, rows start at odd multiples of 4 bytes: the vectors are then
    // loaded and stored at 4-byte aligned addresses, and a row's last vector is moved back
    // so that it ends with the row (it overlaps the one before; both lanes hold the same
    // sums for the shared columns).  Scalar lanes are left for N < 4.
    const uintptr_t align = reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Y);
    const int mode = N < 4 ? 2 : (N % 4 == 0 && ld % 4 == 0 && align % 16 == 0) ? 0 : 1;
    const int vec = mode == 2 ? 1 : 4;

    // partial sums of the pieces of split rows: the handle's buffer (allocated here when a
    // run needs more than it holds), or this GPU's static array, which is never allocated
    float *partial = h->partial;
    const bool uses_handle_partial = !static_partial && h->n_long_units > 0;
    // the capture status is only asked for where something depends on it: a buffer that would
    // have to grow, or a stream the handle would have to order against another
    const bool must_grow = uses_handle_partial && h->partial_floats < (size_t)h->n_long_units * (size_t)ld;
    const bool capturing = (must_grow || needs_capture_status(h, stream)) && stream_is_capturing(stream);
    if (static_partial) {
        partial = nullptr;
        const size_t need = (size_t)h->n_long_units * (size_t)ld;
        if (need > kStaticScratchFloats) {
            set_error("accel_run_static: this matrix needs %zu floats of partial sums at N = %d "
                      "(%lld pieces of split rows x N), the static scratch holds %zu",
                      need, N, (long long)h->n_long_units, kStaticScratchFloats);
            return ACCEL_ERR_ARG;
        }
        if (need > 0)
            if (int rc = static_scratch_address(&partial)) return rc;
    } else if (uses_handle_partial) {
        const size_t need = (size_t)h->n_long_units * (size_t)ld;
        if (h->partial_floats < need) {
            if (capturing) {
                set_error("the partial-sum buffer has to grow for N = %d and the stream is capturing: "
                          "call accel_reserve(h, N) before the capture", N);
                return ACCEL_ERR_STATE;
            }
            if (int rc = reserve_partial(h, need)) return rc;
        }
        partial = h->partial;
    }
    // The buffer is shared by all runs of this handle, and a value update may still be
    // rewriting what this run reads: a run on another stream than the one that used them
    // last waits for that stream on the device (runs queued on one stream are ordered anyway).
    hipEvent_t run_done = nullptr;                  // to be bound to the run's last kernel
    if (int rc = order_run(h, stream, uses_handle_partial, capturing, &run_done)) return rc;
    // split rows are added up by the gather kernel itself (the wavefront that stores a row's
    // last piece), or, when the handle has no counters for that, by a second kernel
    int *row_done = h->fused_reduce ? h->row_done : nullptr;
    const bool has_reduce = h->n_split_rows > 0 && !row_done;
    // Wide operands are computed one column panel at a time (all units for the first
    // panel, then all units for the next): a panel's slice of X is what the L2s have
    // to hold, and a narrower slice means more rows of X fit.
    // Measured (panel 64 against one pass): N = 256 on the hub graph -12 %, N = 128 on the
    // dense and the power-law 100 M-non-zero graphs -7 % and -4 %; no gain when the
    // columns have no popularity skew or the rows are very short, and a loss when N is
    // not a multiple of the panel (N = 100: 64 + 36 leaves lanes idle).
    int panel = N;
    const int want = h->plan_panel_option > 0 ? h->plan_panel_option : kPanel;
    const bool forced = h->plan_panel_option > 0;
    if (mode == 0 && N > want &&
        (forced || (N % want == 0 && h->nnz >= kPanelMinNnz && h->nnz >= 16 * h->rows)))
        panel = want;
    // operands below 4 GiB are addressed with 32-bit byte offsets (see gather_row)
    const bool wide = (uint64_t)h->cols * (uint64_t)ld * 4u > 0xFFFFFFFFull;
    const int4 *wk = reinterpret_cast<const int4 *>(h->work);
    const int64_t entry_groups = h->plan_team ? h->n_units : h->n_units / kWaves;
    for (int c0 = 0; c0 < N; c0 += panel) {
        const int n = std::min(panel, N - c0);
        int L = 1;                                   // lanes per row: one per vector, a power of two
        while (L * vec < n && L < 64) L <<= 1;
        // zero-fill workgroups come first; their count is rounded up to a multiple of the
        // queue count so that entry group i still lands on die i % 8 (surplus ones exit at once)
        const int zr = zero_rows_per_group(n);
        int64_t zero_groups = (h->n_zero_rows + zr - 1) / zr;
        zero_groups = (zero_groups + h->plan_queues - 1) / h->plan_queues * h->plan_queues;
        const int64_t groups = entry_groups + zero_groups;
        if (groups > 0x7fffffffLL) {
            set_error("launch of %lld workgroups exceeds the grid limit", (long long)groups);
            return ACCEL_ERR_ARG;
        }
        if (groups == 0) break;
        const dim3 grid((unsigned)groups);
        const float *Xp = X ? X + c0 : X;
        float *Yp = Y + c0, *Pp = partial ? partial + c0 : nullptr;
        const float *bp = bias ? bias + c0 : nullptr;
        const bool first = c0 == 0, last = c0 + panel >= N;
        hipEvent_t stop = last ? main_stop : nullptr;
        if (last && !stop && !has_reduce) stop = run_done;      // the run ends with this launch
        const LaunchArgs la{h->plan_team, grid, stream, wk, (int)h->n_units, h->s_idx, h->s_val, h->perm,
                            Xp, Yp, Pp, n, ld, (int)h->n_zero_rows, (int)zero_groups, bp, relu,
                            h->long_slot, (int)(h->rows - h->n_split_rows), row_done,
                            first ? main_start : nullptr, stop};
        const int rc = launch_for_mode(mode, wide, L, la);
        if (rc) return rc;
    }
    if (!has_reduce && run_done && main_stop)       // the one launch cannot carry both events
        ACCEL_HIP(hipEventRecord(run_done, stream));
    if (has_reduce) {
        // one launch: rows with very many slots (the last n_big rows) get a workgroup each, the
        // others share one: as many rows per workgroup as leaves a row one thread per vector
        // of columns (16 at least, so that a row's loads stay coalesced)
        const int n_split = (int)h->n_split_rows, n_big = (int)h->n_big_rows, n_shared = n_split - n_big;
        const int rvec = mode == 0 ? 4 : 1;          // 16-byte accesses need the same as the gather kernel's
        const int nv = (N + rvec - 1) / rvec;
        int threads_per_row = 16;
        while (threads_per_row < nv && threads_per_row < kReduceThreads) threads_per_row <<= 1;
        const int rpw = kReduceThreads / threads_per_row;
        const int shared_groups = (n_shared + rpw - 1) / rpw;
        const dim3 rgrid((unsigned)(shared_groups + n_big));
        auto kernel = rvec == 4 ? long_row_reduce_kernel<4> : long_row_reduce_kernel<1>;
        if (run_done)
            hipExtLaunchKernelGGL(kernel, rgrid, dim3(kReduceThreads), 0, stream, nullptr, run_done,
                                  0, (const float *)partial, (const int32_t *)h->long_slot, (const int32_t *)h->perm,
                                  (int64_t)(h->rows - h->n_split_rows), n_shared, shared_groups, rpw, n_split, Y, nv,
                                  ld, bias, relu);
        else
            kernel<<<rgrid, dim3(kReduceThreads), 0, stream>>>(
                partial, h->long_slot, h->perm, h->rows - h->n_split_rows, n_shared, shared_groups, rpw,
                n_split, Y, nv, ld, bias, relu);
    }
    ACCEL_HIP(hipGetLastError());
    return ACCEL_OK;
}

}  // namespace accel
