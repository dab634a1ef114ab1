// Shared declarations of the library's translation units (not installed).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "accel_gcn.h"

namespace accel {

constexpr int kDegBound = ACCEL_DEG_BOUND;            // non-zeros per block4 entry
constexpr int kSlices = ACCEL_SLICES_PER_BLOCK;       // slices per entry (metadata ABI)
constexpr int kSliceNz = kDegBound / kSlices;         // 32
constexpr int kXcds = 8;                              // accelerator dies, each with its own L2
constexpr int kCusPerDie = 32;                        // compute units per die: 256 on the whole GPU
constexpr int kWavesPerGroup = 4;                     // wavefronts (work units) per workgroup (1, 2, 8: within 2 %)

constexpr int kMaxGroups = 64;                        // column groups of the launch plan (8..64)

// Column group of a non-zero.  Eight consecutive columns share a group so that
// neighbouring short rows of X (one 128-byte line holds 8 rows at N = 4) stay
// together.  Group g belongs to die g % 8; with more than 8 groups a die works
// through its groups one after the other, so that the share of X its L2 has to
// hold at any time is 1/groups of the matrix.
__host__ __device__ inline int col_group(int c, int groups) { return (c >> 3) & (groups - 1); }

// Column groups a split row of degree d is stored in: as many as leave a group about
// kGroupMinPiece non-zeros, 8 at least, 64 at most (a power of two); `forced`
// (8..64) overrides the rule.  Short split rows keep few, long pieces; very long rows
// are spread over many groups, whose share of X is small enough to stay in one L2.
constexpr int kGroupMinPiece = 96;                    // 48 and 192 measured: each better on one workload, worse on another
__host__ __device__ inline int row_groups(int d, int forced)
{
    if (forced) return forced;
    int g = kXcds;
    while (g < kMaxGroups && d / (2 * g) >= kGroupMinPiece) g *= 2;
    return g;
}
// Pieces are binned by (groups of their row, group): 8 + 16 + 32 + 64 bins.
constexpr int kPlanBins = 120;
__host__ __device__ inline int plan_bin(int groups, int g) { return groups - kXcds + g; }

// last-error string of the calling thread
void set_error(const char *fmt, ...);
const char *get_error();
void clear_error();

#define ACCEL_HIP(call)                                                                     \
    do {                                                                                    \
        hipError_t e_ = (call);                                                             \
        if (e_ != hipSuccess) {                                                             \
            accel::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),         \
                             __FILE__, __LINE__);                                           \
            return ACCEL_ERR_HIP;                                                           \
        }                                                                                   \
    } while (0)

// Slice rule of the block4 metadata for a row degree 1..384
// (block_level_partition.py:12-21 tables, :56-63 defaults beyond the table).
__host__ __device__ inline void slice_rule(int d, int &w_nz, int &rows_per_block)
{
    if (d >= kDegBound / 2) { w_nz = kSliceNz; rows_per_block = 1; return; }
    const int split = d <= 32 ? 1 : d <= 64 ? 2 : d <= 96 ? 3 : d <= 128 ? 4 : 6;
    w_nz = (d + split - 1) / split;
    rows_per_block = kSlices / split;
}

}  // namespace accel

// The operator state behind the opaque C handle.
struct accel_handle {
    static constexpr int kXcds = accel::kXcds;
    int64_t rows = 0, cols = 0, nnz = 0;
    int device = 0;
    // caller's CSR on the device (owned when uploaded from the host)
    const int32_t *indptr = nullptr;
    const int32_t *idx = nullptr;
    const float *val = nullptr;
    bool owns_input = false;
    // preprocess products
    bool ready = false;
    bool identity_perm = false;       // input already degree-sorted: perm == iota
    int32_t *perm = nullptr;          // [rows] new row -> caller's row (nullptr when identity)
    int32_t *s_indptr = nullptr;      // [rows+1] degree-sorted CSR
    const int32_t *s_idx = nullptr;   // [nnz]  (aliases idx when identity)
    const float *s_val = nullptr;     // [nnz]  (aliases val when identity)
    bool owns_sorted = false;
    void *slab = nullptr;             // when set: perm, s_indptr and the owned s_idx / s_val live in this one allocation
    int32_t *block4 = nullptr;        // [4*n_blocks]  the .block4 metadata (upstream ABI)
    // launch plan derived from block4 (see preprocess.hip, "work list")
    int32_t *work = nullptr;          // [4*n_units] one int4 per wavefront
    int64_t n_units = 0;              // multiple of 4 * plan_queues
    int64_t n_long_units = 0;         // units that write a partial sum
    int32_t *long_slot = nullptr;     // [n_split_rows+1] partial-sum slots of each split row
    int32_t *row_done = nullptr;      // [n_split_rows] pieces of each split row stored so far in the running
                                      // launch; zero between launches (part of the long_slot allocation)
    int plan_reduce_option = 0;       // 0: choose (in the gather kernel); 1: in the gather kernel; 2: second kernel
    bool fused_reduce = true;         // split rows are added up by the gather kernel itself
    // plan granularity: rows with more than plan_split non-zeros are cut into pieces of at
    // most plan_unit (through partial sums); block4 entries of shorter rows are cut into
    // units of whole rows holding at most plan_unit non-zeros.  384 = one unit per entry.
    int plan_unit_option = 0;         // 0: choose from the size of the matrix
    int plan_unit = ACCEL_DEG_BOUND;
    int plan_split_option = 0;        // 0: choose
    int plan_split = ACCEL_DEG_BOUND; // rows with more non-zeros than this are cut into pieces (<= plan_unit)
    int plan_groups = 0;              // 0: by row length (row_groups); 8..64: the same for all rows
    int plan_team_option = 0;         // 0: choose from the size of the matrix; 1: wavefront units; 2: workgroup units
    int plan_panel_option = 0;        // 0: choose; else the column-panel width of wide operands
    int plan_queues_option = 0;       // 0: from the device's shape; 1 or 8
    int plan_queues = accel::kXcds;   // interleaved queues of the launch plan: 8 (one per die), or 1
    int device_cus = 0;               // compute units of the device the handle was created on
    bool plan_team = false;           // a unit is worked on by a whole workgroup (small matrices)
    bool local = false;               // most non-zeros lie near the diagonal (sampled)
    int64_t n_split_rows = 0;         // rows with more than plan_split non-zeros
    int64_t n_big_rows = 0;           // of those, rows with more than 32 * plan_split
    int64_t nnz_short = 0;            // non-zeros of the rows that are not split
    int64_t n_wide_rows = 0;          // rows with more than 1,024 non-zeros (regrouped by a workgroup each)
    int64_t n_blocks = 0, n_long_blocks = 0, n_long_rows = 0, n_zero_rows = 0;
    int32_t max_degree = 0;
    double preprocess_ms = 0.0;
    // scratch for the partial sums of long-row segments: [n_long_blocks * N]
    float *partial = nullptr;
    size_t partial_floats = 0;
    // sorted position -> position in the caller's arrays, built by the first value update
    int32_t *src_pos = nullptr;
    // the handle's own copy of the caller's values (owns_input) is behind the sorted copy: a value
    // update from a device array went into the sorted copy only (restore_own_values brings it back)
    bool val_stale = false;
    // Which streams use the handle's mutable device memory (see order_run / order_update in
    // capi.hip).  Runs read the sorted values and, with split rows, write and read `partial`;
    // a value update rewrites the sorted values.  As long as all of that happens on one stream
    // (`home`), the stream orders it and nothing is tracked.  The first use on a second stream
    // waits for the device once and switches the handle to tracking: from then on a run leaves
    // an event, bound to its last kernel, in the slot of its stream.  Nothing is ever asked of
    // a stream after the call that used it has returned (the caller may have destroyed it).
    hipStream_t home = nullptr;              // the one stream the handle has been used on so far
    bool has_home = false;
    bool multi_stream = false;               // a second stream has turned up: runs are tracked
    static constexpr int kMaxStreams = 4;
    struct StreamSlot {
        hipStream_t stream = nullptr;
        hipEvent_t done = nullptr;           // bound to the last kernel of the last tracked run on `stream`
        bool live = false;                   // a run has been queued there since the last value update
    } slot[kMaxStreams];
    int next_victim = 0;                     // slot reused when a fifth stream turns up
    int partial_slot = -1;                   // slot of the last run that used `partial`
    hipStream_t writer = nullptr;            // stream of the last value update
    bool writer_pending = false;             // ... which may still be running
    hipEvent_t writer_done = nullptr;        // recorded behind it
};

namespace accel {
// preprocess.hip
struct SavedOrder {               // a degree-sort order read from a saved state
    bool identity;                // the rows were already in order: no permutation stored
    const uint32_t *perm_dev;     // [rows] on the device otherwise
};
int preprocess_device(accel_handle *h, const SavedOrder *given = nullptr);
int build_source_positions(accel_handle *h, hipStream_t s);
int gather_values(accel_handle *h, const float *val, hipStream_t s);
int restore_own_values(accel_handle *h, hipStream_t s);
// capi.hip
void release_products(accel_handle *h);
bool stream_is_capturing(hipStream_t s);
bool needs_capture_status(const accel_handle *h, hipStream_t s);
int order_run(accel_handle *h, hipStream_t s, bool uses_partial, bool capturing, hipEvent_t *run_done);
int order_update(accel_handle *h, hipStream_t s, bool capturing);
int note_update(accel_handle *h, hipStream_t s, bool capturing);
// spmm.hip
int spmm_launch(accel_handle *h, const float *X, float *Y, int N, hipStream_t stream,
                hipEvent_t main_start = nullptr, hipEvent_t main_stop = nullptr, const float *bias = nullptr,
                int relu = 0, bool static_partial = false, int ld = 0);
int reserve_partial(accel_handle *h, size_t floats);
int fill_u32(void *dst, uint32_t v, size_t n, hipStream_t s);
int copy_u32(void *dst, const void *src, size_t n, hipStream_t s);
}  // namespace accel
