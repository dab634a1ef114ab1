/*
 * accel_gcn.h - C ABI of the MI355X (gfx950) build of Accel-GCN's SpMM hot path.
 *
 * The path: Y = A * X, A a CSR adjacency (int32 indices, fp32 values), X and Y
 * dense row-major fp32 with N columns; rows are degree-sorted and cut into
 * blocks of at most 384 non-zeros described by int32 quadruples (the ".block4"
 * metadata).  Every entry point below names the upstream interface it replaces
 * (paths relative to the upstream tree).
 *
 * Conventions
 *   - plain pointers and sizes only; every function returns an accel_status
 *     (0 = ok, negative = error) and accel_last_error() describes the last
 *     failure on the calling thread;
 *   - a handle is not thread-safe; distinct handles are independent;
 *   - "device pointer" = anything the GPU can dereference (hipMalloc,
 *     hipMallocManaged, as upstream's data.h:15 uses);
 *   - nothing here falls back to the CPU: the *_host functions are explicit
 *     host utilities, every other call needs a GPU and fails with
 *     ACCEL_ERR_HIP without one.
 */
#ifndef ACCEL_GCN_H
#define ACCEL_GCN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum accel_status {
    ACCEL_OK = 0,
    ACCEL_ERR_ARG = -1,    /* null pointer, non-positive size, N <= 0, ... */
    ACCEL_ERR_CSR = -2,    /* indptr not monotone / not starting at 0 / not ending at nnz, column out of range */
    ACCEL_ERR_ALLOC = -3,  /* host or device allocation failed */
    ACCEL_ERR_HIP = -4,    /* HIP runtime error (includes "no GPU") */
    ACCEL_ERR_META = -5,   /* supplied .block4 metadata does not describe this CSR */
    ACCEL_ERR_STATE = -6,  /* call order violated (run before preprocess, ...), another GPU current than the
                              handle's, or a call that would have to allocate while its stream is capturing */
    ACCEL_ERR_IO = -7      /* file missing / truncated */
} accel_status;

/* accel_create flags */
#define ACCEL_PTR_HOST 0   /* indptr/idx/val are host arrays: copied to the GPU */
#define ACCEL_PTR_DEVICE 1 /* device pointers: borrowed, must outlive the handle */

/* metadata ABI shared with upstream (spmm_accel.cu:11-12, block_level_partition.py:7-8) */
#define ACCEL_DEG_BOUND 384
#define ACCEL_SLICES_PER_BLOCK 12

typedef struct accel_handle accel_handle;

/* Message for the most recent error on this thread ("" if none). */
const char *accel_last_error(void);
/* Library version, major*10000 + minor*100 + patch. */
int accel_version(void);

/* ---- host utilities -------------------------------------------------------
 * accel_partition_host: the walk of block_level_partition.py:48-103 with the
 * tables of :7-21, on the host.  Writes up to cap quadruples
 * (degree,row_begin,loc_begin,info) to block4_out (may be NULL with cap 0 to
 * size the buffer) and the full count to *n_blocks.
 * accel_degree_sort_host: perm_out[new_row] = old_row, ascending degree, ties
 * by row id: the order upstream's *.new_indptr files are in
 * (block_level_partition.py:31,38; tie-break defined by this library). */
int accel_partition_host(const int32_t *indptr, int64_t rows, int32_t *block4_out, int64_t cap,
                         int64_t *n_blocks);
int accel_degree_sort_host(const int32_t *indptr, int64_t rows, int32_t *perm_out);

/* The same partition computed by HIP kernels (scans + one emit kernel) for a
 * host indptr in the row order given, i.e. what block_level_partition.py:38-106
 * produces for one *.new_indptr file.  Bit-exact with accel_partition_host. */
int accel_partition_gpu(const int32_t *indptr, int64_t rows, int32_t *block4_out, int64_t cap,
                        int64_t *n_blocks);

/* ---- raw-array files (data.h:7-34; block_level_partition.py:31-32,105-106) --
 * Whole-file little-endian arrays of 4-byte elements.  accel_file_count
 * returns the element count; accel_file_read fills a host buffer. */
int accel_file_count(const char *path, int64_t *n_elems);
int accel_file_read(const char *path, void *dst, int64_t n_elems);
int accel_file_write(const char *path, const void *src, int64_t n_elems);

/* ---- device memory plumbing (for callers without a HIP binding of their own;
 * upstream uses cudaMallocManaged/cudaFree directly, main.cu:62-88,171-181) -- */
int accel_device_count(int *n);
int accel_dev_malloc(void **p, size_t bytes);
int accel_dev_free(void *p);
int accel_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes);
int accel_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes);
int accel_dev_fill_u32(void *dst_dev, uint32_t value, size_t n_words, void *stream);
/* Plain grid-stride copy kernel of n_words 4-byte words; also the known-size
 * reference against which hardware byte counters are calibrated. */
int accel_dev_copy_u32(void *dst_dev, const void *src_dev, size_t n_words, void *stream);
int accel_stream_sync(void *stream); /* NULL = default stream */

/* ---- the operator ----------------------------------------------------------
 * init: replaces SPMM_BASE's constructor (spmm_base.h:9-20) for the CSR part:
 * stores (ACCEL_PTR_DEVICE) or uploads (ACCEL_PTR_HOST) the CSR.  The CSR may
 * be in any row order.  Arrays passed as ACCEL_PTR_DEVICE are borrowed until
 * accel_destroy and must be memory the GPU can read, of at least rows + 1, nnz and nnz
 * elements: a host address or a smaller allocation is ACCEL_ERR_ARG here and again
 * in accel_preprocess / accel_load_state, before any kernel reads them. */
int accel_create(const int32_t *indptr, const int32_t *idx, const float *val, int64_t rows,
                 int64_t cols, int64_t nnz, int flags, accel_handle **out);

/* preprocess: replaces the first half of SPMM_ACCEL::do_test (spmm_accel.cu:
 * 122-132, which loads a .block4 file written by block_level_partition.py) and
 * the offline degree sort behind upstream's *.new_* files.  On the GPU:
 * validates the CSR, stable-sorts rows by degree (skipped when already
 * sorted), gathers the permuted CSR, and builds the block4 metadata. */
int accel_preprocess(accel_handle *h);

/* Granularity of the launch plan (no counterpart upstream, whose unit is always one
 * block4 entry): the most non-zeros one wavefront takes, 16..384, or 0 to let the
 * library choose from the size of the matrix (the default).  Rows above the split
 * threshold (see accel_set_plan_split) are cut into pieces of at most this size,
 * added up through partial sums; block4 entries of shorter rows are cut into
 * units of whole rows of at most this size.  The block4 metadata itself
 * never changes.  Call before accel_preprocess. */
int accel_set_plan_unit(accel_handle *h, int unit_nz);
/* Rows with more non-zeros than this (16..384, never above the unit size; 0 = let
 * the library choose: 192, or 384 when most non-zeros of the matrix lie near its
 * diagonal) are the ones stored by column group and cut into pieces. */
int accel_set_plan_split(accel_handle *h, int split_nz);
/* Number of column groups the pieces of split rows are sorted into: 8, 16, 32 or
 * 64 for every row, or 0 (the default) to choose per row: 8 groups, doubled while
 * a group would still get about 96 non-zeros of the row, up to 64.  Group g =
 * (column >> 3) & (groups - 1) is worked on by die g % 8, one group after the
 * other.  Call before accel_preprocess. */
int accel_set_plan_groups(accel_handle *h, int groups);
/* Who works on one unit of the launch plan (no counterpart upstream, where a block4
 * entry always gets one thread block, spmm_accel.cu:128): 1 = one wavefront (four units per
 * workgroup, the layout described at accel_get_plan); 2 = a whole workgroup of four
 * wavefronts, which share the unit's rows or, for a long row, its non-zeros; 0 (the
 * default) = the library chooses: workgroup units for small matrices, whose run time
 * is the longest chain of dependent gathers rather than memory bandwidth.  Call
 * before accel_preprocess. */
int accel_set_plan_team(accel_handle *h, int mode);

/* Saved preprocessing state.  Upstream persists its preprocessing as a file
 * (block_level_partition.py:105-106 writes <graph>.block4) and its operator loads
 * that file instead of recomputing (spmm_accel.cu:122).  On this GPU every product of
 * accel_preprocess but one is rebuilt faster than a file of its size can be read, so
 * accel_save_state writes that one, the degree-sort permutation (4 bytes per row), and
 * the plan options of the handle.  accel_load_state takes the place of accel_preprocess
 * on a handle created on the same CSR: it runs the preprocessing with the sort replaced
 * by the stored order.  Nothing in the file is trusted: the order is used only after a
 * kernel has found it to be exactly the degree order of this CSR (ascending degree,
 * ties by row id: there is only one), so a file saved for another matrix, written by
 * another library version or damaged gives ACCEL_ERR_META and leaves the handle
 * un-preprocessed and its options as they were; a missing or short file gives
 * ACCEL_ERR_IO.  After a successful load the handle is the one that was saved: the same
 * options, and the results of accel_run are the same bits; accel_info.preprocess_ms is
 * the time of the load.  The load is not faster than accel_preprocess (reading the file
 * costs more than the sort it replaces); it exists for callers that want the operator's
 * state to travel with the graph, as upstream's metadata file does. */
int accel_save_state(const accel_handle *h, const char *path);
int accel_load_state(accel_handle *h, const char *path);

/* New values for the non-zeros of an unchanged structure (indptr and idx as they were
 * at accel_create), e.g. edge weights that change between training steps.  Upstream's
 * kernel reads the caller's `val` on every launch (spmm_accel.cu:75), so a caller that
 * rewrites the array sees the new weights at once; this library computes from its
 * degree-sorted copy, which these calls bring up to date: one kernel that gathers the
 * values through a map from sorted position to the caller's position (sort, metadata
 * and launch plan are kept).  The first update of a handle builds that map (one device
 * allocation of 4 bytes per non-zero, kept until the next accel_preprocess); later ones
 * allocate nothing.
 *
 * accel_update_values_async: val_dev = nnz floats on the device in the order of the CSR
 * given to accel_create; the kernel is queued on `stream` (a hipStream_t, NULL = default
 * stream) and the call returns without waiting.  On the stream the handle's runs use it
 * is ordered by that stream.  On another stream the handle orders it on the device behind
 * its runs that are still in flight, and later runs on other streams behind it (see
 * accel_run: the first call on a second stream waits for the device once), so "update,
 * then run" needs no host synchronisation whatever the streams are.  It can be captured into a HIP graph together with the runs that follow
 * (after one update outside the capture has built the map; a capturing stream is only
 * ordered against itself).  A handle that borrows device arrays borrows val_dev from now
 * on (it may be the same array, rewritten in place); a handle that uploaded its CSR keeps
 * its own copy of the caller's order, which it brings up to date from the sorted copy only
 * if the handle is preprocessed again.
 *
 * accel_update_values: the same for an array in host memory (ACCEL_PTR_HOST: copied to the
 * device first; only for handles that own their CSR) or on the device (ACCEL_PTR_DEVICE),
 * on the default stream, and it returns when the update is done.  Not while capturing.
 *
 * A saved state holds no values and stays valid.  The sorted copy is rewritten where it
 * is, so HIP graphs captured from runs of this handle stay valid and compute with the new
 * values (exception: a CSR that was already sorted and has no split row is read in place,
 * so passing a different array changes the address a captured run reads). */
int accel_update_values(accel_handle *h, const float *val, int flags);
int accel_update_values_async(accel_handle *h, const float *val_dev, void *stream);

/* Interleaved queues of the launch plan (no counterpart upstream, whose grid is the block4
 * list in order, spmm_accel.cu:128).  The plan is laid out for the way the whole MI355X
 * hands out workgroups: workgroup i runs on die i % 8, so the list is eight interleaved
 * queues, one per die and its L2 (see accel_get_plan).  0 (the default) = from the device
 * the handle was created on: 8 when it has the 256 compute units of the whole GPU, 1 on
 * any other shape (a partition of the GPU, where that mapping does not hold): the same
 * units in one queue, column group after column group.  1 or 8 force the layout.  Call
 * before accel_preprocess; accel_info.plan_queues tells what was used. */
int accel_set_plan_queues(accel_handle *h, int queues);

/* Where the partial sums of split rows are added up.  Upstream's run is one launch
 * (spmm_accel.cu:104-108) whose blocks add long rows into vout with atomicAdd (:84,97).
 * Here every piece of a split row stores its sum to a slot of its own and the slots are
 * added in a fixed order (results are the same bits on every run): 1 = by the gather
 * kernel itself, one launch: each piece counts itself in on a per-row counter and the
 * wavefront that stores the row's last piece adds the row up; 2 = by a second, small
 * kernel behind the gather kernel; 0 (the default) = the library chooses: 1 when the
 * plan holds at most 16,384 pieces (launch-bound matrices, where a second launch costs
 * more than the wait each piece then ends on), 2 otherwise.
 * Call before accel_preprocess. */
int accel_set_plan_reduce(accel_handle *h, int mode);

/* Column panels (no counterpart upstream, which always walks all N columns of a row
 * at once, spmm_accel.cu:37-48): one accel_run computes Y one panel of `columns`
 * columns at a time (the last one narrower when N is not a multiple), all work units
 * for the first panel before the next, so that the caches only have to hold that slice
 * of X.  0 (the default) lets the library choose from N and the size of the matrix
 * (panels of 64 for N = 128, 192, ... on large matrices).
 * Takes effect at the next accel_run; needs N % 4 == 0 and 16-byte aligned X and Y. */
int accel_set_plan_panel(accel_handle *h, int columns);

/* Check externally produced metadata (a .block4 file) against what
 * accel_preprocess built for this CSR; ACCEL_ERR_META if any int differs. */
int accel_check_block4(accel_handle *h, const int32_t *block4_host, int64_t n_blocks);

typedef struct accel_info {
    int64_t rows, cols, nnz;
    int64_t n_blocks;       /* block4 entries */
    int64_t n_long_blocks;  /* entries that are segments of rows with degree > 384 */
    int64_t n_long_rows;    /* rows with degree > 384 */
    int64_t n_zero_rows;    /* rows with degree 0 */
    int32_t max_degree;
    int32_t already_sorted; /* 1: input rows were already in ascending degree order */
    double preprocess_ms;   /* wall time of the last accel_preprocess */
    int64_t n_plan_units;   /* wavefronts of one launch (launch plan, incl. padding) */
    int64_t n_split_rows;   /* rows cut into pieces that go through partial sums */
    int32_t plan_unit_nz;   /* most non-zeros one wavefront takes (<= 384) */
    int32_t plan_groups;    /* 0: column groups chosen per row from its length; 8..64: forced */
    int32_t plan_split_nz;  /* rows with more non-zeros than this are cut into pieces */
    int32_t plan_team;      /* 1: a unit is worked on by a whole workgroup, 0: by one wavefront */
    int32_t plan_queues;    /* interleaved queues of the launch plan: 8 (one per die) or 1 */
    int32_t plan_reduce;    /* 1: the gather kernel adds split rows up itself, 2: a second kernel does */
    int64_t n_plan_pieces;  /* units of the plan that are pieces of split rows (each has a partial-sum slot) */
} accel_info;
int accel_get_info(const accel_handle *h, accel_info *out);

/* Copies to host: block4 (4*n_blocks int32), perm (rows int32), and the
 * degree-sorted CSR (rows+1 / nnz / nnz); any pointer may be NULL to skip. */
int accel_get_block4(const accel_handle *h, int32_t *out, int64_t cap_blocks);
int accel_get_perm(const accel_handle *h, int32_t *out, int64_t cap_rows);
int accel_get_sorted_csr(const accel_handle *h, int32_t *indptr, int32_t *idx, float *val);

/* The launch plan derived from block4 (no counterpart upstream, where the grid
 * is simply one thread block per block4 entry, spmm_accel.cu:128): one int4
 * (x, y, z, w) per wavefront, four per workgroup (per workgroup when
 * accel_info.plan_team is 1; the list has the same form).  x <= 384: a block4 entry of
 * whole rows, verbatim.  x > 384: a piece of a long row: partial-sum slot
 * x - 385, sorted row y, first non-zero z, length w <= 384.  w == 0: padding.
 * With accel_info.plan_queues == 1 the list is one queue in the order described below;
 * with 8: workgroup i runs on die i % 8, so units 4*i .. 4*i+3 belong to queue i % 8;
 * the pieces of split rows in queue g only hold columns c with (c >> 3) & 7 == g,
 * ordered by column group ((c >> 3) & (groups - 1)) when there are more than 8, and
 * inside a group by the caller's row id (rows of 8 groups; longer rows: largest
 * first).  Behind them a queue holds its share of the
 * whole-row units: those are ordered by the caller's row id of their first row, and
 * that order is cut into eight consecutive shares of about equal load, so that a die
 * works on a narrow band of the caller's rows at any time (the last 2048 units of
 * few non-zeros of a share are held back to the end of their queue).
 * Writes up to cap_units quadruples to out (may be NULL) and the count to *n_units. */
int accel_get_plan(const accel_handle *h, int32_t *out, int64_t cap_units, int64_t *n_units);

/* run: replaces SPMM_ACCEL::run (spmm_accel.cu:104-108).  Y = A X with beta = 0:
 * every row of Y is written exactly once, rows of degree 0 receive zeros (the
 * upstream kernel leaves them untouched and accumulates into the rest,
 * spmm_accel.cu:84,97).  X has cols(A) rows, Y has rows(A) rows, both with
 * leading dimension N (spmm_accel.cu:75,84 index row*feat_in+lane).  Rows of Y
 * are in the caller's original row order.  Asynchronous on `stream` (a
 * hipStream_t, NULL = default stream); X and Y are device pointers: an address the
 * GPU cannot read, or an allocation too small for cols x N (X) or rows x N (Y) floats,
 * is refused with ACCEL_ERR_ARG where the runtime can tell (it is asked on every call,
 * except while `stream` is capturing: the runtime answers no such query during a capture),
 * and a call with another GPU current than the one the handle was created on with
 * ACCEL_ERR_STATE.  The partial-sum buffer of a matrix with split rows is shared by all
 * runs of the handle.  A handle used on one stream needs nothing beyond the stream's own
 * order.  The first call on a second stream waits for the device once; from then on every
 * run of the handle carries an event and a run on another stream than the previous one is
 * made to wait for that one on the device (no error, no host wait; distinct handles are
 * independent).  A stream that is capturing is not ordered against other streams: the
 * caller orders a graph against other uses of the handle. */
int accel_run(accel_handle *h, const float *X, float *Y, int32_t N, void *stream);

/* run with the rest of a GCN layer fused into the store: Y = act(A X + bias).
 * No counterpart upstream (its kernel stops at A X); this is the step a GCN layer
 * applies right after the aggregation, done here while the row is in registers
 * instead of as a second pass over Y.  bias: N floats on the device, or NULL.
 * flags: 0 or ACCEL_EPILOGUE_RELU.  Rows of degree 0 receive act(bias). */
#define ACCEL_EPILOGUE_RELU 1
int accel_run_epilogue(accel_handle *h, const float *X, float *Y, int32_t N, const float *bias,
                       int flags, void *stream);

/* accel_run on operands whose rows are `ld` floats apart (ld >= N; accel_run is ld = N,
 * the only layout upstream's kernel knows: it indexes row * feat_in + lane,
 * spmm_accel.cu:75,84).  What it is for: the time of a run is set by the 128-byte lines a
 * gathered row of X touches.  Rows of N = 127 floats packed back to back straddle five
 * lines each, padded to ld = 128 they touch four; N = 50 at ld = 64 two instead of two and
 * a half.  A caller that keeps X padded to a multiple of 32 floats gets the time of the
 * next multiple for any N.  The columns N .. ld-1 of X are never read and those of Y never
 * written.  The partial-sum buffer is sized for ld (accel_reserve(h, ld)). */
int accel_run_strided(accel_handle *h, const float *X, float *Y, int32_t N, int32_t ld, void *stream);

/* The run with every option at once: rows `ld` floats apart (0 = packed, ld = N), bias
 * and/or ReLU in the store, on `stream`.  accel_run, accel_run_epilogue and
 * accel_run_strided are this call with the other fields left at zero; what it adds is
 * their combination (a GCN layer on a padded feature matrix: Y = relu(A X + b) with rows
 * a multiple of 32 floats apart).  No counterpart upstream, whose launch has one form
 * (spmm_accel.cu:104-108). */
typedef struct accel_run_args {
    const float *X;    /* cols x N floats, rows ld apart */
    float *Y;          /* rows x N floats, rows ld apart */
    int32_t N;         /* columns computed */
    int32_t ld;        /* floats between rows of X and of Y; 0 = N */
    const float *bias; /* N floats on the device, or NULL */
    int32_t flags;     /* 0 or ACCEL_EPILOGUE_RELU */
    void *stream;      /* hipStream_t; NULL = default stream */
} accel_run_args;
int accel_run_ex(accel_handle *h, const accel_run_args *args);

/* accel_run keeps the partial sums of split rows (pieces x N floats) in a buffer of the
 * handle.  It is allocated by the first accel_run with a given N and replaced by a larger
 * one when a later run brings a larger N; a HIP graph captured with the old buffer must
 * then be captured again.  accel_reserve allocates it for every N up to max_N at once, so
 * that no later accel_run with N <= max_N allocates or frees: call it before capturing a
 * graph or entering a loop that must not allocate (a run that would have to grow the
 * buffer while its stream is capturing fails with ACCEL_ERR_STATE).  No counterpart
 * upstream, whose kernel adds split rows up with atomicAdd (spmm_accel.cu:84,97). */
int accel_reserve(accel_handle *h, int32_t max_N);

/* accel_run for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart upstream.  The only scratch of a run, the partial sums of the
 * pieces of split rows (pieces x N floats), lives in a static device array of
 * ACCEL_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until the
 * process ends, instead of the handle's buffer that accel_run allocates on its
 * first call with a given N.  This call allocates and frees nothing.  A matrix
 * whose partial sums at this N do not fit is refused with ACCEL_ERR_ARG and a
 * message that names both sizes (matrices without split rows need none and always
 * fit).  All handles on one GPU share the array: two calls that overlap in time
 * on the same GPU (different streams or different handles) race; calls queued on
 * one stream are safe.  Every slot a run reads is written by that run first, so
 * nothing needs clearing between calls.  Same result, bit for bit, as accel_run. */
#define ACCEL_STATIC_SCRATCH_BYTES (32u << 20)
int accel_run_static(accel_handle *h, const float *X, float *Y, int32_t N, void *stream);

/* Timing protocol of SPMM_BASE::timing_body (spmm_base.h:34-63) with HIP
 * events on `stream`: `warmup` untimed runs, then `iters` runs queued back to back,
 * each bracketed by two recorded events.  ms_total[i] covers everything accel_run
 * launches; ms_main[i] (optional) only the gather kernel, taken from events bound to
 * that kernel's own start and end (hipExtLaunchKernel), which put nothing between the
 * kernels of a run.  Either array may be NULL. */
int accel_time(accel_handle *h, const float *X, float *Y, int32_t N, int warmup, int iters,
               float *ms_total, float *ms_main, void *stream);

/* The same protocol on a run with every option (rows `ld` apart, bias, ReLU): accel_time is
 * this call with those fields at zero. */
int accel_time_ex(accel_handle *h, const accel_run_args *args, int warmup, int iters, float *ms_total,
                  float *ms_main);

/* Z = X W in fp32: the dense product of a GCN layer, whose result is the dense operand of
 * accel_run (layer: Y = act(A (X W) + bias) = accel_dense_xw, then accel_run_epilogue).  No
 * counterpart upstream, whose operator takes the product as given (spmm_accel.cu:16-102 stops
 * at A X).  X: rows x K floats, rows ldx floats apart (0 = K); W: K x N floats, packed
 * row-major; Z: rows x N floats, rows ldz apart (0 = N; the columns N .. ldz-1 are not
 * written); all three on the device, Z overlapping neither input.  Any rows >= 0, K >= 1,
 * N >= 1; rows of X that start and end on 16-byte boundaries (X aligned, ldx and K multiples
 * of 4) are read as 16-byte vectors.  Needs no handle; asynchronous on `stream`; allocates nothing.
 * Computed on the fp32 matrix cores: sums of K products in fp32, whose order differs from a
 * sequential loop (compare against a higher-precision product, as for accel_run).  Built for
 * the shapes of a layer: many rows and N up to 128, where the product is bound by streaming
 * X; for wider outputs (N = 256 and more) a BLAS is the better tool. */
int accel_dense_xw(const float *X, const float *W, float *Z, int64_t rows, int32_t K, int32_t N,
                   int32_t ldx, int32_t ldz, void *stream);

int accel_destroy(accel_handle *h);

#ifdef __cplusplus
}
#endif
#endif /* ACCEL_GCN_H */
