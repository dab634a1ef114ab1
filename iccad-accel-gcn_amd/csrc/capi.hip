// extern "C" surface of the library (declared in include/accel_gcn.h).
#include <algorithm>
#include <cstring>
#include <fstream>
#include <new>
#include <vector>

#include "internal.h"

namespace accel {

static thread_local std::string g_error;

void set_error(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
}
const char *get_error() { return g_error.c_str(); }
void clear_error() { g_error.clear(); }

int partition_only_device(const int32_t *indptr_dev, int64_t rows, int64_t nnz,
                          int32_t **block4_dev, int64_t *n_blocks);
bool stream_is_capturing(hipStream_t s);
int dense_xw_launch(const float *X, const float *W, float *Z, int64_t rows, int K, int N, int64_t ldx, int64_t ldz,
                    hipStream_t stream);      // dense.hip

void release_products(accel_handle *h)
{
    if (h->slab) {
        (void)hipFree(h->slab);
        h->slab = nullptr;
    } else {
        if (h->perm) (void)hipFree(h->perm);
        if (h->s_indptr) (void)hipFree(h->s_indptr);
        if (h->owns_sorted) {
            if (h->s_idx) (void)hipFree(const_cast<int32_t *>(h->s_idx));
            if (h->s_val) (void)hipFree(const_cast<float *>(h->s_val));
        }
    }
    if (h->work) (void)hipFree(h->work);
    if (h->long_slot) (void)hipFree(h->long_slot);
    if (h->block4) (void)hipFree(h->block4);
    if (h->partial) (void)hipFree(h->partial);
    if (h->src_pos) (void)hipFree(h->src_pos);
    h->src_pos = nullptr;
    h->val_stale = false;
    // what other streams still hold was queued against the memory freed above (hipFree waits
    // for the device), so the bookkeeping starts afresh
    if (h->writer_done) (void)hipEventDestroy(h->writer_done);
    for (auto &sl : h->slot) {
        if (sl.done) (void)hipEventDestroy(sl.done);
        sl = accel_handle::StreamSlot();
    }
    h->writer_done = nullptr; h->writer = nullptr; h->writer_pending = false;
    h->partial_slot = -1; h->next_victim = 0;
    h->has_home = false; h->home = nullptr; h->multi_stream = false;
    h->perm = nullptr; h->s_indptr = nullptr; h->s_idx = nullptr; h->s_val = nullptr;
    h->work = nullptr; h->long_slot = nullptr; h->row_done = nullptr; h->block4 = nullptr; h->partial = nullptr;
    h->n_units = h->n_long_units = 0;
    h->partial_floats = 0; h->owns_sorted = false; h->ready = false;
}

static int need_gpu()
{
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        set_error("no HIP device available (%s); this library has no CPU fallback",
                  e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        return ACCEL_ERR_HIP;
    }
    return ACCEL_OK;
}

// A dense operand must be memory the GPU can read: a host address handed to a kernel is a
// memory fault, not an error code.  The runtime is asked what the address is and, where it
// knows the allocation, whether `bytes` fit behind it.  It is asked on every call: an answer
// remembered from an earlier call says nothing once the caller has freed the buffer and a
// smaller one has taken its address (allocators that recycle addresses do this all the time).
// Not while a stream is capturing: the runtime counts these queries among the calls that
// end a capture in error, so a captured run takes its operands unchecked (check_run).
static int check_operand(const void *p, size_t bytes, const char *fn, const char *name)
{
    if (!p || bytes == 0) return ACCEL_OK;
    hipPointerAttribute_t at;
    const hipError_t qe = hipPointerGetAttributes(&at, p);
    if (qe == hipErrorStreamCaptureUnsupported || qe == hipErrorStreamCaptureImplicit) {
        (void)hipGetLastError();            // another stream of this process is capturing: nothing can be asked
        return ACCEL_OK;
    }
    if (qe != hipSuccess || at.type == hipMemoryTypeUnregistered) {
        (void)hipGetLastError();
        set_error("%s: %s (%p) is not memory the GPU can access (a host array? copy it to the device first)",
                  fn, name, p);
        return ACCEL_ERR_ARG;
    }
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, const_cast<void *>(p)) == hipSuccess && base) {
        const size_t off = (size_t)(static_cast<const char *>(p) - static_cast<const char *>(base));
        if (off > size || size - off < bytes) {
            set_error("%s: %s needs %zu bytes, its allocation holds %zu from that address", fn, name, bytes,
                      off > size ? (size_t)0 : size - off);
            return ACCEL_ERR_ARG;
        }
    } else {
        (void)hipGetLastError();
    }
    return ACCEL_OK;
}

// A CSR borrowed from the caller (ACCEL_PTR_DEVICE) must be device memory of the stated sizes.
int check_borrowed_csr(const accel_handle *h, const char *fn)
{
    if (h->owns_input) return ACCEL_OK;
    if (int rc = check_operand(h->indptr, sizeof(int32_t) * (size_t)(h->rows + 1), fn, "indptr")) return rc;
    if (int rc = check_operand(h->idx, sizeof(int32_t) * (size_t)h->nnz, fn, "idx")) return rc;
    return check_operand(h->val, sizeof(float) * (size_t)h->nnz, fn, "val");
}

// The handle's device memory belongs to the GPU it was created on; a launch with another GPU
// current would hand that GPU addresses it cannot use.
static int check_device(const accel_handle *h, const char *fn)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); dev = -1; }
    if (dev != h->device) {
        set_error("%s: the handle was created on GPU %d, the current device is %d (hipSetDevice(%d) first)", fn,
                  h->device, dev, h->device);
        return ACCEL_ERR_STATE;
    }
    return ACCEL_OK;
}

// argument checks shared by the run entry points
static int check_run(accel_handle *h, const float *X, float *Y, int32_t N, const float *bias, const char *fn,
                     hipStream_t stream, int32_t ld = 0)
{
    if (!h) { set_error("%s: null handle", fn); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("%s: call accel_preprocess first", fn); return ACCEL_ERR_STATE; }
    if (N <= 0) { set_error("%s: N must be positive, got %d", fn, N); return ACCEL_ERR_ARG; }
    if (int rc = check_device(h, fn)) return rc;
    if ((h->rows > 0 && !Y) || (h->nnz > 0 && !X)) { set_error("%s: null dense operand", fn); return ACCEL_ERR_ARG; }
    if (h->rows == 0) return ACCEL_OK;
    if (stream_is_capturing(stream)) return ACCEL_OK;    // see check_operand
    if (ld <= 0) ld = N;
    // the last row only has to hold N floats
    const size_t x_floats = h->cols > 0 ? (size_t)(h->cols - 1) * (size_t)ld + (size_t)N : 0;
    const size_t y_floats = (size_t)(h->rows - 1) * (size_t)ld + (size_t)N;
    if (int rc = check_operand(X, x_floats * sizeof(float), fn, "X")) return rc;
    if (int rc = check_operand(Y, y_floats * sizeof(float), fn, "Y")) return rc;
    return check_operand(bias, (size_t)N * sizeof(float), fn, "bias");
}

// ---------------------------------------------------------------------------
// Stream order of a handle's mutable device memory.  Runs read the sorted values and, when
// the matrix has split rows, write and then read the partial-sum buffer; a value update
// rewrites the sorted values.  Work queued on one stream is ordered by the stream, and as
// long as a handle is used on one stream only nothing else happens (an event per run costs
// the run some 2 us on the device, a fifth of a launch-bound matrix's run).  The first use on
// a second stream waits for the device once; from then on the handle orders its uses itself,
// on the device, without making the host wait: a run binds an event to its last kernel, kept
// in the slot of its stream, and whatever has to come after that run on another stream waits
// for the event.  A stream is never touched after the call that used it has returned, so the
// caller may destroy it at any time.  A stream that is capturing is left alone (an event of
// work outside a capture cannot be waited for inside one, and the device cannot be waited
// for): the caller orders a graph against other uses of the handle.
// ---------------------------------------------------------------------------
bool stream_is_capturing(hipStream_t s)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cap != hipStreamCaptureStatusNone;
}

// Whether a call on s has to find out if s is capturing: only when it would do something a
// capture does not allow.
bool needs_capture_status(const accel_handle *h, hipStream_t s)
{
    return h->multi_stream || (h->has_home && s != h->home);
}

// One stream so far, or the switch to tracking when a second one turns up.  *single: the
// handle still lives on one stream.
static int single_stream(accel_handle *h, hipStream_t s, bool *single)
{
    *single = false;
    if (h->multi_stream) return ACCEL_OK;
    if (!h->has_home) { h->home = s; h->has_home = true; }
    if (s == h->home) { *single = true; return ACCEL_OK; }
    ACCEL_HIP(hipDeviceSynchronize());      // once per handle: what the first stream holds left no events
    h->multi_stream = true;
    h->writer_pending = false;
    return ACCEL_OK;
}

// Before a run is queued on s.  *run_done receives the event to bind to the run's last kernel
// (null: this run is not tracked).
int order_run(accel_handle *h, hipStream_t s, bool uses_partial, bool capturing, hipEvent_t *run_done)
{
    *run_done = nullptr;
    if (capturing) return ACCEL_OK;
    bool single = false;
    if (int rc = single_stream(h, s, &single)) return rc;
    if (single) return ACCEL_OK;
    if (h->writer_pending && s != h->writer) {
        if (hipEventQuery(h->writer_done) == hipSuccess) {
            h->writer_pending = false;
        } else {
            (void)hipGetLastError();
            ACCEL_HIP(hipStreamWaitEvent(s, h->writer_done, 0));
        }
    }
    int mine = -1;
    for (int i = 0; i < accel_handle::kMaxStreams; i++)
        if (h->slot[i].done && h->slot[i].stream == s) mine = i;
    if (mine < 0) {
        for (int i = 0; i < accel_handle::kMaxStreams && mine < 0; i++)
            if (!h->slot[i].done) mine = i;
        if (mine < 0) {
            // a fifth stream: it takes over a slot and waits for what that slot's stream held,
            // so that whoever waits for this run also waits for those
            mine = h->next_victim;
            h->next_victim = (h->next_victim + 1) % accel_handle::kMaxStreams;
            ACCEL_HIP(hipStreamWaitEvent(s, h->slot[mine].done, 0));
        } else {
            ACCEL_HIP(hipEventCreateWithFlags(&h->slot[mine].done, hipEventDisableTiming));
        }
        h->slot[mine].stream = s;
    }
    if (uses_partial) {
        if (h->partial_slot >= 0 && h->partial_slot != mine)
            ACCEL_HIP(hipStreamWaitEvent(s, h->slot[h->partial_slot].done, 0));
        h->partial_slot = mine;
    }
    h->slot[mine].live = true;
    *run_done = h->slot[mine].done;
    return ACCEL_OK;
}

// Before a value update is queued on s: it has to come after every run that reads the
// values it rewrites, and after an earlier update on another stream.
int order_update(accel_handle *h, hipStream_t s, bool capturing)
{
    if (capturing) return ACCEL_OK;
    bool single = false;
    if (int rc = single_stream(h, s, &single)) return rc;
    if (single) return ACCEL_OK;
    for (auto &sl : h->slot)
        if (sl.live && sl.stream != s) ACCEL_HIP(hipStreamWaitEvent(s, sl.done, 0));
    if (h->writer_pending && h->writer != s) ACCEL_HIP(hipStreamWaitEvent(s, h->writer_done, 0));
    return ACCEL_OK;
}

// Behind a value update queued on s.
int note_update(accel_handle *h, hipStream_t s, bool capturing)
{
    if (capturing || !h->multi_stream) return ACCEL_OK;
    if (!h->writer_done) ACCEL_HIP(hipEventCreateWithFlags(&h->writer_done, hipEventDisableTiming));
    ACCEL_HIP(hipEventRecord(h->writer_done, s));
    h->writer = s;
    h->writer_pending = true;
    for (auto &sl : h->slot) sl.live = false;   // later runs order themselves behind this update
    return ACCEL_OK;
}

}  // namespace accel

using namespace accel;

extern "C" {

const char *accel_last_error(void) { return get_error(); }
int accel_version(void) { return 200; }   // 0.2.0: saved state, value updates, strided and static runs

// ---------------------------------------------------------------------------
// host utilities
// ---------------------------------------------------------------------------
int accel_partition_host(const int32_t *indptr, int64_t rows, int32_t *block4_out, int64_t cap,
                         int64_t *n_blocks)
{
    clear_error();
    if (!indptr || rows < 0 || !n_blocks || cap < 0 || (cap > 0 && !block4_out)) {
        set_error("accel_partition_host: bad argument");
        return ACCEL_ERR_ARG;
    }
    if (indptr[0] != 0) {
        set_error("indptr must start at 0");
        return ACCEL_ERR_CSR;
    }
    int64_t nb = 0;
    auto put = [&](int d, int64_t row, int64_t loc, int info) {
        if (nb < cap) {
            int32_t *q = block4_out + 4 * nb;
            q[0] = d; q[1] = (int32_t)row; q[2] = (int32_t)loc; q[3] = info;
        }
        nb++;
    };
    // one pass over maximal runs of equal degree
    int64_t r = 0;
    while (r < rows) {
        const int64_t d64 = (int64_t)indptr[r + 1] - indptr[r];
        if (d64 < 0) {
            set_error("indptr decreases at row %lld", (long long)r);
            return ACCEL_ERR_CSR;
        }
        int64_t end = r + 1;
        while (end < rows && (int64_t)indptr[end + 1] - indptr[end] == d64) end++;
        const int d = (int)d64;
        if (d > kDegBound) {
            for (int64_t q = r; q < end; q++)
                for (int off = 0; off < d; off += kDegBound)
                    put(d, q, (int64_t)indptr[q] + off, std::min(kDegBound, d - off));
        } else if (d > 0) {
            int w, rpb;
            slice_rule(d, w, rpb);
            for (int64_t q = r; q < end; q += rpb)
                put(d, q, indptr[q], (w << 16) + (int)std::min<int64_t>(rpb, end - q));
        }
        r = end;
    }
    *n_blocks = nb;
    return ACCEL_OK;
}

int accel_degree_sort_host(const int32_t *indptr, int64_t rows, int32_t *perm_out)
{
    clear_error();
    if (!indptr || rows < 0 || (rows > 0 && !perm_out)) {
        set_error("accel_degree_sort_host: bad argument");
        return ACCEL_ERR_ARG;
    }
    std::vector<uint64_t> keys;
    try {
        keys.resize((size_t)rows);
    } catch (const std::bad_alloc &) {
        set_error("host allocation failed");
        return ACCEL_ERR_ALLOC;
    }
    for (int64_t r = 0; r < rows; r++) {
        const int64_t d = (int64_t)indptr[r + 1] - indptr[r];
        if (d < 0) {
            set_error("indptr decreases at row %lld", (long long)r);
            return ACCEL_ERR_CSR;
        }
        keys[(size_t)r] = ((uint64_t)d << 32) | (uint64_t)r;   // unique keys: any sort is stable
    }
    std::sort(keys.begin(), keys.end());
    for (int64_t r = 0; r < rows; r++) perm_out[r] = (int32_t)(keys[(size_t)r] & 0xFFFFFFFFu);
    return ACCEL_OK;
}

// ---------------------------------------------------------------------------
// raw-array files
// ---------------------------------------------------------------------------
int accel_file_count(const char *path, int64_t *n_elems)
{
    clear_error();
    if (!path || !n_elems) { set_error("accel_file_count: bad argument"); return ACCEL_ERR_ARG; }
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) { set_error("cannot open %s", path); return ACCEL_ERR_IO; }
    const std::streamoff len = f.tellg();
    if (len < 0 || len % 4 != 0) {
        set_error("%s: size %lld is not a whole number of 4-byte elements", path, (long long)len);
        return ACCEL_ERR_IO;
    }
    *n_elems = (int64_t)(len / 4);
    return ACCEL_OK;
}

int accel_file_read(const char *path, void *dst, int64_t n_elems)
{
    clear_error();
    if (!path || n_elems < 0 || (n_elems > 0 && !dst)) {
        set_error("accel_file_read: bad argument");
        return ACCEL_ERR_ARG;
    }
    std::ifstream f(path, std::ios::binary);
    if (!f) { set_error("cannot open %s", path); return ACCEL_ERR_IO; }
    f.read(static_cast<char *>(dst), (std::streamsize)(n_elems * 4));
    if (f.gcount() != (std::streamsize)(n_elems * 4)) {
        set_error("%s: short read (%lld of %lld bytes)", path, (long long)f.gcount(),
                  (long long)(n_elems * 4));
        return ACCEL_ERR_IO;
    }
    return ACCEL_OK;
}

int accel_file_write(const char *path, const void *src, int64_t n_elems)
{
    clear_error();
    if (!path || n_elems < 0 || (n_elems > 0 && !src)) {
        set_error("accel_file_write: bad argument");
        return ACCEL_ERR_ARG;
    }
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    if (!f) { set_error("cannot create %s", path); return ACCEL_ERR_IO; }
    f.write(static_cast<const char *>(src), (std::streamsize)(n_elems * 4));
    f.close();
    if (!f) { set_error("write to %s failed", path); return ACCEL_ERR_IO; }
    return ACCEL_OK;
}

// ---------------------------------------------------------------------------
// device plumbing
// ---------------------------------------------------------------------------
int accel_device_count(int *n)
{
    clear_error();
    if (!n) { set_error("accel_device_count: null argument"); return ACCEL_ERR_ARG; }
    *n = 0;
    const hipError_t e = hipGetDeviceCount(n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *n = 0;
        set_error("hipGetDeviceCount: %s", hipGetErrorString(e));
        return ACCEL_ERR_HIP;
    }
    return ACCEL_OK;
}

int accel_dev_malloc(void **p, size_t bytes)
{
    clear_error();
    if (!p) { set_error("accel_dev_malloc: null argument"); return ACCEL_ERR_ARG; }
    *p = nullptr;
    if (int rc = need_gpu()) return rc;
    if (hipMalloc(p, bytes ? bytes : 4) != hipSuccess) {
        (void)hipGetLastError();
        *p = nullptr;
        set_error("device allocation of %zu bytes failed", bytes);
        return ACCEL_ERR_ALLOC;
    }
    return ACCEL_OK;
}

int accel_dev_free(void *p)
{
    clear_error();
    if (p) ACCEL_HIP(hipFree(p));
    return ACCEL_OK;
}

int accel_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
    clear_error();
    if (bytes && (!dst || !src)) { set_error("accel_memcpy_h2d: null argument"); return ACCEL_ERR_ARG; }
    if (bytes) ACCEL_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return ACCEL_OK;
}

int accel_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    clear_error();
    if (bytes && (!dst || !src)) { set_error("accel_memcpy_d2h: null argument"); return ACCEL_ERR_ARG; }
    if (bytes) ACCEL_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return ACCEL_OK;
}

int accel_dev_fill_u32(void *dst, uint32_t value, size_t n_words, void *stream)
{
    clear_error();
    if (n_words && !dst) { set_error("accel_dev_fill_u32: null argument"); return ACCEL_ERR_ARG; }
    if (!stream_is_capturing(static_cast<hipStream_t>(stream)))          // see check_operand
        if (int rc = check_operand(dst, n_words * 4, "accel_dev_fill_u32", "dst")) return rc;
    return fill_u32(dst, value, n_words, static_cast<hipStream_t>(stream));
}

int accel_dev_copy_u32(void *dst_dev, const void *src_dev, size_t n_words, void *stream)
{
    clear_error();
    if (n_words && (!dst_dev || !src_dev)) { set_error("accel_dev_copy_u32: null argument"); return ACCEL_ERR_ARG; }
    if (!stream_is_capturing(static_cast<hipStream_t>(stream))) {
        if (int rc = check_operand(dst_dev, n_words * 4, "accel_dev_copy_u32", "dst")) return rc;
        if (int rc = check_operand(src_dev, n_words * 4, "accel_dev_copy_u32", "src")) return rc;
    }
    return copy_u32(dst_dev, src_dev, n_words, static_cast<hipStream_t>(stream));
}

int accel_stream_sync(void *stream)
{
    clear_error();
    ACCEL_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return ACCEL_OK;
}

// ---------------------------------------------------------------------------
// operator
// ---------------------------------------------------------------------------
int accel_create(const int32_t *indptr, const int32_t *idx, const float *val, int64_t rows,
                 int64_t cols, int64_t nnz, int flags, accel_handle **out)
{
    clear_error();
    if (!out) { set_error("accel_create: null handle pointer"); return ACCEL_ERR_ARG; }
    *out = nullptr;
    if (rows < 0 || cols < 0 || nnz < 0 || rows >= 0x7fffffffLL || cols > 0x7fffffffLL ||
        nnz > 0x7fffffffLL) {
        set_error("accel_create: rows/cols/nnz must be non-negative and fit int32");
        return ACCEL_ERR_ARG;
    }
    if (!indptr || (nnz > 0 && (!idx || !val))) {
        set_error("accel_create: null CSR array");
        return ACCEL_ERR_ARG;
    }
    if (flags != ACCEL_PTR_HOST && flags != ACCEL_PTR_DEVICE) {
        set_error("accel_create: unknown flags %d", flags);
        return ACCEL_ERR_ARG;
    }
    if (int rc = need_gpu()) return rc;
    accel_handle *h = new (std::nothrow) accel_handle();
    if (!h) { set_error("host allocation failed"); return ACCEL_ERR_ALLOC; }
    h->rows = rows; h->cols = cols; h->nnz = nnz;
    (void)hipGetDevice(&h->device);
    if (hipDeviceGetAttribute(&h->device_cus, hipDeviceAttributeMultiprocessorCount, h->device) != hipSuccess) {
        (void)hipGetLastError();
        h->device_cus = 0;
    }
    if (flags == ACCEL_PTR_DEVICE) {
        h->indptr = indptr; h->idx = idx; h->val = val;
        h->owns_input = false;
        // the kernels of accel_preprocess read these arrays: a host address would be a memory fault
        if (int rc = check_borrowed_csr(h, "accel_create")) { delete h; return rc; }
    } else {
        void *a = nullptr, *b = nullptr, *c = nullptr;
        const size_t sa = sizeof(int32_t) * (size_t)(rows + 1);
        const size_t sb = sizeof(int32_t) * (size_t)nnz, sc = sizeof(float) * (size_t)nnz;
        if (hipMalloc(&a, sa) != hipSuccess || hipMalloc(&b, sb ? sb : 4) != hipSuccess ||
            hipMalloc(&c, sc ? sc : 4) != hipSuccess) {
            (void)hipGetLastError();
            if (a) (void)hipFree(a);
            if (b) (void)hipFree(b);
            if (c) (void)hipFree(c);
            delete h;
            set_error("device allocation for the CSR (%zu bytes) failed", sa + sb + sc);
            return ACCEL_ERR_ALLOC;
        }
        h->indptr = static_cast<int32_t *>(a);
        h->idx = static_cast<int32_t *>(b);
        h->val = static_cast<float *>(c);
        h->owns_input = true;
        hipError_t e = hipMemcpy(a, indptr, sa, hipMemcpyHostToDevice);
        if (e == hipSuccess && sb) e = hipMemcpy(b, idx, sb, hipMemcpyHostToDevice);
        if (e == hipSuccess && sc) e = hipMemcpy(c, val, sc, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            set_error("upload of the CSR failed: %s", hipGetErrorString(e));
            accel_destroy(h);
            return ACCEL_ERR_HIP;
        }
    }
    *out = h;
    return ACCEL_OK;
}

int accel_destroy(accel_handle *h)
{
    if (!h) return ACCEL_OK;
    release_products(h);
    if (h->owns_input) {
        (void)hipFree(const_cast<int32_t *>(h->indptr));
        (void)hipFree(const_cast<int32_t *>(h->idx));
        (void)hipFree(const_cast<float *>(h->val));
    }
    delete h;
    return ACCEL_OK;
}

int accel_set_plan_unit(accel_handle *h, int unit_nz)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_unit: null handle"); return ACCEL_ERR_ARG; }
    if (unit_nz != 0 && (unit_nz < 16 || unit_nz > kDegBound)) {
        set_error("accel_set_plan_unit: unit must be 0 (automatic) or 16..384, got %d", unit_nz);
        return ACCEL_ERR_ARG;
    }
    h->plan_unit_option = unit_nz;
    return ACCEL_OK;
}

int accel_set_plan_split(accel_handle *h, int split_nz)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_split: null handle"); return ACCEL_ERR_ARG; }
    if (split_nz != 0 && (split_nz < 16 || split_nz > kDegBound)) {
        set_error("accel_set_plan_split: threshold must be 0 (automatic) or 16..384, got %d", split_nz);
        return ACCEL_ERR_ARG;
    }
    h->plan_split_option = split_nz;
    return ACCEL_OK;
}

int accel_set_plan_groups(accel_handle *h, int groups)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_groups: null handle"); return ACCEL_ERR_ARG; }
    if (groups != 0 && groups != 8 && groups != 16 && groups != 32 && groups != 64) {
        set_error("accel_set_plan_groups: groups must be 0 (automatic), 8, 16, 32 or 64, got %d", groups);
        return ACCEL_ERR_ARG;
    }
    h->plan_groups = groups;
    return ACCEL_OK;
}

int accel_set_plan_team(accel_handle *h, int mode)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_team: null handle"); return ACCEL_ERR_ARG; }
    if (mode < 0 || mode > 2) {
        set_error("accel_set_plan_team: mode must be 0 (automatic), 1 (wavefront units) or 2 "
                  "(workgroup units), got %d", mode);
        return ACCEL_ERR_ARG;
    }
    h->plan_team_option = mode;
    return ACCEL_OK;
}

int accel_set_plan_queues(accel_handle *h, int queues)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_queues: null handle"); return ACCEL_ERR_ARG; }
    if (queues != 0 && queues != 1 && queues != kXcds) {
        set_error("accel_set_plan_queues: queues must be 0 (from the device), 1 or %d, got %d", kXcds, queues);
        return ACCEL_ERR_ARG;
    }
    h->plan_queues_option = queues;
    return ACCEL_OK;
}

int accel_set_plan_reduce(accel_handle *h, int mode)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_reduce: null handle"); return ACCEL_ERR_ARG; }
    if (mode < 0 || mode > 2) {
        set_error("accel_set_plan_reduce: mode must be 0 (automatic), 1 (in the gather kernel) or 2 (second "
                  "kernel), got %d", mode);
        return ACCEL_ERR_ARG;
    }
    h->plan_reduce_option = mode;
    return ACCEL_OK;
}

int accel_set_plan_panel(accel_handle *h, int columns)
{
    clear_error();
    if (!h) { set_error("accel_set_plan_panel: null handle"); return ACCEL_ERR_ARG; }
    if (columns != 0 && (columns < 4 || columns > 1024 || columns % 4 != 0)) {
        set_error("accel_set_plan_panel: width must be 0 (automatic) or a multiple of 4 in 4..1024, got %d",
                  columns);
        return ACCEL_ERR_ARG;
    }
    h->plan_panel_option = columns;
    return ACCEL_OK;
}

int accel_preprocess(accel_handle *h)
{
    clear_error();
    if (!h) { set_error("accel_preprocess: null handle"); return ACCEL_ERR_ARG; }
    if (int rc = check_device(h, "accel_preprocess")) return rc;
    if (int rc = check_borrowed_csr(h, "accel_preprocess")) return rc;     // still there, still large enough
    if (h->val_stale) {                     // value updates since: the handle's copy of the values first
        if (hipDeviceSynchronize() != hipSuccess) (void)hipGetLastError();
        if (int rc = restore_own_values(h, nullptr)) return rc;
    }
    release_products(h);
    const int rc = preprocess_device(h);
    if (rc) release_products(h);
    return rc;
}

// Common part of the two value updates: val_dev holds the new values on the device, in the
// order of the caller's CSR; everything is queued on `stream`.
static int update_values_on_stream(accel_handle *h, const float *val_dev, hipStream_t stream, const char *fn)
{
    (void)hipGetLastError();                // launch errors are read back below: start from a clean slate
    const bool capturing = stream_is_capturing(stream);
    if (h->owns_sorted && !h->src_pos) {
        if (capturing) {
            set_error("%s: the first value update of a handle builds its position map (one allocation); "
                      "do it once before the capture", fn);
            return ACCEL_ERR_STATE;
        }
        if (int rc = build_source_positions(h, stream)) return rc;
    }
    if (int rc = order_update(h, stream, capturing)) return rc;
    if (!h->owns_input) h->val = val_dev;   // borrowed from now on (it may be the same array, rewritten)
    if (h->owns_sorted) {
        // one kernel: the new values into the sorted copy.  A handle's own copy of the caller's
        // order is not rewritten here; it is brought back from the sorted copy if a new
        // preprocessing of the handle ever needs it (restore_own_values).
        if (int rc = gather_values(h, val_dev, stream)) return rc;
        if (h->owns_input && val_dev != h->val) h->val_stale = true;
    } else if (h->owns_input) {
        // the kernels read the handle's copy of the caller's order in place
        if (val_dev != h->val)
            if (int rc = copy_u32(const_cast<float *>(h->val), val_dev, (size_t)h->nnz, stream)) return rc;
    } else {
        h->s_val = h->val;                  // the kernels read the caller's array in place
    }
    return note_update(h, stream, capturing);
}

int accel_update_values_async(accel_handle *h, const float *val_dev, void *stream)
{
    clear_error();
    if (!h) { set_error("accel_update_values_async: null handle"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_update_values_async: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (int rc = check_device(h, "accel_update_values_async")) return rc;
    if (h->nnz == 0) return ACCEL_OK;
    if (!val_dev) { set_error("accel_update_values_async: null array"); return ACCEL_ERR_ARG; }
    if (!stream_is_capturing(static_cast<hipStream_t>(stream)))
        if (int rc = check_operand(val_dev, sizeof(float) * (size_t)h->nnz, "accel_update_values_async", "val"))
            return rc;
    return update_values_on_stream(h, val_dev, static_cast<hipStream_t>(stream), "accel_update_values_async");
}

int accel_update_values(accel_handle *h, const float *val, int flags)
{
    clear_error();
    if (!h) { set_error("accel_update_values: null handle"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_update_values: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (flags != ACCEL_PTR_HOST && flags != ACCEL_PTR_DEVICE) {
        set_error("accel_update_values: unknown flags %d", flags);
        return ACCEL_ERR_ARG;
    }
    if (int rc = check_device(h, "accel_update_values")) return rc;
    if (h->nnz == 0) return ACCEL_OK;
    if (!val) { set_error("accel_update_values: null array"); return ACCEL_ERR_ARG; }
    const size_t bytes = sizeof(float) * (size_t)h->nnz;
    if (flags == ACCEL_PTR_DEVICE)
        if (int rc = check_operand(val, bytes, "accel_update_values", "val")) return rc;
    if (!h->owns_input && flags != ACCEL_PTR_DEVICE) {
        set_error("accel_update_values: this handle borrows its CSR from device memory; pass the new "
                  "values as a device array (ACCEL_PTR_DEVICE)");
        return ACCEL_ERR_ARG;
    }
    hipStream_t s = nullptr;
    if (stream_is_capturing(s)) {
        set_error("accel_update_values waits for its own work; use accel_update_values_async in a capture");
        return ACCEL_ERR_STATE;
    }
    if (flags == ACCEL_PTR_HOST) {
        // into the handle's own copy of the caller's order, behind the runs that may still read it
        if (int rc = order_update(h, s, false)) return rc;
        ACCEL_HIP(hipMemcpyAsync(const_cast<float *>(h->val), val, bytes, hipMemcpyHostToDevice, s));
        val = h->val;
    }
    if (int rc = update_values_on_stream(h, val, s, "accel_update_values")) return rc;
    ACCEL_HIP(hipStreamSynchronize(s));
    h->writer_pending = false;
    if (flags == ACCEL_PTR_HOST) h->val_stale = false;   // the handle's copy was written first
    return ACCEL_OK;
}

int accel_get_info(const accel_handle *h, accel_info *out)
{
    clear_error();
    if (!h || !out) { set_error("accel_get_info: null argument"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_get_info: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    out->rows = h->rows; out->cols = h->cols; out->nnz = h->nnz;
    out->n_blocks = h->n_blocks; out->n_long_blocks = h->n_long_blocks;
    out->n_long_rows = h->n_long_rows; out->n_zero_rows = h->n_zero_rows;
    out->max_degree = h->max_degree; out->already_sorted = h->identity_perm ? 1 : 0;
    out->preprocess_ms = h->preprocess_ms;
    out->n_plan_units = h->n_units;
    out->n_split_rows = h->n_split_rows;
    out->plan_unit_nz = h->plan_unit;
    out->plan_groups = h->plan_groups;
    out->plan_split_nz = h->plan_split;
    out->plan_team = h->plan_team ? 1 : 0;
    out->plan_queues = h->plan_queues;
    out->plan_reduce = h->fused_reduce ? 1 : 2;
    out->n_plan_pieces = h->n_long_units;
    return ACCEL_OK;
}

int accel_get_block4(const accel_handle *h, int32_t *out, int64_t cap_blocks)
{
    clear_error();
    if (!h || (!out && h->n_blocks > 0)) { set_error("accel_get_block4: null argument"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_get_block4: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (cap_blocks < h->n_blocks) {
        set_error("accel_get_block4: buffer holds %lld blocks, %lld needed", (long long)cap_blocks,
                  (long long)h->n_blocks);
        return ACCEL_ERR_ARG;
    }
    if (h->n_blocks)
        ACCEL_HIP(hipMemcpy(out, h->block4, sizeof(int32_t) * 4 * (size_t)h->n_blocks,
                            hipMemcpyDeviceToHost));
    return ACCEL_OK;
}

int accel_get_perm(const accel_handle *h, int32_t *out, int64_t cap_rows)
{
    clear_error();
    if (!h || (!out && h->rows > 0)) { set_error("accel_get_perm: null argument"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_get_perm: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (cap_rows < h->rows) { set_error("accel_get_perm: buffer too small"); return ACCEL_ERR_ARG; }
    if (h->identity_perm) {
        for (int64_t r = 0; r < h->rows; r++) out[r] = (int32_t)r;
    } else {
        ACCEL_HIP(hipMemcpy(out, h->perm, sizeof(int32_t) * (size_t)h->rows, hipMemcpyDeviceToHost));
    }
    return ACCEL_OK;
}

int accel_get_sorted_csr(const accel_handle *h, int32_t *indptr, int32_t *idx, float *val)
{
    clear_error();
    if (!h) { set_error("accel_get_sorted_csr: null handle"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_get_sorted_csr: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (h->rows == 0) {
        if (indptr) indptr[0] = 0;
        return ACCEL_OK;
    }
    if (indptr)
        ACCEL_HIP(hipMemcpy(indptr, h->s_indptr, sizeof(int32_t) * (size_t)(h->rows + 1),
                            hipMemcpyDeviceToHost));
    if (idx && h->nnz)
        ACCEL_HIP(hipMemcpy(idx, h->s_idx, sizeof(int32_t) * (size_t)h->nnz, hipMemcpyDeviceToHost));
    if (val && h->nnz)
        ACCEL_HIP(hipMemcpy(val, h->s_val, sizeof(float) * (size_t)h->nnz, hipMemcpyDeviceToHost));
    return ACCEL_OK;
}

int accel_get_plan(const accel_handle *h, int32_t *out, int64_t cap_units, int64_t *n_units)
{
    clear_error();
    if (!h || !n_units || cap_units < 0) { set_error("accel_get_plan: bad argument"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_get_plan: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    *n_units = h->n_units;
    const int64_t take = std::min(cap_units, h->n_units);
    if (out && take > 0)
        ACCEL_HIP(hipMemcpy(out, h->work, sizeof(int32_t) * 4 * (size_t)take, hipMemcpyDeviceToHost));
    return ACCEL_OK;
}

int accel_check_block4(accel_handle *h, const int32_t *block4_host, int64_t n_blocks)
{
    clear_error();
    if (!h || n_blocks < 0 || (n_blocks > 0 && !block4_host)) {
        set_error("accel_check_block4: bad argument");
        return ACCEL_ERR_ARG;
    }
    if (!h->ready) { set_error("accel_check_block4: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (n_blocks != h->n_blocks) {
        set_error("metadata has %lld blocks, this CSR partitions into %lld", (long long)n_blocks,
                  (long long)h->n_blocks);
        return ACCEL_ERR_META;
    }
    std::vector<int32_t> mine((size_t)n_blocks * 4);
    if (n_blocks)
        ACCEL_HIP(hipMemcpy(mine.data(), h->block4, sizeof(int32_t) * mine.size(), hipMemcpyDeviceToHost));
    for (size_t i = 0; i < mine.size(); i++)
        if (mine[i] != block4_host[i]) {
            set_error("metadata differs at block %zu field %zu: file %d, CSR %d", i / 4, i % 4,
                      block4_host[i], mine[i]);
            return ACCEL_ERR_META;
        }
    return ACCEL_OK;
}

// Partition a row order as given, on the GPU: what block_level_partition.py
// computes for one *.new_indptr file (lines 38-106).  indptr is a host array.
int accel_partition_gpu(const int32_t *indptr, int64_t rows, int32_t *block4_out, int64_t cap,
                        int64_t *n_blocks)
{
    clear_error();
    if (!indptr || rows < 0 || rows >= 0x7fffffffLL || !n_blocks || cap < 0 ||
        (cap > 0 && !block4_out)) {
        set_error("accel_partition_gpu: bad argument");
        return ACCEL_ERR_ARG;
    }
    if (int rc = need_gpu()) return rc;
    *n_blocks = 0;
    if (rows == 0) return ACCEL_OK;
    void *dptr = nullptr;
    if (hipMalloc(&dptr, sizeof(int32_t) * (size_t)(rows + 1)) != hipSuccess) {
        (void)hipGetLastError();
        set_error("device allocation failed");
        return ACCEL_ERR_ALLOC;
    }
    int rc = ACCEL_OK;
    int32_t *b4 = nullptr;
    int64_t nb = 0;
    if (hipMemcpy(dptr, indptr, sizeof(int32_t) * (size_t)(rows + 1), hipMemcpyHostToDevice) != hipSuccess) {
        set_error("upload of indptr failed");
        rc = ACCEL_ERR_HIP;
    }
    if (!rc) rc = partition_only_device(static_cast<int32_t *>(dptr), rows, indptr[rows], &b4, &nb);
    if (!rc) {
        *n_blocks = nb;
        const int64_t take = std::min(nb, cap);
        if (take > 0 &&
            hipMemcpy(block4_out, b4, sizeof(int32_t) * 4 * (size_t)take, hipMemcpyDeviceToHost) != hipSuccess) {
            set_error("download of the metadata failed");
            rc = ACCEL_ERR_HIP;
        }
    }
    if (b4) (void)hipFree(b4);
    (void)hipFree(dptr);
    return rc;
}

int accel_run(accel_handle *h, const float *X, float *Y, int32_t N, void *stream)
{
    clear_error();
    if (int rc = check_run(h, X, Y, N, nullptr, "accel_run", static_cast<hipStream_t>(stream))) return rc;
    return spmm_launch(h, X, Y, N, static_cast<hipStream_t>(stream));
}

int accel_run_strided(accel_handle *h, const float *X, float *Y, int32_t N, int32_t ld, void *stream)
{
    clear_error();
    if (ld < N) { set_error("accel_run_strided: the row stride (%d) must be at least N (%d)", ld, N); return ACCEL_ERR_ARG; }
    if (int rc = check_run(h, X, Y, N, nullptr, "accel_run_strided", static_cast<hipStream_t>(stream), ld)) return rc;
    return spmm_launch(h, X, Y, N, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, 0, false, ld);
}

int accel_run_ex(accel_handle *h, const accel_run_args *a)
{
    clear_error();
    if (!a) { set_error("accel_run_ex: null arguments"); return ACCEL_ERR_ARG; }
    const int32_t ld = a->ld == 0 ? a->N : a->ld;
    if (ld < a->N) { set_error("accel_run_ex: the row stride (%d) must be 0 or at least N (%d)", a->ld, a->N); return ACCEL_ERR_ARG; }
    if (a->flags & ~ACCEL_EPILOGUE_RELU) { set_error("accel_run_ex: unknown flags %d", a->flags); return ACCEL_ERR_ARG; }
    if (int rc = check_run(h, a->X, a->Y, a->N, a->bias, "accel_run_ex", static_cast<hipStream_t>(a->stream), ld)) return rc;
    return spmm_launch(h, a->X, a->Y, a->N, static_cast<hipStream_t>(a->stream), nullptr, nullptr, a->bias,
                       (a->flags & ACCEL_EPILOGUE_RELU) ? 1 : 0, false, ld);
}

int accel_reserve(accel_handle *h, int32_t max_N)
{
    clear_error();
    if (!h) { set_error("accel_reserve: null handle"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_reserve: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    if (max_N <= 0) { set_error("accel_reserve: N must be positive, got %d", max_N); return ACCEL_ERR_ARG; }
    return reserve_partial(h, (size_t)h->n_long_units * (size_t)max_N);
}

int accel_run_static(accel_handle *h, const float *X, float *Y, int32_t N, void *stream)
{
    clear_error();
    if (int rc = check_run(h, X, Y, N, nullptr, "accel_run_static", static_cast<hipStream_t>(stream))) return rc;
    return spmm_launch(h, X, Y, N, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, 0, true);
}

int accel_run_epilogue(accel_handle *h, const float *X, float *Y, int32_t N, const float *bias,
                       int flags, void *stream)
{
    clear_error();
    if (int rc = check_run(h, X, Y, N, bias, "accel_run_epilogue", static_cast<hipStream_t>(stream))) return rc;
    if (flags & ~ACCEL_EPILOGUE_RELU) { set_error("accel_run_epilogue: unknown flags %d", flags); return ACCEL_ERR_ARG; }
    return spmm_launch(h, X, Y, N, static_cast<hipStream_t>(stream), nullptr, nullptr, bias,
                       (flags & ACCEL_EPILOGUE_RELU) ? 1 : 0);
}

// The timing protocol on any form of run: a->stream carries the launches.
static int time_runs(accel_handle *h, const accel_run_args *a, int32_t ld, int warmup, int iters, float *ms_total,
                     float *ms_main)
{
    hipStream_t s = static_cast<hipStream_t>(a->stream);
    const int relu = (a->flags & ACCEL_EPILOGUE_RELU) ? 1 : 0;
    for (int i = 0; i < warmup; i++)
        if (int rc = spmm_launch(h, a->X, a->Y, a->N, s, nullptr, nullptr, a->bias, relu, false, ld)) return rc;
    ACCEL_HIP(hipStreamSynchronize(s));
    if (iters == 0) return ACCEL_OK;
    // All launches are queued back to back; the events are read after one final wait.  Per
    // run: two events recorded around it, and two bound to the gather kernel itself (its
    // start and its end: these put nothing between the run's kernels).
    std::vector<hipEvent_t> ev((size_t)iters * 4, nullptr);
    int rc = ACCEL_OK;
    for (auto &e : ev)
        if (hipEventCreate(&e) != hipSuccess) { rc = ACCEL_ERR_HIP; set_error("hipEventCreate failed"); break; }
    for (int i = 0; i < iters && !rc; i++) {
        hipError_t e = hipEventRecord(ev[4 * i], s);
        if (e == hipSuccess)
            rc = spmm_launch(h, a->X, a->Y, a->N, s, ms_main ? ev[4 * i + 1] : nullptr,
                             ms_main ? ev[4 * i + 2] : nullptr, a->bias, relu, false, ld);
        if (!rc && e == hipSuccess) e = hipEventRecord(ev[4 * i + 3], s);
        if (!rc && e != hipSuccess) { set_error("hipEventRecord: %s", hipGetErrorString(e)); rc = ACCEL_ERR_HIP; }
    }
    if (!rc && hipStreamSynchronize(s) != hipSuccess) { set_error("stream synchronisation failed"); rc = ACCEL_ERR_HIP; }
    for (int i = 0; i < iters && !rc; i++) {
        float t = 0.f;
        hipError_t e = hipEventElapsedTime(&t, ev[4 * i], ev[4 * i + 3]);
        if (e == hipSuccess && ms_total) ms_total[i] = t;
        if (e == hipSuccess && ms_main) {
            e = hipEventElapsedTime(&t, ev[4 * i + 1], ev[4 * i + 2]);
            ms_main[i] = t;
        }
        if (e != hipSuccess) { set_error("event timing failed: %s", hipGetErrorString(e)); rc = ACCEL_ERR_HIP; }
    }
    for (auto e : ev)
        if (e) (void)hipEventDestroy(e);
    return rc;
}

int accel_time(accel_handle *h, const float *X, float *Y, int32_t N, int warmup, int iters,
               float *ms_total, float *ms_main, void *stream)
{
    clear_error();
    if (warmup < 0 || iters < 0) { set_error("accel_time: bad warmup/iters"); return ACCEL_ERR_ARG; }
    if (int rc = check_run(h, X, Y, N, nullptr, "accel_time", static_cast<hipStream_t>(stream))) return rc;
    const accel_run_args a{X, Y, N, 0, nullptr, 0, stream};
    return time_runs(h, &a, N, warmup, iters, ms_total, ms_main);
}

int accel_time_ex(accel_handle *h, const accel_run_args *a, int warmup, int iters, float *ms_total,
                  float *ms_main)
{
    clear_error();
    if (!a) { set_error("accel_time_ex: null arguments"); return ACCEL_ERR_ARG; }
    if (warmup < 0 || iters < 0) { set_error("accel_time_ex: bad warmup/iters"); return ACCEL_ERR_ARG; }
    const int32_t ld = a->ld == 0 ? a->N : a->ld;
    if (ld < a->N) { set_error("accel_time_ex: the row stride (%d) must be 0 or at least N (%d)", a->ld, a->N); return ACCEL_ERR_ARG; }
    if (a->flags & ~ACCEL_EPILOGUE_RELU) { set_error("accel_time_ex: unknown flags %d", a->flags); return ACCEL_ERR_ARG; }
    if (int rc = check_run(h, a->X, a->Y, a->N, a->bias, "accel_time_ex", static_cast<hipStream_t>(a->stream), ld)) return rc;
    return time_runs(h, a, ld, warmup, iters, ms_total, ms_main);
}

int accel_dense_xw(const float *X, const float *W, float *Z, int64_t rows, int32_t K, int32_t N, int32_t ldx,
                   int32_t ldz, void *stream)
{
    clear_error();
    const char *fn = "accel_dense_xw";
    if (int rc = need_gpu()) return rc;
    if (rows < 0 || K <= 0 || N <= 0) {
        set_error("%s: bad shape (%lld rows, K = %d, N = %d)", fn, (long long)rows, K, N);
        return ACCEL_ERR_ARG;
    }
    if (ldx == 0) ldx = K;
    if (ldz == 0) ldz = N;
    if (ldx < K || ldz < N) {
        set_error("%s: row strides (%d, %d) must be 0 or at least K (%d) and N (%d)", fn, ldx, ldz, K, N);
        return ACCEL_ERR_ARG;
    }
    if (rows == 0) return ACCEL_OK;
    if (!X || !W || !Z) { set_error("%s: null operand", fn); return ACCEL_ERR_ARG; }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!stream_is_capturing(s)) {              // see check_operand
        const size_t x_bytes = ((size_t)(rows - 1) * (size_t)ldx + (size_t)K) * sizeof(float);
        const size_t z_bytes = ((size_t)(rows - 1) * (size_t)ldz + (size_t)N) * sizeof(float);
        if (int rc = check_operand(X, x_bytes, fn, "X")) return rc;
        if (int rc = check_operand(W, (size_t)K * (size_t)N * sizeof(float), fn, "W")) return rc;
        if (int rc = check_operand(Z, z_bytes, fn, "Z")) return rc;
        const char *zb = reinterpret_cast<const char *>(Z), *xb = reinterpret_cast<const char *>(X),
                   *wb = reinterpret_cast<const char *>(W);
        if ((zb < xb + x_bytes && xb < zb + z_bytes) ||
            (zb < wb + (size_t)K * N * sizeof(float) && wb < zb + z_bytes)) {
            set_error("%s: Z overlaps an input", fn);
            return ACCEL_ERR_ARG;
        }
    }
    return dense_xw_launch(X, W, Z, rows, K, N, ldx, ldz, s);
}

}  // extern "C"
