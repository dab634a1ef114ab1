// Saved preprocessing state: the part of accel_preprocess that a file can stand in for.
//
// Upstream persists its preprocessing as a file: block_level_partition.py:105-106 writes
// <graph>.block4 once and SPMM_ACCEL::do_test loads it on every call (spmm_accel.cu:122).
// Here every product of the preprocessing except one is rebuilt on the GPU faster than a
// file of its size can be read (block4, the sorted indptr, the launch plan and the
// partial-sum slots together take well under a millisecond for 125 M non-zeros), and the
// sorted copy of the non-zeros is as large as the CSR itself.  The state therefore holds
// the one product that is an input to all the others, the degree-sort permutation, plus
// the plan options the handle was preprocessed with.  accel_load_state reads it and runs
// the preprocessing with the sort replaced by the stored order.
//
// Nothing in the file is trusted: the stored order is accepted only if a kernel finds it
// to be exactly the order the sort would produce for this CSR's indptr (that order is
// unique), so a state of another matrix, of another library version or with flipped bits
// is refused with ACCEL_ERR_META, and everything that indexes memory is computed afresh
// by the code that is running.
#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>

#include "internal.h"

namespace accel {
int check_borrowed_csr(const accel_handle *h, const char *fn);      // capi.hip
namespace {

constexpr char kMagic[8] = {'A', 'C', 'G', 'C', 'N', 'S', 'T', '2'};
constexpr uint32_t kStateVersion = 2;

struct StateHeader {
    char magic[8];
    uint32_t version, header_bytes;
    int32_t library_version;          // accel_version() of the writer (informative)
    int32_t identity_perm;            // 1: the rows were already in degree order, no permutation follows
    int64_t rows, cols, nnz;
    int32_t plan_unit_option, plan_split_option, plan_groups, plan_team_option, plan_queues_option;
    int32_t plan_reduce_option;
    int64_t perm_words;               // rows, or 0 with identity_perm
    uint64_t header_hash;             // FNV-1a of this header with header_hash = 0
};

uint64_t header_hash(StateHeader hd)
{
    hd.header_hash = 0;
    const unsigned char *b = reinterpret_cast<const unsigned char *>(&hd);
    uint64_t x = 0xCBF29CE484222325ull;
    for (size_t i = 0; i < sizeof hd; i++) x = (x ^ b[i]) * 0x100000001B3ull;
    return x;
}

struct File {
    FILE *f = nullptr;
    ~File() { if (f) fclose(f); }
};

struct PinnedBuf {   // host memory the GPU copies from and to directly
    void *p = nullptr;
    ~PinnedBuf() { if (p) (void)hipHostFree(p); }
    int alloc(size_t bytes)
    {
        if (hipHostMalloc(&p, bytes ? bytes : 4, hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            p = nullptr;
            set_error("allocation of %zu bytes of pinned host memory failed", bytes);
            return ACCEL_ERR_ALLOC;
        }
        return ACCEL_OK;
    }
};

struct DevMem {
    void *p = nullptr;
    ~DevMem() { if (p) (void)hipFree(p); }
};

}  // namespace
}  // namespace accel

using namespace accel;

extern "C" {

int accel_save_state(const accel_handle *h, const char *path)
{
    clear_error();
    if (!h || !path) { set_error("accel_save_state: null argument"); return ACCEL_ERR_ARG; }
    if (!h->ready) { set_error("accel_save_state: call accel_preprocess first"); return ACCEL_ERR_STATE; }
    StateHeader hd;
    std::memset(&hd, 0, sizeof hd);
    std::memcpy(hd.magic, kMagic, sizeof kMagic);
    hd.version = kStateVersion;
    hd.header_bytes = (uint32_t)sizeof(StateHeader);
    hd.library_version = accel_version();
    hd.identity_perm = h->identity_perm ? 1 : 0;
    hd.rows = h->rows; hd.cols = h->cols; hd.nnz = h->nnz;
    hd.plan_unit_option = h->plan_unit_option; hd.plan_split_option = h->plan_split_option;
    hd.plan_groups = h->plan_groups; hd.plan_team_option = h->plan_team_option;
    hd.plan_queues_option = h->plan_queues_option;
    hd.plan_reduce_option = h->plan_reduce_option;
    hd.perm_words = h->identity_perm ? 0 : h->rows;
    hd.header_hash = header_hash(hd);
    PinnedBuf host;
    if (hd.perm_words > 0) {
        if (int rc = host.alloc(sizeof(int32_t) * (size_t)hd.perm_words)) return rc;
        ACCEL_HIP(hipMemcpy(host.p, h->perm, sizeof(int32_t) * (size_t)hd.perm_words, hipMemcpyDeviceToHost));
    }
    // write to a temporary name and rename, so that a reader never sees half a file
    const std::string tmp = std::string(path) + ".tmp";
    {
        File out;
        out.f = fopen(tmp.c_str(), "wb");
        if (!out.f) { set_error("cannot create %s", tmp.c_str()); return ACCEL_ERR_IO; }
        bool ok = fwrite(&hd, sizeof hd, 1, out.f) == 1;
        if (ok && hd.perm_words > 0)
            ok = fwrite(host.p, sizeof(int32_t), (size_t)hd.perm_words, out.f) == (size_t)hd.perm_words;
        ok = ok && fflush(out.f) == 0;
        if (!ok) {
            set_error("write to %s failed", tmp.c_str());
            fclose(out.f);
            out.f = nullptr;
            (void)remove(tmp.c_str());
            return ACCEL_ERR_IO;
        }
    }
    if (rename(tmp.c_str(), path) != 0) {
        set_error("cannot rename %s to %s", tmp.c_str(), path);
        (void)remove(tmp.c_str());
        return ACCEL_ERR_IO;
    }
    return ACCEL_OK;
}

int accel_load_state(accel_handle *h, const char *path)
{
    clear_error();
    if (!h || !path) { set_error("accel_load_state: null argument"); return ACCEL_ERR_ARG; }
    if (int rc = check_borrowed_csr(h, "accel_load_state")) return rc;
    const auto t0 = std::chrono::steady_clock::now();
    File in;
    in.f = fopen(path, "rb");
    if (!in.f) { set_error("cannot open %s", path); return ACCEL_ERR_IO; }
    StateHeader hd;
    if (fread(&hd, sizeof hd, 1, in.f) != 1) { set_error("%s: truncated header", path); return ACCEL_ERR_IO; }
    if (std::memcmp(hd.magic, kMagic, sizeof kMagic) != 0 || hd.version != kStateVersion ||
        hd.header_bytes != sizeof(StateHeader)) {
        set_error("%s is not a state file of this library version", path);
        return ACCEL_ERR_META;
    }
    if (hd.header_hash != header_hash(hd)) {
        set_error("%s: header does not match its hash (damaged file)", path);
        return ACCEL_ERR_META;
    }
    if (hd.rows != h->rows || hd.cols != h->cols || hd.nnz != h->nnz) {
        set_error("%s was saved for a %lld x %lld matrix with %lld non-zeros, this one is %lld x %lld with %lld",
                  path, (long long)hd.rows, (long long)hd.cols, (long long)hd.nnz, (long long)h->rows,
                  (long long)h->cols, (long long)h->nnz);
        return ACCEL_ERR_META;
    }
    // the header must be consistent with itself and hold options the setters would accept
    auto unit_ok = [](int v) { return v == 0 || (v >= 16 && v <= kDegBound); };
    const bool sane = (hd.identity_perm == 0 || hd.identity_perm == 1) &&
                      hd.perm_words == (hd.identity_perm ? 0 : hd.rows) && unit_ok(hd.plan_unit_option) &&
                      unit_ok(hd.plan_split_option) &&
                      (hd.plan_groups == 0 || hd.plan_groups == 8 || hd.plan_groups == 16 ||
                       hd.plan_groups == 32 || hd.plan_groups == 64) &&
                      hd.plan_team_option >= 0 && hd.plan_team_option <= 2 &&
                      (hd.plan_queues_option == 0 || hd.plan_queues_option == 1 || hd.plan_queues_option == kXcds) &&
                      hd.plan_reduce_option >= 0 && hd.plan_reduce_option <= 2;
    if (!sane) { set_error("%s: inconsistent header", path); return ACCEL_ERR_META; }
    // the file must be exactly as long as the header says, before anything is allocated from it
    {
        const int64_t expect = (int64_t)sizeof(StateHeader) + 4 * hd.perm_words;
        const long at = ftell(in.f);
        if (at < 0 || fseek(in.f, 0, SEEK_END) != 0) { set_error("%s: cannot seek", path); return ACCEL_ERR_IO; }
        const long len = ftell(in.f);
        if (fseek(in.f, at, SEEK_SET) != 0) { set_error("%s: cannot seek", path); return ACCEL_ERR_IO; }
        if ((int64_t)len != expect) {
            set_error("%s: %lld bytes, the header describes %lld (truncated or damaged file)", path,
                      (long long)len, (long long)expect);
            return ACCEL_ERR_IO;
        }
    }
    // the file goes into pinned memory, from which the GPU copies it in one transfer
    PinnedBuf host;
    DevMem dev;
    SavedOrder order{hd.identity_perm != 0, nullptr};
    if (hd.perm_words > 0) {
        const size_t bytes = sizeof(int32_t) * (size_t)hd.perm_words;
        if (int rc = host.alloc(bytes)) return rc;
        if (fread(host.p, 1, bytes, in.f) != bytes) { set_error("%s: truncated", path); return ACCEL_ERR_IO; }
        if (hipMalloc(&dev.p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            dev.p = nullptr;
            set_error("device allocation of %zu bytes failed", bytes);
            return ACCEL_ERR_ALLOC;
        }
        ACCEL_HIP(hipMemcpyAsync(dev.p, host.p, bytes, hipMemcpyHostToDevice, nullptr));
        order.perm_dev = static_cast<const uint32_t *>(dev.p);
    }
    if (h->val_stale) {                     // value updates since: the handle's copy of the values first
        if (hipDeviceSynchronize() != hipSuccess) (void)hipGetLastError();
        if (int rc = restore_own_values(h, nullptr)) return rc;
    }
    release_products(h);
    // the options of the state replace the handle's, so that the handle ends up as the one
    // that was saved; they come back if the load fails
    const int keep[6] = {h->plan_unit_option, h->plan_split_option, h->plan_groups, h->plan_team_option,
                         h->plan_queues_option, h->plan_reduce_option};
    h->plan_unit_option = hd.plan_unit_option; h->plan_split_option = hd.plan_split_option;
    h->plan_groups = hd.plan_groups; h->plan_team_option = hd.plan_team_option;
    h->plan_queues_option = hd.plan_queues_option;
    h->plan_reduce_option = hd.plan_reduce_option;
    const int rc = preprocess_device(h, &order);
    (void)hipStreamSynchronize(nullptr);            // the staging buffers go away with this scope
    if (rc) {
        release_products(h);
        h->plan_unit_option = keep[0]; h->plan_split_option = keep[1]; h->plan_groups = keep[2];
        h->plan_team_option = keep[3]; h->plan_queues_option = keep[4]; h->plan_reduce_option = keep[5];
        return rc;
    }
    h->preprocess_ms =
        std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return ACCEL_OK;
}

}  // extern "C"
