// Saved preprocessing state: what accel_preprocess produced for one CSR, written to a
// file and loaded into a new handle on the same CSR instead of being recomputed.
//
// Upstream persists its preprocessing the same way: block_level_partition.py:105-106
// writes <graph>.block4 once and SPMM_ACCEL::do_test loads it on every call
// (spmm_accel.cu:122).  Here the state is the block4 metadata plus the other products
// of the GPU preprocessing: the degree-sort permutation, the sorted indptr, the launch
// plan and the partial-sum slots of the split rows.  The sorted copy of the non-zeros is
// not stored (it is as large as the CSR itself); it is gathered again from the caller's
// arrays by two kernels.
//
// The file is keyed by content hashes of indptr and idx (computed on the GPU), so a
// state saved for another graph is refused with ACCEL_ERR_META, and every stored array
// carries its own hash, so a damaged file is refused before any kernel uses it.
#include <cstring>
#include <chrono>
#include <cstdio>
#include <memory>
#include <new>
#include <vector>

#include "internal.h"

namespace accel {
namespace {

constexpr char kMagic[8] = {'A', 'C', 'G', 'C', 'N', 'S', 'T', '1'};
constexpr uint32_t kStateVersion = 1;
constexpr uint64_t kSeedIndptr = 0x11, kSeedIdx = 0x22, kSeedArray = 0x100;

enum ArrayId { kPerm = 0, kSortedIndptr, kBlock4, kWork, kLongSlot, kNumArrays };

struct StateHeader {
    char magic[8];
    uint32_t version, header_bytes;
    int64_t rows, cols, nnz;
    uint64_t hash_indptr, hash_idx;
    int64_t n_blocks, n_long_blocks, n_long_rows, n_zero_rows, n_units, n_long_units, n_split_rows,
        n_big_rows, n_wide_rows;
    int32_t max_degree, identity_perm, plan_unit, plan_split, plan_groups, plan_team, local,
        waves_per_group;
    int64_t words[kNumArrays];        // 4-byte words of each stored array (0: absent)
    uint64_t hash[kNumArrays];        // content hash of each stored array
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

struct DevU64 {
    uint64_t *p = nullptr;
    ~DevU64() { if (p) (void)hipFree(p); }
    int alloc(int n)
    {
        if (hipMalloc(reinterpret_cast<void **>(&p), sizeof(uint64_t) * (size_t)n) != hipSuccess) {
            (void)hipGetLastError();
            p = nullptr;
            set_error("device allocation failed");
            return ACCEL_ERR_ALLOC;
        }
        return ACCEL_OK;
    }
};

// hashes of several device arrays in one go: out_host[i] = hash of arrays[i]
int hash_arrays(const void *const *arrays, const int64_t *words, const uint64_t *seeds, int n,
                uint64_t *out_host)
{
    DevU64 d;
    if (int rc = d.alloc(n)) return rc;
    if (int rc = fill_u32(d.p, 0u, (size_t)n * 2, nullptr)) return rc;
    for (int i = 0; i < n; i++)
        if (int rc = hash_words_device(arrays[i], words[i], seeds[i], d.p + i, nullptr)) return rc;
    ACCEL_HIP(hipMemcpy(out_host, d.p, sizeof(uint64_t) * (size_t)n, hipMemcpyDeviceToHost));
    return ACCEL_OK;
}

int csr_hashes(const accel_handle *h, uint64_t *hash_indptr, uint64_t *hash_idx)
{
    const void *arrays[2] = {h->indptr, h->idx};
    const int64_t words[2] = {h->rows + 1, h->nnz};
    const uint64_t seeds[2] = {kSeedIndptr, kSeedIdx};
    uint64_t out[2] = {0, 0};
    if (int rc = hash_arrays(arrays, words, seeds, 2, out)) return rc;
    *hash_indptr = out[0];
    *hash_idx = out[1];
    return ACCEL_OK;
}

void stored_arrays(const accel_handle *h, const void **arrays, int64_t *words)
{
    arrays[kPerm] = h->perm;
    words[kPerm] = h->perm ? h->rows : 0;
    arrays[kSortedIndptr] = h->s_indptr;
    words[kSortedIndptr] = h->s_indptr ? h->rows + 1 : 0;
    arrays[kBlock4] = h->block4;
    words[kBlock4] = 4 * h->n_blocks;
    arrays[kWork] = h->work;
    words[kWork] = 4 * h->n_units;
    arrays[kLongSlot] = h->long_slot;
    words[kLongSlot] = h->long_slot ? h->n_split_rows + 1 : 0;
}

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
    hd.rows = h->rows; hd.cols = h->cols; hd.nnz = h->nnz;
    hd.n_blocks = h->n_blocks; hd.n_long_blocks = h->n_long_blocks; hd.n_long_rows = h->n_long_rows;
    hd.n_zero_rows = h->n_zero_rows; hd.n_units = h->n_units; hd.n_long_units = h->n_long_units;
    hd.n_split_rows = h->n_split_rows; hd.n_big_rows = h->n_big_rows; hd.n_wide_rows = h->n_wide_rows;
    hd.max_degree = h->max_degree; hd.identity_perm = h->identity_perm ? 1 : 0;
    hd.plan_unit = h->plan_unit; hd.plan_split = h->plan_split; hd.plan_groups = h->plan_groups;
    hd.plan_team = h->plan_team ? 1 : 0; hd.local = h->local ? 1 : 0;
    hd.waves_per_group = kWavesPerGroup;
    const void *arrays[kNumArrays];
    stored_arrays(h, arrays, hd.words);
    if (h->rows > 0) {
        if (int rc = csr_hashes(h, &hd.hash_indptr, &hd.hash_idx)) return rc;
        uint64_t seeds[kNumArrays];
        for (int i = 0; i < kNumArrays; i++) seeds[i] = kSeedArray + (uint64_t)i;
        if (int rc = hash_arrays(arrays, hd.words, seeds, kNumArrays, hd.hash)) return rc;
    }
    hd.header_hash = header_hash(hd);
    // write to a temporary name and rename, so that a reader never sees half a file
    const std::string tmp = std::string(path) + ".tmp";
    {
        File out;
        out.f = fopen(tmp.c_str(), "wb");
        if (!out.f) { set_error("cannot create %s", tmp.c_str()); return ACCEL_ERR_IO; }
        bool ok = fwrite(&hd, sizeof hd, 1, out.f) == 1;
        int rc = ACCEL_OK;
        std::vector<uint32_t> host;
        for (int i = 0; i < kNumArrays && ok && !rc; i++) {
            if (hd.words[i] == 0) continue;
            try {
                host.resize((size_t)hd.words[i]);
            } catch (const std::bad_alloc &) {
                set_error("host allocation of %lld bytes failed", (long long)hd.words[i] * 4);
                rc = ACCEL_ERR_ALLOC;
                break;
            }
            const hipError_t e =
                hipMemcpy(host.data(), arrays[i], sizeof(uint32_t) * host.size(), hipMemcpyDeviceToHost);
            if (e != hipSuccess) {
                set_error("download of the state failed: %s", hipGetErrorString(e));
                rc = ACCEL_ERR_HIP;
                break;
            }
            ok = fwrite(host.data(), sizeof(uint32_t), host.size(), out.f) == host.size();
        }
        ok = ok && fflush(out.f) == 0;
        if (!rc && !ok) {
            set_error("write to %s failed", tmp.c_str());
            rc = ACCEL_ERR_IO;
        }
        if (rc) {
            fclose(out.f);
            out.f = nullptr;
            (void)remove(tmp.c_str());
            return rc;
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
    const auto t0 = std::chrono::steady_clock::now();
    File in;
    in.f = fopen(path, "rb");
    if (!in.f) { set_error("cannot open %s", path); return ACCEL_ERR_IO; }
    StateHeader hd;
    if (fread(&hd, sizeof hd, 1, in.f) != 1) { set_error("%s: truncated header", path); return ACCEL_ERR_IO; }
    if (std::memcmp(hd.magic, kMagic, sizeof kMagic) != 0 || hd.version != kStateVersion ||
        hd.header_bytes != sizeof(StateHeader) || hd.waves_per_group != kWavesPerGroup) {
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
    // the header must be consistent with itself before anything is sized from it
    const int64_t want[kNumArrays] = {hd.identity_perm ? 0 : hd.rows, hd.rows > 0 ? hd.rows + 1 : 0,
                                      4 * hd.n_blocks, 4 * hd.n_units,
                                      hd.rows > 0 ? hd.n_split_rows + 1 : 0};
    bool sane = hd.n_blocks >= 0 && hd.n_units >= 0 && hd.n_split_rows >= 0 && hd.n_split_rows <= hd.rows &&
                hd.n_big_rows >= 0 && hd.n_big_rows <= hd.n_split_rows && hd.n_wide_rows >= 0 &&
                hd.n_wide_rows <= hd.rows && hd.n_zero_rows >= 0 &&
                hd.n_zero_rows <= hd.rows && hd.n_long_units >= 0 && hd.n_long_units <= hd.n_units &&
                hd.n_blocks <= hd.rows + hd.nnz && hd.n_units <= 0x7fffffffLL &&
                hd.n_units % (kXcds * kWavesPerGroup) == 0 &&
                (hd.plan_groups == 0 || hd.plan_groups == 8 || hd.plan_groups == 16 || hd.plan_groups == 32 ||
                 hd.plan_groups == 64);
    for (int i = 0; i < kNumArrays && sane; i++) sane = hd.words[i] == want[i];
    if (!sane) { set_error("%s: inconsistent header", path); return ACCEL_ERR_META; }
    // the file must be exactly as long as the header says, before anything is allocated from it
    {
        int64_t expect = (int64_t)sizeof(StateHeader);
        for (int i = 0; i < kNumArrays; i++) expect += 4 * hd.words[i];
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

    release_products(h);
    if (h->rows == 0) {
        h->identity_perm = true;
        h->ready = true;
        return ACCEL_OK;
    }
    uint64_t hi = 0, hx = 0;
    if (int rc = csr_hashes(h, &hi, &hx)) return rc;
    if (hi != hd.hash_indptr || hx != hd.hash_idx) {
        set_error("%s was saved for a different CSR (content hash of %s differs)", path,
                  hi != hd.hash_indptr ? "indptr" : "idx");
        return ACCEL_ERR_META;
    }
    // upload the stored arrays; on any failure the handle is left without products
    void *dev[kNumArrays] = {};
    auto fail = [&](int rc) {
        for (auto p : dev)
            if (p) (void)hipFree(p);
        return rc;
    };
    std::vector<uint32_t> host;
    for (int i = 0; i < kNumArrays; i++) {
        if (hd.words[i] == 0) continue;
        try {
            host.resize((size_t)hd.words[i]);
        } catch (const std::bad_alloc &) {
            set_error("host allocation of %lld bytes failed", (long long)hd.words[i] * 4);
            return fail(ACCEL_ERR_ALLOC);
        }
        if (fread(host.data(), sizeof(uint32_t), host.size(), in.f) != host.size()) {
            set_error("%s: truncated", path);
            return fail(ACCEL_ERR_IO);
        }
        if (hipMalloc(&dev[i], sizeof(uint32_t) * host.size()) != hipSuccess) {
            (void)hipGetLastError();
            dev[i] = nullptr;
            set_error("device allocation of %zu bytes failed", sizeof(uint32_t) * host.size());
            return fail(ACCEL_ERR_ALLOC);
        }
        if (hipMemcpy(dev[i], host.data(), sizeof(uint32_t) * host.size(), hipMemcpyHostToDevice) != hipSuccess) {
            set_error("upload of the saved state failed");
            return fail(ACCEL_ERR_HIP);
        }
    }
    {
        uint64_t seeds[kNumArrays], got[kNumArrays];
        for (int i = 0; i < kNumArrays; i++) seeds[i] = kSeedArray + (uint64_t)i;
        if (int rc = hash_arrays(dev, hd.words, seeds, kNumArrays, got)) return fail(rc);
        for (int i = 0; i < kNumArrays; i++)
            if (got[i] != hd.hash[i]) {
                set_error("%s: stored array %d does not match its hash (damaged file)", path, i);
                return fail(ACCEL_ERR_META);
            }
    }
    h->perm = static_cast<int32_t *>(dev[kPerm]);
    h->s_indptr = static_cast<int32_t *>(dev[kSortedIndptr]);
    h->block4 = static_cast<int32_t *>(dev[kBlock4]);
    h->work = static_cast<int32_t *>(dev[kWork]);
    h->long_slot = static_cast<int32_t *>(dev[kLongSlot]);
    h->identity_perm = hd.identity_perm != 0;
    h->n_blocks = hd.n_blocks; h->n_long_blocks = hd.n_long_blocks; h->n_long_rows = hd.n_long_rows;
    h->n_zero_rows = hd.n_zero_rows; h->n_units = hd.n_units; h->n_long_units = hd.n_long_units;
    h->n_split_rows = hd.n_split_rows; h->n_big_rows = hd.n_big_rows; h->n_wide_rows = hd.n_wide_rows;
    h->max_degree = hd.max_degree;
    h->plan_unit = hd.plan_unit; h->plan_split = hd.plan_split; h->plan_groups = hd.plan_groups;
    h->plan_team = hd.plan_team != 0; h->local = hd.local != 0;
    // non-zeros of the rows that are not split = sorted indptr at the first split row
    const int64_t first_long = h->rows - h->n_split_rows;
    int32_t nz_short32 = 0;
    int rc = ACCEL_OK;
    if (hipMemcpy(&nz_short32, h->s_indptr + first_long, sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) {
        set_error("read-back of the sorted indptr failed");
        rc = ACCEL_ERR_HIP;
    }
    if (!rc && (nz_short32 < 0 || (int64_t)nz_short32 > h->nnz)) {
        set_error("%s: sorted indptr out of range", path);
        rc = ACCEL_ERR_META;
    }
    if (!rc) rc = rebuild_sorted_csr(h, nz_short32, nullptr);
    if (rc) {
        release_products(h);
        return rc;
    }
    h->ready = true;
    h->preprocess_ms =
        std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return ACCEL_OK;
}

}  // extern "C"
