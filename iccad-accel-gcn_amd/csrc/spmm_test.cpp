// spmm_test: command-line harness for the SPMM_ACCEL operator, the counterpart of
// upstream's main.cu for the accel operator only.
//
//   spmm_test <graph> <dim>      check against a host CSR loop, then time (main.cu:186-194)
//   spmm_test                    time every <graphs>/*.config for dim 16..128 (main.cu:195-219)
//   options: --graphs DIR (default ../graphs/)  --meta DIR (default ../block_level_meta/)
//            --save-state   write <meta>/<graph>.accelstate after preprocessing; a later run
//                           takes the row order from it instead of sorting (as upstream loads
//                           its .block4, spmm_accel.cu:122) and says so on stderr
//            --natural      read the graph in its own vertex order, <graph>.graph.ptrdump and
//                           <graph>.graph.edgedump (the files upstream gives to its baselines,
//                           main.cu:64-65), and hand that CSR to the operator, which sorts the
//                           rows by degree itself and returns vout in the order given.  On graphs
//                           whose numbering has locality this is the faster input: the launch plan
//                           follows the caller's row ids, which the pre-sorted files have lost.
//
// Input files, as upstream reads them (main.cu:62-65, data.h:7-21): <graph>.new_indptr and
// <graph>.new_indices (rows in ascending degree order), or the two .graph.* files with
// --natural; raw little-endian int32 (held in device memory here, not managed memory).  Values are all 1 and vin ~ U[0,1) from
// std::default_random_engine seeded with 123 (main.cu:90-93,114-121, value mode 3).
// Output lines follow main.cu:40-49 and :161-167:
//   err sum = <x>  validation pass!|fail!
//   <i>/<n> <graph> <dim> accel <microseconds>
// The check is upstream's: mean |out - ref| < 1e-3 (main.cu:18-51), with the reference
// product computed here by a plain host loop where upstream calls cuSPARSE (main.cu:143-155).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <filesystem>
#include <iostream>
#include <random>
#include <vector>

#include "accel_gcn.h"
#include "spmm_accel.h"

namespace {

std::string base_dir = "../graphs/";
std::string meta_dir = "../block_level_meta/";
int dim_min = 16, dim_max = 128, interval = 1;
int total_file_cnt = 0, current_file_cnt = 0;
bool save_state = false;
bool natural_order = false;

// Upstream keeps every array in managed memory (data.h:15) and lets the pages migrate.
// Here the arrays live in device memory and are copied explicitly: on a GPU that runs
// without page migration a managed allocation stays in host memory, and every gather
// would cross the host link (measured: 9.7 ms instead of 0.1 ms per launch on a
// 1.2 M-non-zero graph).
template <class T>
bool to_device(const std::vector<T> &host, T **dev)
{
    const size_t bytes = std::max<size_t>(host.size(), 1) * sizeof(T);
    if (hipMalloc(reinterpret_cast<void **>(dev), bytes) != hipSuccess) {
        std::cerr << "hipMalloc of " << bytes << " bytes failed" << std::endl;
        return false;
    }
    if (!host.empty() && hipMemcpy(*dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) {
        std::cerr << "copy to the device failed" << std::endl;
        return false;
    }
    return true;
}

template <class T>
bool read_file(const std::string &path, std::vector<T> &out)
{
    int64_t n = 0;
    int rc = accel_file_count(path.c_str(), &n);
    if (rc == ACCEL_OK) {
        out.resize((size_t)n);
        rc = accel_file_read(path.c_str(), out.data(), n);
    }
    if (rc != ACCEL_OK) std::cerr << accel_last_error() << std::endl;
    return rc == ACCEL_OK;
}

// the role cuSPARSE plays upstream: an independent product to check against
void host_reference(const int *ptr, const int *idx, const float *val, const float *vin, float *out,
                    int v_num, int dim)
{
    for (int r = 0; r < v_num; r++) {
        float *y = out + (size_t)r * dim;
        std::fill(y, y + dim, 0.0f);
        for (int p = ptr[r]; p < ptr[r + 1]; p++) {
            const float a = val[p];
            const float *x = vin + (size_t)idx[p] * dim;
            for (int j = 0; j < dim; j++) y[j] += a * x[j];
        }
    }
}

double check_err(const float *out, const float *ref, size_t len, bool &has_err)
{
    double err_sum = 0;
    has_err = false;
    for (size_t i = 0; i < len; i++) {
        const double err = std::fabs((double)out[i] - (double)ref[i]);
        err_sum += err;
        if (err > 0.1 && !has_err) {
            has_err = true;
            std::cout << "err at " << i << std::endl;
        }
    }
    std::cout << "err sum = " << err_sum << "  ";
    std::cout << (err_sum / (double)len < 0.001 ? "validation pass!" : "validation fail!") << std::endl;
    return err_sum;
}

int test_graph(const std::string &graph, int spec_dim, bool checking, bool timing)
{
    int lo = dim_min, hi = dim_max;
    if (spec_dim > 0) lo = hi = spec_dim;

    std::vector<int> h_ptr, h_idx;
    const std::string ptr_file = graph + (natural_order ? ".graph.ptrdump" : ".new_indptr");
    const std::string idx_file = graph + (natural_order ? ".graph.edgedump" : ".new_indices");
    if (!read_file(base_dir + ptr_file, h_ptr)) return 1;
    if (!read_file(base_dir + idx_file, h_idx)) return 1;
    if (h_ptr.empty()) {
        std::cerr << ptr_file << " is empty" << std::endl;
        return 1;
    }
    const int v_num = (int)h_ptr.size() - 1, e_num = (int)h_idx.size();
    const size_t dense = (size_t)v_num * hi;
    std::default_random_engine engine;
    engine.seed(123);
    std::uniform_real_distribution<float> rd(0, 1);
    std::vector<float> h_val((size_t)e_num, 1.0f), h_vin(dense), h_out(dense);
    std::generate(h_vin.begin(), h_vin.end(), [&]() { return rd(engine); });

    int *indptr = nullptr, *indices = nullptr;
    float *val = nullptr, *vin = nullptr, *vout = nullptr;
    if (!to_device(h_ptr, &indptr) || !to_device(h_idx, &indices) || !to_device(h_val, &val) ||
        !to_device(h_vin, &vin) || !to_device(h_out, &vout))
        return 1;

    SPMM_ACCEL accel(graph, indptr, indices, val, vin, vout, v_num, e_num, hi);
    accel.set_meta_dir(meta_dir);
    accel.set_save_state(save_state);
    bool said = false;
    int rc = 0;
    std::vector<float> ref;
    for (int dim = lo; dim <= hi && rc == 0; dim += interval) {
        if (checking) {
            std::cout << "CHECKING ..." << std::endl;
            if (accel.do_test(false, dim) < 0) {
                std::cerr << "accel: " << accel.error() << std::endl;
                rc = 1;
                break;
            }
            if (!said && accel.loaded_from_state()) std::cerr << "accel: preprocessing loaded from saved state" << std::endl;
            said = true;
            ref.resize((size_t)v_num * dim);
            host_reference(h_ptr.data(), h_idx.data(), h_val.data(), h_vin.data(), ref.data(), v_num, dim);
            if (hipMemcpy(h_out.data(), vout, ref.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) {
                std::cerr << "copy from the device failed" << std::endl;
                rc = 1;
                break;
            }
            bool has_err = false;
            std::cout << "checking accel" << std::endl;
            const double e = check_err(h_out.data(), ref.data(), ref.size(), has_err);
            if (!(e / (double)std::max<size_t>(ref.size(), 1) < 0.001)) rc = 2;
        }
        if (timing) {
            std::cout << "TIMING ..." << std::endl;
            const double t = accel.do_test(true, dim);
            if (t < 0) {
                std::cerr << "accel: " << accel.error() << std::endl;
                rc = 1;
                break;
            }
            std::cout << current_file_cnt << "/" << total_file_cnt << " " << graph << " " << dim
                      << " accel " << t * 1e6 << std::endl;
        }
    }
    (void)hipFree(indptr);
    (void)hipFree(indices);
    (void)hipFree(val);
    (void)hipFree(vin);
    (void)hipFree(vout);
    return rc;
}

}  // namespace

int main(int argc, char *argv[])
{
    std::vector<std::string> pos;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        if (a == "--graphs" && i + 1 < argc) base_dir = argv[++i];
        else if (a == "--meta" && i + 1 < argc) meta_dir = argv[++i];
        else if (a == "--save-state") save_state = true;
        else if (a == "--natural") natural_order = true;
        else pos.push_back(a);
    }
    if (!base_dir.empty() && base_dir.back() != '/') base_dir += '/';
    if (!meta_dir.empty() && meta_dir.back() != '/') meta_dir += '/';
    int n_dev = 0;
    if (accel_device_count(&n_dev) != ACCEL_OK || n_dev < 1) {
        std::cerr << "spmm_test: no GPU (" << accel_last_error() << ")" << std::endl;
        return 3;
    }
    if (pos.size() >= 2) {
        std::cout << "dir = " << base_dir << std::endl;
        return test_graph(pos[0], std::atoi(pos[1].c_str()), true, true);
    }
    namespace fs = std::filesystem;
    std::error_code ec;
    std::vector<std::string> graphs;
    for (const auto &f : fs::directory_iterator(base_dir, ec))
        if (f.path().extension() == ".config") graphs.push_back(f.path().stem().string());
    if (ec) {
        std::cerr << "spmm_test: cannot list " << base_dir << std::endl;
        return 1;
    }
    std::sort(graphs.begin(), graphs.end());
    total_file_cnt = (int)graphs.size();
    int rc = 0;
    for (const auto &g : graphs) {
        current_file_cnt++;
        rc |= test_graph(g, 0, false, true);
        (void)hipDeviceSynchronize();
    }
    return rc;
}
