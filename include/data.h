/*
 * Raw-array file readers of the benchmark framework (upstream: data.h:7-34).
 *
 * A graph file is a whole-file array of fixed-size elements.  Upstream's
 * cuda_read_array (data.h:7-21) reads one into managed memory and returns the
 * element count; read_array (data.h:22-34) reads into a new[] host array.
 *
 *   hip_read_array  the device-side reader: the file is read into a host buffer
 *                   and copied into a hipMalloc allocation (managed memory is
 *                   accepted by the operators as well, but on a GPU that runs
 *                   without page migration it stays on the host and every gather
 *                   crosses the host link).  *arr is a device pointer; release it
 *                   with hipFree.
 *   read_array      same file, host array from new[]; release it with delete[].
 *
 * Both return the element count, or -1 when the file cannot be read or the
 * device allocation or copy fails (upstream returns a garbage count for a
 * missing file).
 */
#pragma once
#include <hip/hip_runtime.h>

#include <fstream>
#include <string>
using namespace std;   /* as upstream's data.h:4: its callers name `string` unqualified */

template <typename scalar_t>
int read_array(scalar_t **arr, string file)
{
    *arr = nullptr;
    std::ifstream input(file, std::ios::in | std::ios::binary | std::ios::ate);
    if (!input) return -1;
    const std::streamoff bytes = input.tellg();
    if (bytes < 0) return -1;
    const size_t cnt = (size_t)bytes / sizeof(scalar_t);
    input.seekg(0, std::ios::beg);
    scalar_t *host = new scalar_t[cnt ? cnt : 1];
    input.read(reinterpret_cast<char *>(host), (std::streamsize)(cnt * sizeof(scalar_t)));
    if ((size_t)input.gcount() != cnt * sizeof(scalar_t)) {
        delete[] host;
        return -1;
    }
    *arr = host;
    return (int)cnt;
}

template <typename scalar_t>
int hip_read_array(scalar_t **arr, string file)
{
    *arr = nullptr;
    scalar_t *host = nullptr;
    const int cnt = read_array(&host, file);
    if (cnt < 0) return -1;
    void *dev = nullptr;
    const size_t bytes = (size_t)cnt * sizeof(scalar_t);
    bool ok = hipMalloc(&dev, bytes ? bytes : sizeof(scalar_t)) == hipSuccess;
    if (ok && bytes) ok = hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice) == hipSuccess;
    delete[] host;
    if (!ok) {
        if (dev) (void)hipFree(dev);
        return -1;
    }
    *arr = static_cast<scalar_t *>(dev);
    return cnt;
}
