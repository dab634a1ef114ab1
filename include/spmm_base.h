/*
 * Operator interface of the SpMM benchmark framework, HIP edition.
 *
 * Mirrors upstream's spmm_base.h:6-65 member for member so that code written
 * against it keeps compiling: same constructor signature (:9-20), the same two
 * pure virtuals do_test(timing, dim) (:23) and run(dim) (:33), the same
 * protected fields including the launch geometry `grid`/`block` (:30), and the
 * same timing protocol in timing_body: 4 warm-up launches, then 4 launches each
 * timed on the host with a device synchronisation, arithmetic mean in seconds,
 * 0 when timing is off (:34-63).  The only change is the runtime: HIP's dim3 and
 * hipDeviceSynchronize, and a steady clock instead of system_clock (util.h:4-9).
 *
 * What a translation unit gets from including this file is part of the
 * interface too: upstream's header pulls in util.h (:2, the timestamp /
 * getDuration helpers) and <string> and opens namespace std (:4), and its own
 * caller relies on that (main.cu:10 names `string` before its own using-
 * directive).  This header does the same.
 */
#pragma once
#include <hip/hip_runtime.h>

#include <chrono>
#include <string>

#include "util.h"
using namespace std;

class SPMM_BASE
{
public:
    SPMM_BASE(std::string _graph, int *ptr, int *idx, float *val, float *vin, float *vout,
              int num_v, int num_e, int dim)
        : _graph(_graph), ptr(ptr), idx(idx), val(val), vin(vin), vout(vout), num_v(num_v),
          num_e(num_e), dim(dim)
    {
    }
    ~SPMM_BASE() {}

    /* Preprocess, then run once (timing == false, returns 0) or run the timing
     * protocol (returns mean seconds per launch; negative on error). */
    virtual double do_test(bool timing, int dim) = 0;

protected:
    std::string _graph;
    int *ptr, *idx;
    float *val, *vin, *vout;
    int num_v, num_e, dim;
    dim3 grid, block;

    /* One asynchronous launch of the operator on the default stream. */
    virtual void run(int dim) = 0;

    double timing_body(bool timing, int dim)
    {
        if (!timing) {
            run(dim);
            (void)hipDeviceSynchronize();
            return 0.0;
        }
        const int times = 4;
        for (int i = 0; i < times; i++) run(dim);
        (void)hipDeviceSynchronize();
        double measured = 0.0;
        for (int i = 0; i < times; i++) {
            const auto t0 = std::chrono::steady_clock::now();
            run(dim);
            (void)hipDeviceSynchronize();
            const auto t1 = std::chrono::steady_clock::now();
            measured += std::chrono::duration<double>(t1 - t0).count();
        }
        return measured / times;
    }
};
