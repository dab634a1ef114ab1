/*
 * Host-clock helpers of the benchmark framework (upstream: util.h:4-9).
 *
 * Upstream's callers write `timestamp(t0); ...; timestamp(t1); getDuration(t0, t1)`
 * around a launch plus a device synchronisation (spmm_base.h:53-57) and get
 * seconds as a double.  The same two names are provided here so that such
 * code compiles unchanged; spmm_base.h includes this file as upstream's does.
 */
#pragma once
#include <chrono>

/* Declares a variable holding the present wall-clock time. */
#define timestamp(__var__) auto __var__ = std::chrono::system_clock::now();

/* Seconds from a to b. */
inline double getDuration(std::chrono::system_clock::time_point a, std::chrono::system_clock::time_point b)
{
    return std::chrono::duration_cast<std::chrono::duration<double>>(b - a).count();
}
