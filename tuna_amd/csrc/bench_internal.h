// Declarations of the diagnostic build only (libtuna_amd_bench.so): the yardstick launches of bench_kernels.hip.
#pragma once
#include "../../include/tuna_amd_bench.h"
#include "tuna_internal.h"

namespace tuna {

hipError_t launch_copy(const void *src, void *dst, size_t bytes, hipStream_t stream);
hipError_t launch_division_selftest(unsigned long long *counts, hipStream_t stream);
hipError_t launch_empty(void *sink, int blocks, int threads, hipStream_t stream);
hipError_t run_handover_yardstick(int stride, int npairs, int store_sc1, int load_sc1, int reuse, int iters, hipStream_t stream, double *out);
hipError_t launch_read(const void *src, void *sink, size_t bytes, int blocks, int variant, hipStream_t stream);
hipError_t launch_unit_rate(int unit, int cus, uint32_t *sink, double *work, hipStream_t stream);

}  // namespace tuna
