// Routing choices and launch counters that only a diagnostic build can change or read.
//
// The library picks between kernels that compute identical results (lean twin or general kernel, weights through
// registers or through LDS, workgroup shape of the batched kernel, kernel family of the blockwise GEMM).  Tests and
// A/B timings want to force each choice and to see which kernel ran.  Those switches are process-wide state, which
// a product library must not have: libtuna_amd.so links diag_off.cpp, where every choice is a constant and
// counting does nothing; libtuna_amd_bench.so links diag_on.cpp, where they are atomics behind the tuna_set_* /
// tuna_*_launches entry points of tuna_amd_bench.h.  Every other object file is the same in both libraries.
#pragma once

namespace tuna {
namespace diag {

int lean_kernels();          // 1: launches that qualify take the lean / streaming twins of the general kernel
int weight_path();           // 1: launches that have an LDS-staged twin run it whatever their config says
int multi_waves_m();         // batched kernel: waves along the rows (0: the library's choice)
int multi_prefetch();        // batched kernel: ring depth (0: the library's choice)
int multi_lds();             // 1: batches with a ring of two stage weights and x through LDS
int multi_min_batch();       // batches shorter than this are launched problem by problem (2)
int blockwise_scales_lds();  // 1: the narrow-row blockwise kernel keeps a workgroup's scales in LDS

enum Counter { kLeanLaunches, kMultiLaunches, kBlockwiseNarrow, kBlockwiseMulti, kBlockwiseTiled, kBlockwiseMid, kNumCounters };
void count(Counter c);

}  // namespace diag
}  // namespace tuna
