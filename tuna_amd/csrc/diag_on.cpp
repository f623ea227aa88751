// Diagnostic build (libtuna_amd_bench.so): the routing choices of diag.h as process-wide atomics, set and read
// through the entry points of tuna_amd_bench.h.
#include <atomic>

#include "bench_internal.h"
#include "diag.h"
#include "tuna_internal.h"

namespace tuna {
namespace diag {

static std::atomic<int> g_lean{1}, g_weight_path{0}, g_multi_waves_m{0}, g_multi_prefetch{0}, g_multi_lds{0}, g_multi_min_batch{2},
    g_blockwise_scales_lds{1};
static std::atomic<unsigned long long> g_counters[kNumCounters];

static inline int get(const std::atomic<int> &v) { return v.load(std::memory_order_relaxed); }

int lean_kernels() { return get(g_lean); }
int weight_path() { return get(g_weight_path); }
int multi_waves_m() { return get(g_multi_waves_m); }
int multi_prefetch() { return get(g_multi_prefetch); }
int multi_lds() { return get(g_multi_lds); }
int multi_min_batch() { return get(g_multi_min_batch); }
int blockwise_scales_lds() { return get(g_blockwise_scales_lds); }
void count(Counter c) { g_counters[c].fetch_add(1, std::memory_order_relaxed); }

}  // namespace diag
}  // namespace tuna

using namespace tuna;
using namespace tuna::diag;

extern "C" {

TUNA_EXPORT int tuna_set_lean_kernels(int enabled) { return g_lean.exchange(enabled ? 1 : 0); }
TUNA_EXPORT int tuna_set_weight_path(int through_lds) { return g_weight_path.exchange(through_lds ? 1 : 0); }
TUNA_EXPORT unsigned long long tuna_lean_launches(void) { return g_counters[kLeanLaunches].load(); }

TUNA_EXPORT int tuna_set_multi_shape(int waves_m, int prefetch)
{
    g_multi_waves_m.store(waves_m);
    g_multi_prefetch.store(prefetch);
    return TUNA_OK;
}
TUNA_EXPORT int tuna_set_multi_weight_path(int through_lds) { return g_multi_lds.exchange(through_lds ? 1 : 0); }
TUNA_EXPORT int tuna_set_multi_min_batch(int count) { return g_multi_min_batch.exchange(count < 1 ? 1 : count); }
TUNA_EXPORT unsigned long long tuna_multi_launches(void) { return g_counters[kMultiLaunches].load(); }

TUNA_EXPORT unsigned long long tuna_blockwise_launches(int kernel)
{
    return kernel >= 0 && kernel < 4 ? g_counters[kBlockwiseNarrow + kernel].load(std::memory_order_relaxed) : 0ull;
}
TUNA_EXPORT int tuna_set_blockwise_scales_lds(int enabled) { return g_blockwise_scales_lds.exchange(enabled ? 1 : 0); }
}  // extern "C"
