// Diagnostic build (libtuna_amd_bench.so): the routing choices of diag.h as process-wide atomics, set and read
// through the entry points of tuna_amd_bench.h.
#include <atomic>

#include "bench_internal.h"
#include "diag.h"
#include "tuna_internal.h"

namespace tuna {
namespace diag {

static std::atomic<int> g_lean{1}, g_weight_path{0}, g_multi_waves_m{0}, g_multi_prefetch{0}, g_multi_lds{0}, g_multi_min_batch{2},
    g_blockwise_stream{1}, g_blockwise_scales_lds{1}, g_blockwise_shape[3];
static std::atomic<unsigned long long> g_counters[kNumCounters];

static inline int get(const std::atomic<int> &v) { return v.load(std::memory_order_relaxed); }

int lean_kernels() { return get(g_lean); }
int weight_path() { return get(g_weight_path); }
int multi_waves_m() { return get(g_multi_waves_m); }
int multi_prefetch() { return get(g_multi_prefetch); }
int multi_lds() { return get(g_multi_lds); }
int multi_min_batch() { return get(g_multi_min_batch); }
int blockwise_stream() { return get(g_blockwise_stream); }
int blockwise_scales_lds() { return get(g_blockwise_scales_lds); }
int blockwise_shape(int i) { return i >= 0 && i < 3 ? get(g_blockwise_shape[i]) : 0; }
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
TUNA_EXPORT int tuna_set_blockwise_stream(int enabled)
{
    return g_blockwise_stream.exchange(enabled < 0 ? 0 : enabled > 3 ? 3 : enabled, std::memory_order_relaxed);
}
TUNA_EXPORT int tuna_set_blockwise_scales_lds(int enabled) { return g_blockwise_scales_lds.exchange(enabled ? 1 : 0); }
TUNA_EXPORT int tuna_set_blockwise_shape(int rows, int waves_k, int prefetch)
{
    if ((rows || waves_k || prefetch) && !blockwise_variant_exists(rows, waves_k, prefetch))
        return fail(TUNA_ERR_INVALID_ARG, "no blockwise GEMM variant with %d rows, %d waves, ring %d", rows, waves_k, prefetch);
    g_blockwise_shape[0].store(rows);
    g_blockwise_shape[1].store(waves_k);
    g_blockwise_shape[2].store(prefetch);
    return TUNA_OK;
}

}  // extern "C"
