// Product build (libtuna_amd.so): the library's routing choices are constants and nothing is counted.
#include "diag.h"

namespace tuna {
namespace diag {

int lean_kernels() { return 1; }
int weight_path() { return 0; }
int multi_waves_m() { return 0; }
int multi_prefetch() { return 0; }
int multi_lds() { return 0; }
int multi_min_batch() { return 2; }
int blockwise_scales_lds() { return 1; }
void count(Counter) {}

}  // namespace diag
}  // namespace tuna
