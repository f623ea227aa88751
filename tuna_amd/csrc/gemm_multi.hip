// Instantiations and launcher of the batched persistent kernel (gemm_multi.hpp).

#include "gemm_multi.hpp"

namespace tuna {

typedef void (*MultiKernelFn)(const MultiArgs);
static const struct {
    int u;
    MultiKernelFn fn;
} kMulti[] = {{2, gemm_multi_kernel<2>}, {4, gemm_multi_kernel<4>}, {-2, gemm_multi_kernel<2, true, true>},  // (-2: ring of 2, weights and x through LDS)
              {12, gemm_multi_kernel<2, true, false, true>}, {14, gemm_multi_kernel<4, true, false, true>},  // (10 + ring: a scale per block of a row)
              {22, gemm_multi_kernel<2, true, false, false, true>}, {24, gemm_multi_kernel<4, true, false, false, true>}};  // (20 + ring: fused epilogues)
static constexpr int kNumMulti = sizeof(kMulti) / sizeof(kMulti[0]);

static OptInFlag g_multi_attr_done[16][kNumMulti];

bool multi_variant_exists(int prefetch)
{
    for (int i = 0; i < kNumMulti; ++i)
        if (kMulti[i].u == prefetch) return true;
    return false;
}

size_t multi_lds_bytes() { return (size_t)kLutBytes + 2 * 32 * 1024 + 32 * 1024; }  // table, two x buffers, reduction area

hipError_t launch_gemm_multi(const MultiArgs &args, int prefetch, int dev, hipStream_t stream)
{
    int vi = -1;
    for (int i = 0; i < kNumMulti; ++i)
        if (kMulti[i].u == prefetch) vi = i;
    if (vi < 0 || dev < 0 || dev >= 16) return hipErrorInvalidConfiguration;
    const hipError_t e = ensure_lds_opt_in(g_multi_attr_done[dev][vi], reinterpret_cast<const void *>(kMulti[vi].fn));
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kMulti[vi].fn, dim3((unsigned)args.n_wg), dim3(1024), multi_lds_bytes(), stream, args);
    return hipGetLastError();
}

}  // namespace tuna
