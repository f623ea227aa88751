// Instantiations and launcher of the batched persistent kernel (gemm_multi.hpp).
#include <mutex>

#include "gemm_multi.hpp"

namespace tuna {

typedef void (*MultiKernelFn)(const MultiArgs);
static const struct {
    int u;
    MultiKernelFn fn;
} kMulti[] = {{2, gemm_multi_kernel<2>}, {4, gemm_multi_kernel<4>}};
static constexpr int kNumMulti = sizeof(kMulti) / sizeof(kMulti[0]);

static std::mutex g_multi_attr_mutex;
static unsigned char g_multi_attr_done[16][kNumMulti];

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
    {
        std::lock_guard<std::mutex> lock(g_multi_attr_mutex);
        if (!g_multi_attr_done[dev][vi]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kMulti[vi].fn),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
            if (e != hipSuccess) return e;
            g_multi_attr_done[dev][vi] = 1;
        }
    }
    hipLaunchKernelGGL(kMulti[vi].fn, dim3((unsigned)args.n_wg), dim3(1024), multi_lds_bytes(), stream, args);
    return hipGetLastError();
}

}  // namespace tuna
