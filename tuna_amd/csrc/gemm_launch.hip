// Instantiations of the GEMM kernel and the variant dispatcher.
#include <mutex>

#include "gemm_kernel.hpp"

namespace tuna {

typedef void (*GemmKernelFn)(const GemmArgs);

struct Variant {
    int rw, u, tt, dec, maxt;
    GemmKernelFn fn;
};

#define V(RW, U, TT, DEC, MAXT) {RW, U, TT, DEC, MAXT, gemm_kernel<RW, U, TT, DEC, MAXT>}
#define V_TT(RW, U, MAXT) V(RW, U, 1, TUNA_DECODE_GEMM, MAXT), V(RW, U, 2, TUNA_DECODE_GEMM, MAXT), V(RW, U, 4, TUNA_DECODE_GEMM, MAXT)

static const Variant kVariants[] = {
    // Only variants that compile without register spills are listed (checked with
    // -Rpass-analysis=kernel-resource-usage); tuna_amd/make_configs.py mirrors this list.
    // rows_per_wave = 64
    V_TT(1, 2, 512), V_TT(1, 4, 512), V_TT(1, 8, 512),
    // rows_per_wave = 128
    V(2, 2, 1, TUNA_DECODE_GEMM, 512), V(2, 2, 2, TUNA_DECODE_GEMM, 512),
    V(2, 4, 1, TUNA_DECODE_GEMM, 512), V(2, 4, 2, TUNA_DECODE_GEMM, 512),
    V(2, 8, 1, TUNA_DECODE_GEMM, 512),
    // rows_per_wave = 256
    V(4, 2, 1, TUNA_DECODE_GEMM, 512),
    // 16-wave workgroups (128 VGPRs per lane): single token tile only
    V(1, 4, 1, TUNA_DECODE_GEMM, 1024), V(1, 8, 1, TUNA_DECODE_GEMM, 1024),
    // dequant-rounding decode (correctness mode, not tuned)
    V(1, 2, 1, TUNA_DECODE_DEQUANT, 512), V(1, 2, 2, TUNA_DECODE_DEQUANT, 512), V(1, 2, 4, TUNA_DECODE_DEQUANT, 512),
};
#undef V
#undef V_TT
static constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

static const Variant *find_variant(int rw, int u, int tt, int dec, int threads)
{
    const int maxt = threads <= 512 ? 512 : 1024;
    for (int i = 0; i < kNumVariants; ++i) {
        const Variant &v = kVariants[i];
        if (v.rw == rw && v.u == u && v.tt == tt && v.dec == dec && v.maxt == maxt) return &v;
    }
    return nullptr;
}

bool gemm_variant_exists(int rw, int prefetch, int token_tiles, int decode, int threads)
{
    return find_variant(rw, prefetch, token_tiles, decode, threads) != nullptr;
}

// Dynamic LDS above 64 KB needs a one-time opt-in per kernel and device.
static std::mutex g_attr_mutex;
static unsigned char g_attr_done[16][kNumVariants];

hipError_t launch_gemm(const GemmPlan &plan, hipStream_t stream)
{
    const Variant *v = find_variant(plan.rw, plan.prefetch, plan.token_tiles, plan.decode, plan.threads);
    if (!v) return hipErrorInvalidConfiguration;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    const int vi = (int)(v - kVariants);
    {
        std::lock_guard<std::mutex> lock(g_attr_mutex);
        if (!g_attr_done[dev][vi]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(v->fn),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
            if (e != hipSuccess) return e;
            g_attr_done[dev][vi] = 1;
        }
    }
    hipLaunchKernelGGL(v->fn, plan.grid, dim3(plan.threads), plan.lds_bytes, stream, plan.args);
    return hipGetLastError();
}

}  // namespace tuna
