// The quantizer's division by a block maximum (dequant_kernel.hip) and nothing else: shared with the
// self-test kernel of the diagnostic build (bench_kernels.hip), which runs it on every pair of fp16 values.
#pragma once
#include <hip/hip_runtime.h>

namespace tuna {

// fp32(w) / a, correctly rounded, for the quotients this kernel forms: w an fp16 value, a the
// largest |fp16| of its block, so |w| <= a and both are normal binary32 numbers (or w is zero).
// y is the reciprocal of a refined once from v_rcp_f32 (computed once per block); the quotient is one
// multiply and one fused correction step.  No denormal-mode switches, no scaling: the ranges rule
// out what the general division sequence guards against.  Equality with the IEEE division is
// checked for every pair (w, a) of fp16 values with |w| <= a in tests/test_gpu_parity.py.
__device__ __forceinline__ float refined_rcp(float a)
{
    const float y = __builtin_amdgcn_rcpf(a);
    return __builtin_fmaf(__builtin_fmaf(-a, y, 1.0f), y, y);
}

__device__ __forceinline__ float div_by_block_max(float w, float a, float y)
{
    const float q = w * y;
    return __builtin_fmaf(__builtin_fmaf(-q, a, w), y, q);
}

}  // namespace tuna
