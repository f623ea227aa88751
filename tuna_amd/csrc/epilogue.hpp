// Device-side types and the fused output epilogues shared by the GEMM kernels.
#pragma once
#include "tuna_internal.h"

namespace tuna {

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint32_t lds_u32;

// Final store of 4 consecutive output features (columns col .. col+3 of a row of `out` that is
// ld long) of one token, with the fused epilogues:
//   TUNA_EPILOGUE_NONE      out = fp16(v)
//   TUNA_EPILOGUE_RESIDUAL  out = fp16(v + residual), residual fp16 with the layout of out
//   TUNA_EPILOGUE_SILU_MUL  weight rows interleaved (2i: gate_i, 2i+1: up_i): the four values are
//                           (g0, u0, g1, u1) and out, ld/2 long, gets fp16(silu(g) * u) for both
__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + __expf(-g)) * u; }

__device__ __forceinline__ void store_features4(f16 *out, const f16 *residual, int epilogue, size_t tok, int ld, int col,
                                                float v0, float v1, float v2, float v3)
{
    if (epilogue == TUNA_EPILOGUE_SILU_MUL) {
        const f16x2 h = {(f16)silu_mul(v0, v1), (f16)silu_mul(v2, v3)};
        *reinterpret_cast<f16x2 *>(out + tok * (size_t)(ld >> 1) + (col >> 1)) = h;
        return;
    }
    const size_t at = tok * (size_t)ld + col;
    if (epilogue == TUNA_EPILOGUE_RESIDUAL) {
        const f16x4 r = *reinterpret_cast<const f16x4 *>(residual + at);
        v0 += (float)r[0], v1 += (float)r[1], v2 += (float)r[2], v3 += (float)r[3];
    }
    *reinterpret_cast<f16x4 *>(out + at) = f16x4{(f16)v0, (f16)v1, (f16)v2, (f16)v3};
}

}  // namespace tuna
