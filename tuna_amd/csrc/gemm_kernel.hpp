// FP16-activation x 4-bit-codebook-weight GEMM for gfx950 (CDNA4, wave64).
//
//   out[n, m] = x[n, k] . W[m, k]^T,   W[r, c] = fp16(code[nib(r, c)]) *fp16 fp16(absmax[r])
//
// Replaces the reference's Tuna<...> kernel (kernel.cu:2850-2960) and its
// Deq4GemmIterator (kernel.cu:1043-2505); nothing of their structure is kept.
//
// Mapping to the machine
//   * MFMA v_mfma_f32_16x16x32_f16 with the WEIGHTS as the A operand (16 rows x 32 k)
//     and the activations as B (32 k x 16 tokens).  Lane l = (i = l % 16, g = l / 16)
//     supplies, for A, one weight row and 8 consecutive k: exactly one dword of the
//     packed layout (row mb*8 + r of block (mb, kb) is dword r of the 32-byte record).
//   * One global_load_dwordx4 per lane fetches 4 consecutive rows of one 8x8 block, so
//     the 4 dwords feed 4 MFMAs that share the B fragment.  Lane (i, g) reads block row
//     i/2, half i%2 of block column kb0 + g: a wave instruction covers 64 rows x 32 k as
//     8 fully used 128-byte segments.  MFMA #j, row index i is weight row 4*i + j of the
//     wave's 64: the row permutation is undone for free when the accumulators are stored
//     (a lane ends up owning 16 consecutive output features of one token).
//   * Packed weights are used exactly once, so they go global -> registers through a
//     ring of `U` k-steps per wave (nontemporal loads); there is nothing to share in LDS.
//   * Activations are re-used by every wave: the workgroup stages its k-slice of x in
//     LDS in chunks and each wave reads its B fragments with ds_read_b128.
//   * Decode: the codebook is a run-time input, so it is a table.  LDS holds, for every
//     byte value, the half2 {code[hi nibble], code[lo nibble]} replicated once per lane
//     (row stride 256 B).  A lane's address is (byte << 8) | (lane << 2), built by one
//     v_perm_b32, and lands in the lane's own bank column: no bank conflicts for any
//     data.  One v_pk_mul_f16 applies the row's fp16 scale - the same single fp16
//     rounding as the reference's `smemCode.get(nib) * absMax` (kernel.cu:2178-2192).
//     Cost: 1 perm + 1 ds_read_b32 + 1 pk_mul per two weights.
//   * Split-K: waves_k waves of a workgroup cover interleaved k-steps and are summed in
//     LDS in a fixed order; split_k workgroups write fp32 partials to a workspace and the
//     last one to arrive (device-scope counter) sums them in split order and stores fp16.
//     No atomics on the output (unlike kernel.cu:2739-2745), no pre-zeroing, and the
//     result does not depend on arrival order.
#pragma once
#include "tuna_internal.h"

namespace tuna {

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint32_t lds_u32;

__device__ __forceinline__ uint32_t f16_bits(f16 h)
{
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

// Decode one packed dword (one weight row, 8 consecutive k) into the MFMA A operand.
template <int DEC>
__device__ __forceinline__ f16x8 decode_dword(uint32_t d, const unsigned char *lut, uint32_t lane4,
                                              f16x2 sc16, float sc32)
{
    if constexpr (DEC == TUNA_DECODE_GEMM) {
        // address = (byte_n << 8) | (lane << 2): byte 0 from lane4, byte 1 from d, rest zero
        const uint32_t a0 = __builtin_amdgcn_perm(d, lane4, 0x0c0c0400u);
        const uint32_t a1 = __builtin_amdgcn_perm(d, lane4, 0x0c0c0500u);
        const uint32_t a2 = __builtin_amdgcn_perm(d, lane4, 0x0c0c0600u);
        const uint32_t a3 = __builtin_amdgcn_perm(d, lane4, 0x0c0c0700u);
        // The table starts at LDS address 0 (the kernel has no static LDS), so the
        // permuted value IS the LDS address: no base add per lookup.
        const uint32_t t0 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a0);
        const uint32_t t1 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a1);
        const uint32_t t2 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a2);
        const uint32_t t3 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a3);
        const f16x2 h0 = __builtin_bit_cast(f16x2, t0) * sc16;
        const f16x2 h1 = __builtin_bit_cast(f16x2, t1) * sc16;
        const f16x2 h2 = __builtin_bit_cast(f16x2, t2) * sc16;
        const f16x2 h3 = __builtin_bit_cast(f16x2, t3) * sc16;
        f16x8 r;
        r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];
        r[4] = h2[0]; r[5] = h2[1]; r[6] = h3[0]; r[7] = h3[1];
        return r;
    } else {
        // fp32 multiply then round (kernel.cu:3222-3228); lut holds the 16 fp32 codes
        const float *cf = reinterpret_cast<const float *>(lut);
        f16x8 r;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t nib = (d >> (8 * (e >> 1) + 4 * (1 - (e & 1)))) & 15u;
            r[e] = (f16)(cf[nib] * sc32);
        }
        return r;
    }
}

template <int RW, int U, int TT, int DEC, int MAXT>
__global__ __launch_bounds__(MAXT) void gemm_kernel(const GemmArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int NACC = RW * 4 * TT;
    constexpr int LUT_B = (DEC == TUNA_DECODE_GEMM) ? kLutBytes : 64;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave % a.waves_k;
    const int wm = wave / a.waves_k;
    const int i16 = lane & 15;
    const int g = lane >> 4;

    int id = blockIdx.x;
    if (a.xcd_swizzle) {
        const int total = gridDim.x;
        if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    }
    const int row_tile = id / a.split_k;
    const int ks = id - row_tile * a.split_k;
    const int tok0 = blockIdx.y * (TT * 16);
    const int row0 = (row_tile * a.waves_m + wm) * (RW * kRowsPerLoad);

    const int sb = ks * a.steps_per_split;
    const int se = min(a.steps_total, sb + a.steps_per_split);
    const int nsteps = max(se - sb, 0);
    const int n_it = nsteps > wk ? (nsteps - wk + a.waves_k - 1) / a.waves_k : 0;

    // ---- packed-weight stream: per-lane base pointers and the prefetch ring ----------
    const int kb_total = a.k >> 3;
    const int mb_last = (a.m >> 3) - 1;
    const unsigned char *wp[RW];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        const int mb = min(((row0 + rw * kRowsPerLoad) >> 3) + (i16 >> 1), mb_last);
        wp[rw] = a.q + ((size_t)mb * (size_t)kb_total) * 32 + (i16 & 1) * 16;
    }
    // Small operands first, all unconditional, so that every later wait on them can be an
    // exact s_waitcnt vmcnt(N) that leaves the weight prefetches in flight.
    const float code_lane = a.code[lane & 15];
    float sc32[RW][4];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = row0 + rw * kRowsPerLoad + i16 * 4 + j;
            sc32[rw][j] = a.absmax[min(row, a.m - 1)];  // rows past m are never stored
        }

    u32x4 wq[U][RW];
    const int kstride = a.waves_k * 4;  // block columns between this wave's consecutive steps
    const int kb_first = (sb + wk) * 4 + g;
    // Unconditional by design: a load whose step lies beyond this wave's share is clamped
    // to a valid block column and its data is never used.  Only loads that are always
    // issued let the compiler count outstanding loads exactly (s_waitcnt vmcnt(N > 0)).
#define TUNA_LOAD_STEP(u, it)                                                                  \
    {                                                                                          \
        const int kb_ = min(kb_first + (it) * kstride, kb_total - 1);                          \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) wq[u][rw] =                          \
            __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wp[rw] + (size_t)kb_ * 32)); \
    }
#pragma unroll
    for (int u = 0; u < U; ++u) TUNA_LOAD_STEP(u, u)

    // ---- per-row scales (fp16 like the reference's staging, kernel.cu:2770) -----------
    f16x2 sc16[RW][4];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f16 h = (f16)sc32[rw][j];
            sc16[rw][j] = f16x2{h, h};
        }

    // ---- decode table -------------------------------------------------------------------
    unsigned char *lut = smem;
    if constexpr (DEC == TUNA_DECODE_GEMM) {
        // Lane l holds fp16(code[l % 16]) (kernel.cu:2800 rounds the codebook to fp16);
        // entries are gathered across lanes, no memory traffic.
        // piece p: 16 bytes of row (p >> 4); all 64 slots of a row hold the same half2
        const int code_bits = (int)f16_bits((f16)code_lane);
        for (int p = tid; p < kLutBytes / 16; p += blockDim.x) {
            const int e = p >> 4;
            const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
            const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
            const uint32_t v = hi | (lo << 16);
            reinterpret_cast<u32x4 *>(lut)[p] = u32x4{v, v, v, v};
        }
    } else {
        if (tid < 16) reinterpret_cast<float *>(lut)[tid] = code_lane;
    }
    const uint32_t lane4 = (uint32_t)lane << 2;

    // ---- x staging ----------------------------------------------------------------------
    unsigned char *xs = smem + LUT_B;
    const int xs_stride = a.chunk_steps * 64 + 16;  // bytes per token row (+16: bank skew)
    const f16 *xg = reinterpret_cast<const f16 *>(a.x);

    f32x4 acc[RW][4][TT];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // One k-step of this wave: B fragments from LDS, decode 4*RW dwords, 4*RW*TT MFMAs.
#define TUNA_CONSUME(u, xoff)                                                                   \
    {                                                                                          \
        f16x8 b_[TT];                                                                          \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) b_[tt] =                             \
            *reinterpret_cast<const f16x8 *>(xb + tt * 16 * xs_stride + (xoff));               \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) _Pragma("unroll") for (int j = 0; j < 4; ++j) \
        {                                                                                      \
            const f16x8 av_ = decode_dword<DEC>(wq[u][rw][j], lut, lane4, sc16[rw][j], sc32[rw][j]); \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] =                 \
                __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_[tt], acc[rw][j][tt], 0, 0, 0);  \
        }                                                                                      \
    }

    const int ipc = a.chunk_steps / a.waves_k;  // iterations per chunk per wave (multiple of U)
    const int n_chunks = (nsteps + a.chunk_steps - 1) / a.chunk_steps;
    const int wstep = a.waves_k * 64;           // LDS bytes between this wave's consecutive steps
    int it = 0;                                 // this wave's next iteration (multiple of U)
    for (int c = 0; c < n_chunks; ++c) {
        if (c) __syncthreads();
        {
            const int kbase = (sb + c * a.chunk_steps) * kStepK;
            const int xc8 = a.chunk_steps * 4;  // 16-byte pieces per token row
            for (int r = wave; r < TT * 16; r += (int)(blockDim.x >> 6)) {
                const int tok = tok0 + r;
                for (int c8 = lane; c8 < xc8; c8 += 64) {
                    const int kk = kbase + c8 * 8;
                    u32x4 v = u32x4{0u, 0u, 0u, 0u};
                    if (tok < a.n && kk < a.k)
                        v = *reinterpret_cast<const u32x4 *>(xg + (size_t)tok * a.k + kk);
                    *reinterpret_cast<u32x4 *>(xs + r * xs_stride + c8 * 16) = v;
                }
            }
        }
        __syncthreads();
        const int it_chunk0 = c * ipc;
        const int it_end = min(it_chunk0 + ipc, n_it);
        const unsigned char *xb = xs + i16 * xs_stride + g * 16 + wk * 64 - it_chunk0 * wstep;
        // steady state: every slot is consumed and refilled, no branches inside the group
        while (it + U <= it_end && it + 2 * U <= n_it) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                TUNA_CONSUME(u, (it + u) * wstep)
                TUNA_LOAD_STEP(u, it + u + U)
                // keep the refill right behind its consume: the scheduler would otherwise
                // sink all U loads to the end of the group and empty the ring every group
                __builtin_amdgcn_sched_barrier(0);
            }
            it += U;
        }
        if (it + U <= it_end && it + U == n_it) {
            // last full group of the wave: drain the ring, nothing left to fetch
#pragma unroll
            for (int u = 0; u < U; ++u) TUNA_CONSUME(u, (it + u) * wstep)
            it += U;
        } else {
            // ragged tail (fewer than U steps left in the wave or in the chunk)
            while (it < it_end) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (it + u < it_end) {
                        TUNA_CONSUME(u, (it + u) * wstep)
                        if (it + u + U < n_it) TUNA_LOAD_STEP(u, it + u + U)
                    }
                }
                it += U;
            }
        }
    }
#undef TUNA_CONSUME
#undef TUNA_LOAD_STEP

    // ---- reduce the waves_k partial sums of the workgroup in LDS, fixed order ---------
    f32x4 *red = reinterpret_cast<f32x4 *>(smem);
    if (a.waves_k > 1) {
        __syncthreads();  // table and x are dead from here on
        if (wk > 0) {
            f32x4 *dst = red + ((size_t)((wk - 1) * a.waves_m + wm) * NACC) * 64 + lane;
#pragma unroll
            for (int rw = 0; rw < RW; ++rw)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) dst[((rw * 4 + j) * TT + tt) * 64] = acc[rw][j][tt];
        }
        __syncthreads();
        if (wk == 0) {
            for (int w = 1; w < a.waves_k; ++w) {
                const f32x4 *src = red + ((size_t)((w - 1) * a.waves_m + wm) * NACC) * 64 + lane;
#pragma unroll
                for (int rw = 0; rw < RW; ++rw)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] += src[((rw * 4 + j) * TT + tt) * 64];
            }
        }
    }

    // ---- reduce across the split_k workgroups through the workspace --------------------
    // Partials travel as device-scope relaxed atomics (write-through stores, L2-bypassing
    // loads): they are coherent across the 8 XCD L2s without the L2 write-back/invalidate
    // that a device-scope release/acquire fence costs on every workgroup.  Order is given by
    // "all my stores have completed" (workgroup-scope release = s_waitcnt vmcnt(0)) before
    // the barrier that precedes the arrival counter's atomic increment.
    if (a.split_k > 1) {
        const size_t tile = (size_t)blockIdx.y * a.row_tiles + row_tile;
        float *wst = a.ws + (tile * a.split_k * a.waves_m) * (size_t)(NACC * 256);
        if (wk == 0) {
            float *dst = wst + ((size_t)(ks * a.waves_m + wm) * NACC) * 256 + lane;
#pragma unroll
            for (int rw = 0; rw < RW; ++rw)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            __hip_atomic_store(dst + (((rw * 4 + j) * TT + tt) * 4 + v) * 64, acc[rw][j][tt][v],
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        }
        __syncthreads();
        volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(smem + a.lds_bytes - 16);
        if (tid == 0)
            *ticket = __hip_atomic_fetch_add(a.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*ticket != (unsigned)(a.split_k - 1)) return;
        // last workgroup of this tile: every partial is in memory; sum them in split order
        if (tid == 0) __hip_atomic_store(a.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (wk == 0) {
#pragma unroll
            for (int rw = 0; rw < RW; ++rw)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int s = 0; s < a.split_k; ++s) {
                const float *src = wst + ((size_t)(s * a.waves_m + wm) * NACC) * 256 + lane;
#pragma unroll
                for (int rw = 0; rw < RW; ++rw)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                            for (int v = 0; v < 4; ++v)
                                acc[rw][j][tt][v] += __hip_atomic_load(src + (((rw * 4 + j) * TT + tt) * 4 + v) * 64,
                                                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }

    // ---- store: lane (token i16, group g) owns 16 consecutive output features ---------
    if (wk == 0) {
        f16 *outp = reinterpret_cast<f16 *>(a.out);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const int tok = tok0 + tt * 16 + i16;
            if (tok >= a.n) continue;
#pragma unroll
            for (int rw = 0; rw < RW; ++rw) {
                const int rb = row0 + rw * kRowsPerLoad + g * 16;
                f16x8 lo, hi;
#pragma unroll
                for (int v = 0; v < 2; ++v)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        lo[v * 4 + j] = (f16)acc[rw][j][tt][v];
                        hi[v * 4 + j] = (f16)acc[rw][j][tt][v + 2];
                    }
                f16 *dst = outp + (size_t)tok * a.m + rb;
                if (rb + 8 <= a.m) *reinterpret_cast<f16x8 *>(dst) = lo;
                if (rb + 16 <= a.m) *reinterpret_cast<f16x8 *>(dst + 8) = hi;
            }
        }
    }
}

}  // namespace tuna
