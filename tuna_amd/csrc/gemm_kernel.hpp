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
//     LDS in chunks, as 16-byte pieces ordered [8-k slot][token], so that both the staging
//     writes and the ds_read_b128 of a B fragment (16 lanes = 16 tokens of one slot = 256
//     contiguous bytes) are bank-conflict free without padding.
//   * Decode: the codebook is a run-time input, so it is a table.  LDS holds, for every
//     byte value, the half2 {code[hi nibble], code[lo nibble]} replicated once per lane
//     (row stride 256 B).  A lane's address is (byte << 8) | (lane << 2), built by one
//     v_perm_b32, and lands in the lane's own bank column: no bank conflicts for any
//     data.  One v_pk_mul_f16 applies the row's fp16 scale - the same single fp16
//     rounding as the reference's `smemCode.get(nib) * absMax` (kernel.cu:2178-2192).
//     Cost: 1 perm + 1 ds_read_b32 + 1 pk_mul per two weights.
//   * Split-K: waves_k waves of a workgroup cover interleaved k-steps; their accumulators
//     meet in LDS and every thread sums a 1/waves_k share in wave order.  split_k
//     workgroups write those fp32 sums to a workspace and the last one to arrive
//     (device-scope counter) adds them in split order.  The fp16 result is transposed
//     through LDS and stored with 16-byte, fully coalesced writes.  No atomics on the
//     output (unlike kernel.cu:2739-2745), no pre-zeroing, and the result does not depend
//     on arrival order.
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
#if defined(TUNA_ABLATE) && TUNA_ABLATE == 1  /* development only: no table reads */
        const uint32_t t0 = a0, t1 = a1, t2 = a2, t3 = a3;
#else
        const uint32_t t0 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a0);
        const uint32_t t1 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a1);
        const uint32_t t2 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a2);
        const uint32_t t3 = *reinterpret_cast<const lds_u32 *>((uintptr_t)a3);
#endif
#if defined(TUNA_ABLATE) && TUNA_ABLATE == 2  /* development only: no scale multiply */
        const f16x2 h0 = __builtin_bit_cast(f16x2, t0), h1 = __builtin_bit_cast(f16x2, t1);
        const f16x2 h2 = __builtin_bit_cast(f16x2, t2), h3 = __builtin_bit_cast(f16x2, t3);
#else
        const f16x2 h0 = __builtin_bit_cast(f16x2, t0) * sc16;
        const f16x2 h1 = __builtin_bit_cast(f16x2, t1) * sc16;
        const f16x2 h2 = __builtin_bit_cast(f16x2, t2) * sc16;
        const f16x2 h3 = __builtin_bit_cast(f16x2, t3) * sc16;
#endif
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

// x staging, global -> registers -> LDS, in batches of kXBatch 16-byte pieces per thread.
// Piece p of a chunk is token row (p % (16*TT)), 8-k slot (p / (16*TT)) and lives at LDS
// byte 16*p.  All loads of a batch are issued before the first LDS write (addresses are
// clamped so the loads are unconditional; invalid pieces are zeroed by a select).
constexpr int kXBatch = 4;

struct XStage {
    u32x4 v[kXBatch];
};

template <int TT>
__device__ __forceinline__ void x_stage_load(XStage &st, const f16 *xg, int base, int nthreads, int tid, int pieces,
                                             int tok0, int kbase, int n, int k)
{
#pragma unroll
    for (int b = 0; b < kXBatch; ++b) {
        const int p = min(base + b * nthreads + tid, pieces - 1);
        const int r = p & (16 * TT - 1);
        const int c8 = p / (16 * TT);
        const int tok = min(tok0 + r, n - 1);
        const int kk = min(kbase + c8 * 8, k - 8);
        st.v[b] = *reinterpret_cast<const u32x4 *>(xg + (size_t)tok * k + kk);
    }
}

template <int TT>
__device__ __forceinline__ void x_stage_store(const XStage &st, unsigned char *xs, int base, int nthreads, int tid,
                                              int pieces, int tok0, int kbase, int n, int k)
{
#pragma unroll
    for (int b = 0; b < kXBatch; ++b) {
        const int p = base + b * nthreads + tid;
        if (p < pieces) {
            const int r = p & (16 * TT - 1);
            const int c8 = p / (16 * TT);
            const bool ok = (tok0 + r < n) && (kbase + c8 * 8 < k);
            *reinterpret_cast<u32x4 *>(xs + (size_t)p * 16) = ok ? st.v[b] : u32x4{0u, 0u, 0u, 0u};
        }
    }
}

template <int RW, int U, int TT, int DEC, int MAXT, int MINW>
__global__ __launch_bounds__(MAXT, MINW) void gemm_kernel(const GemmArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int NACC = RW * 4 * TT;  // float4 accumulator planes per lane
    constexpr int LUT_B = (DEC == TUNA_DECODE_GEMM) ? kLutBytes : 64;

    const int tid = threadIdx.x;
#ifdef TUNA_TRACE
#define TUNA_MARK(i) if (a.trace && tid == 0) a.trace[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + (i)] = wall_clock64();
#else
#define TUNA_MARK(i)
#endif
    TUNA_MARK(0)
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave & (a.waves_k - 1);
    const int wm = wave >> a.wk_log2;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int nthreads = (int)blockDim.x;

    int id = blockIdx.x;
    if (a.xcd_swizzle) {
        const int total = gridDim.x;
        if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    }
    const int row_tile = id / a.split_k;
    const int ks = id - row_tile * a.split_k;
    const int tok0 = blockIdx.y * (TT * 16);
    const int rows_wg = a.waves_m * (RW * kRowsPerLoad);
    const int row0 = row_tile * rows_wg + wm * (RW * kRowsPerLoad);  // first weight row of this wave

    const int sb = ks * a.steps_per_split;
    const int se = min(a.steps_total, sb + a.steps_per_split);
    const int nsteps = max(se - sb, 0);
    const int n_it = nsteps > wk ? (nsteps - wk + a.waves_k - 1) >> a.wk_log2 : 0;

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

    // ---- packed-weight stream ------------------------------------------------------------
    // address = q + [uniform: 128 bytes per k-step] + [per lane: block row, row half, g]:
    // the uniform part rides in SGPRs, so a load costs no vector ALU work.
    const int kb_total = a.k >> 3;
    const int mb_last = (a.m >> 3) - 1;
    const int g_last = min(g, kb_total - 1 - (a.steps_total - 1) * 4);  // last k-step may be short
    uint32_t lb[RW], lb_last[RW];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) {
        const int mb = min(((row0 + rw * kRowsPerLoad) >> 3) + (i16 >> 1), mb_last);
        const uint32_t rowb = (uint32_t)mb * (uint32_t)kb_total * 32u + (uint32_t)(i16 & 1) * 16u;
        lb[rw] = rowb + (uint32_t)g * 32u;
        lb_last[rw] = rowb + (uint32_t)g_last * 32u;
    }
    u32x4 wq[U][RW];
    const int s_first = sb + wk;            // this wave's first k-step
    const int s_stride = a.waves_k;         // k-steps between its consecutive iterations
    // Unconditional by design: a load whose step lies beyond this wave's share is clamped
    // to the last k-step and its data is never used.  Only loads that are always issued
    // let the compiler count outstanding loads exactly (s_waitcnt vmcnt(N > 0)).
#define TUNA_LOAD_STEP(u, it)                                                                  \
    {                                                                                          \
        const int s_ = min(s_first + (it) * s_stride, a.steps_total - 1);                      \
        const unsigned char *base_ = a.q + (size_t)s_ * 128;                                   \
        const bool last_ = s_ == a.steps_total - 1;                                            \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) wq[u][rw] = __builtin_nontemporal_load( \
            reinterpret_cast<const u32x4 *>(base_ + (last_ ? lb_last[rw] : lb[rw])));          \
    }
#pragma unroll
    for (int u = 0; u < U; ++u) TUNA_LOAD_STEP(u, u)

    // first batch of the first x chunk: in flight while the decode table is built
    const f16 *xg = reinterpret_cast<const f16 *>(a.x);
    const int x_pieces = (TT * 16 * 4) << a.chunk_log2;  // 16-byte pieces per chunk
    XStage xst;
    x_stage_load<TT>(xst, xg, 0, nthreads, tid, x_pieces, tok0, sb * kStepK, a.n, a.k);

    TUNA_MARK(1)
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
#pragma unroll 4
        for (int p = tid; p < kLutBytes / 16; p += nthreads) {
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
    TUNA_MARK(2)

    unsigned char *xs = smem + LUT_B;

    f32x4 acc[RW][4][TT];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

#ifndef TUNA_DWORD_GROUP
#define TUNA_DWORD_GROUP 0
#endif
    // One k-step of this wave: B fragments from LDS, decode 4*RW dwords, 4*RW*TT MFMAs.
#define TUNA_CONSUME(u, xoff)                                                                   \
    {                                                                                          \
        f16x8 b_[TT];                                                                          \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) b_[tt] =                             \
            *reinterpret_cast<const f16x8 *>(xb + tt * 256 + (xoff));                          \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) _Pragma("unroll") for (int j = 0; j < 4; ++j) \
        {                                                                                      \
            const f16x8 av_ = decode_dword<DEC>(wq[u][rw][j], lut, lane4, sc16[rw][j], sc32[rw][j]); \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] =                 \
                __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_[tt], acc[rw][j][tt], 0, 0, 0);  \
            if (TUNA_DWORD_GROUP > 0 && (j % TUNA_DWORD_GROUP) == TUNA_DWORD_GROUP - 1) __builtin_amdgcn_sched_barrier(0); \
        }                                                                                      \
    }

    // One group = U consecutive iterations of this wave: every ring slot is consumed and
    // refilled, no branches inside (refill addresses are clamped, see TUNA_LOAD_STEP).
#define TUNA_GROUP()                                                                            \
    {                                                                                          \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                          \
        {                                                                                      \
            TUNA_CONSUME(u, (it + u) * wstep)                                                  \
            TUNA_LOAD_STEP(u, it + u + U)                                                      \
            /* keep the refill right behind its consume: the scheduler would otherwise sink */ \
            /* all U loads to the end of the group and empty the ring every group */           \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        it += U;                                                                               \
    }

    const int ipc = a.chunk_steps >> a.wk_log2;  // iterations per chunk per wave (multiple of U)
    const int n_chunks = (nsteps + a.chunk_steps - 1) >> a.chunk_log2;
    const int wstep = a.waves_k * (1024 * TT);   // LDS bytes between this wave's consecutive steps
    int it = 0;                                  // this wave's next iteration (multiple of U)

    // chunk 0 of x: loaded above, written here
    if (n_chunks > 0) x_stage_store<TT>(xst, xs, 0, nthreads, tid, x_pieces, tok0, sb * kStepK, a.n, a.k);
    __syncthreads();
    TUNA_MARK(3)

    for (int c = 0; c < n_chunks; ++c) {
        const int it_chunk0 = c * ipc;
        const bool has_next = c + 1 < n_chunks;
        // B fragment of lane (token i16, k-group g), local step sl: slot sl*4+g, piece slot*16*TT + i16
        const unsigned char *xb = xs + g * (256 * TT) + i16 * 16 + wk * (1024 * TT) - it_chunk0 * wstep;
        if (has_next) {
            // A chunk with a successor is full: every wave owns all ipc iterations of it.
            const int it_peel = it_chunk0 + ipc - U;
            while (it < it_peel) TUNA_GROUP()
            // Last group of the chunk: the next chunk of x is fetched into registers first, so
            // that after the group exactly U*RW younger loads are in flight and the wait before
            // the LDS write below is an exact vmcnt, not a drain of the weight ring.
            const int kbase = (sb + (c + 1) * a.chunk_steps) * kStepK;
            x_stage_load<TT>(xst, xg, 0, nthreads, tid, x_pieces, tok0, kbase, a.n, a.k);
            TUNA_GROUP()
            __syncthreads();  // every wave is done reading chunk c
            x_stage_store<TT>(xst, xs, 0, nthreads, tid, x_pieces, tok0, kbase, a.n, a.k);
            __syncthreads();
        } else {
            const int it_end = min(it_chunk0 + ipc, n_it);
            // steady state while both the group and its refills lie inside this wave's share
            while (it + U <= it_end && it + 2 * U <= n_it) TUNA_GROUP()
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
    }
#undef TUNA_GROUP
#undef TUNA_CONSUME
#undef TUNA_LOAD_STEP
    TUNA_MARK(4)

    // ---- workgroup reduction: accumulators meet in LDS, every thread sums a share ------
    // A wave's accumulators are the float array [plane][lane][4] (NACC*256 floats); thread
    // (wk, lane) of row group wm owns floats f = (i*waves_k + wk)*64 + lane, i < nf.
    __syncthreads();  // table and x are dead from here on
    {
        f32x4 *dst = reinterpret_cast<f32x4 *>(smem) + (size_t)(wm * a.waves_k + wk) * (NACC * 64) + lane;
#pragma unroll
        for (int rw = 0; rw < RW; ++rw)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) dst[((rw * 4 + j) * TT + tt) * 64] = acc[rw][j][tt];
    }
    __syncthreads();
    TUNA_MARK(5)
    const float *redf = reinterpret_cast<const float *>(smem) + (size_t)wm * a.waves_k * (NACC * 256);
    const int nf = (NACC * 4) >> a.wk_log2;
    f16 *tile = reinterpret_cast<f16 *>(smem + a.red_bytes);  // [token][rows_wg + 8] fp16
    const int tile_ld = rows_wg + 8;
    // float f = (plane*64 + l)*4 + v is token (plane % TT)*16 + l%16, weight row
    // (plane / (4*TT))*64 + 16*(l/16) + 4*v + (plane / TT) % 4 of the wave
#define TUNA_TILE_PUT(f, val)                                                                   \
    {                                                                                          \
        const int pl_ = (f) >> 8, l_ = ((f) >> 2) & 63, v_ = (f) & 3;                          \
        const int tok_ = (pl_ % TT) * 16 + (l_ & 15);                                          \
        const int row_ = wm * (RW * kRowsPerLoad) + (pl_ / (4 * TT)) * 64 + (l_ >> 4) * 16 + v_ * 4 + (pl_ / TT) % 4; \
        tile[tok_ * tile_ld + row_] = (f16)(val);                                              \
    }

    if (a.split_k == 1) {
        for (int i = 0; i < nf; ++i) {
            const int f = ((i << a.wk_log2) + wk) * 64 + lane;
            float s = 0.f;
            for (int w = 0; w < a.waves_k; ++w) s += redf[(size_t)w * (NACC * 256) + f];
            TUNA_TILE_PUT(f, s)
        }
    } else {
        // Partials travel as device-scope relaxed atomics (write-through stores, L2-bypassing
        // loads): coherent across the 8 XCD L2s without the L2 write-back/invalidate that a
        // device-scope release/acquire fence costs on every workgroup.  Order is given by
        // "all my stores have completed" (workgroup-scope release = s_waitcnt vmcnt(0))
        // before the barrier that precedes the arrival counter's increment.
        const size_t tile_id = (size_t)blockIdx.y * a.row_tiles + row_tile;
        float *wst = a.ws + (tile_id * a.split_k * a.waves_m) * (size_t)(NACC * 256);
        float *mine = wst + ((size_t)ks * a.waves_m + wm) * (NACC * 256);
        for (int i = 0; i < nf; ++i) {
            const int f = ((i << a.wk_log2) + wk) * 64 + lane;
            float s = 0.f;
            for (int w = 0; w < a.waves_k; ++w) s += redf[(size_t)w * (NACC * 256) + f];
            __hip_atomic_store(mine + f, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        TUNA_MARK(6)
        volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(smem + a.lds_bytes - 16);
        if (tid == 0)
            *ticket = __hip_atomic_fetch_add(a.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        TUNA_MARK(7)
        if (*ticket != (unsigned)(a.split_k - 1)) return;
        // last workgroup of this tile: every partial is in memory; add them in split order
        if (tid == 0) __hip_atomic_store(a.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int i = 0; i < nf; ++i) {
            const int f = ((i << a.wk_log2) + wk) * 64 + lane;
            const float *src = wst + (size_t)wm * (NACC * 256) + f;
            float s = 0.f;
            for (int sp = 0; sp < a.split_k; ++sp)
                s += __hip_atomic_load(src + (size_t)sp * a.waves_m * (NACC * 256), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            TUNA_TILE_PUT(f, s)
        }
    }
#undef TUNA_TILE_PUT
    __syncthreads();
    TUNA_MARK(8)

    // ---- store the [tokens][rows_wg] fp16 tile: 16 bytes per thread, rows contiguous ---
    {
        f16 *outp = reinterpret_cast<f16 *>(a.out);
        constexpr int RW_LOG2 = RW == 1 ? 0 : (RW == 2 ? 1 : 2);
        const int r8_log2 = a.wm_log2 + RW_LOG2 + 3;  // log2(rows_wg / 8)
        const int pieces = (TT * 16) << r8_log2;
        for (int p = tid; p < pieces; p += nthreads) {
            const int tok = p >> r8_log2;
            const int r8 = p & ((1 << r8_log2) - 1);
            const int row = row_tile * rows_wg + r8 * 8;
            if (tok0 + tok < a.n && row + 8 <= a.m)
                *reinterpret_cast<u32x4 *>(outp + (size_t)(tok0 + tok) * a.m + row) =
                    *reinterpret_cast<const u32x4 *>(tile + tok * tile_ld + r8 * 8);
        }
    }
    TUNA_MARK(9)
#undef TUNA_MARK
}

}  // namespace tuna
