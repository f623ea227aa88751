// Narrow-row GEMM kernel for the smallest launches (gfx950, wave64): 16, 32 or 64 weight rows per
// workgroup, all waves of the workgroup along k, no split across workgroups.
//
// With 64 rows per wave a 4096..8192-row projection has only 64..128 row groups, so filling
// 256 CUs takes a split of k across workgroups, and its hand-over (partial sums through
// memory, an arrival counter, a finishing pass) costs three dependent round trips: 2 us of an
// 8 us launch.  Here a workgroup owns 16*LW rows (LW = 1, 2, 4): 256..512 workgroups from the
// rows alone, the k range is divided over the WK waves of the workgroup, and the only
// reduction is the one through LDS.
//   * MFMA v_mfma_f32_16x16x32_f16 as in gemm_kernel.hpp (weights = A, activations = B).  Lane
//     (i = lane % 16, g = lane / 16) loads LW consecutive dwords of one 8x8 block: weight rows
//     LW*i + j, j < LW, of the workgroup's 16*LW, block column 4*step + g.  A wave instruction
//     covers 2*LW block rows x 128 contiguous bytes.
//   * Every wave has its own k range, so nothing of x is shared inside the workgroup: B fragments
//     come straight from global memory (L2 hits: x is 128 KB per 16 tokens and read by everyone),
//     one 16-byte load per lane and k-step, loaded contiguously and moved to the lane that needs
//     them by cross-lane reads; no staging, no barrier before the main loop.  Token rows past n
//     are clamped, not zeroed: a B column only feeds its own output column, which is never stored.
//   * Weights and B fragments travel through one ring of U k-steps per wave.
//   * Decode table and decode as in gemm_kernel.hpp (bit-identical weights).
//   * Reduction: the WK waves put their LW accumulator planes in LDS; each thread sums two
//     adjacent output features of one token in wave order and stores them (fused epilogues of
//     epilogue.hpp).  Deterministic; no workspace, no counters.
//   * BLK variants: one scale per block of 64 << blk_shift consecutive weights of a row, absmax
//     [m, k / block] (the layout the reference's quantizer writes for block_size < k, test.py:15-17).
//     A wave's double step of 64 k lies inside one block; the scales of a ring slot's block travel
//     through the ring with its weights and are rounded to fp16 when the slot is consumed - the
//     decode is fp16(code) * fp16(absmax of the block), the GEMM's rounding with a finer scale.
//     The workgroup's scales ([rows][k / block], contiguous in memory) are copied into LDS once at
//     the start (a_slds; rows one float apart from a multiple of the bank count) and read from
//     there when a ring slot is refilled: a wave's scale load from global memory touches sixteen
//     cache lines for sixteen values, as much address work as sixteen weight loads.  Without
//     a_slds (slices that do not fit beside table and reduction planes) they come from memory.
// Requires k % (32*WK*U) == 0, m % (16*LW) == 0, dense launches; a workgroup takes 16*TT tokens
// (TT = token_tiles = 1, 2, 4: every decoded weight fragment feeds TT MFMAs), more tokens are
// gridDim.y chunks.  Selected by rows_per_wave = 16 or 32 in the config,
// or by rows_per_wave = 64 with waves_m = 0.
#pragma once
#include "gemm_kernel.hpp"

namespace tuna {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// The arguments are separate scalars, the ones the first loads need in front: the first 16
// dwords of a kernel's arguments can be preloaded into scalar registers with the wave (built
// with -amdgpu-kernarg-preload-count=16), which takes the argument fetch - a round trip to
// memory - off the start of every wave.  A struct passed by value is not preloaded.
template <int LW, int WK, int U, bool PERM, int TT, bool BLK = false, int ROWS = 16 * LW>
__global__ __launch_bounds__(WK * 64) void gemm_narrow_kernel(const uint8_t *a_q, const void *a_x, const float *a_code,
                                                              const float *a_absmax, int a_k, int a_n, int a_n_it, int a_m,
                                                              void *a_out, int a_epilogue, const void *a_residual,
                                                              int a_blk_shift, int a_nblk, int a_slds)
{
    struct {
        const uint8_t *q;
        const void *x;
        const float *code;
        const float *absmax;
        void *out;
        const void *residual;
        int epilogue, m, n, k, n_it;
    } const a = {a_q, a_x, a_code, a_absmax, a_out, a_residual, a_epilogue, a_m, a_n, a_k, a_n_it};
    extern __shared__ __align__(16) unsigned char smem[];
    static_assert(LW == 1 || LW == 2 || LW == 4, "16, 32 or 64 rows per workgroup");
    static_assert(ROWS % 8 == 0 && ROWS % LW == 0 && ROWS <= 16 * LW && ROWS > 8 * LW, "rows of a partly filled tile");
    unsigned char *lut = smem;
    float *red = reinterpret_cast<float *>(smem + kLutBytes);  // [wave][row plane][token tile][lane][4]
    // BLK with a_slds: [row][a_nblk + 1] scales of the workgroup, each rounded to fp16 and stored twice in a dword
    uint32_t *sbuf = reinterpret_cast<uint32_t *>(red + WK * LW * TT * 256);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int wk = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int nthreads = WK * 64;
    const uint32_t lane4 = (uint32_t)lane << 2;
    const int row0 = blockIdx.x * ROWS;
    // ROWS < 16 * LW (24 rows with LW = 2: 6144 rows make 256 workgroups instead of 192): the lanes whose rows lie
    // beyond the tile load the rows of other lanes again - valid addresses, sums nobody stores
    const int ia = ROWS == 16 * LW ? i16 : (i16 < ROWS / LW ? i16 : i16 - ROWS / LW);
    const int tok0 = blockIdx.y * (16 * TT);  // TT tiles of 16 tokens share every decoded weight fragment

    // ---- requests: codebook and scales, then the first ring turn (x fragment, weights) --------
    const float code_lane = a.code[i16];
    float sc32[LW] = {};
    if constexpr (BLK) {
        // (per block: loaded with the ring below)
    } else if constexpr (LW == 1) {
        sc32[0] = a.absmax[row0 + ia];
    } else if constexpr (LW == 2) {
        const f32x2 s2 = *reinterpret_cast<const f32x2 *>(a.absmax + row0 + 2 * ia);
        sc32[0] = s2[0];
        sc32[1] = s2[1];
    } else {
        const f32x4 s4 = *reinterpret_cast<const f32x4 *>(a.absmax + row0 + 4 * ia);
#pragma unroll
        for (int j = 0; j < 4; ++j) sc32[j] = s4[j];
    }
    const uint32_t kb_total = (uint32_t)a.k >> 3;
    // A wave walks k in double steps of 64 (two MFMAs, one 128-byte line of x per token): wave wk
    // owns double steps wk, wk + WK, ...
    // Weights, per lane: block row and dwords of the block, block column 4*step + g.
    const uint32_t lb = ((uint32_t)(row0 >> 3) + (uint32_t)((LW * ia) >> 3)) * kb_total * 32u +
                        (uint32_t)((LW * ia) & 7) * 4u + (uint32_t)g * 32u;
    // B fragments: the MFMA wants lane (token i16, group g) to hold x[token][32*step + 8g ..], i.e.
    // four consecutive lanes on four different token rows - a wave instruction loading it that
    // way touches 16 rows with no two neighbouring lanes on one line and takes about three times
    // as long in the address path as a contiguous one.  PERM: lane l LOADS token l / 4, 8-k group
    // l % 4 (each quad of lanes reads 64 contiguous bytes) and the fragment goes to the lane that
    // needs it by a cross-lane read (ds_bpermute: no LDS memory, no barrier) when it is consumed:
    // lane (i16, g) takes the piece lane 4*i16 + g loaded.  Without PERM every lane loads its own
    // fragment: cheaper for one to four tokens, where the clamped rows coincide anyway.
    uint32_t xoff[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
        xoff[tt] = PERM ? ((uint32_t)min(tt * 16 + (lane >> 2), a.n - 1 - tok0) * (uint32_t)a.k + (uint32_t)(lane & 3) * 8u) * 2u
                        : ((uint32_t)min(tt * 16 + i16, a.n - 1 - tok0) * (uint32_t)a.k + (uint32_t)g * 8u) * 2u;
    const int x_src = (i16 * 4 + g) << 2;  // byte address of the source lane for ds_bpermute
    // uniform: this wave's double step 0; one ring turn (U/2 double steps) further per group
    const unsigned char *qp = a.q + (size_t)wk * 256;
    const unsigned char *xp = reinterpret_cast<const unsigned char *>(a.x) + (size_t)tok0 * a.k * 2 + (size_t)wk * 128;
    uint32_t wq[U][LW];
    u32x4 xq[U][TT];
    uint32_t sq[BLK ? U : 1][LW];  // BLK: the scales of the ring slot's block, rounded to fp16, twice in a dword
    const auto pack_scale = [](float s_) {
        const uint32_t h_ = (uint32_t)f16_bits((f16)s_);
        return h_ | (h_ << 16);
    };
    // BLK: lane's first scale, and the double step of ring slot 0 in the turn being loaded
    const float *sp = a.absmax + (size_t)(row0 + LW * ia) * (size_t)(BLK ? a_nblk : 1);
    int dstep = wk;
    static_assert(U % 2 == 0, "whole double steps");
#define TUNA_NARROW_LOAD(u)                                                                     \
    {                                                                                          \
        const size_t xo_ = (size_t)((u) >> 1) * (WK * 128) + ((u) & 1) * 64;               \
        const size_t qo_ = (size_t)((u) >> 1) * (WK * 256) + ((u) & 1) * 128;              \
        if constexpr (BLK) {                                                                   \
            const int blk_ = (dstep + ((u) >> 1) * WK) >> a_blk_shift;                         \
            if (a_slds) {                                                                      \
                /* (the two slots of a double step lie in one block: the second copies the first) */ \
                if (dstep != wk) {                                                             \
                    _Pragma("unroll") for (int j = 0; j < LW; ++j) sq[u][j] =                  \
                        ((u) & 1) ? sq[(u) & ~1][j] : sbuf[(LW * ia + j) * (a_nblk + 1) + blk_]; \
                }                                                                              \
            } else {                                                                           \
                _Pragma("unroll") for (int j = 0; j < LW; ++j) sq[u][j] = pack_scale(sp[(size_t)j * a_nblk + blk_]); \
            }                                                                                  \
        }                                                                                      \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) xq[u][tt] = *reinterpret_cast<const u32x4 *>(xp + xo_ + xoff[tt]); \
        if constexpr (LW == 1) {                                                               \
            wq[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(qp + qo_ + lb)); \
        } else if constexpr (LW == 2) {                                                        \
            const u32x2 w2_ = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(qp + qo_ + lb)); \
            wq[u][0] = w2_[0];                                                                 \
            wq[u][1] = w2_[1];                                                                 \
        } else {                                                                               \
            const u32x4 w4_ = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qp + qo_ + lb)); \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) wq[u][j] = w4_[j];                   \
        }                                                                                      \
    }
#pragma unroll
    for (int u = 0; u < U; ++u) TUNA_NARROW_LOAD(u)
    qp += (size_t)(U / 2) * (WK * 256);
    xp += (size_t)(U / 2) * (WK * 128);
    dstep += (U / 2) * WK;
    // BLK, scales through LDS: the first eight scales per thread of the workgroup's slice are requested here and
    // stored behind the table build; longer slices follow in further rounds
    constexpr int SB = 8;
    float sv[BLK ? SB : 1];
    const int s_count = BLK ? ROWS * a_nblk : 0;
    const float *s_src = a.absmax + (size_t)row0 * (size_t)(BLK ? a_nblk : 1);
    if constexpr (BLK) {
        if (a_slds) {
#pragma unroll
            for (int i = 0; i < SB; ++i) sv[i] = s_src[min(tid + i * nthreads, s_count - 1)];
        }
    }

    // ---- decode table (see gemm_kernel.hpp), built while the loads are in flight ------------
    {
        const int code_bits = (int)f16_bits((f16)code_lane);
        for (int p0 = tid; p0 < kLutBytes / 16; p0 += 4 * nthreads) {
            uint32_t v[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int e = (p0 + b * nthreads) >> 4;
                const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
                const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
                v[b] = hi | (lo << 16);
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int p = p0 + b * nthreads;
                if (p < kLutBytes / 16) reinterpret_cast<u32x4 *>(lut)[p] = u32x4{v[b], v[b], v[b], v[b]};
            }
        }
    }
    f16x2 sc16[LW];
#pragma unroll
    for (int j = 0; j < LW; ++j) {
        const f16 h = (f16)sc32[j];
        sc16[j] = f16x2{h, h};
    }
    if constexpr (BLK) {
        if (a_slds) {
            const int pitch = a_nblk + 1;
            for (int base = 0; base < s_count; base += SB * nthreads) {
                if (base) {
#pragma unroll
                    for (int i = 0; i < SB; ++i) sv[i] = s_src[min(base + tid + i * nthreads, s_count - 1)];
                }
#pragma unroll
                for (int i = 0; i < SB; ++i) {
                    const int idx = base + tid + i * nthreads;
                    const int r = idx / a_nblk;
                    if (idx < s_count) sbuf[r * pitch + (idx - r * a_nblk)] = pack_scale(sv[i]);
                }
            }
        }
    }
    __syncthreads();  // the table (and the scales) are complete
    if constexpr (BLK) {
        if (a_slds) {
            // the first ring turn's scales (its weights were requested before the scales were in LDS)
            const uint32_t *sl = sbuf + LW * ia * (a_nblk + 1);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int blk_ = (wk + (u >> 1) * WK) >> a_blk_shift;
#pragma unroll
                for (int j = 0; j < LW; ++j) sq[u][j] = sl[j * (a_nblk + 1) + blk_];
            }
        }
    }

    // ---- main loop: n_it / U ring turns, the last one without refills ------------------------
    f32x4 acc[LW][TT];
#pragma unroll
    for (int j = 0; j < LW; ++j)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#define TUNA_NARROW_CONSUME(u)                                                                  \
    {                                                                                          \
        f16x8 b_[TT];                                                                          \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt)                                      \
        {                                                                                      \
            u32x4 xb_ = xq[u][tt];                                                             \
            if constexpr (PERM) {                                                              \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) xb_[e] = (uint32_t)__builtin_amdgcn_ds_bpermute(x_src, (int)xq[u][tt][e]); \
            }                                                                                  \
            b_[tt] = __builtin_bit_cast(f16x8, xb_);                                           \
        }                                                                                      \
        _Pragma("unroll") for (int j = 0; j < LW; ++j)                                         \
        {                                                                                      \
            f16x2 s_ = sc16[j];                                                                \
            if constexpr (BLK) s_ = __builtin_bit_cast(f16x2, sq[u][j]);                       \
            const f16x8 av_ = decode_dword<TUNA_DECODE_GEMM>(wq[u][j], lut, lane4, s_, 0.f);   \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) acc[j][tt] =                     \
                __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_[tt], acc[j][tt], 0, 0, 0);      \
        }                                                                                      \
    }
    for (int it = U; it < a.n_it; it += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            TUNA_NARROW_CONSUME(u)
            TUNA_NARROW_LOAD(u)
            __builtin_amdgcn_sched_barrier(0);  // keep each refill right behind its consume
        }
        qp += (size_t)(U / 2) * (WK * 256);
        xp += (size_t)(U / 2) * (WK * 128);
        dstep += (U / 2) * WK;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) TUNA_NARROW_CONSUME(u)
#undef TUNA_NARROW_CONSUME
#undef TUNA_NARROW_LOAD

    // ---- reduction over the waves and store -----------------------------------------------------
    // Plane (j, tt) of a wave: lane l, element v is token 16*tt + l % 16, MFMA row 4*(l/16) + v,
    // weight row LW*(MFMA row) + j of the workgroup's 16*LW.
#pragma unroll
    for (int j = 0; j < LW; ++j)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
            reinterpret_cast<f32x4 *>(red)[(size_t)((wk * LW + j) * TT + tt) * 64 + lane] = acc[j][tt];
    __syncthreads();
    f16 *outp = reinterpret_cast<f16 *>(a.out);
    const f16 *resp = reinterpret_cast<const f16 *>(a.residual);
    constexpr int PAIRS = 128 * LW * TT;  // pairs of adjacent rows x 16*TT tokens
#pragma unroll
    for (int p0 = 0; p0 < PAIRS; p0 += nthreads) {
        const int pi = p0 + tid;
        if (PAIRS % nthreads != 0 && pi >= PAIRS) break;
        const int tt = pi / (128 * LW);                                // token tile
        const int tk = (pi / (8 * LW)) % 16, rp = pi % (8 * LW);       // token of the tile, row pair: rows 2*rp and 2*rp + 1
        // float index of row 2*rp in wave 0's planes; row 2*rp + 1 is the next element (LW 1) or
        // the same element of the next row plane (LW 2, 4)
        const int mr = (2 * rp) / LW, j0 = (2 * rp) % LW;  // MFMA row and plane of row 2*rp
        const int f0 = (j0 * TT + tt) * 256 + (((mr >> 2) * 16 + tk) << 2) + (mr & 3);
        constexpr int f1_off = LW == 1 ? 1 : TT * 256;
        float v0[WK], v1[WK];
#pragma unroll
        for (int w = 0; w < WK; ++w) {
            v0[w] = red[(size_t)w * (LW * TT * 256) + f0];
            v1[w] = red[(size_t)w * (LW * TT * 256) + f0 + f1_off];
        }
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < WK; ++w) {
            s0 += v0[w];
            s1 += v1[w];
        }
        const int tok = tok0 + tt * 16 + tk;
        if (tok >= a.n || (ROWS != 16 * LW && 2 * rp >= ROWS)) continue;
        const int col = row0 + 2 * rp;
        if (a.epilogue == TUNA_EPILOGUE_SILU_MUL) {
            outp[(size_t)tok * (size_t)(a.m >> 1) + (col >> 1)] = (f16)silu_mul(s0, s1);
        } else {
            const size_t at = (size_t)tok * (size_t)a.m + col;
            if (a.epilogue == TUNA_EPILOGUE_RESIDUAL) {
                const f16x2 r = *reinterpret_cast<const f16x2 *>(resp + at);
                s0 += (float)r[0], s1 += (float)r[1];
            }
            *reinterpret_cast<f16x2 *>(outp + at) = f16x2{(f16)s0, (f16)s1};
        }
    }
}

}  // namespace tuna
