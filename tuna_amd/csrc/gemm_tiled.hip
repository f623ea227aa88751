// FP16-activation x 4-bit-codebook-weight GEMM for MANY tokens (64 ... thousands) on gfx950.
//
//   out[n, m] = x[n, k] . W[m, k]^T,   W[r, c] = fp16(code[nib(r, c)]) *fp16 fp16(absmax[r])
//
// Counterpart of the reference's larger-n kernel configurations (kernel.cu:3037-3155 select
// them by token bucket).  With many tokens the op is bound by the matrix cores and by the
// decode, not by HBM, so unlike the streaming kernel (gemm_kernel.hpp: weights straight into
// registers, every wave decodes what it multiplies) a weight is decoded ONCE per workgroup
// tile and shared by all tokens of the tile through LDS:
//
//   * workgroup tile: BM = WM*TM*16 weight rows x BN = WN*TN*16 tokens, k in steps of 64;
//     WM x WN waves, a wave owns TM x TN MFMA tiles (v_mfma_f32_16x16x32_f16, weights = A).
//   * per k-step the 512 threads fetch BM x 64 packed weights (16 bytes per thread: 4
//     consecutive rows x 8 k; 16 threads cover 256 contiguous bytes of a block row) and
//     BN x 64 activations into registers, four steps ahead of their use (HBM latency is
//     longer than two steps of matrix work);
//   * two LDS tile buffers: while the matrix cores work on step s from one buffer, step
//     s+1 is decoded and staged into the other - one barrier per step, and the decode's
//     VALU/LDS work runs in the shadow of the MFMAs of the other wave on the SIMD;
//   * decode through the same conflict-free byte-pair table as the streaming kernel
//     (one v_perm_b32 + ds_read_b32 + v_pk_mul_f16 per two weights, bit-identical to
//     kernel.cu:2178-2192), then one ds_write_b128 per decoded dword into the A tile;
//   * A and X tiles are [row][64 k] fp16 = 128-byte rows whose eight 16-byte slots are
//     XOR-swizzled with (row & 7): the decode writes, the activation writes and the
//     ds_read_b128 fragment reads (8 lanes = 8 consecutive rows of one slot) all touch every
//     bank exactly once - no padding, no bank conflicts;
//   * fp32 accumulators stay in registers for the whole k range; a lane ends up with 4
//     consecutive output features of one token per MFMA tile: 8-byte stores.
//   * M32 variants multiply with v_mfma_f32_32x32x16_f16 instead (the counterpart of the reference's
//     wider MMA shapes, kernel.cu:411-465): a wave's TM x TN tiles of 16 x 16 become (TM/2) x (TN/2)
//     tiles of 32 x 32, a k-step of 64 is four MFMA steps of 16 instead of two of 32.  Lane l
//     supplies row / token l % 32 and the 8 k of half l / 32 of the step: the same 16-byte
//     fragment reads from the same tiles (8 consecutive lanes still read 8 consecutive rows of one
//     slot), half as many MFMA instructions for the same bytes read from LDS.  The sums are the
//     same products added in another order, so results differ from the 16 x 16 variants in the
//     last bits of the fp32 accumulation only.
#include "epilogue.hpp"

namespace tuna {


constexpr int kTiledThreads = 512;
constexpr int kTiledStepK = 64;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t tiled_u32x2 __attribute__((ext_vector_type(2)));

template <int WM, int TM, int WN, int TN, int NSETS, bool M32 = false, bool BLK = false>
__global__ __launch_bounds__(kTiledThreads, 2) void gemm_tiled_kernel(const TiledArgs a)
{
    static_assert(WM * WN * 64 == kTiledThreads, "8 waves");
    static_assert(!M32 || (TM % 2 == 0 && TN % 2 == 0), "32 x 32 MFMA tiles pair up the 16 x 16 ones");
    constexpr int BM = WM * TM * 16;
    constexpr int BN = WN * TN * 16;
    constexpr int DW = BM / 64;            // packed dwords (weight rows of one 8-k block) a thread decodes per k-step
    constexpr int P = 8 / DW;              // threads per 32-byte block of the packed layout
    constexpr int L = 4 * DW;              // table lookups (byte pairs) per thread and k-step
    constexpr int X_PER_THREAD = BN / 64;  // 16-byte activation pieces per thread per k-step
    static_assert(DW == 1 || DW == 2 || DW == 4, "64, 128 or 256 weight rows per workgroup");
    static_assert(X_PER_THREAD >= 1, "tile shape");
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *lut = smem;                       // byte-pair table at LDS address 0
    constexpr int BUF = (BM + BN) * 128;             // one buffer: weight tile [BM][128 B] + activation tile [BN][128 B]
    unsigned char *a_tile = smem + kLutBytes;
    unsigned char *x_tile = a_tile + BM * 128;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm_i = wave / WN, wn_i = wave % WN;
    const int i16 = lane & 15, g = lane >> 4;
    const uint32_t lane4 = (uint32_t)lane << 2;

    // One-dimensional grid over (row tile, token tile) with the token tiles of a row tile next to
    // each other in launch order, so that the workgroups resident at one time share their weights
    // through the caches (rows-major order streams all weights from HBM once per token tile).  When
    // the row tile count is a multiple of 8 the token tiles of a row tile also share an XCD and its
    // L2: workgroups are dealt to the 8 XCDs in turn, workgroup L sits on XCD L % 8.
    int row_tile, tok_tile;
    if ((a.row_tiles & 7) == 0) {
        const unsigned slot = blockIdx.x >> 3;
        tok_tile = (int)(slot % (unsigned)a.tok_tiles);
        row_tile = (int)(slot / (unsigned)a.tok_tiles) * 8 + (int)(blockIdx.x & 7);
    } else {
        tok_tile = (int)(blockIdx.x % (unsigned)a.tok_tiles);
        row_tile = (int)(blockIdx.x / (unsigned)a.tok_tiles);
    }
    const int row_base = row_tile * BM;
    const int tok_base = tok_tile * BN;
    const int kb_total = a.k >> 3;
    const int mb_last = (a.m >> 3) - 1;
    const f16 *xg = reinterpret_cast<const f16 *>(a.x);

    // ---- this thread's share of the loads ------------------------------------------------
    // weights: every thread takes DW consecutive rows of one 8 x 8 block per k-step - block row
    // tid / (8 P) of the tile, k-block (tid / P) % 8 of the step, rows DW * (tid % P) .. of the block:
    // a wave's load covers whole 32-byte blocks, 8 P consecutive threads 256 contiguous bytes
    const int a_piece = tid % P, a_kb = (tid / P) & 7, a_mbl = tid / (8 * P);
    const int a_mb = min((row_base >> 3) + a_mbl, mb_last);
    const unsigned char *a_src = a.q + (size_t)a_mb * kb_total * 32 + a_piece * (4 * DW);
    const int a_row = a_mbl * 8 + a_piece * DW;      // first of the DW tile rows this thread decodes
    // one scale per row - or (BLK) per block of 64 << blk_shift weights of a row: a k-step of 64 lies inside one
    // block, its scales travel through the register sets with its weights
    f16x2 sc16[DW];
    const float *sc_src[DW];
    const int nblk = BLK ? a.k >> (6 + a.blk_shift) : 1;
#pragma unroll
    for (int j = 0; j < DW; ++j) {
        sc_src[j] = a.absmax + (size_t)min(row_base + a_row + j, a.m - 1) * (size_t)nblk;
        if constexpr (!BLK) {
            const f16 h = (f16)sc_src[j][0];
            sc16[j] = f16x2{h, h};
        }
    }
    // activations: piece p = tid + i*512: token p / 8 of the tile, 8-k slot p % 8 of the step
    const f16 *x_src[X_PER_THREAD];
    bool x_tok_ok[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; ++i) {
        const int p = tid + i * kTiledThreads;
        const int tok = tok_base + (p >> 3);
        x_tok_ok[i] = tok < a.n;
        x_src[i] = xg + (size_t)min(tok, a.n - 1) * a.k + (p & 7) * 8;
    }

    // NSETS register sets: steps s .. s+NSETS-1 in flight (4; 8 for the 64-token tiles, whose steps
    // are short against the HBM latency)
    static_assert(NSETS == 4 || NSETS == 8, "register sets");
    // (256-token tiles keep two sets of activations: four would not leave room for both halves' fragments, and
    // activations come from the L2, not from HBM)
    constexpr int XSETS = X_PER_THREAD == 4 ? 2 : NSETS;
    uint32_t wq[NSETS][DW];
    float sq[BLK ? NSETS : 1][DW];
    u32x4 xr[XSETS][X_PER_THREAD];
    // Unconditional, clamped loads (exact s_waitcnt counts); what lies beyond k is zeroed in x.
#define TUNA_TILED_LOAD(set, s)                                                                 \
    {                                                                                          \
        const int kb_ = min((s) * 8 + a_kb, kb_total - 1);                                     \
        const unsigned char *p_ = a_src + (size_t)kb_ * 32;                                    \
        if constexpr (BLK) {                                                                   \
            const int blk_ = min((s) >> a.blk_shift, nblk - 1);                                \
            _Pragma("unroll") for (int j = 0; j < DW; ++j) sq[set][j] = sc_src[j][blk_];       \
        }                                                                                      \
        if constexpr (DW == 4) {                                                               \
            const u32x4 w_ = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p_));  \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) wq[set][j] = w_[j];                  \
        } else if constexpr (DW == 2) {                                                        \
            const tiled_u32x2 w_ = __builtin_nontemporal_load(reinterpret_cast<const tiled_u32x2 *>(p_)); \
            wq[set][0] = w_[0];                                                                \
            wq[set][DW - 1] = w_[1];                                                           \
        } else {                                                                               \
            wq[set][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p_));   \
        }                                                                                      \
    }
#define TUNA_TILED_LOAD_X(set, s)                                                               \
    _Pragma("unroll") for (int i = 0; i < X_PER_THREAD; ++i)                                   \
    {                                                                                          \
        const int kk_ = min((s) * kTiledStepK, a.k - 8 - ((tid + i * kTiledThreads) & 7) * 8); \
        xr[set][i] = *reinterpret_cast<const u32x4 *>(x_src[i] + kk_);                         \
    }

    const int s0 = blockIdx.z * a.steps_per_split;
    const int s1 = min(a.steps_total, s0 + a.steps_per_split);
#pragma unroll
    for (int u = 0; u < NSETS; ++u) {
        TUNA_TILED_LOAD(u, min(s0 + u, a.steps_total - 1))
        if (u < XSETS) TUNA_TILED_LOAD_X(u, min(s0 + u, a.steps_total - 1))
    }

    // ---- decode table (as in the streaming kernel) ------------------------------------------
    {
        const int code_bits = (int)(uint32_t)__builtin_bit_cast(uint16_t, (f16)a.code[lane & 15]);
#pragma unroll 4
        for (int p = tid; p < kLutBytes / 16; p += kTiledThreads) {
            const int e = p >> 4;
            const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
            const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
            const uint32_t v = hi | (lo << 16);
            reinterpret_cast<u32x4 *>(lut)[p] = u32x4{v, v, v, v};
        }
    }

    // Accumulators as TM * TN float4 "slots" in both variants.  16 x 16 tiles: slot tm * TN + tn, element
    // v of lane l is weight row 16*tm + 4*(l/16) + v, token 16*tn + l%16.  32 x 32 tiles: tile t holds 16
    // floats per lane, float 4*q + v being weight row 8*q + 4*(l/32) + v, token l%32 of the tile; its
    // four float4s are the slots 4*t + q.
    constexpr int TM2 = M32 ? TM / 2 : 1, TN2 = M32 ? TN / 2 : 1;
    f32x4 acc[M32 ? 1 : TM][M32 ? 1 : TN];
    f32x16 acc32[TM2][TN2];
    if constexpr (M32) {
#pragma unroll
        for (int tm = 0; tm < TM2; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN2; ++tn)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc32[tm][tn][e] = 0.f;
    } else {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int i32 = lane & 31, h32 = lane >> 5;

    // fragment addresses: row (i16) of MFMA tile tm / tn, slot (kh*4 + g) ^ (row & 7)
    const unsigned char *a_frag = a_tile + (wm_i * TM * 16 + (M32 ? i32 : i16)) * 128;
    const unsigned char *x_frag = x_tile + (wn_i * TN * 16 + (M32 ? i32 : i16)) * 128;
    const int sw = (M32 ? i32 : i16) & 7;

    // ---- the pieces of one k-step --------------------------------------------------------------
    // A k-step of 64 is two halves of 32 k.  Fragments of half h of a step, TM of the weight tile and TN
    // of the activation tile (32 x 32 tiles: two k-quarters of TM/2 and TN/2):
    f16x8 fa[2][TM], fb[2][TN];
#define TUNA_TILED_READ(h, buf)                                                                  \
    {                                                                                          \
        if constexpr (M32) {                                                                   \
            _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                                   \
            {                                                                                  \
                const int slot_ = (((((h) * 2 + kk) * 2 + h32) ^ sw) << 4) + (buf) * BUF;      \
                _Pragma("unroll") for (int tn = 0; tn < TN2; ++tn)                             \
                    fb[h][kk * TN2 + tn] = *reinterpret_cast<const f16x8 *>(x_frag + tn * (32 * 128) + slot_); \
                _Pragma("unroll") for (int tm = 0; tm < TM2; ++tm)                             \
                    fa[h][kk * TM2 + tm] = *reinterpret_cast<const f16x8 *>(a_frag + tm * (32 * 128) + slot_); \
            }                                                                                  \
        } else {                                                                               \
            const int slot_ = ((((h) * 4 + g) ^ sw) << 4) + (buf) * BUF;                       \
            _Pragma("unroll") for (int tn = 0; tn < TN; ++tn)                                  \
                fb[h][tn] = *reinterpret_cast<const f16x8 *>(x_frag + tn * (16 * 128) + slot_); \
            _Pragma("unroll") for (int tm = 0; tm < TM; ++tm)                                  \
                fa[h][tm] = *reinterpret_cast<const f16x8 *>(a_frag + tm * (16 * 128) + slot_); \
        }                                                                                      \
    }
    // MFMA q of the NM of a half
    constexpr int NM = M32 ? 2 * TM2 * TN2 : TM * TN;
    constexpr int QS = NM / 4;
#define TUNA_TILED_MFMA1(h, q)                                                                   \
    {                                                                                          \
        if constexpr (M32) {                                                                   \
            const int kk_ = (q) / (TM2 * TN2), tm_ = ((q) % (TM2 * TN2)) / TN2, tn_ = (q) % TN2; \
            acc32[tm_][tn_] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[h][kk_ * TM2 + tm_], fb[h][kk_ * TN2 + tn_], \
                                                                     acc32[tm_][tn_], 0, 0, 0); \
        } else {                                                                               \
            acc[(q) / TN][(q) % TN] =                                                          \
                __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[h][(q) / TN], fb[h][(q) % TN], acc[(q) / TN][(q) % TN], 0, 0, 0); \
        }                                                                                      \
    }
    // Staging of a k-step from register set `set`: the table reads of its L byte pairs ...
    uint32_t lt[L];
    f16x2 hh[L];
#define TUNA_TILED_LUT(set)                                                                      \
    _Pragma("unroll") for (int j = 0; j < DW; ++j)                                             \
    {                                                                                          \
        const uint32_t d_ = wq[set][j];                                                        \
        if constexpr (BLK) {                                                                   \
            const f16 h_ = (f16)sq[set][j];                                                    \
            sc16[j] = f16x2{h_, h_};                                                           \
        }                                                                                      \
        lt[4 * j + 0] = *reinterpret_cast<const lds_u32 *>((uintptr_t)__builtin_amdgcn_perm(d_, lane4, 0x0c0c0400u)); \
        lt[4 * j + 1] = *reinterpret_cast<const lds_u32 *>((uintptr_t)__builtin_amdgcn_perm(d_, lane4, 0x0c0c0500u)); \
        lt[4 * j + 2] = *reinterpret_cast<const lds_u32 *>((uintptr_t)__builtin_amdgcn_perm(d_, lane4, 0x0c0c0600u)); \
        lt[4 * j + 3] = *reinterpret_cast<const lds_u32 *>((uintptr_t)__builtin_amdgcn_perm(d_, lane4, 0x0c0c0700u)); \
    }
    // ... the scaling of pair l (bit-identical to kernel.cu:2178-2192), the fourth pair of a dword storing
    // its eight weights into row a_row + l / 4 of weight tile `buf` ...
#define TUNA_TILED_DECODE(l, buf)                                                                \
    {                                                                                          \
        hh[l] = __builtin_bit_cast(f16x2, lt[l]) * sc16[(l) >> 2];                             \
        if (((l) & 3) == 3) {                                                                  \
            const int r_ = a_row + ((l) >> 2);                                                 \
            const f16x8 w_ = {hh[(l) - 3][0], hh[(l) - 3][1], hh[(l) - 2][0], hh[(l) - 2][1],  \
                              hh[(l) - 1][0], hh[(l) - 1][1], hh[l][0],       hh[l][1]};       \
            *reinterpret_cast<f16x8 *>(a_tile + (buf) * BUF + r_ * 128 + ((a_kb ^ (r_ & 7)) << 4)) = w_; \
        }                                                                                      \
    }
    // ... and activation piece i of step s (zero beyond n and k) into activation tile `buf`.
#define TUNA_TILED_XSTAGE(set, i, buf, s)                                                        \
    {                                                                                          \
        const int p_ = tid + (i) * kTiledThreads;                                              \
        const int t_ = p_ >> 3, sl_ = p_ & 7;                                                  \
        const bool ok_ = x_tok_ok[i] && ((s) * kTiledStepK + sl_ * 8 < a.k);                   \
        *reinterpret_cast<u32x4 *>(x_tile + (buf) * BUF + t_ * 128 + ((sl_ ^ (t_ & 7)) << 4)) = \
            ok_ ? xr[set][i] : u32x4{0u, 0u, 0u, 0u};                                          \
    }
    // Iteration i of a tile's k-steps, k-step `step`, whose tiles are complete in buffer i & 1 (a barrier
    // has passed).  The matrix cores must not wait for the staging of the next step, nor for the
    // fragments of this one, so the order is written out and pinned:
    //   fragments of this step's first half are requested, and the table reads of step + 1;
    //   the MFMAs of the PREVIOUS step's second half run meanwhile (their fragments were read before the
    //     barrier), with the scaling and the weight-tile stores of step + 1 between them;
    //   fragments of this step's second half are requested;
    //   the MFMAs of this step's first half run, with the activation stores of step + 1 and the
    //     refill of the register set between them;
    //   barrier.
    // FIRST: no previous step.  The second half of the last step follows the loop.
#define TUNA_TILED_ITER(i, step, FIRST)                                                          \
    {                                                                                          \
        const int set_ = ((i) + 1) % NSETS, xset_ = ((i) + 1) % XSETS, cur_ = (i) & 1, nxt_ = cur_ ^ 1; \
        TUNA_TILED_READ(0, cur_)                                                               \
        TUNA_TILED_LUT(set_)                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                     \
        _Pragma("unroll") for (int q = 0; q < NM; ++q)                                         \
        {                                                                                      \
            if (!(FIRST)) TUNA_TILED_MFMA1(1, q)                                               \
            /* (none behind the first quarter of the MFMAs: the table reads are still on their way) */ \
            _Pragma("unroll") for (int l = max(q - QS, 0) * L / (NM - QS); l < max(q - QS + 1, 0) * L / (NM - QS); ++l) \
                TUNA_TILED_DECODE(l, nxt_)                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        TUNA_TILED_READ(1, cur_)                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                     \
        _Pragma("unroll") for (int q = 0; q < NM; ++q)                                         \
        {                                                                                      \
            TUNA_TILED_MFMA1(0, q)                                                             \
            _Pragma("unroll") for (int xi = 0; xi < X_PER_THREAD; ++xi)                        \
                if (q == xi * NM / X_PER_THREAD) TUNA_TILED_XSTAGE(xset_, xi, nxt_, (step) + 1) \
            if (q == NM - 1) {                                                                 \
                /* (activations first: the wait for them two steps on then leaves this step's weights in flight) */ \
                TUNA_TILED_LOAD_X(xset_, min((step) + 1 + XSETS, a.steps_total - 1))           \
                TUNA_TILED_LOAD(set_, min((step) + 1 + NSETS, a.steps_total - 1))              \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        __syncthreads(); /* the staged tiles are complete; this step's tiles are free */       \
    }

    int s = s0;
    __syncthreads();  // decode table complete
    // the first step, staged with nothing to hide behind
    TUNA_TILED_LUT(0)
#pragma unroll
    for (int l = 0; l < L; ++l) TUNA_TILED_DECODE(l, 0)
#pragma unroll
    for (int xi = 0; xi < X_PER_THREAD; ++xi) TUNA_TILED_XSTAGE(0, xi, 0, s)
    TUNA_TILED_LOAD(0, min(s + NSETS, a.steps_total - 1))
    TUNA_TILED_LOAD_X(0, min(s + XSETS, a.steps_total - 1))
    __syncthreads();
    TUNA_TILED_ITER(0, s, true)
    ++s;
    for (; s + NSETS - 1 < s1; s += NSETS) {
#pragma unroll
        for (int it = 0; it < NSETS; ++it) TUNA_TILED_ITER(it + 1, s + it, false)
    }
    // tail: up to NSETS - 1 more steps (the staging of a step past the end is harmless: its loads
    // are clamped and nothing reads the tiles)
#pragma unroll
    for (int it = 0; it < NSETS - 1; ++it)
        if (s + it < s1) TUNA_TILED_ITER(it + 1, s + it, false)
    // second half of the last step
#pragma unroll
    for (int q = 0; q < NM; ++q) TUNA_TILED_MFMA1(1, q)
#undef TUNA_TILED_ITER
#undef TUNA_TILED_XSTAGE
#undef TUNA_TILED_DECODE
#undef TUNA_TILED_LUT
#undef TUNA_TILED_MFMA1
#undef TUNA_TILED_READ
#undef TUNA_TILED_LOAD_X
#undef TUNA_TILED_LOAD

    // ---- epilogue -----------------------------------------------------------------------------
    // slot sl = tm * TN + tn (see the accumulators above): its float4 of this lane, first weight row, token
    auto slot_value = [&](int sl) {
        if constexpr (M32) {
            const int t32 = sl >> 2, q = sl & 3;  // slots of a 32 x 32 tile are consecutive here: sl = tile * 4 + q
            const f32x16 &t = acc32[t32 / TN2][t32 % TN2];
            return f32x4{t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
        } else {
            return acc[sl / TN][sl % TN];
        }
    };
    auto slot_row = [&](int sl) {
        if constexpr (M32) return row_base + wm_i * TM * 16 + ((sl >> 2) / TN2) * 32 + (sl & 3) * 8 + h32 * 4;
        else return row_base + (wm_i * TM + sl / TN) * 16 + g * 4;
    };
    auto slot_tok = [&](int sl) {
        if constexpr (M32) return tok_base + wn_i * TN * 16 + ((sl >> 2) % TN2) * 32 + i32;
        else return tok_base + (wn_i * TN + sl % TN) * 16 + i16;
    };
    f16 *outp = reinterpret_cast<f16 *>(a.out);
    const f16 *resp = reinterpret_cast<const f16 *>(a.residual);
    if (a.split_k == 1) {
#pragma unroll
        for (int sl = 0; sl < TM * TN; ++sl) {
            const int row = slot_row(sl), tok = slot_tok(sl);
            if (tok < a.n && row + 4 <= a.m) {
                const f32x4 v = slot_value(sl);
                store_features4(outp, resp, a.epilogue, (size_t)tok, a.m, row, v[0], v[1], v[2], v[3]);
            }
        }
        return;
    }
    // split-K: fp32 partial tiles [split][tile][wave][tm][tn][lane] as float4, the last workgroup of
    // a tile to arrive adds them in split order (deterministic, no atomics on out)
    const size_t tile_id = (size_t)tok_tile * a.row_tiles + row_tile;
    constexpr size_t kTileF4 = (size_t)8 * TM * TN * 64;  // float4s per partial tile
    f32x4 *ws4 = reinterpret_cast<f32x4 *>(a.ws);
    f32x4 *mine = ws4 + (tile_id * a.split_k + blockIdx.z) * kTileF4 + (size_t)wave * (TM * TN * 64) + lane;
#pragma unroll
    for (int sl = 0; sl < TM * TN; ++sl) {
        const f32x4 v = slot_value(sl);
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0" : : "v"(mine + sl * 64), "v"(v) : "memory");
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the partial sums have left this CU
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(a_tile);
    if (tid == 0) *ticket = __hip_atomic_fetch_add(a.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket != (unsigned)(a.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(a.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The partial tiles come back as 16-byte loads that bypass this CU's and this XCD's caches (sc1: the writers sit
    // on any XCD), two slots x two splits requested before the first is awaited - the pass is a chain of memory
    // round trips, and four requests of 16 bytes per lane in flight take a third of the time of one of 4 bytes.
    // Each slot's sum still adds its splits in ascending order.
    const f32x4 *src = ws4 + tile_id * a.split_k * kTileF4 + (size_t)wave * (TM * TN * 64) + lane;
    static_assert((TM * TN) % 2 == 0, "slots are finished in pairs");
    for (int sl = 0; sl < TM * TN; sl += 2) {
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
        int sp = 0;
        for (; sp + 1 < a.split_k; sp += 2) {
            const f32x4 *p = src + (size_t)sp * kTileF4 + sl * 64;
            f32x4 a0, a1, b0, b1;
            asm volatile("global_load_dwordx4 %0, %4, off sc1\n\t"
                         "global_load_dwordx4 %1, %5, off sc1\n\t"
                         "global_load_dwordx4 %2, %6, off sc1\n\t"
                         "global_load_dwordx4 %3, %7, off sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(a0), "=&v"(a1), "=&v"(b0), "=&v"(b1)
                         : "v"(p), "v"(p + 64), "v"(p + kTileF4), "v"(p + kTileF4 + 64)
                         : "memory");
            s0 += a0, s1 += a1;
            s0 += b0, s1 += b1;
        }
        if (sp < a.split_k) {
            const f32x4 *p = src + (size_t)sp * kTileF4 + sl * 64;
            f32x4 a0, a1;
            asm volatile("global_load_dwordx4 %0, %2, off sc1\n\t"
                         "global_load_dwordx4 %1, %3, off sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(a0), "=&v"(a1)
                         : "v"(p), "v"(p + 64)
                         : "memory");
            s0 += a0, s1 += a1;
        }
        {
            const int row = slot_row(sl), tok = slot_tok(sl);
            if (tok < a.n && row + 4 <= a.m) store_features4(outp, resp, a.epilogue, (size_t)tok, a.m, row, s0[0], s0[1], s0[2], s0[3]);
        }
        {
            const int row = slot_row(sl + 1), tok = slot_tok(sl + 1);
            if (tok < a.n && row + 4 <= a.m) store_features4(outp, resp, a.epilogue, (size_t)tok, a.m, row, s1[0], s1[1], s1[2], s1[3]);
        }
    }
}

typedef void (*TiledFn)(const TiledArgs);
struct TiledVariant {
    int bm, bn;
    TiledFn fn;
    TiledFn fn32;   // the same tile with 32 x 32 x 16 MFMAs, or null
    TiledFn fn_blk; // the same tile (16 x 16 x 32 MFMAs) with a scale per block of a row
};
// (WM, TM, WN, TN): rows x tokens of the workgroup tile
static const TiledVariant kTiled[] = {
    {256, 128, gemm_tiled_kernel<4, 4, 2, 4, 4>, gemm_tiled_kernel<4, 4, 2, 4, 4, true>, gemm_tiled_kernel<4, 4, 2, 4, 4, false, true>},
    {256, 64, gemm_tiled_kernel<4, 4, 2, 2, 8>, gemm_tiled_kernel<4, 4, 2, 2, 8, true>, gemm_tiled_kernel<4, 4, 2, 2, 8, false, true>},
    {128, 256, gemm_tiled_kernel<2, 4, 4, 4, 4>, gemm_tiled_kernel<2, 4, 4, 4, 4, true>, gemm_tiled_kernel<2, 4, 4, 4, 4, false, true>},
    {128, 128, gemm_tiled_kernel<2, 4, 4, 2, 4>, gemm_tiled_kernel<2, 4, 4, 2, 4, true>, gemm_tiled_kernel<2, 4, 4, 2, 4, false, true>},
    {64, 256, gemm_tiled_kernel<1, 4, 8, 2, 4>, gemm_tiled_kernel<1, 4, 8, 2, 4, true>, gemm_tiled_kernel<1, 4, 8, 2, 4, false, true>},
    {64, 128, gemm_tiled_kernel<1, 4, 8, 1, 4>, nullptr, gemm_tiled_kernel<1, 4, 8, 1, 4, false, true>},
};
static constexpr int kNumTiled = sizeof(kTiled) / sizeof(kTiled[0]);

bool tiled_variant_exists(int bm, int bn, bool mfma32)
{
    if (bm == 256 && bn == 256) return true;  // gemm_wide.hip
    for (int i = 0; i < kNumTiled; ++i)
        if (kTiled[i].bm == bm && kTiled[i].bn == bn) return !mfma32 || kTiled[i].fn32 != nullptr;
    return false;
}

size_t tiled_lds_bytes(int bm, int bn)
{
    if (bm == 256 && bn == 256) return wide_lds_bytes();
    return (size_t)kLutBytes + 2 * (size_t)(bm + bn) * 128;  // two tile buffers
}

static OptInFlag g_tiled_attr[16][kNumTiled][3];

hipError_t launch_gemm_tiled(const TiledArgs &args, int bm, int bn, bool mfma32, hipStream_t stream, bool scale_blocks)
{
    if (bm == 256 && bn == 256) return !scale_blocks ? launch_gemm_wide(args, mfma32, stream) : hipErrorInvalidConfiguration;
    int vi = -1;
    for (int i = 0; i < kNumTiled; ++i)
        if (kTiled[i].bm == bm && kTiled[i].bn == bn) vi = i;
    if (vi < 0 || (scale_blocks && mfma32)) return hipErrorInvalidConfiguration;
    const TiledFn fn = scale_blocks ? kTiled[vi].fn_blk : mfma32 ? kTiled[vi].fn32 : kTiled[vi].fn;
    if (!fn) return hipErrorInvalidConfiguration;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    if ((e = ensure_lds_opt_in(g_tiled_attr[dev][vi][scale_blocks ? 2 : mfma32], reinterpret_cast<const void *>(fn))) != hipSuccess) return e;
    TiledArgs a = args;
    a.row_tiles = ceil_div_i(args.m, bm);
    a.tok_tiles = ceil_div_i(args.n, bn);
    if ((long long)a.row_tiles * a.tok_tiles > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    const dim3 grid((unsigned)(a.row_tiles * a.tok_tiles), 1, (unsigned)args.split_k);
    hipLaunchKernelGGL(fn, grid, dim3(kTiledThreads), tiled_lds_bytes(bm, bn), stream, a);
    return hipGetLastError();
}

}  // namespace tuna
