// FP16-activation x 4-bit-codebook-weight GEMM for MANY tokens, 256 weight rows x 256 tokens per workgroup.
//
// The many-token kernel of gemm_tiled.hip spends most of its LDS time per flop on fragment reads, decode-table
// reads and tile stores.  All three shrink with the tile: a weight is decoded once per 256 tokens, an activation
// staged once per 256 rows, and a wave that owns 128 x 128 of the tile reads half the fragments per flop of a
// 64 x 64 one.  Such a wave needs 256 accumulator registers, so this kernel runs ONE wave per SIMD (4 waves of
// 512 registers: the accumulators in the AGPR half) and hides every latency inside that wave's own instruction
// stream instead of behind a second wave:
//
//   * a k-step of 64 is four phases; the fragments of a phase are requested between the MFMAs of the phase
//     before, the staging of step s + 1 (scaling and tile stores of the decoded weights, activation stores) sits
//     between the MFMAs of phases 0..2 of step s with ONE barrier behind phase 2, the table reads of a packed
//     dword come a phase before the stores that use them (a ring of four dwords' reads), the register sets are
//     refilled as they come free;
//   * v_mfma_f32_16x16x32_f16 by default (rows_per_wave = 64 in the config; 8 x 8 tiles per wave, a phase is
//     four weight tiles x eight token tiles): with operands of real data the chip gives that shape about 14 %
//     more flops than v_mfma_f32_32x32x16_f16 (launch_unit_rate, units 10..13) - which variant M32 keeps
//     (rows_per_wave = 32; 4 x 4 tiles per wave, a phase is a quarter of 16 k);
//   * same tiles as gemm_tiled.hip: [row][64 k] fp16 = 128-byte rows, 16-byte slots XOR-swizzled with row & 7,
//     two buffers of (256 + 256) rows = 128 KB; the byte-pair decode table has a copy per 32 lanes instead of
//     per 64 (32 KB: reads at the same rate, the LDS takes a wave's 4-byte reads 32 lanes at a time), which is
//     what lets table and tiles share the 160 KB;
//   * a thread decodes one 32-byte record (8 rows x 8 k) per k-step; 8 consecutive threads read the 256
//     contiguous bytes of a block row's k-step; weights and activations come through buffer loads (descriptor in
//     scalar registers, one 32-bit offset per lane, the k-step as a scalar offset): no 64-bit address
//     arithmetic in the loop, which a single wave per SIMD would pay for in MFMA issue slots.
// KTAIL: k is any multiple of 8.  The last k-step is then partly beyond k: a thread whose 8-k slot of that step
// lies beyond k loads the last slot inside k instead (no access leaves a row, whatever the descriptor's range
// check covers), and the activations of those slots are stored as zeros, so the products vanish whatever the
// weight slots hold (finite values: table entries times the row's own scale).  k a multiple of 64 runs the
// variant without the selects.
//
// Decode and rounding are those of the other kernels (bit-identical to kernel.cu:2178-2192); the sums are the
// same products in the same order as the variants of gemm_tiled.hip with the same MFMA shape.
#include "epilogue.hpp"

namespace tuna {

constexpr int kWideThreads = 256;
constexpr int kWideLutBytes = 256 * 32 * 4;
constexpr int kWideRows = 256, kWideTokens = 256;
constexpr int kWideBuf = (kWideRows + kWideTokens) * 128;

typedef float wide_f32x16 __attribute__((ext_vector_type(16)));

template <int NSETS, bool M32, bool KTAIL>
__global__ __launch_bounds__(kWideThreads, 1) void gemm_wide_kernel(const TiledArgs a)
{
    static_assert(NSETS == 2 || NSETS == 4, "register sets of packed weights");
    constexpr int XSETS = 2;
    constexpr int BUF = kWideBuf;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *lut = smem;  // byte-pair table at LDS address 0: entry (byte << 7) | ((lane & 31) << 2)
    unsigned char *a_tile = smem + kWideLutBytes;
    unsigned char *x_tile = a_tile + kWideRows * 128;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm_i = wave >> 1, wn_i = wave & 1;
    const int i32 = lane & 31, h32 = lane >> 5;  // 32 x 32 tiles: row / token and k-half of a lane's fragments
    const int i16 = lane & 15, g = lane >> 4;    // 16 x 16 tiles: row / token and k-group
    const uint32_t lane8 = (uint32_t)(lane & 31) << 3;

    // grid order as in gemm_tiled.hip: the token tiles of a row tile next to each other (and on one XCD when the
    // row tile count is a multiple of 8)
    int row_tile, tok_tile;
    if ((a.row_tiles & 7) == 0) {
        const unsigned slot = blockIdx.x >> 3;
        tok_tile = (int)(slot % (unsigned)a.tok_tiles);
        row_tile = (int)(slot / (unsigned)a.tok_tiles) * 8 + (int)(blockIdx.x & 7);
    } else {
        tok_tile = (int)(blockIdx.x % (unsigned)a.tok_tiles);
        row_tile = (int)(blockIdx.x / (unsigned)a.tok_tiles);
    }
    const int row_base = row_tile * kWideRows;
    const int tok_base = tok_tile * kWideTokens;
    const int kb_total = a.k >> 3;
    const int mb_last = (a.m >> 3) - 1;

    // weights: thread -> block row tid / 8 of the tile, k-block tid % 8 of the step (rows beyond the matrix are
    // clamped: their products are never stored).  Addresses are a uniform base - the tile's first block row, first
    // token - that advances with the k-step, plus a 32-bit offset per thread inside the tile: no 64-bit vector
    // arithmetic in the loop, short address operands, no limit on the size of q or x.
    const int a_kb = tid & 7, a_mbl = tid >> 3;
    const uint32_t a_off = ((uint32_t)(min((row_base >> 3) + a_mbl, mb_last) - (row_base >> 3)) * (uint32_t)kb_total + (uint32_t)a_kb) * 32u;
    f16x2 sc16[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const f16 h = (f16)a.absmax[min(row_base + a_mbl * 8 + j, a.m - 1)];
        sc16[j] = f16x2{h, h};
    }
    unsigned char *a_dst = a_tile + a_mbl * 8 * 128;  // row a_mbl * 8 + j: + j * 128 + ((a_kb ^ j) << 4)
    // activations: piece i of a thread is token tid / 8 + 32 i of the tile, 8-k slot tid % 8 of the step (tokens
    // beyond n read the last token's row: their outputs are never stored)
    uint32_t x_off[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int tok = tok_base + (tid >> 3) + 32 * i;
        x_off[i] = ((uint32_t)(min(tok, a.n - 1) - tok_base) * (uint32_t)a.k + (uint32_t)(tid & 7) * 8u) * 2u;
    }
    unsigned char *x_dst = x_tile + (tid >> 3) * 128 + (((tid & 7) ^ ((tid >> 3) & 7)) << 4);  // piece i: + i * 4096
    // KTAIL: the thread's slot of k-step s lies inside k while 64 s < x_k_left; in the last step a slot beyond k
    // steps back to the last one inside (in bytes: 32 per slot of packed weights, 16 per slot of activations)
    const int x_k_left = a.k - (tid & 7) * 8;
    const int slots_back = KTAIL ? max(0, (tid & 7) - (((a.k >> 3) - 1) & 7)) : 0;
    const uint32_t a_back = (uint32_t)slots_back * 32u, x_back = (uint32_t)slots_back * 16u;

    u32x4 wq[NSETS][2];
    u32x4 xr[XSETS][8];
    // buffer loads: descriptor + 32-bit offset per lane + uniform offset of the k-step (weights without the
    // nontemporal hint: the token tiles of a row tile run side by side and share them through the L2)
    const size_t q_rest = (size_t)(a.m - row_base) * (size_t)(a.k >> 1), x_rest = (size_t)(a.n - tok_base) * (size_t)a.k * 2;
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(a.q) + (size_t)(row_base >> 3) * kb_total * 32, 0, (int)(uint32_t)min(q_rest, (size_t)0xffffffffu), 0x00020000);
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<unsigned char *>(const_cast<void *>(a.x)) + (size_t)tok_base * a.k * 2, 0,
        (int)(uint32_t)min(x_rest, (size_t)0xffffffffu), 0x00020000);
#define TUNA_WIDE_LOAD(set, s)                                                                  \
    {                                                                                          \
        const uint32_t o_ = KTAIL && (s) == s_last ? a_off - a_back : a_off;                   \
        wq[set][0] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, (int)o_, (s) * 256, 0);     \
        wq[set][1] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, (int)o_ + 16, (s) * 256, 0); \
    }
#define TUNA_WIDE_LOAD_X(set, s)                                                                \
    {                                                                                          \
        const uint32_t b_ = KTAIL && (s) == s_last ? x_back : 0u;                              \
        _Pragma("unroll") for (int i = 0; i < 8; ++i)                                          \
            xr[set][i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)(x_off[i] - b_), (s) * 128, 0); \
    }

    const int s0 = blockIdx.z * a.steps_per_split;
    const int s1 = min(a.steps_total, s0 + a.steps_per_split);
    const int s_last = a.steps_total - 1;
#pragma unroll
    for (int u = 0; u < NSETS; ++u) {
        TUNA_WIDE_LOAD(u, min(s0 + u, s_last))
        if (u < XSETS) TUNA_WIDE_LOAD_X(u, min(s0 + u, s_last))
    }

    // decode table: entry e = 128 bytes = 32 copies of fp16(code[e >> 4]) | fp16(code[e & 15]) << 16
    {
        const int code_bits = (int)(uint32_t)__builtin_bit_cast(uint16_t, (f16)a.code[lane & 15]);
#pragma unroll 4
        for (int p = tid; p < kWideLutBytes / 16; p += kWideThreads) {
            const int e = p >> 3;
            const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
            const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
            const uint32_t v = hi | (lo << 16);
            reinterpret_cast<u32x4 *>(lut)[p] = u32x4{v, v, v, v};
        }
    }

    // accumulators of the wave's 128 x 128.  32 x 32 tiles (tm, tn): float 4*q + v of lane l is weight row
    // 32 tm + 8 q + 4 (l / 32) + v, token 32 tn + l % 32.  16 x 16 tiles: element v of lane l is weight row
    // 16 tm + 4 (l / 16) + v, token 16 tn + l % 16.
    wide_f32x16 acc[M32 ? 4 : 1][M32 ? 4 : 1];
    f32x4 acc16[M32 ? 1 : 8][M32 ? 1 : 8];
    if constexpr (M32) {
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
#pragma unroll
            for (int tn = 0; tn < 4; ++tn)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[tm][tn][e] = 0.f;
    } else {
#pragma unroll
        for (int tm = 0; tm < 8; ++tm)
#pragma unroll
            for (int tn = 0; tn < 8; ++tn) acc16[tm][tn] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // fragment addresses: row i32 of 32 x 32 tile t, slot (2 quarter + h32) ^ (row & 7)
    const unsigned char *a_frag = a_tile + (wm_i * 128 + i32) * 128;
    const unsigned char *x_frag = x_tile + (wn_i * 128 + i32) * 128;
    const int swz = (h32 ^ (i32 & 7)) << 4;  // slot << 4 = (32 * quarter) ^ swz

    // fragments of a quarter: [0..3] weight tiles, [4..7] token tiles
    f16x8 fr[2][8];
#define TUNA_WIDE_READ1(f, kq, buf, t)                                                           \
    {                                                                                          \
        const int o_ = ((32 * (kq)) ^ swz) + (buf) * BUF + ((t) & 3) * (32 * 128);             \
        fr[f][t] = *reinterpret_cast<const f16x8 *>(((t) < 4 ? a_frag : x_frag) + o_);        \
    }
#define TUNA_WIDE_MFMA1(f, i)                                                                    \
    acc[(i) >> 2][(i) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[f][(i) >> 2], fr[f][4 + ((i) & 3)], acc[(i) >> 2][(i) & 3], 0, 0, 0);
    // 16 x 16 tiles: a k-step is two halves of 32 k, a half two phases of 32 MFMAs (weight tiles 0..3, then 4..7,
    // against all eight token tiles, token tile by token tile): two sets of four weight fragments, and ONE set of
    // eight token fragments - in the second phase of a half a token fragment is replaced by the next half's right
    // behind its last MFMA, 29 MFMAs before its first use
    const unsigned char *a_frag16 = a_tile + (wm_i * 128 + i16) * 128;
    const unsigned char *x_frag16 = x_tile + (wn_i * 128 + i16) * 128;
    const int swz16 = (g ^ (i16 & 7)) << 4;  // slot << 4 = (64 * half) ^ swz16
    f16x8 fa[2][4], fb[8];
#define TUNA_WIDE_READ_A(ab, h, buf, t)                                                          \
    fa[ab][(t) & 3] = *reinterpret_cast<const f16x8 *>(a_frag16 + ((64 * (h)) ^ swz16) + (buf) * BUF + (t) * (16 * 128));
#define TUNA_WIDE_READ_B(h, buf, t)                                                              \
    fb[t] = *reinterpret_cast<const f16x8 *>(x_frag16 + ((64 * (h)) ^ swz16) + (buf) * BUF + (t) * (16 * 128));
    // (written out with the accumulator pinned to the AGPR half of the register file: left to itself the
    // register allocator spreads 64 four-register accumulators over both halves and then spills in the loop;
    // accumulators are next touched 63 MFMAs later, and the epilogue waits out the last ones before it reads them)
#define TUNA_WIDE_MFMA16(ab, tm, tn)                                                             \
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc16[tm][tn]) : "v"(fa[ab][(tm) & 3]), "v"(fb[tn]));

    // table reads of the four byte pairs of packed dword j of register set `set` ...
    uint32_t lt[16];  // a ring of four dwords: dword j in entries 4 (j % 4) ..
#define TUNA_WIDE_LUT(set, j)                                                                    \
    {                                                                                          \
        const uint32_t d_ = wq[set][(j) >> 2][(j) & 3];                                        \
        lt[4 * ((j) & 3) + 0] = *reinterpret_cast<const lds_u32 *>((uintptr_t)(__builtin_amdgcn_perm(d_, lane8, 0x0c0c0400u) >> 1)); \
        lt[4 * ((j) & 3) + 1] = *reinterpret_cast<const lds_u32 *>((uintptr_t)(__builtin_amdgcn_perm(d_, lane8, 0x0c0c0500u) >> 1)); \
        lt[4 * ((j) & 3) + 2] = *reinterpret_cast<const lds_u32 *>((uintptr_t)(__builtin_amdgcn_perm(d_, lane8, 0x0c0c0600u) >> 1)); \
        lt[4 * ((j) & 3) + 3] = *reinterpret_cast<const lds_u32 *>((uintptr_t)(__builtin_amdgcn_perm(d_, lane8, 0x0c0c0700u) >> 1)); \
    }
    // ... their scaling (bit-identical to kernel.cu:2178-2192) and the store of the dword's eight weights into
    // row a_mbl * 8 + j of weight tile `buf` ...
#define TUNA_WIDE_DECODE(j, buf)                                                                 \
    {                                                                                          \
        const f16x2 h0_ = __builtin_bit_cast(f16x2, lt[4 * ((j) & 3) + 0]) * sc16[j];                \
        const f16x2 h1_ = __builtin_bit_cast(f16x2, lt[4 * ((j) & 3) + 1]) * sc16[j];                \
        const f16x2 h2_ = __builtin_bit_cast(f16x2, lt[4 * ((j) & 3) + 2]) * sc16[j];                \
        const f16x2 h3_ = __builtin_bit_cast(f16x2, lt[4 * ((j) & 3) + 3]) * sc16[j];                \
        const f16x8 w_ = {h0_[0], h0_[1], h1_[0], h1_[1], h2_[0], h2_[1], h3_[0], h3_[1]};     \
        *reinterpret_cast<f16x8 *>(a_dst + (buf) * BUF + (j) * 128 + ((a_kb ^ (j)) << 4)) = w_; \
    }
    // ... and activation piece i into activation tile `buf`.
#define TUNA_WIDE_XSTAGE(set, i, buf, s)                                                         \
    {                                                                                          \
        u32x4 v_ = xr[set][i];                                                                 \
        if constexpr (KTAIL) {                                                                 \
            if ((s) * 64 >= x_k_left) v_ = u32x4{0u, 0u, 0u, 0u};                              \
        }                                                                                      \
        *reinterpret_cast<u32x4 *>(x_dst + (buf) * BUF + (i) * 4096) = v_;                     \
    }
    // Iteration `it` (k-step `step`) of a tile: its tiles are complete in buffer it & 1, the fragments of its
    // first quarter in fr[0], the table reads of dwords 0..3 of step + 1 in lt.  Side work between the MFMAs:
    //   quarter 0: fragments of quarter 1; weights 0..3 of step + 1 scaled and stored into the other buffer, each
    //              followed by the table reads of dword 4..7 into the freed ring entry; refill of that register set
    //   quarter 1: fragments of quarter 2; weights 4..7; activations 0..1
    //   quarter 2: fragments of quarter 3; activations 2..7 and the refill of their register set; barrier
    //   quarter 3: fragments of quarter 0 of step + 1; table reads of dwords 0..3 of step + 2
#define TUNA_WIDE_ITER(it, step)                                                                 \
    {                                                                                          \
        const int cur_ = (it) & 1, nxt_ = cur_ ^ 1, xset_ = ((it) + 1) % XSETS;                \
        const int set1_ = ((it) + 1) % NSETS, set2_ = ((it) + 2) % NSETS;                      \
        _Pragma("unroll") for (int i = 0; i < 16; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA1(0, i)                                                              \
            if (i < 8) TUNA_WIDE_READ1(1, 1, cur_, i)                                          \
            if (i >= 8 && (i & 1) == 0) TUNA_WIDE_DECODE((i - 8) >> 1, nxt_)                   \
            if (i >= 8 && (i & 1) == 1) TUNA_WIDE_LUT(set1_, 4 + ((i - 9) >> 1))               \
            if (i == 15) TUNA_WIDE_LOAD(set1_, min((step) + 1 + NSETS, s_last))                \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        _Pragma("unroll") for (int i = 0; i < 16; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA1(1, i)                                                              \
            if (i < 8) TUNA_WIDE_READ1(0, 2, cur_, i)                                          \
            if (i >= 8 && (i & 1) == 0) TUNA_WIDE_DECODE(4 + ((i - 8) >> 1), nxt_)             \
            if (i == 13 || i == 15) TUNA_WIDE_XSTAGE(xset_, (i - 13) >> 1, nxt_, (step) + 1)   \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        _Pragma("unroll") for (int i = 0; i < 16; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA1(0, i)                                                              \
            if (i < 8) TUNA_WIDE_READ1(1, 3, cur_, i)                                          \
            if (i >= 8 && i < 14) TUNA_WIDE_XSTAGE(xset_, 2 + (i - 8), nxt_, (step) + 1)       \
            if (i == 14) TUNA_WIDE_LOAD_X(xset_, min((step) + 1 + XSETS, s_last))              \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        __syncthreads(); /* the staged tiles are complete; this step's tiles are free once quarter 3 is read */ \
        _Pragma("unroll") for (int i = 0; i < 16; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA1(1, i)                                                              \
            if (i < 8) TUNA_WIDE_READ1(0, 0, nxt_, i)                                          \
            if (i >= 8 && (i & 1) == 0) TUNA_WIDE_LUT(set2_, (i - 8) >> 1)                     \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
    }

    // The same iteration with 16 x 16 tiles: four phases of 32 MFMAs.  Side work:
    //   phase 0 (half 0, weight tiles 0..3): weight fragments 4..7 of half 0; weights 0..3 of step + 1 and the
    //            table reads of dwords 4..7; refill
    //   phase 1 (half 0, tiles 4..7): weight fragments 0..3 of half 1, token fragments of half 1 as they come
    //            free; weights 4..7; activations 0..1
    //   phase 2 (half 1, tiles 0..3): weight fragments 4..7 of half 1; activations 2..7 and their refill; barrier
    //   phase 3 (half 1, tiles 4..7): weight fragments 0..3 and token fragments of half 0 of step + 1; table reads
    //            of dwords 0..3 of step + 2
#define TUNA_WIDE_ITER16(it, step)                                                               \
    {                                                                                          \
        const int cur_ = (it) & 1, nxt_ = cur_ ^ 1, xset_ = ((it) + 1) % XSETS;                \
        const int set1_ = ((it) + 1) % NSETS, set2_ = ((it) + 2) % NSETS;                      \
        _Pragma("unroll") for (int i = 0; i < 32; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA16(0, i & 3, i >> 2)                                                 \
            if (i < 4) TUNA_WIDE_READ_A(1, 0, cur_, 4 + i)                                     \
            if (i >= 8 && (i - 8) % 6 == 0) TUNA_WIDE_DECODE((i - 8) / 6, nxt_)                \
            if (i >= 11 && (i - 11) % 6 == 0) TUNA_WIDE_LUT(set1_, 4 + (i - 11) / 6)           \
            if (i == 31) TUNA_WIDE_LOAD(set1_, min((step) + 1 + NSETS, s_last))                \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        _Pragma("unroll") for (int i = 0; i < 32; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA16(1, 4 + (i & 3), i >> 2)                                           \
            if (i < 4) TUNA_WIDE_READ_A(0, 1, cur_, i)                                         \
            if ((i & 3) == 3) TUNA_WIDE_READ_B(1, cur_, i >> 2)                                \
            if (i >= 13 && i < 29 && (i - 13) % 4 == 0) TUNA_WIDE_DECODE(4 + (i - 13) / 4, nxt_) \
            if (i == 29 || i == 30) TUNA_WIDE_XSTAGE(xset_, i - 29, nxt_, (step) + 1)          \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        _Pragma("unroll") for (int i = 0; i < 32; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA16(0, i & 3, i >> 2)                                                 \
            if (i < 4) TUNA_WIDE_READ_A(1, 1, cur_, 4 + i)                                     \
            if (i >= 8 && i < 32 && (i - 8) % 4 == 0) TUNA_WIDE_XSTAGE(xset_, 2 + (i - 8) / 4, nxt_, (step) + 1) \
            if (i == 30) TUNA_WIDE_LOAD_X(xset_, min((step) + 1 + XSETS, s_last))              \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        __syncthreads(); /* the staged tiles are complete; this step's tiles are free once the last fragments are read */ \
        _Pragma("unroll") for (int i = 0; i < 32; ++i)                                         \
        {                                                                                      \
            TUNA_WIDE_MFMA16(1, 4 + (i & 3), i >> 2)                                           \
            if (i < 4) TUNA_WIDE_READ_A(0, 0, nxt_, i)                                         \
            if ((i & 3) == 3) TUNA_WIDE_READ_B(0, nxt_, i >> 2)                                \
            if (i >= 13 && i < 29 && (i - 13) % 4 == 0) TUNA_WIDE_LUT(set2_, (i - 13) / 4)     \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
    }

    __syncthreads();  // decode table complete
    // the first step staged with nothing to hide behind, and the table reads of the second step's dwords 0..3
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int j = 0; j < 4; ++j) TUNA_WIDE_LUT(0, 4 * h + j)
#pragma unroll
        for (int j = 0; j < 4; ++j) TUNA_WIDE_DECODE(4 * h + j, 0)
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) TUNA_WIDE_XSTAGE(0, i, 0, s0)
    TUNA_WIDE_LOAD(0, min(s0 + NSETS, s_last))
    TUNA_WIDE_LOAD_X(0, min(s0 + XSETS, s_last))
    __syncthreads();
    // (fragments first, table reads behind them: the order in which the loop leaves them)
    if constexpr (M32) {
#pragma unroll
        for (int t = 0; t < 8; ++t) TUNA_WIDE_READ1(0, 0, 0, t)
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) TUNA_WIDE_READ_A(0, 0, 0, t)
#pragma unroll
        for (int t = 0; t < 8; ++t) TUNA_WIDE_READ_B(0, 0, t)
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) TUNA_WIDE_LUT(1 % NSETS, j)

    int s = s0;
    for (; s + NSETS - 1 < s1; s += NSETS) {
#pragma unroll
        for (int it = 0; it < NSETS; ++it) {
            if constexpr (M32) TUNA_WIDE_ITER(it, s + it)
            else TUNA_WIDE_ITER16(it, s + it)
        }
    }
    // tail: up to NSETS - 1 more steps (the staging of a step past the end is harmless: its loads are clamped
    // and nothing uses the tiles)
#pragma unroll
    for (int it = 0; it < NSETS - 1; ++it)
        if (s + it < s1) {
            if constexpr (M32) TUNA_WIDE_ITER(it, s + it)
            else TUNA_WIDE_ITER16(it, s + it)
        }
#undef TUNA_WIDE_ITER16
#undef TUNA_WIDE_ITER
#undef TUNA_WIDE_MFMA16
#undef TUNA_WIDE_READ_B
#undef TUNA_WIDE_READ_A
#undef TUNA_WIDE_XSTAGE
#undef TUNA_WIDE_DECODE
#undef TUNA_WIDE_LUT
#undef TUNA_WIDE_MFMA1
#undef TUNA_WIDE_READ1
#undef TUNA_WIDE_LOAD_X
#undef TUNA_WIDE_LOAD

    if constexpr (!M32) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the last MFMAs have written their accumulators
    // ---- epilogue: slot sl (32 x 32 tiles: 4 * tile + q; 16 x 16 tiles: 8 tm + tn) is a float4 of this lane:
    // 4 consecutive weight rows of one token ------
    auto slot_value = [&](int sl) {
        if constexpr (M32) {
            const wide_f32x16 &t = acc[(sl >> 2) >> 2][(sl >> 2) & 3];
            const int q = sl & 3;
            return f32x4{t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
        } else {
            return acc16[sl >> 3][sl & 7];
        }
    };
    auto slot_row = [&](int sl) {
        if constexpr (M32) return row_base + wm_i * 128 + ((sl >> 2) >> 2) * 32 + (sl & 3) * 8 + h32 * 4;
        else return row_base + wm_i * 128 + (sl >> 3) * 16 + g * 4;
    };
    auto slot_tok = [&](int sl) {
        if constexpr (M32) return tok_base + wn_i * 128 + ((sl >> 2) & 3) * 32 + i32;
        else return tok_base + wn_i * 128 + (sl & 7) * 16 + i16;
    };
    f16 *outp = reinterpret_cast<f16 *>(a.out);
    const f16 *resp = reinterpret_cast<const f16 *>(a.residual);
    if (a.split_k == 1) {
#pragma unroll
        for (int sl = 0; sl < 64; ++sl) {
            const int row = slot_row(sl), tok = slot_tok(sl);
            if (tok < a.n && row + 4 <= a.m) {
                const f32x4 v = slot_value(sl);
                store_features4(outp, resp, a.epilogue, (size_t)tok, a.m, row, v[0], v[1], v[2], v[3]);
            }
        }
        return;
    }
    // split-K: fp32 partial tiles [split][tile][wave][slot][lane] as float4, the last workgroup of a tile to
    // arrive adds them in split order (deterministic, no atomics on out)
    const size_t tile_id = (size_t)tok_tile * a.row_tiles + row_tile;
    constexpr size_t kTileF4 = (size_t)4 * 64 * 64;  // float4s per partial tile
    f32x4 *ws4 = reinterpret_cast<f32x4 *>(a.ws);
    f32x4 *mine = ws4 + (tile_id * a.split_k + blockIdx.z) * kTileF4 + (size_t)wave * (64 * 64) + lane;
#pragma unroll
    for (int sl = 0; sl < 64; ++sl) {
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
    // (16-byte loads past this CU's and this XCD's caches - the writers sit on any XCD - two slots x two splits
    // requested before the first is awaited, as in gemm_tiled.hip; a slot's sum adds its splits in ascending order)
    const f32x4 *src = ws4 + tile_id * a.split_k * kTileF4 + (size_t)wave * (64 * 64) + lane;
    for (int sl = 0; sl < 64; sl += 2) {
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

size_t wide_lds_bytes() { return (size_t)kWideLutBytes + 2 * (size_t)kWideBuf; }

static OptInFlag g_wide_attr[16][4];

hipError_t launch_gemm_wide(const TiledArgs &args, bool mfma32, hipStream_t stream)
{
    const bool ktail = args.k % 64 != 0;
    const auto fn = ktail ? (mfma32 ? gemm_wide_kernel<2, true, true> : gemm_wide_kernel<2, false, true>)
                          : (mfma32 ? gemm_wide_kernel<2, true, false> : gemm_wide_kernel<2, false, false>);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    if ((e = ensure_lds_opt_in(g_wide_attr[dev][2 * ktail + mfma32], reinterpret_cast<const void *>(fn))) != hipSuccess) return e;
    TiledArgs a = args;
    a.row_tiles = ceil_div_i(args.m, kWideRows);
    a.tok_tiles = ceil_div_i(args.n, kWideTokens);
    if ((long long)a.row_tiles * a.tok_tiles > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    const dim3 grid((unsigned)(a.row_tiles * a.tok_tiles), 1, (unsigned)args.split_k);
    hipLaunchKernelGGL(fn, grid, dim3(kWideThreads), wide_lds_bytes(), stream, a);
    return hipGetLastError();
}

}  // namespace tuna
