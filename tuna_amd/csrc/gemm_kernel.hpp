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
//     LDS in chunks, as 16-byte pieces ordered [8-k slot][token], so that the ds_read_b128 of
//     a B fragment (16 lanes = 16 tokens of one slot = 256 contiguous bytes) is bank-conflict
//     free without padding; the staging reads global memory with every quad of lanes on 64
//     contiguous bytes of one token row and writes one k-step (4 slots x 16 tokens = 1 KB
//     contiguous) per wave instruction.
//   * Decode: the codebook is a run-time input, so it is a table.  LDS holds, for every
//     byte value, the half2 {code[hi nibble], code[lo nibble]} replicated once per lane
//     (row stride 256 B).  A lane's address is (byte << 8) | (lane << 2), built by one
//     v_perm_b32, and lands in the lane's own bank column: no bank conflicts for any
//     data.  One v_pk_mul_f16 applies the row's fp16 scale - the same single fp16
//     rounding as the reference's `smemCode.get(nib) * absMax` (kernel.cu:2178-2192).
//     Cost: 1 perm + 1 ds_read_b32 + 1 pk_mul per two weights.
//   * Persistent workgroups: the grid is at most (CUs x workgroups per CU); a workgroup
//     builds the decode table once (while its first tile's loads are in flight) and then
//     walks tiles (row tile, k segment).  The next tile's weight ring is requested BEFORE
//     the current tile's reduction and store, so the HBM stream never idles between tiles;
//     the small operands (row scales, first x chunk - mostly L2 hits) follow at the start of
//     the tile, where they do not hold registers across the epilogue.
//   * Split-K inside a workgroup: waves_k waves cover interleaved k-steps; their
//     accumulators meet in LDS and every thread sums a 1/waves_k share in wave order.  After
//     the four planes of a 64-row group a thread owns 4 consecutive output features of one
//     token.  With waves_k == 1 and no k split the accumulators are stored straight from
//     registers (16-byte stores, no LDS, no barrier).
//   * Split-K across workgroups, two schemes.  Fixed (split_k >= 1): tile t is (row tile
//     t / split_k, part t % split_k), parts of equal length.  Balanced (split_k == 0): the
//     k-steps of all row tiles, in units of 2^unit_log2 steps, are laid end to end and cut
//     into one contiguous range per workgroup, so every workgroup streams the same number
//     of bytes; a range covers whole row tiles plus at most two partial segments.  Either
//     way partial fp32 sums go to a workspace with device-coherent stores and the last
//     contributor to arrive (device-scope ticket counter) adds them in k order.  No atomics
//     on the output (unlike kernel.cu:2739-2745), no pre-zeroing, and the result does not
//     depend on arrival order.
//   * k_stagger: row tile r starts r * k_stagger steps into its k segment and wraps, so
//     that workgroups running side by side do not all walk the same 2^n-strided columns of
//     the weight matrix (and the same HBM channels) in lockstep.
//   * GRP variants (grouped GEMM, one weight matrix per group of tokens): row tiles count
//     over the groups that have tokens; the token range, output column base and weight rows
//     of a tile come from the group's entry of the offset list in the kernel arguments.
//   * The store applies the fused epilogue (none / + residual / SiLU(gate) * up on
//     interleaved rows), see epilogue.hpp.
#pragma once
#include "epilogue.hpp"

namespace tuna {


__device__ __forceinline__ uint32_t f16_bits(f16 h)
{
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

// s_waitcnt immediate for "at most n vector memory operations outstanding", the other counters
// unconstrained (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
constexpr int wait_vmcnt(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

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

// One 16-byte device-coherent store of partial sums: the write-through form (sc1) the
// compiler emits for a relaxed device-scope atomic store, which it only offers 4 bytes wide
// (four of those cost four 32-byte-granular writes to memory for every 16 bytes).  The
// caller orders it with an explicit s_waitcnt vmcnt(0) before signalling.
__device__ __forceinline__ void store_partial(float *dst, f32x4 v)
{
    // the s_nop covers the wait state a store wider than 8 bytes needs before its data
    // registers may be overwritten (the compiler does not see inside the asm)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0" : : "v"(dst), "v"(v) : "memory");
}

// Four 16-byte device-coherent loads of partial sums (the counterpart of store_partial) and the
// wait for them, in one statement: the compiler does not know that the results arrive later,
// so nothing of its own may come between the loads and the wait.
__device__ __forceinline__ void load_partials4(const float *s0, const float *s1, const float *s2, const float *s3, f32x4 &p0,
                                               f32x4 &p1, f32x4 &p2, f32x4 &p3)
{
    asm volatile(
        "global_load_dwordx4 %0, %4, off sc1\n\t"
        "global_load_dwordx4 %1, %5, off sc1\n\t"
        "global_load_dwordx4 %2, %6, off sc1\n\t"
        "global_load_dwordx4 %3, %7, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(p0), "=&v"(p1), "=&v"(p2), "=&v"(p3)
        : "v"(s0), "v"(s1), "v"(s2), "v"(s3)
        : "memory");
}

// Cross-wave sum of NP accumulator planes for thread (wk, lane) of a row group.  A plane
// buffer holds, per wave of the row group, 256 floats; the thread sums float
// f = (i*WK + wk)*64 + lane of every wave, in wave order, for each i with f < 256.  WK (the
// number of waves along k) is a template argument so that all WK*NP loads of a thread are
// issued before the first add: with a run-time wave count the loop took one LDS round trip
// per wave and plane (32 of them, 1.3 us, for 8 waves).
template <int WK, int NP, int LIM>
__device__ __forceinline__ void sum_planes(const float *buf, size_t plane_floats, int wm, int wk, int lane,
                                           float (&o)[4][4], int j0)
{
    if constexpr (LIM == 0) {
        // register-starved variants (two workgroups per CU): one LDS round trip at a time
#pragma unroll
        for (int j = 0; j < NP; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int f = (i * WK + wk) * 64 + lane;
                float sum = 0.f;
                if (f < 256)
                    for (int w = 0; w < WK; ++w) sum += buf[j * plane_floats + (size_t)(wm * WK + w) * 256 + f];
                o[i][j0 + j] = sum;
            }
        return;
    }
    constexpr int NI = WK >= 4 ? 1 : 4 / WK;                        // values of i that can give f < 256
    constexpr int LIM1 = LIM > 0 ? LIM : 1;
    constexpr int JB = LIM1 / (WK * NI) < NP ? (LIM1 / (WK * NI) > 0 ? LIM1 / (WK * NI) : 1) : NP;  // planes per batch of <= LIM loads
    const float *base = buf + (size_t)wm * (WK * 256);
    if (WK > 4 && wk >= 4) return;  // (wave-uniform) the 256 floats of a plane are owned by waves 0..3
#pragma unroll
    for (int jb = 0; jb < NP; jb += JB) {
        float v[JB][NI][WK];
#pragma unroll
        for (int j = 0; j < JB; ++j)
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int f = min((i * WK + wk) * 64 + lane, 255);  // clamped: unused sums are discarded by the caller
#pragma unroll
                for (int w = 0; w < WK; ++w) v[j][i][w] = base[(jb + j) * plane_floats + (size_t)w * 256 + f];
            }
        // all loads of the batch before the first add (the scheduler otherwise pairs each load
        // with its add to save registers, which is the serial chain again)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < JB; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float sum = 0.f;
                if (i < NI) {
#pragma unroll
                    for (int w = 0; w < WK; ++w) sum += v[j][i < NI ? i : 0][w];
                }
                o[i][j0 + jb + j] = sum;
            }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int NP, int LIM>
__device__ __forceinline__ void sum_planes_any(int wk_log2, const float *buf, size_t plane_floats, int wm, int wk, int lane,
                                               float (&o)[4][4], int j0)
{
    switch (wk_log2) {
    case 0: sum_planes<1, NP, LIM>(buf, plane_floats, wm, wk, lane, o, j0); break;
    case 1: sum_planes<2, NP, LIM>(buf, plane_floats, wm, wk, lane, o, j0); break;
    case 2: sum_planes<4, NP, LIM>(buf, plane_floats, wm, wk, lane, o, j0); break;
    case 3: sum_planes<8, NP, LIM>(buf, plane_floats, wm, wk, lane, o, j0); break;
    default: sum_planes<16, NP, LIM>(buf, plane_floats, wm, wk, lane, o, j0); break;
    }
}

// x staging, global -> registers -> LDS, XB 16-byte pieces per thread (4, or 8 for the deepest
// prefetch ring, whose smallest chunk is twice as long).
// Piece p of a chunk is token row (p % (16*TT)), 8-k slot (p / (16*TT)) and lives at LDS
// byte 16*p.  All loads of a batch are issued before the first LDS write (addresses are
// clamped so the loads are unconditional; invalid pieces are zeroed by a select).
template <int XB>
struct XStage {
    u32x4 v[XB];
};

// Where a segment's k range [hi_k - span_k, hi_k) starts: the walk begins rot_k elements into
// it and wraps around (all in k elements, multiples of 32).
struct KRot {
    int rot_k, hi_k, span_k;
};

__device__ __forceinline__ int k_physical(int k_logical, const KRot &kr)
{
    const int kp = k_logical + kr.rot_k;
    return kp >= kr.hi_k ? kp - kr.span_k : kp;
}

// Piece p = tid + b*nthreads of a chunk: its lane (p % 64) picks token row lane / 4 of a 16-token
// tile and 8-k group lane % 4 of a k-step, p / 64 picks the k-step and (TT > 1) the token tile.
// Every quad of lanes reads 64 contiguous bytes of one token row - with neighbouring lanes on
// different rows (the order the MFMA wants) a wave instruction takes about three times as long
// in the address path - and a wave instruction writes the 16 rows x 4 slots of one k-step and
// tile: with the layout byte = slot*(256*TT) + row*16 that is 4 runs of 256 contiguous bytes,
// bank-conflict free without padding, and the 16 rows of a slot are a contiguous B fragment.
template <int TT, int XB>
__device__ __forceinline__ void x_stage_load(XStage<XB> &st, const f16 *xg, int nthreads, int tid, int tok0, int kbase, int n,
                                             int k, const KRot &kr)
{
    // uniform 64-bit base (the tile's first token row) + a 32-bit per-lane offset: a tile spans
    // at most 16*TT rows of at most 2^23 k, so no 64-bit address lives in vector registers.
    // Rows past n and slots past the chunk or k are clamped here and zeroed by x_stage_store.
    const unsigned char *row0 = reinterpret_cast<const unsigned char *>(xg + (size_t)tok0 * k);
    const uint32_t row_bytes = (uint32_t)k * 2u;
    const int r_max = n - 1 - tok0;
    // (an opaque copy of the thread id: the per-piece offsets below do not depend on the chunk,
    // and hoisted out of the chunk loop they would sit in registers across the MFMA loop)
    asm volatile("" : "+v"(tid));
    const int row_l = (tid & 63) >> 2, grp = tid & 3;
#pragma unroll
    for (int b = 0; b < XB; ++b) {
        const int wv = (tid + b * nthreads) >> 6;  // wave instruction of the chunk: k-step wv / TT, token tile wv % TT
        const int row = (wv % TT) * 16 + row_l;
        const int kk = min(k_physical(kbase + (wv / TT) * 32 + grp * 8, kr), k - 8);
        st.v[b] = *reinterpret_cast<const u32x4 *>(row0 + (__umul24((uint32_t)min(row, r_max), row_bytes) + (uint32_t)kk * 2u));
    }
}

template <int TT, int XB>
__device__ __forceinline__ void x_stage_store(const XStage<XB> &st, unsigned char *xs, int nthreads, int tid, int pieces,
                                              int tok0, int kbase, int n, int k, const KRot &kr)
{
    asm volatile("" : "+v"(tid));  // (as in x_stage_load)
    const int row_l = (tid & 63) >> 2, grp = tid & 3;
#pragma unroll
    for (int b = 0; b < XB; ++b) {
        const int p = b * nthreads + tid;
        if (p < pieces) {
            const int wv = p >> 6;
            const int row = (wv % TT) * 16 + row_l, slot = (wv / TT) * 4 + grp;
            const int kl = kbase + slot * 8;
            const bool ok = tok0 + row < n && kl < kr.hi_k && k_physical(kl, kr) < k;
            *reinterpret_cast<u32x4 *>(xs + slot * (256 * TT) + row * 16) = ok ? st.v[b] : u32x4{0u, 0u, 0u, 0u};
        }
    }
}

// MODE 0: persistent workgroups walking tiles; 1: the same for grouped launches (GRP below);
// 2: the launch has one workgroup per tile and a fixed split (ONE below) - no tile walk, no
// balanced split: the lean path for the small shapes, whose time is instruction issue between
// the first and the last memory access rather than bandwidth.
template <int RW, int U, int TT, int DEC, int MAXT, int MINW, int MODE>
__global__ __launch_bounds__(MAXT, MINW) void gemm_kernel(const GemmArgs a)
{
    constexpr bool GRP = MODE == 1;
    constexpr bool ONE = MODE == 2;
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int NACC = RW * 4 * TT;  // float4 accumulator planes per lane
    constexpr int LUT_B = (DEC == TUNA_DECODE_GEMM) ? kLutBytes : 64;
    constexpr int RED_LIM = MINW >= 4 ? 0 : 32;  // LDS loads in flight per thread in the cross-wave sums (0: unbatched)

    const int tid = threadIdx.x;
    // Every kernel argument the first tile needs is requested here, in one batch with one wait:
    // left to itself the compiler fetches them where they are first used, three to four
    // dependent round trips to memory before the first weight load can be issued.  (Not a
    // volatile asm: that would count as a store and turn the codebook's scalar loads below
    // into vector loads.  Its result, zero, is folded into the wave index to pin it here.)
    int args_here;
    asm("s_mov_b32 %0, 0"
        : "=s"(args_here)
        : "s"(a.q), "s"(a.x), "s"(a.code), "s"(a.absmax), "s"(a.ws), "s"(a.counters), "s"(a.epilogue), "s"(a.m), "s"(a.n), "s"(a.k), "s"(a.waves_m), "s"(a.waves_k),
          "s"(a.split_k), "s"(a.wk_log2), "s"(a.steps_total), "s"(a.steps_per_split), "s"(a.chunk_steps), "s"(a.chunk_log2),
          "s"(a.row_tiles), "s"(a.xcd_swizzle), "s"(a.k_stagger), "s"(a.tiles_total), "s"(a.balanced), "s"(a.unit_log2),
          "s"(a.units_per_tile), "s"(a.units_total), "s"(gridDim.x), "s"(blockDim.x));
    const bool bal = ONE ? false : (a.balanced != 0);
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6) + args_here;
    const int wk = wave & (a.waves_k - 1);
    const int wm = wave >> a.wk_log2;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int nthreads = (int)blockDim.x;
    // tokens of the tile being fetched / computed: [tok0, min(tok0 + 16*TT, n_tok)); rows of
    // `out` are out_ld long and the tile's group starts at weight row out_row0
    int tok0 = blockIdx.y * (TT * 16), n_tok = a.n, out_row0 = 0;
    const int out_ld = GRP ? a.group_rows : a.m;
    const int rows_wg = a.waves_m * (RW * kRowsPerLoad);
    const int kb_total = a.k >> 3;
    const int mb_last = (a.m >> 3) - 1;
    const int g_last = min(g, kb_total - 1 - (a.steps_total - 1) * 4);  // last k-step may be short
    const f16 *xg = reinterpret_cast<const f16 *>(a.x);
    const int x_pieces = (TT * 16 * 4) << a.chunk_log2;  // 16-byte pieces per x chunk
    const int s_stride = a.waves_k;                      // k-steps between a wave's consecutive iterations

    // LDS: [decode table | work area].  The work area holds the x chunk during a tile's main
    // loop and the reduction planes + fp16 output tile during its epilogue; the table is never
    // overwritten, it serves every tile of this workgroup.
    unsigned char *lut = smem;
    unsigned char *work = smem + LUT_B;
    const uint32_t lane4 = (uint32_t)lane << 2;

    // ---- persistent tile walk -------------------------------------------------------------
    int wg = blockIdx.x;
    const int n_wg = gridDim.x;
    if (a.xcd_swizzle && (n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);

    // The walk.  Fixed split: tile t = (row tile, k split) for t = wg, wg + n_wg, ... below
    // row_tiles * split_k.  Balanced split: the k range of every row tile is cut into units
    // of 2^unit_log2 k-steps, all units of all row tiles form one sequence, workgroup w owns
    // units [w*T/n_wg, (w+1)*T/n_wg) of it and walks them as segments that end at row tile
    // boundaries.  `part` is the segment's slot among the partial sums of its row tile
    // (-1: the segment is the whole row tile, its sums are final).
    int t_begin = wg, t_end = a.tiles_total;
    if (a.balanced) {
        t_begin = balanced_begin((unsigned)wg, (unsigned)n_wg, (unsigned)a.units_total);
        t_end = balanced_begin((unsigned)wg + 1u, (unsigned)n_wg, (unsigned)a.units_total);
    }
    // state of the tile being fetched / computed
    int row_tile = 0, part = -1, sb = 0, nsteps = 0, n_it = 0, s_first = 0, t_next = 0;
    int seg_hi = 0, s_clamp = 0, rot = 0, row_base = 0;
    uint32_t lb[RW], lb_last[RW];
    u32x4 wq[U][RW];
    constexpr int XB = U == 8 ? 8 : 4;
    XStage<XB> xst;

    // Unconditional by design: a load whose step lies beyond this wave's share is clamped
    // to the segment's last k-step and its data is never used.  Only loads that are always issued
    // let the compiler count outstanding loads exactly (s_waitcnt vmcnt(N > 0)).
    // address = q + [uniform: 128 bytes per k-step, in SGPRs] + [per lane: block row, half, g]
#define TUNA_LOAD_STEP(u, it)                                                                  \
    {                                                                                          \
        int s_ = min(s_first + (it) * s_stride, s_clamp) + rot;                                \
        if (s_ >= seg_hi) s_ -= nsteps;                                                        \
        const unsigned char *base_ = a.q + (size_t)s_ * 128;                                   \
        const bool last_ = s_ == a.steps_total - 1;                                            \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) wq[u][rw] = __builtin_nontemporal_load( \
            reinterpret_cast<const u32x4 *>(base_ + (last_ ? lb_last[rw] : lb[rw])));          \
    }

    // Grouped launches: a tile whose group has no tokens in this token chunk is not walked at
    // all (its weights are never read).  Advances `t` to the workgroup's next tile with work.
#define TUNA_SKIP_EMPTY(t)                                                                      \
    if constexpr (GRP) {                                                                        \
        while ((t) < t_end) {                                                                  \
            int rt_, nx_;                                                                      \
            if (a.balanced) {                                                                  \
                const Segment sg_ = balanced_segment((t), t_begin, t_end, a.units_per_tile, a.unit_log2, a.steps_total); \
                rt_ = sg_.row_tile;                                                            \
                nx_ = sg_.next;                                                                \
            } else {                                                                           \
                rt_ = (t) / a.split_k;                                                         \
                nx_ = (t) + n_wg;                                                              \
            }                                                                                  \
            const int e_ = a.act[rt_ / a.tiles_per_group];                                     \
            if (a.tok_off[e_] + (int)blockIdx.y * (TT * 16) < a.tok_off[e_ + 1]) break;        \
            (t) = nx_;                                                                         \
        }                                                                                      \
    }

    // Request what tile `t` streams from HBM first: the weight ring.  (The row scales and the
    // first x chunk are small and mostly L2 hits; they are requested at the start of the tile,
    // behind these loads: prefetched here they would cost 20 registers across the previous
    // tile's epilogue.)
#define TUNA_TILE_FETCH(t)                                                                      \
    {                                                                                          \
        if (a.balanced) {                                                                      \
            const Segment sg_ = balanced_segment((t), t_begin, t_end, a.units_per_tile, a.unit_log2, a.steps_total); \
            row_tile = sg_.row_tile;                                                           \
            sb = sg_.sb;                                                                       \
            nsteps = sg_.nsteps;                                                               \
            part = sg_.part;                                                                   \
            t_next = sg_.next;                                                                 \
        } else {                                                                               \
            row_tile = (t) / a.split_k;                                                        \
            part = (t) - row_tile * a.split_k;                                                 \
            sb = part * a.steps_per_split;                                                     \
            nsteps = max(min(a.steps_total, sb + a.steps_per_split) - sb, 0);                  \
            if (a.split_k == 1) part = -1;                                                     \
            t_next = (t) + n_wg;                                                               \
        }                                                                                      \
        row_base = row_tile * rows_wg;                                                         \
        if constexpr (GRP) {                                                                    \
            /* row tiles count over the groups that have tokens only (a.act lists them) */     \
            const int slot_ = row_tile / a.tiles_per_group;                                    \
            const int e_ = a.act[slot_];                                                       \
            tok0 = a.tok_off[e_] + (int)blockIdx.y * (TT * 16);                                \
            n_tok = a.tok_off[e_ + 1];                                                         \
            out_row0 = e_ * a.group_rows;                                                      \
            row_base = out_row0 + (row_tile - slot_ * a.tiles_per_group) * rows_wg;            \
        }                                                                                      \
        const int row0_ = row_base + wm * (RW * kRowsPerLoad);                                 \
        n_it = nsteps > wk ? (nsteps - wk + a.waves_k - 1) >> a.wk_log2 : 0;                   \
        s_first = sb + wk;                                                                     \
        /* stagger: this row tile walks its k range starting rot steps in, wrapping around */  \
        seg_hi = sb + nsteps;                                                                  \
        s_clamp = min(seg_hi, a.steps_total) - 1;                                              \
        rot = (a.k_stagger && nsteps > 1) ? (int)(((unsigned)row_tile * (unsigned)a.k_stagger) % (unsigned)nsteps) : 0; \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw)                                      \
        {                                                                                      \
            const int mb_ = min(((row0_ + rw * kRowsPerLoad) >> 3) + (i16 >> 1), mb_last);     \
            const uint32_t rowb_ = (uint32_t)mb_ * (uint32_t)kb_total * 32u + (uint32_t)(i16 & 1) * 16u; \
            lb[rw] = rowb_ + (uint32_t)g * 32u;                                                \
            lb_last[rw] = rowb_ + (uint32_t)g_last * 32u;                                      \
        }                                                                                      \
        _Pragma("unroll") for (int u = 0; u < U; ++u) TUNA_LOAD_STEP(u, u)                     \
    }

    // The small operands of a tile: row scales and the first x chunk (mostly L2 hits).
#define TUNA_TILE_SMALL_LOADS()                                                                 \
    {                                                                                          \
        const int row0_ = row_base + wm * (RW * kRowsPerLoad);                                 \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) _Pragma("unroll") for (int j = 0; j < 4; ++j) \
        {                                                                                      \
            const int row_ = row0_ + rw * kRowsPerLoad + i16 * 4 + j;                          \
            sc32c[rw][j] = a.absmax[min(row_, a.m - 1)]; /* rows past m are never stored */    \
        }                                                                                      \
        krot = KRot{rot * kStepK, seg_hi * kStepK, nsteps * kStepK};                           \
        x_stage_load<TT, XB>(xst, xg, nthreads, tid, tok0, sb * kStepK, n_tok, a.k, krot); \
    }

    int t = t_begin;
    // The 16 codes are uniform and read before the kernel's first store, so they come through
    // the scalar cache: waiting for them does not wait for the weight loads (vector loads
    // return in order).
    const float *__restrict__ code_ptr = a.code;
    float code_s[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) code_s[i] = code_ptr[i];
    // scales and first x chunk of the tile about to be computed (requested right behind its
    // weight ring: at the start for the first tile, after the epilogue for the following ones)
    float sc32c[RW][4] = {};
    KRot krot{0, 0, 0};
    TUNA_SKIP_EMPTY(t)
    if (t < t_end) {
        TUNA_TILE_FETCH(t)
        if constexpr (!GRP) TUNA_TILE_SMALL_LOADS()
        // ---- decode table, once per workgroup, built while the first tile's loads are in flight
        float code_lane = 0.f;  // (a select between two loads would be turned back into a vector load)
#pragma unroll
        for (int i = 0; i < 16; ++i) code_lane = i16 == i ? code_s[i] : code_lane;
        if constexpr (DEC == TUNA_DECODE_GEMM) {
            // Lane l holds fp16(code[l % 16]) (kernel.cu:2800 rounds the codebook to fp16);
            // entries are gathered across lanes, no memory traffic.
            // piece p: 16 bytes of row (p >> 4); all 64 slots of a row hold the same half2
            const int code_bits = (int)f16_bits((f16)code_lane);
            // four pieces per thread and round: the eight cross-lane reads of a round are in
            // flight together instead of one LDS round trip per piece
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
        } else {
            if (tid < 16) reinterpret_cast<float *>(lut)[tid] = code_lane;
        }
    }

    // One k-step of this wave: B fragments from LDS, decode 4*RW dwords, 4*RW*TT MFMAs.
#define TUNA_CONSUME(u, xoff)                                                                   \
    {                                                                                          \
        f16x8 b_[TT];                                                                          \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) b_[tt] =                             \
            *reinterpret_cast<const f16x8 *>(xb + tt * 256 + (xoff));                          \
        _Pragma("unroll") for (int rw = 0; rw < RW; ++rw) _Pragma("unroll") for (int j = 0; j < 4; ++j) \
        {                                                                                      \
            const f16x8 av_ = decode_dword<DEC>(wq[u][rw][j], lut, lane4, sc16[rw][j], sc32c[rw][j]); \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] =                 \
                __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_[tt], acc[rw][j][tt], 0, 0, 0);  \
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
    const int wstep = a.waves_k * (1024 * TT);   // LDS bytes between this wave's consecutive steps

    while (t < t_end) {
        // (grouped variants request them here for every tile: with a second place of request
        // the compiler keeps two copies of the staging registers)
        if constexpr (GRP) TUNA_TILE_SMALL_LOADS()
        // ---- this tile's scales (fp16 like the reference's staging, kernel.cu:2770) and the
        //      first x chunk, requested behind the ring loads already in flight
        f16x2 sc16[RW][4];
#pragma unroll
        for (int rw = 0; rw < RW; ++rw)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f16 h = (f16)sc32c[rw][j];
                sc16[rw][j] = f16x2{h, h};
            }
        f32x4 acc[RW][4][TT];
#pragma unroll
        for (int rw = 0; rw < RW; ++rw)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) acc[rw][j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int cur_row_tile = row_tile, cur_part = part, cur_sb = sb;
        const int cur_tok0 = tok0, cur_ntok = n_tok, cur_out_row0 = out_row0, cur_row_base = row_base;
        const int n_chunks = (nsteps + a.chunk_steps - 1) >> a.chunk_log2;
        int it = 0;  // this wave's next iteration (multiple of U)

        // the work area is free again once every wave has left the previous tile's epilogue
        __syncthreads();
        if (n_chunks > 0) x_stage_store<TT, XB>(xst, work, nthreads, tid, x_pieces, cur_tok0, cur_sb * kStepK, cur_ntok, a.k, krot);
        // The x pieces are the youngest loads in flight, so a thread that stored one has waited for
        // everything; a thread with no piece to store has not, and the compiler then carries its
        // staging registers as pending loads through the tile: reusing one of them inside the main
        // loop gets a wait for ALL loads there, which empties the weight ring once per group.
        // The explicit wait makes "nothing pending" a fact on every path.
        __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
        __syncthreads();

        for (int c = 0; c < n_chunks; ++c) {
            const int it_chunk0 = c * ipc;
            const bool has_next = c + 1 < n_chunks;
            // B fragment of lane (token i16, k-group g), local step sl: slot sl*4+g, piece slot*16*TT + i16
            const unsigned char *xb = work + g * (256 * TT) + i16 * 16 + wk * (1024 * TT) - it_chunk0 * wstep;
            if (has_next) {
                // A chunk with a successor is full: every wave owns all ipc iterations of it.
                const int it_peel = it_chunk0 + ipc - U;
                while (it < it_peel) TUNA_GROUP()
                // Last group of the chunk: the next chunk of x is fetched into registers first, so
                // that after the group exactly U*RW younger loads are in flight and the wait before
                // the LDS write below is an exact vmcnt, not a drain of the weight ring.
                const int kbase = (cur_sb + (c + 1) * a.chunk_steps) * kStepK;
                x_stage_load<TT, XB>(xst, xg, nthreads, tid, cur_tok0, kbase, cur_ntok, a.k, krot);
                TUNA_GROUP()
                __syncthreads();  // every wave is done reading chunk c
                // exactly the group's U*RW refills are younger than the x pieces (see above)
                __builtin_amdgcn_s_waitcnt(wait_vmcnt(U * RW));
                x_stage_store<TT, XB>(xst, work, nthreads, tid, x_pieces, cur_tok0, kbase, cur_ntok, a.k, krot);
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

        // ---- next tile: get its loads going before this tile's reduction and store ---------
        if constexpr (ONE) {
            t = t_end;
        } else {
            t = t_next;
            TUNA_SKIP_EMPTY(t)
            if (t < t_end) TUNA_TILE_FETCH(t)
        }

        // ---- workgroup reduction and store ---------------------------------------------------
        // A plane is one float4 per lane = 256 floats [lane][4].  The waves_k waves of a row
        // group put their copies of a plane side by side in LDS (two buffers alternate, so one
        // barrier per plane - or per four planes when the work area holds eight of them) and
        // thread (wk, lane) sums the floats f = (i*waves_k + wk)*64 + lane
        // of it in wave order.  Float f = l*4 + v of the plane of MFMA j is token l%16 and
        // weight row 16*(l/16) + 4*v + j of the wave's 64: after the four planes j = 0..3 a
        // thread owns 4 consecutive output features of one token and stores them as 8 bytes.
        // The per-thread index arithmetic does not depend on the tile; an opaque copy of the
        // lane id keeps the compiler from hoisting it out of the tile loop into registers that
        // would stay live across the main loop.
        int lane_e = lane, wk_e = wk, wm_e = wm;
        asm volatile("" : "+v"(lane_e));
        asm volatile("" : "+s"(wk_e), "+s"(wm_e));
        const size_t plane_floats = (size_t)(a.waves_m * a.waves_k) * 256;  // one buffer
        float *redf = reinterpret_cast<float *>(work);
        const size_t tile_id = (size_t)blockIdx.y * a.row_tiles + cur_row_tile;
        // Partial sums of a segment: [wm][rw][tt][f][j] floats.  Fixed split: the row tile's
        // split_k segments lie side by side in split order.  Balanced split: a workgroup owns
        // two slots (a workgroup has at most two segments that are not whole row tiles: the
        // one that starts at its first unit - slot 0 - and the one that ends at its last -
        // slot 1).  The contributors of a row tile are consecutive workgroups in k order, and
        // only the first of them can have used its slot 1.  Contributor c of this row tile is
        // at src0 + c*src_stride - (c > 0 ? src_adj : 0).
        const bool partial = cur_part >= 0;
        const size_t seg_floats = (size_t)a.waves_m * (NACC * 256);
        const float *src0 = a.ws;
        size_t src_stride = 0, src_adj = 0;
        float *mine = a.ws;
        unsigned n_contrib = 1;
        if (partial) {
            if (a.balanced) {
                const unsigned nw = (unsigned)n_wg;
                unsigned w_lo, first_slot;
                balanced_contributors((unsigned)cur_row_tile, (unsigned)a.units_per_tile, (unsigned)a.units_total, nw, &w_lo,
                                      &n_contrib, &first_slot);
                float *wsy = a.ws + (size_t)blockIdx.y * nw * 2 * seg_floats;
                src0 = wsy + ((size_t)w_lo * 2 + first_slot) * seg_floats;
                src_stride = 2 * seg_floats;
                src_adj = first_slot * seg_floats;
                mine = wsy + ((size_t)wg * 2 + (unsigned)cur_part) * seg_floats + (size_t)wm_e * (NACC * 256);
            } else {
                float *wst = a.ws + (tile_id * a.split_k) * seg_floats;
                src0 = wst;
                src_stride = seg_floats;
                mine = wst + (size_t)cur_part * seg_floats + (size_t)wm_e * (NACC * 256);
                n_contrib = (unsigned)a.split_k;
            }
        }
        f16 *outp = reinterpret_cast<f16 *>(a.out);
        const f16 *resp = reinterpret_cast<const f16 *>(a.residual);
        bool write_out = true;
        if (a.waves_k == 1 && !partial) {
            // No k split at all: the wave's accumulators are final.  Lane (token i16, group g)
            // owns 16 consecutive output features, acc[rw][j][tt][v] being feature 4*v + j of
            // them: two 16-byte stores per 64-row group, no LDS, no barrier.
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                const int tok = cur_tok0 + tt * 16 + (lane_e & 15);
#pragma unroll
                for (int rw = 0; rw < RW; ++rw) {
                    const int rb = cur_row_base + wm_e * (RW * kRowsPerLoad) + rw * 64 + (lane_e >> 4) * 16;
                    if (a.epilogue == TUNA_EPILOGUE_NONE) {
                        f16x8 lo, hi;
#pragma unroll
                        for (int v = 0; v < 2; ++v)
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                lo[v * 4 + j] = (f16)acc[rw][j][tt][v];
                                hi[v * 4 + j] = (f16)acc[rw][j][tt][v + 2];
                            }
                        f16 *dst = outp + (size_t)tok * out_ld + (rb - cur_out_row0);
                        if (tok < cur_ntok && rb + 8 <= a.m) *reinterpret_cast<f16x8 *>(dst) = lo;
                        if (tok < cur_ntok && rb + 16 <= a.m) *reinterpret_cast<f16x8 *>(dst + 8) = hi;
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (tok < cur_ntok && rb + v * 4 + 4 <= a.m)
                                store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, rb + v * 4 - cur_out_row0,
                                                acc[rw][0][tt][v], acc[rw][1][tt][v], acc[rw][2][tt][v], acc[rw][3][tt][v]);
                    }
                }
            }
            if constexpr (MODE == 0) if (t < t_end) TUNA_TILE_SMALL_LOADS()
            continue;
        }
        __syncthreads();  // every wave has left the main loop: the work area is free
#pragma unroll
        for (int rw = 0; rw < RW; ++rw)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                float o[4][4];  // [i][j]
                if (a.planes_log2 == 2) {
                    // the work area holds all four planes of a row group at once: one barrier
                    float *buf = redf + (size_t)((rw * TT + tt) % 2) * 4 * plane_floats;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        reinterpret_cast<f32x4 *>(buf + j * plane_floats)[(size_t)(wm_e * a.waves_k + wk_e) * 64 + lane_e] =
                            acc[rw][j][tt];
                    __syncthreads();
                    sum_planes_any<4, RED_LIM>(a.wk_log2, buf, plane_floats, wm_e, wk_e, lane_e, o, 0);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float *buf = redf + ((rw * TT + tt) * 4 + j) % 2 * plane_floats;
                        reinterpret_cast<f32x4 *>(buf)[(size_t)(wm_e * a.waves_k + wk_e) * 64 + lane_e] = acc[rw][j][tt];
                        __syncthreads();
                        sum_planes_any<1, RED_LIM>(a.wk_log2, buf, plane_floats, wm_e, wk_e, lane_e, o, j);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int f = ((i << a.wk_log2) + wk_e) * 64 + lane_e;
                    if (f >= 256) continue;
                    if (!partial) {
                        const int l = f >> 2, v = f & 3;
                        const int tok = cur_tok0 + tt * 16 + (l & 15);
                        const int row = cur_row_base + wm_e * (RW * kRowsPerLoad) + rw * 64 + (l >> 4) * 16 + v * 4;
                        if (tok < cur_ntok && row + 4 <= a.m)
                            store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, row - cur_out_row0, o[i][0], o[i][1],
                                            o[i][2], o[i][3]);
                    } else {
                        float *dst = mine + ((size_t)(rw * TT + tt) * 256 + f) * 4;
                        store_partial(dst, f32x4{o[i][0], o[i][1], o[i][2], o[i][3]});
                    }
                }
            }

        if (partial) {
            // Partials travel as device-scope relaxed atomics (write-through stores, L2-bypassing
            // loads): coherent across the 8 XCD L2s without the L2 write-back/invalidate that a
            // device-scope release/acquire fence costs on every workgroup.  Order is given by
            // "all my stores have completed" (an explicit s_waitcnt vmcnt(0)) before the barrier
            // that precedes the arrival counter's increment.
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): a workgroup-scope fence does not wait for global stores
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();  // also: every read of the reduction buffers is done
            volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(work);
            if (wk_e + wm_e == 0 && lane_e == 0)
                *ticket = __hip_atomic_fetch_add(a.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            write_out = *ticket == n_contrib - 1u;
            if (write_out) {
                // last workgroup of this row tile: every partial is in memory; add them in k order
                if (wk_e + wm_e == 0 && lane_e == 0)
                    __hip_atomic_store(a.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                for (int rt = 0; rt < RW * TT; ++rt)
                    for (int i = 0; i < 4; ++i) {
                        const int f = ((i << a.wk_log2) + wk_e) * 64 + lane_e;
                        if (f >= 256) break;
                        const float *src = src0 + (size_t)wm_e * (NACC * 256) + ((size_t)rt * 256 + f) * 4;
                        // several contributors per round trip (indices are clamped so that the loads
                        // are unconditional and all in flight together); summed in k order
                        float s4[4] = {0.f, 0.f, 0.f, 0.f};
                        constexpr unsigned FB = 4;
                        for (unsigned sp0 = 0; sp0 < n_contrib; sp0 += FB) {
                            float pv[FB][4];
#pragma unroll
                            for (unsigned b = 0; b < FB; ++b) {
                                const unsigned sp = min(sp0 + b, n_contrib - 1u);
                                const float *sps = src + (size_t)sp * src_stride - (sp ? src_adj : 0);
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    pv[b][j] = __hip_atomic_load(sps + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            }
#pragma unroll
                            for (unsigned b = 0; b < FB; ++b)
                                if (sp0 + b < n_contrib) {
#pragma unroll
                                    for (int j = 0; j < 4; ++j) s4[j] += pv[b][j];
                                }
                        }
                        const int rw = rt / TT, tt = rt % TT;
                        const int l = f >> 2, v = f & 3;
                        const int tok = cur_tok0 + tt * 16 + (l & 15);
                        const int row = cur_row_base + wm_e * (RW * kRowsPerLoad) + rw * 64 + (l >> 4) * 16 + v * 4;
                        if (tok < cur_ntok && row + 4 <= a.m)
                            store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, row - cur_out_row0, s4[0], s4[1], s4[2],
                                            s4[3]);
                    }
            }
        }
        if constexpr (MODE == 0) if (t < t_end) TUNA_TILE_SMALL_LOADS()
    }
#undef TUNA_GROUP
#undef TUNA_CONSUME
#undef TUNA_TILE_FETCH
#undef TUNA_SKIP_EMPTY
#undef TUNA_TILE_SMALL_LOADS
#undef TUNA_LOAD_STEP
}

}  // namespace tuna
