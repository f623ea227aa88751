// Several independent 1..16-token GEMMs in ONE launch of persistent workgroups (gfx950, wave64).
//
// At 16 tokens a projection of a 7B..70B model is 8..235 MB of packed weights: 1..30 us of HBM
// time, against which a launch of its own costs 2.5 us kernel-to-kernel plus the ramp of the
// memory system at its start and the uneven finish of its workgroups at its end.  Here the k
// ranges of all row tiles of all problems of a batch, cut into units of one ring turn of a
// workgroup, form one sequence that is divided evenly over one workgroup per compute unit
// (a balanced split across problems): a workgroup streams one contiguous share of the batch and
// the launch has one start and one end.
//   * Operand mapping, decode table, decode and MFMA as in gemm_kernel.hpp: 64 weight rows per
//     wave, waves_m x waves_k waves (16 in all), wave (wm, wk) takes the k-steps wk, wk + waves_k,
//     ... of its segment; lane (i16, g) loads 16 bytes = 4 rows of one 8x8 block per k-step.
//   * The weight ring (U k-steps per wave) never drains between segments: the last ring turn of a
//     segment is refilled with the first steps of the workgroup's next segment - another row
//     tile, or another problem - so that segment's first weights are in registers when its loop
//     begins, and the reduction and store of the finished segment run under loads in flight.
//   * x: the segment's k range in chunks of 1024 k, double-buffered in LDS as in gemm_mid.hpp
//     ([8-k slot][token] pieces: conflict-free writes and B-fragment reads).  The last chunk of a
//     segment prefetches the first chunk and the scales of the next segment instead, so a segment
//     switch is an ordinary chunk switch and the reduction of the finished segment (through an LDS
//     area of its own, two accumulator planes at a time) is the only work between two main loops.
//   * A segment that is a whole row tile stores its output; a partial one hands its fp32 sums over
//     through the workspace (write-through stores, explicit wait, arrival ticket) and the last of
//     the row tile's contributors to arrive adds them in k order: deterministic, no atomics on the
//     output, counters return to zero (the scheme of gemm_kernel.hpp's balanced split).
//   * LDSW variants (ring of 2): packed weights and x go global -> LDS with global_load_lds_dwordx4 as in
//     the LDSW twins of gemm_mid.hpp (per-wave weight ring read back with ds_read_b128, x chunks of
//     512 k straight into the chunk buffer, every wait for a load written out, bare barriers, stores
//     into LDS the compiler does not look into).  Same arithmetic in the same order: same bits.
//   * BLK variants: one scale per block of 64 << blk_shift weights of a row (absmax [m, k / block]) instead of one per
//     row.  x chunks of 512 k; beside each x chunk the scales of the workgroup's rows for the chunk's blocks are
//     staged in LDS ([block of the chunk][row]: coalesced 8-byte reads of a row's consecutive blocks, one 16-byte
//     LDS read of a lane's four rows per k-step) and rounded to fp16 when a step is decoded: the decode is
//     fp16(code) * fp16(absmax of the block), the GEMM's rounding with a finer scale.
// Requires, for every problem: n <= 16, m a multiple of 64*waves_m, k a multiple of
// 32*waves_k*U, 16-byte aligned scales; the host falls back to separate launches otherwise.
#pragma once
#include "gemm_lean.hpp"
#include "gemm_mid.hpp"

namespace tuna {

constexpr int kMaxMultiProblems = 32;

struct MultiProblem {
    const uint8_t *q;
    const void *x;
    const float *absmax;
    void *out;
    const void *residual;  // EPI variants: fp16 with the layout of out, added before the rounding (TUNA_EPILOGUE_RESIDUAL)
    int m, n, k;
    int units_per_tile;  // k / (32 * waves_k * U)
    int tile_begin;      // id of its first row tile (arrival counters)
    int epilogue;        // EPI variants: TUNA_EPILOGUE_* of this problem's stores
};

struct MultiArgs {
    const float *code;
    float *ws;           // two slots of waves_m * 4 KB per workgroup
    unsigned *counters;  // one per row tile of the batch, zero between launches
    int n_problems;
    int units_total;     // (units_total + 1) * n_wg < 2^31
    int waves_m, wk_log2;
    int n_wg;
    int swizzle;         // n_wg is a multiple of 8: consecutive shares sit on one XCD
    int blk_shift;       // BLK variants: a scale per 64 << blk_shift weights of a row (every problem of the launch)
    // first unit of every problem in the batch's sequence, and the problem that holds the first unit of
    // every workgroup: a workgroup finds the problem of a unit by walking on from there (its share
    // rarely spans more than two problems), not through a chain of dependent fetches from problem 0
    int unit_begin[kMaxMultiProblems];
    unsigned char first_problem[kMaxCus];
    MultiProblem prob[kMaxMultiProblems];
};

// EPI: the problems carry fused epilogues (epilogue.hpp): a segment remembers its problem and the two places that
// store outputs look the problem's epilogue and residual up there (the other variants carry none of it).
template <int U, bool DEFER = true, bool LDSW = false, bool BLK = false, bool EPI = false>
__global__ __launch_bounds__(1024, 4) void gemm_multi_kernel(const MultiArgs a)
{
    static_assert(!LDSW || U == 2, "LDS is full with a ring of two: table 64 KB, x 2 x 16 KB, rings 32 KB, reduction 32 KB");
    static_assert(!(LDSW && BLK), "scale blocks: register-staged variants only");
    constexpr int XB = BLK ? 1 : 2;        // 16-byte x pieces per thread and chunk: 16 tokens x 1024 (BLK: 512) k x 2 B / 1024 threads
    constexpr int kChunkSteps = (LDSW || BLK) ? 16 : 32;        // k-steps per x chunk (LDSW: one wave instruction per wave)
    constexpr uint32_t kXBuf = ((LDSW || BLK) ? 16 : 32) * 1024;  // bytes of one x buffer
    constexpr uint32_t kSBuf = BLK ? 8 * 256 * 4 : 0;           // BLK: bytes of one scale buffer, [block of the chunk (8)][row (256)]
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *lut = smem;
    unsigned char *xbuf = smem + kLutBytes;  // two x buffers
    unsigned char *sbuf = smem + kLutBytes + 2 * kXBuf;  // BLK: two scale buffers
    // reduction area: two accumulator planes of all 16 waves (32 KB); its first two words double as the
    // arrival tickets of the hand-over, which are written only after every sum has been read
    float *redf = reinterpret_cast<float *>(smem + kLutBytes + 2 * kXBuf + 2 * kSBuf + (LDSW ? 16 * U * 1024 : 0));
    volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(redf);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // LDSW: behind the x buffers the waves' weight rings, U slots of 1 KB each
    unsigned char *wring = smem + kLutBytes + 2 * kXBuf + wave * (U * 1024);
    const int wk_log2 = a.wk_log2;
    const int waves_k = 1 << wk_log2;
    const int wk = wave & (waves_k - 1);
    const int wm = wave >> wk_log2;
    const int rows_wg = a.waves_m * 64;
    const int unit_log2 = wk_log2 + (U == 2 ? 1 : U == 4 ? 2 : 3);  // log2(k-steps per unit)
    const int chunk_its = kChunkSteps >> wk_log2;                  // iterations of one wave per full chunk, a multiple of U
    const uint32_t lane4 = (uint32_t)lane << 2;
    const uint32_t wq_stride = 128u << wk_log2;  // bytes between a wave's consecutive k-steps

    int wg = blockIdx.x;
    if (a.swizzle) wg = (wg & 7) * (a.n_wg >> 3) + (wg >> 3);
    const int t_begin = balanced_begin((unsigned)wg, (unsigned)a.n_wg, (unsigned)a.units_total);
    const int t_end = balanced_begin((unsigned)wg + 1u, (unsigned)a.n_wg, (unsigned)a.units_total);
    if (t_begin >= t_end) return;

    // A segment: units [u, next) of one row tile.  Uniform values; lb is the per-lane byte offset
    // of the lane's 16 bytes within a k-step of the segment's rows.
    struct Seg {
        const uint8_t *q;
        const unsigned char *x;
        const float *absmax;
        f16 *out;
        int m, n, k;
        int row0;     // first weight row of the workgroup's tile
        int sb;       // first k-step
        int nsteps;   // k-steps, a multiple of waves_k * U
        int part;     // -1: the whole row tile; 0 / 1: slot of the workgroup's partial sums
        int next;     // first unit behind the segment
        int tile_id;  // arrival counter
        int u0;       // first unit of the row tile in the batch's sequence
        int upt;      // units per row tile
        int prob;     // EPI: index of the problem
    };
    int p_scan = a.first_problem[wg];  // problem of the last segment looked up (segments are looked up in order)
    auto seg_at = [&](int u) {
        while (p_scan + 1 < a.n_problems && u >= a.unit_begin[p_scan + 1]) ++p_scan;
        const MultiProblem &pr = a.prob[p_scan];
        const int unit_begin_p = a.unit_begin[p_scan];
        Seg s;
        s.q = pr.q;
        s.x = reinterpret_cast<const unsigned char *>(pr.x);
        s.absmax = pr.absmax;
        s.out = reinterpret_cast<f16 *>(pr.out);
        s.m = pr.m, s.n = pr.n, s.k = pr.k;
        s.upt = pr.units_per_tile;
        s.prob = EPI ? p_scan : 0;
        const int ul = u - unit_begin_p;
        const int row_tile = (int)((unsigned)ul / (unsigned)s.upt);
        const int u_in = ul - row_tile * s.upt;
        const int left_tile = s.upt - u_in, left_wg = t_end - u;
        const int seg = left_wg < left_tile ? left_wg : left_tile;
        s.row0 = row_tile * rows_wg;
        s.sb = u_in << unit_log2;
        s.nsteps = seg << unit_log2;
        s.part = seg == s.upt ? -1 : (u == t_begin ? 0 : 1);
        s.next = u + seg;
        s.tile_id = pr.tile_begin + row_tile;
        s.u0 = u - u_in;
        return s;
    };
    auto lane_base = [&](const Seg &s) {
        const uint32_t kb_total = (uint32_t)s.k >> 3;
        return ((uint32_t)((s.row0 + wm * 64) >> 3) + (uint32_t)(i16 >> 1)) * kb_total * 32u + (uint32_t)(i16 & 1) * 16u +
               (uint32_t)g * 32u;
    };

    u32x4 wq[U];
    u32x4 xv[XB];
    f32x4 sc32;
    // x chunk `c` of segment sg (its steps 32c .. 32c+31 in walking order): piece b of this thread is
    // k-step (tid + b*1024) / 64 of the chunk, token row lane / 4, 8-k group lane % 4 (every quad of
    // lanes reads 64 contiguous bytes of one token row).
    const int x_row = lane >> 2, x_grp = lane & 3;
#define TUNA_MULTI_X_LOAD(x_, n_, k_, sb_, nsteps_, c)                                           \
    {                                                                                          \
        const uint32_t row_off_ = (uint32_t)min(x_row, (n_) - 1) * ((uint32_t)(k_) * 2u);      \
        _Pragma("unroll") for (int b = 0; b < XB; ++b)                                         \
        {                                                                                      \
            /* steps past the segment's end: clamped to a valid address, never read */         \
            const int p_ = min((c) * kChunkSteps + ((tid + b * 1024) >> 6), (nsteps_) - 1);    \
            xv[b] = *reinterpret_cast<const u32x4 *>((x_) + row_off_ + (uint32_t)(((sb_) + p_) * 32 + x_grp * 8) * 2u); \
        }                                                                                      \
    }
    // (token rows past n are zeroed, as the other kernels do; they feed output columns that are never stored)
#define TUNA_MULTI_X_STORE(n_, buf)                                                             \
    {                                                                                          \
        const bool ok_ = x_row < (n_);                                                         \
        _Pragma("unroll") for (int b = 0; b < XB; ++b)                                         \
        {                                                                                      \
            const int ks_ = (tid + b * 1024) >> 6;                                             \
            *reinterpret_cast<u32x4 *>((buf) + (ks_ * 4 + x_grp) * 256 + x_row * 16) = ok_ ? xv[b] : u32x4{0u, 0u, 0u, 0u}; \
        }                                                                                      \
    }

    // BLK: the scales of the workgroup's rows for the blocks chunk `c` of a segment touches - thread (row tid / 4,
    // pair tid % 4) fetches blocks 2 * pair and 2 * pair + 1 behind the chunk's first block (a quad of lanes reads
    // 32 contiguous bytes of a row of absmax; block indices clamped to the row, rows to the tile: duplicates)
    const int s_row = min(tid >> 2, rows_wg - 1), s_pair = tid & 3;
    const int blk_sh = a.blk_shift + 1;  // log2(k-steps per scale block)
    float sv[2];
#define TUNA_MULTI_S_LOAD(absmax_, k_, row0_, sb_, nsteps_, c)                                   \
    {                                                                                          \
        const int nblk_ = (k_) >> (5 + blk_sh);                                                \
        const int b0_ = ((sb_) + min((c) * kChunkSteps, (nsteps_) - 1)) >> blk_sh;             \
        const float *sp_ = (absmax_) + (size_t)((row0_) + s_row) * (size_t)nblk_;              \
        sv[0] = sp_[min(b0_ + 2 * s_pair, nblk_ - 1)];                                         \
        sv[1] = sp_[min(b0_ + 2 * s_pair + 1, nblk_ - 1)];                                     \
    }
    /* (stored rounded to fp16, twice in a dword: what the decode multiplies with) */
#define TUNA_MULTI_S_STORE(buf)                                                                 \
    {                                                                                          \
        _Pragma("unroll") for (int e_ = 0; e_ < 2; ++e_)                                       \
        {                                                                                      \
            const uint32_t h_ = (uint32_t)f16_bits((f16)sv[e_]);                               \
            reinterpret_cast<uint32_t *>(buf)[(2 * s_pair + e_) * 256 + (tid >> 2)] = h_ | (h_ << 16); \
        }                                                                                      \
    }

    // LDSW: chunk `c` straight into `buf`, k-step `wave` of the chunk per wave; lane (token i16, 8-k group g)
    // fetches its own B-fragment piece (token rows past n: clamped, their output columns are never stored)
#define TUNA_MULTI_X_DMA(x_, n_, k_, sb_, nsteps_, c, buf)                                       \
    {                                                                                          \
        const int p_ = min((c) * kChunkSteps + wave, (nsteps_) - 1);                           \
        load_weights_to_lds<false>((x_) + (uint32_t)min(i16, (n_) - 1) * ((uint32_t)(k_) * 2u) + (uint32_t)(((sb_) + p_) * 32 + g * 8) * 2u, \
                                   (buf) + wave * 1024);                                       \
    }

    float code_lane;
    if constexpr (LDSW) {
        // through the scalar cache (see gemm_mid.hpp: no vector load into a register while global -> LDS loads fly)
        const float *__restrict__ code_ptr = a.code;
        float cs[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) cs[j] = code_ptr[j];
        code_lane = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) code_lane = i16 == j ? cs[j] : code_lane;
    } else {
        code_lane = a.code[i16];
    }
    Seg cur = seg_at(t_begin);
    uint32_t lb = lane_base(cur);
    // x and the scales first: vector loads return in order, and the first barrier then waits for the x
    // pieces only while the first ring turn stays in flight across it
    if constexpr (LDSW) {
        TUNA_MULTI_X_DMA(cur.x, cur.n, cur.k, cur.sb, cur.nsteps, 0, xbuf)
        // the first segment's scales into this wave's KB of x buffer 1, free until chunk 1 is requested
        load_weights_to_lds<false>(reinterpret_cast<const unsigned char *>(cur.absmax + cur.row0 + wm * 64 + i16 * 4),
                                   xbuf + kXBuf + wave * 1024);
        const unsigned char *qp = cur.q + (size_t)(cur.sb + wk) * 128;
#pragma unroll
        for (int u = 0; u < U; ++u) load_weights_to_lds<true>(qp + (size_t)u * wq_stride + lb, wring + u * 1024);
    } else {
        TUNA_MULTI_X_LOAD(cur.x, cur.n, cur.k, cur.sb, cur.nsteps, 0)
        if constexpr (BLK) TUNA_MULTI_S_LOAD(cur.absmax, cur.k, cur.row0, cur.sb, cur.nsteps, 0)
        else sc32 = *reinterpret_cast<const f32x4 *>(cur.absmax + cur.row0 + wm * 64 + i16 * 4);
        const unsigned char *qp = cur.q + (size_t)(cur.sb + wk) * 128;
#pragma unroll
        for (int u = 0; u < U; ++u) wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qp + (size_t)u * wq_stride + lb));
    }

    // ---- decode table (see gemm_kernel.hpp), built while the first loads are in flight --------
    {
        const int code_bits = (int)f16_bits((f16)code_lane);
        for (int p0 = tid; p0 < kLutBytes / 16; p0 += 4 * 1024) {
            uint32_t v[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int e = (p0 + b * 1024) >> 4;
                const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
                const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
                v[b] = hi | (lo << 16);
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                if constexpr (LDSW) lds_store16_opaque(lut + (size_t)(p0 + b * 1024) * 16, u32x4{v[b], v[b], v[b], v[b]});
                else reinterpret_cast<u32x4 *>(lut)[p0 + b * 1024] = u32x4{v[b], v[b], v[b], v[b]};
            }
        }
    }
    // chunk 0 of the first segment into buffer 0; one barrier publishes it and the table
    if constexpr (LDSW) {
        __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));  // chunk 0 and the scales are older than the ring's U loads
        sc32 = *reinterpret_cast<const f32x4 *>(xbuf + kXBuf + wave * 1024 + lane * 16);
        barrier_lds_only();
    } else {
        TUNA_MULTI_X_STORE(cur.n, xbuf)
        if constexpr (BLK) TUNA_MULTI_S_STORE(sbuf)
        __syncthreads();
    }
    uint32_t xsel = 0;  // buffer that holds the chunk about to be consumed

    // (LDSW: a KB per k-step, lane l's piece at 16*l)
    const uint32_t xb_lane = (LDSW ? (uint32_t)lane * 16u : (uint32_t)g * 256u + (uint32_t)i16 * 16u) + (uint32_t)wk * 1024u;
    const uint32_t wstep = 1024u << wk_log2;  // LDS bytes between this wave's consecutive k-steps
    const size_t seg_floats = (size_t)a.waves_m * 1024;
    const size_t plane_floats = (size_t)16 * 256;  // one accumulator plane of all 16 waves

    // partial segments waiting for their hand-over, by slot (n_contrib == 0: none)
    struct Pending {
        f16 *out;
        int m, n, row0, tile_id, prob;
        unsigned w_lo, n_contrib, first_slot;
    };
    Pending pend0 = {}, pend1 = {};
    // Last contributor of a row tile: every partial is in memory; add them in k order and store.
    auto finish = [&](const Pending &pd) {
        if (tid == 0) __hip_atomic_store(a.counters + pd.tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int epi_ = TUNA_EPILOGUE_NONE;
        const f16 *res_ = nullptr;
        if constexpr (EPI) {
            epi_ = a.prob[pd.prob].epilogue;
            res_ = reinterpret_cast<const f16 *>(a.prob[pd.prob].residual);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = ((i << wk_log2) + wk) * 64 + lane;
            if (f >= 256) continue;
            const float *src = a.ws + ((size_t)pd.w_lo * 2 + pd.first_slot) * seg_floats + (size_t)wm * 1024 + (size_t)f * 4;
            f32x4 s4 = f32x4{0.f, 0.f, 0.f, 0.f};
            for (unsigned sp0 = 0; sp0 < pd.n_contrib; sp0 += 4) {  // four contributors per round trip, summed in k order
                f32x4 pv[4];
                const float *ps[4];
#pragma unroll
                for (unsigned b = 0; b < 4; ++b) {
                    const unsigned sp = min(sp0 + b, pd.n_contrib - 1u);
                    ps[b] = src + (size_t)sp * 2 * seg_floats - (sp ? (size_t)pd.first_slot * seg_floats : (size_t)0);
                }
                load_partials4(ps[0], ps[1], ps[2], ps[3], pv[0], pv[1], pv[2], pv[3]);
#pragma unroll
                for (unsigned b = 0; b < 4; ++b)
                    if (sp0 + b < pd.n_contrib) s4 += pv[b];
            }
            const int l = f >> 2, v = f & 3;
            const int tok = l & 15;
            if (tok < pd.n)
                store_features4(pd.out, res_, epi_, (size_t)tok, pd.m, pd.row0 + wm * 64 + (l >> 4) * 16 + v * 4, s4[0], s4[1], s4[2],
                                s4[3]);
        }
    };

    for (;;) {
        const bool has_next = cur.next < t_end;
        Seg nxt = cur;
        if (has_next) nxt = seg_at(cur.next);
        const uint32_t lb_next = lane_base(nxt);

        f16x2 sc16[4];
        if constexpr (!BLK) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f16 h = (f16)sc32[j];
                sc16[j] = f16x2{h, h};
            }
        }
        f32x4 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int n_it = cur.nsteps >> wk_log2;                                  // this wave's iterations, a multiple of U
        const int n_chunks = (cur.nsteps + kChunkSteps - 1) / kChunkSteps;
        // refills: iteration it + U of this segment; in the last ring turn the first U iterations of
        // the next segment (without one: this segment's last turn again - valid addresses, data unused)
        const unsigned char *rp = cur.q + (size_t)(cur.sb + wk) * 128 + (size_t)U * wq_stride;
        uint32_t rlb = lb;
        const unsigned char *rp_last = has_next ? nxt.q + (size_t)(nxt.sb + wk) * 128
                                                : cur.q + (size_t)(cur.sb + wk) * 128 + (size_t)(n_it - U) * wq_stride;
        const uint32_t rlb_last = has_next ? lb_next : lb;
        int it = 0;
        // the scales of the next segment (without one: this segment's again), needed when this one ends
        f32x4 sc_next = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (!BLK) sc_next = *reinterpret_cast<const f32x4 *>(nxt.absmax + nxt.row0 + wm * 64 + i16 * 4);
        // One ring turn: U of this wave's k-steps consumed and refilled; the refills of the segment's
        // last turn are the first steps of the next segment.
#define TUNA_MULTI_TURN(sl, first)                                                              \
    {                                                                                          \
        if (it + U >= n_it) {                                                                  \
            rp = rp_last;                                                                      \
            rlb = rlb_last;                                                                    \
        }                                                                                      \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                          \
        {                                                                                      \
            if constexpr (LDSW) {                                                              \
                /* the slot's load has landed: U - 1 younger ring loads and, in a chunk's first */ \
                /* turn, the x piece just requested (and the next segment's scales) may fly on */ \
                if (!(first)) __builtin_amdgcn_s_waitcnt(wait_vmcnt(U - 1));                   \
                else if (c == 0) __builtin_amdgcn_s_waitcnt(wait_vmcnt(U + 1));                \
                else __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));                                \
                wq[u] = *reinterpret_cast<const u32x4 *>(wring + u * 1024 + lane * 16);        \
            }                                                                                  \
            const f16x8 b_ = *reinterpret_cast<const f16x8 *>(xb + (size_t)((sl) + u) * wstep); \
            if constexpr (BLK) {                                                               \
                /* the step's scale block, counted from the chunk's first one */               \
                const int rel_ = ((sbc + (((sl) + u) << wk_log2) + wk) >> blk_sh) - (sbc >> blk_sh); \
                const u32x4 s4_ = *reinterpret_cast<const u32x4 *>(sb_lane + (size_t)rel_ * 1024); \
                _Pragma("unroll") for (int j = 0; j < 4; ++j)                                  \
                {                                                                              \
                    const uint32_t e_ = s4_[j]; /* (a copy: bit_cast of a vector element reads element 0) */ \
                    sc16[j] = __builtin_bit_cast(f16x2, e_);                                   \
                }                                                                              \
            }                                                                                  \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                      \
            {                                                                                  \
                const f16x8 av_ = decode_dword<TUNA_DECODE_GEMM>(wq[u][j], lut, lane4, sc16[j], 0.f); \
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_, acc[j], 0, 0, 0);     \
            }                                                                                  \
            if constexpr (LDSW) {                                                              \
                __builtin_amdgcn_sched_barrier(0); /* behind the MFMAs that used the slot's bytes */ \
                load_weights_to_lds<true>(rp + (size_t)u * wq_stride + rlb, wring + u * 1024); \
            } else {                                                                           \
                wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(rp + (size_t)u * wq_stride + rlb)); \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0); /* keep each refill right behind its consume */ \
        }                                                                                      \
        rp += (size_t)U * wq_stride;                                                           \
        it += U;                                                                               \
    }
        for (int c = 0; c < n_chunks; ++c) {
            const bool more = c + 1 < n_chunks;
            // the chunk behind this one: of this segment, or - in its last chunk - the first one of
            // the next segment (no next segment: this chunk again, dropped).  Uniform parameters and
            // ONE unconditional batch of loads: behind a branch the compiler could not count these
            // loads into the waits of the ring and would wait for everything in flight instead.
            {
                const unsigned char *x_ = more ? cur.x : nxt.x;
                const int xn_ = more ? cur.n : nxt.n, xk_ = more ? cur.k : nxt.k, xsb_ = more ? cur.sb : nxt.sb;
                const int xns_ = more ? cur.nsteps : nxt.nsteps, xc_ = more ? c + 1 : (has_next ? 0 : c);
                if constexpr (LDSW) {
                    // (the other buffer was last read in the previous chunk, which ended with a barrier)
                    TUNA_MULTI_X_DMA(x_, xn_, xk_, xsb_, xns_, xc_, xbuf + (xsel ^ 1u) * kXBuf)
                } else {
                    TUNA_MULTI_X_LOAD(x_, xn_, xk_, xsb_, xns_, xc_)
                    if constexpr (BLK) {
                        const float *am_ = more ? cur.absmax : nxt.absmax;
                        const int row0_ = more ? cur.row0 : nxt.row0;
                        TUNA_MULTI_S_LOAD(am_, xk_, row0_, xsb_, xns_, xc_)
                    }
                }
            }
            const unsigned char *xb = xbuf + xsel * kXBuf + xb_lane;
            // BLK: this lane's four rows in the scale buffer of the chunk, and the chunk's first k-step
            const unsigned char *sb_lane = sbuf + xsel * kSBuf + (size_t)(wm * 64 + i16 * 4) * 4;
            const int sbc = cur.sb + c * kChunkSteps;
            const int its = min(chunk_its, n_it - it);
            // (the first ring turn of a chunk is a copy of its own: there the x pieces just requested
            // are in flight behind the ring, and only straight-line code lets the compiler count them
            // into its waits)
            TUNA_MULTI_TURN(0, true)
            for (int sl = U; sl < its; sl += U) TUNA_MULTI_TURN(sl, false)
            // the other buffer was last read in the previous chunk, which ended with a barrier;
            // exactly the last ring turn's U refills are younger than the x pieces
            __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));
            if constexpr (LDSW) {
                barrier_lds_only();
            } else {
                TUNA_MULTI_X_STORE(more ? cur.n : nxt.n, xbuf + (xsel ^ 1u) * kXBuf)
                if constexpr (BLK) TUNA_MULTI_S_STORE(sbuf + (xsel ^ 1u) * kSBuf)
                __syncthreads();
            }
            xsel ^= 1u;
        }
#undef TUNA_MULTI_TURN
        sc32 = sc_next;

        // ---- reduction over the waves along k (layouts of gemm_kernel.hpp), two planes at a time ----
        // (the area was last read before a chunk barrier of this segment; the next segment's first
        // chunk is already staged, so its main loop starts right behind the stores below)
        float o[4][4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h) {  // the first half's sums have been read
                if constexpr (LDSW) barrier_lds_only();
                else __syncthreads();
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float *dst = redf + j * plane_floats + ((size_t)wave * 64 + lane) * 4;
                if constexpr (LDSW) lds_store16_opaque(reinterpret_cast<unsigned char *>(dst), __builtin_bit_cast(u32x4, acc[2 * h + j]));
                else *reinterpret_cast<f32x4 *>(dst) = acc[2 * h + j];
            }
            if constexpr (LDSW) barrier_lds_only();
            else __syncthreads();
            sum_planes_any<2, 32>(wk_log2, redf, plane_floats, wm, wk, lane, o, 2 * h);
        }
        const bool partial = cur.part >= 0;
        int epi_ = TUNA_EPILOGUE_NONE;
        const f16 *res_ = nullptr;
        if constexpr (EPI) {
            epi_ = a.prob[cur.prob].epilogue;
            res_ = reinterpret_cast<const f16 *>(a.prob[cur.prob].residual);
        }
        float *mine = a.ws + ((size_t)wg * 2 + (size_t)(partial ? cur.part : 0)) * seg_floats + (size_t)wm * 1024;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = ((i << wk_log2) + wk) * 64 + lane;
            if (f >= 256) continue;
            if (!partial) {
                const int l = f >> 2, v = f & 3;
                const int tok = l & 15;
                if (tok < cur.n)
                    store_features4(cur.out, res_, epi_, (size_t)tok, cur.m, cur.row0 + wm * 64 + (l >> 4) * 16 + v * 4, o[i][0], o[i][1],
                                    o[i][2], o[i][3]);
            } else {
                store_partial(mine + (size_t)f * 4, f32x4{o[i][0], o[i][1], o[i][2], o[i][3]});
            }
        }
        if (partial) {
            Pending pd;
            pd.out = cur.out;
            pd.m = cur.m, pd.n = cur.n, pd.row0 = cur.row0, pd.tile_id = cur.tile_id, pd.prob = cur.prob;
            const unsigned T = (unsigned)a.units_total, nw = (unsigned)a.n_wg;
            const unsigned u0 = (unsigned)cur.u0, u1 = u0 + (unsigned)cur.upt - 1u;
            pd.w_lo = ((u0 + 1u) * nw - 1u) / T;
            pd.n_contrib = ((u1 + 1u) * nw - 1u) / T - pd.w_lo + 1u;
            pd.first_slot = (pd.w_lo * T) / nw < u0 ? 1u : 0u;
            if constexpr (DEFER) {
                // left to the end of the workgroup's share, where its at most two partial segments (slots 0
                // and 1) are handed over together
                if (cur.part == 0) pend0 = pd;  // (two named copies: an array indexed by the slot would live in scratch memory)
                else pend1 = pd;
            } else {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): a workgroup-scope fence does not wait for global stores
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __syncthreads();  // also: every sum has been read, the ticket word is free
                if (tid == 0) ticket[0] = __hip_atomic_fetch_add(a.counters + pd.tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                if (ticket[0] == pd.n_contrib - 1u) finish(pd);
            }
        }
        if (!has_next) break;
        cur = nxt;
        lb = lb_next;
    }

    // ---- hand-over of the partial segments (see gemm_kernel.hpp): stores complete, barrier, arrival
    //      tickets, and for every row tile whose last contributor this workgroup is, the sum in k order
    if constexpr (DEFER) {
        if (pend0.n_contrib | pend1.n_contrib) {
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): a workgroup-scope fence does not wait for global stores
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();  // also: every sum has been read, the ticket words are free
            if (tid == 0 && pend0.n_contrib)
                ticket[0] = __hip_atomic_fetch_add(a.counters + pend0.tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tid == 64 && pend1.n_contrib)  // (another wave: the two round trips overlap)
                ticket[1] = __hip_atomic_fetch_add(a.counters + pend1.tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (pend0.n_contrib && ticket[0] == pend0.n_contrib - 1u) finish(pend0);
            if (pend1.n_contrib && ticket[1] == pend1.n_contrib - 1u) finish(pend1);
        }
    }
#undef TUNA_MULTI_X_LOAD
#undef TUNA_MULTI_X_DMA
#undef TUNA_MULTI_X_STORE
#undef TUNA_MULTI_S_LOAD
#undef TUNA_MULTI_S_STORE
}

}  // namespace tuna
