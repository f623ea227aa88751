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
//     ([8-k slot][token] pieces: conflict-free writes and B-fragment reads).
//   * A segment that is a whole row tile stores its output; a partial one hands its fp32 sums over
//     through the workspace (write-through stores, explicit wait, arrival ticket) and the last of
//     the row tile's contributors to arrive adds them in k order: deterministic, no atomics on the
//     output, counters return to zero (the scheme of gemm_kernel.hpp's balanced split).
// Requires, for every problem: n <= 16, m a multiple of 64*waves_m, k a multiple of
// 32*waves_k*U, 16-byte aligned scales; the host falls back to separate launches otherwise.
#pragma once
#include "gemm_lean.hpp"

namespace tuna {

constexpr int kMaxMultiProblems = 32;

struct MultiProblem {
    const uint8_t *q;
    const void *x;
    const float *absmax;
    void *out;
    int m, n, k;
    int units_per_tile;  // k / (32 * waves_k * U)
    int unit_begin;      // first unit of this problem in the batch's sequence
    int tile_begin;      // id of its first row tile (arrival counters)
    int pad0, pad1;
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
    MultiProblem prob[kMaxMultiProblems];
};

template <int U>
__global__ __launch_bounds__(1024, 4) void gemm_multi_kernel(const MultiArgs a)
{
    constexpr int XB = 2;                  // 16-byte x pieces per thread and chunk: 16 tokens x 1024 k x 2 B / 1024 threads
    constexpr int kChunkSteps = 32;        // k-steps per x chunk
    constexpr uint32_t kXBuf = 32 * 1024;  // bytes of one x buffer
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *lut = smem;
    unsigned char *xbuf = smem + kLutBytes;                // two x buffers; the reduction planes after a segment's loop
    volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(smem + kLutBytes + 2 * kXBuf);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    };
    int p_scan = 0;  // problem of the last segment looked up (segments are looked up in order)
    auto seg_at = [&](int u) {
        while (p_scan + 1 < a.n_problems && u >= a.prob[p_scan + 1].unit_begin) ++p_scan;
        const MultiProblem &pr = a.prob[p_scan];
        Seg s;
        s.q = pr.q;
        s.x = reinterpret_cast<const unsigned char *>(pr.x);
        s.absmax = pr.absmax;
        s.out = reinterpret_cast<f16 *>(pr.out);
        s.m = pr.m, s.n = pr.n, s.k = pr.k;
        s.upt = pr.units_per_tile;
        const int ul = u - pr.unit_begin;
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
    // x chunk `c` of segment s: piece b of this thread is k-step (tid + b*1024) / 64 of the chunk, token
    // row lane / 4, 8-k group lane % 4 (every quad of lanes reads 64 contiguous bytes of one token row).
    // Steps past the segment's end or k are clamped to valid addresses; their data is never read.
    const int x_row = lane >> 2, x_grp = lane & 3;
#define TUNA_MULTI_X_LOAD(s, c)                                                                 \
    {                                                                                          \
        const uint32_t row_off_ = (uint32_t)min(x_row, (s).n - 1) * ((uint32_t)(s).k * 2u);    \
        _Pragma("unroll") for (int b = 0; b < XB; ++b)                                         \
        {                                                                                      \
            const int ks_ = (tid + b * 1024) >> 6;                                             \
            const int kk_ = min(((s).sb + (c) * kChunkSteps + ks_) * 32 + x_grp * 8, (s).k - 8); \
            xv[b] = *reinterpret_cast<const u32x4 *>((s).x + row_off_ + (uint32_t)kk_ * 2u);   \
        }                                                                                      \
    }
    // (token rows past n are zeroed: they feed output columns that are never stored, but must not be NaN-free garbage either way)
#define TUNA_MULTI_X_STORE(s, buf)                                                              \
    {                                                                                          \
        const bool ok_ = x_row < (s).n;                                                        \
        _Pragma("unroll") for (int b = 0; b < XB; ++b)                                         \
        {                                                                                      \
            const int ks_ = (tid + b * 1024) >> 6;                                             \
            *reinterpret_cast<u32x4 *>((buf) + (ks_ * 4 + x_grp) * 256 + x_row * 16) = ok_ ? xv[b] : u32x4{0u, 0u, 0u, 0u}; \
        }                                                                                      \
    }
#define TUNA_MULTI_SMALL_LOADS(s)                                                               \
    {                                                                                          \
        sc32 = *reinterpret_cast<const f32x4 *>((s).absmax + (s).row0 + wm * 64 + i16 * 4);    \
        TUNA_MULTI_X_LOAD(s, 0)                                                                \
    }

    const float code_lane = a.code[i16];
    Seg cur = seg_at(t_begin);
    uint32_t lb = lane_base(cur);
    {
        const unsigned char *qp = cur.q + (size_t)(cur.sb + wk) * 128;
#pragma unroll
        for (int u = 0; u < U; ++u) wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qp + (size_t)u * wq_stride + lb));
    }
    TUNA_MULTI_SMALL_LOADS(cur)

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
            for (int b = 0; b < 4; ++b) reinterpret_cast<u32x4 *>(lut)[p0 + b * 1024] = u32x4{v[b], v[b], v[b], v[b]};
        }
    }

    const uint32_t xb_lane = (uint32_t)g * 256u + (uint32_t)i16 * 16u + (uint32_t)wk * 1024u;
    const uint32_t wstep = 1024u << wk_log2;  // LDS bytes between this wave's consecutive k-steps
    const size_t seg_floats = (size_t)a.waves_m * 1024;
    const size_t plane_floats = (size_t)16 * 256;  // one accumulator plane of all 16 waves

    for (;;) {
        const bool has_next = cur.next < t_end;
        Seg nxt = cur;
        if (has_next) nxt = seg_at(cur.next);
        const uint32_t lb_next = lane_base(nxt);

        f16x2 sc16[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f16 h = (f16)sc32[j];
            sc16[j] = f16x2{h, h};
        }
        f32x4 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

        // chunk 0 into buffer 0: the x area is free (the barrier that ended the previous segment)
        TUNA_MULTI_X_STORE(cur, xbuf)
        __syncthreads();

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
        for (int c = 0; c < n_chunks; ++c) {
            const bool more = c + 1 < n_chunks;
            TUNA_MULTI_X_LOAD(cur, more ? c + 1 : c)
            const unsigned char *xb = xbuf + (c & 1) * kXBuf + xb_lane;
            const int its = min(chunk_its, n_it - it);
            for (int sl = 0; sl < its; sl += U) {
                if (it + U >= n_it) {
                    rp = rp_last;
                    rlb = rlb_last;
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const f16x8 b_ = *reinterpret_cast<const f16x8 *>(xb + (size_t)(sl + u) * wstep);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const f16x8 av_ = decode_dword<TUNA_DECODE_GEMM>(wq[u][j], lut, lane4, sc16[j], 0.f);
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_, acc[j], 0, 0, 0);
                    }
                    wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(rp + (size_t)u * wq_stride + rlb));
                    __builtin_amdgcn_sched_barrier(0);  // keep each refill right behind its consume
                }
                rp += (size_t)U * wq_stride;
                it += U;
            }
            if (more) TUNA_MULTI_X_STORE(cur, xbuf + ((c + 1) & 1) * kXBuf)
            __syncthreads();
        }

        // ---- the next segment's scales and first x chunk, behind its ring loads --------------------
        const Seg done = cur;
        if (has_next) TUNA_MULTI_SMALL_LOADS(nxt)

        // ---- reduction over the waves along k (layouts of gemm_kernel.hpp) and store ------------------
        float *redf = reinterpret_cast<float *>(xbuf);
#pragma unroll
        for (int j = 0; j < 4; ++j) reinterpret_cast<f32x4 *>(redf + j * plane_floats)[(size_t)wave * 64 + lane] = acc[j];
        __syncthreads();
        float o[4][4];
        sum_planes_any<4, 32>(wk_log2, redf, plane_floats, wm, wk, lane, o, 0);
        const bool partial = done.part >= 0;
        float *mine = a.ws + ((size_t)wg * 2 + (size_t)(partial ? done.part : 0)) * seg_floats + (size_t)wm * 1024;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = ((i << wk_log2) + wk) * 64 + lane;
            if (f >= 256) continue;
            if (!partial) {
                const int l = f >> 2, v = f & 3;
                const int tok = l & 15;
                if (tok < done.n)
                    store_features4(done.out, nullptr, TUNA_EPILOGUE_NONE, (size_t)tok, done.m, done.row0 + wm * 64 + (l >> 4) * 16 + v * 4,
                                    o[i][0], o[i][1], o[i][2], o[i][3]);
            } else {
                store_partial(mine + (size_t)f * 4, f32x4{o[i][0], o[i][1], o[i][2], o[i][3]});
            }
        }
        if (partial) {
            // hand-over (see gemm_kernel.hpp): stores complete, barrier, arrival ticket, the last one sums
            unsigned w_lo, n_contrib, first_slot;
            {
                const unsigned T = (unsigned)a.units_total, nw = (unsigned)a.n_wg;
                const unsigned u0 = (unsigned)done.u0, u1 = u0 + (unsigned)done.upt - 1u;
                w_lo = ((u0 + 1u) * nw - 1u) / T;
                n_contrib = ((u1 + 1u) * nw - 1u) / T - w_lo + 1u;
                first_slot = (w_lo * T) / nw < u0 ? 1u : 0u;
            }
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            if (tid == 0) *ticket = __hip_atomic_fetch_add(a.counters + done.tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (*ticket == n_contrib - 1u) {
                if (tid == 0) __hip_atomic_store(a.counters + done.tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int f = ((i << wk_log2) + wk) * 64 + lane;
                    if (f >= 256) continue;
                    const float *src = a.ws + ((size_t)w_lo * 2 + first_slot) * seg_floats + (size_t)wm * 1024 + (size_t)f * 4;
                    f32x4 s4 = f32x4{0.f, 0.f, 0.f, 0.f};
                    for (unsigned sp0 = 0; sp0 < n_contrib; sp0 += 4) {  // four contributors per round trip, summed in k order
                        f32x4 pv[4];
                        const float *ps[4];
#pragma unroll
                        for (unsigned b = 0; b < 4; ++b) {
                            const unsigned sp = min(sp0 + b, n_contrib - 1u);
                            ps[b] = src + (size_t)sp * 2 * seg_floats - (sp ? (size_t)first_slot * seg_floats : (size_t)0);
                        }
                        load_partials4(ps[0], ps[1], ps[2], ps[3], pv[0], pv[1], pv[2], pv[3]);
#pragma unroll
                        for (unsigned b = 0; b < 4; ++b)
                            if (sp0 + b < n_contrib) s4 += pv[b];
                    }
                    const int l = f >> 2, v = f & 3;
                    const int tok = l & 15;
                    if (tok < done.n)
                        store_features4(done.out, nullptr, TUNA_EPILOGUE_NONE, (size_t)tok, done.m,
                                        done.row0 + wm * 64 + (l >> 4) * 16 + v * 4, s4[0], s4[1], s4[2], s4[3]);
                }
            }
        }
        if (!has_next) break;
        __syncthreads();  // every read of the reduction planes is done: the x area may be written again
        cur = nxt;
        lb = lb_next;
    }
#undef TUNA_MULTI_X_LOAD
#undef TUNA_MULTI_X_STORE
#undef TUNA_MULTI_SMALL_LOADS
}

}  // namespace tuna
