// Lean twin of the streaming GEMM kernel for small launches (gfx950, wave64).
//
// At 1..16 tokens the projections of a 7B..70B model are 8..40 MB of packed weights: 2..7 us
// of HBM time, against which the kernel's own fixed work counts.  A wave issues at most one
// instruction every four cycles, so every 600 instructions between a workgroup's first and
// last memory access cost a microsecond.  This kernel computes exactly what gemm_kernel
// computes for one class of launches and sheds everything that class does not need:
//   * one workgroup per tile, fixed power-of-two split, dense (no tile walk, no balanced split,
//     no groups), 64 rows per wave, one 16-token tile, no stagger;
//   * m a multiple of the workgroup's rows, k a multiple of 32, every wave with the same whole
//     number of ring turns: no clamped or conditional loads, no tails;
//   * the workgroup's whole k slice of x is staged in LDS at once (one barrier covers the decode
//     table and x), waves along k and ring depth are template arguments.
// Same operand mapping, decode, reduction order and split-K hand-over as gemm_kernel (see
// gemm_kernel.hpp), so results are bit-identical to the general kernel run with the same
// config.  launch_gemm picks it when the launch qualifies (lean_applies in gemm_launch.hip).
#pragma once
#include "gemm_kernel.hpp"

namespace tuna {

// What the kernel needs of GemmArgs, as separate scalar arguments with the ones the first loads
// use in front: the first 14 dwords of such arguments are preloaded into scalar registers with
// the wave (build flag -amdgpu-kernarg-preload-count), a struct passed by value is fetched by
// the kernel itself - a round trip to memory before anything else can start.
struct LeanArgs {
    const uint8_t *q;
    const void *x;
    const float *code;
    const float *absmax;
    int k, n, steps_per_split;
    int packed;  // split_log2 | waves_m << 4 | epilogue << 9 | swizzle << 11 | (workgroups / 8) << 12
    int m;
    void *out;
    const void *residual;
    float *ws;
    unsigned *counters;
    int row_tiles;
};

template <int WK, int U, int MAXT, int MINW>
__global__ __launch_bounds__(MAXT, MINW) void gemm_lean_kernel(const uint8_t *a_q, const void *a_x, const float *a_code,
                                                               const float *a_absmax, int a_k, int a_n, int a_sps,
                                                               int a_packed, int a_m, void *a_out,
                                                               const void *a_residual, float *a_ws, unsigned *a_counters,
                                                               int a_row_tiles
)
{
    struct {
        const uint8_t *q;
        const void *x;
        const float *code;
        const float *absmax;
        void *out;
        const void *residual;
        float *ws;
        unsigned *counters;
        int m, n, k, steps_per_split, row_tiles, split_log2, split_k, waves_m, xcd_swizzle, epilogue;
    } const a = {a_q,           a_x,          a_code,          a_absmax,
                 a_out,         a_residual,   a_ws,            a_counters,
                 a_m,           a_n,          a_k,             a_sps,
                 a_row_tiles,   a_packed & 15, 1 << (a_packed & 15), (a_packed >> 4) & 31,
                 (a_packed >> 11) & 1, (a_packed >> 9) & 3
    };
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int WK_LOG2 = WK == 1 ? 0 : WK == 2 ? 1 : WK == 4 ? 2 : WK == 8 ? 3 : 4;
    constexpr int TT = 1;
    unsigned char *lut = smem;
    unsigned char *work = smem + kLutBytes;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave & (WK - 1);
    const int wm = wave >> WK_LOG2;
    const int nthreads = a.waves_m * (WK * 64);  // (blockDim would be a fetch from the argument segment)
    const uint32_t lane4 = (uint32_t)lane << 2;

    int wg = blockIdx.x;
    // (the host sets the swizzle bit only for a workgroup count that is a multiple of 8, and passes
    // an eighth of the count: reading gridDim here would be a fetch from the argument segment)
    if (a.xcd_swizzle) wg = (wg & 7) * (a_packed >> 12) + (wg >> 3);
    const int row_tile = wg >> a.split_log2;
    const int part = wg & (a.split_k - 1);
    const int sb = part * a.steps_per_split;  // first k-step of this workgroup
    const int tok0 = blockIdx.y * 16;
    const int row_base = row_tile * (a.waves_m * 64);
    const int row0 = row_base + wm * 64;
    const int n_it = a.steps_per_split >> WK_LOG2;  // k-steps per wave, a multiple of U

    // ---- requests, in the order their data is needed back (vector loads return in order):
    //      codebook, scales, x slice, first ring turn of weights -----------------------------------
    const float code_lane = a.code[i16];
    const f32x4 sc32 = *reinterpret_cast<const f32x4 *>(a.absmax + row0 + i16 * 4);
    // x slice [16 tokens][k of this split], in 16-byte pieces (one token, one 8-k slot).  Piece
    // p = tid + b*nthreads: lane p % 64 picks token lane / 4 and 8-k group lane % 4, p / 64 the
    // k-step.  Every quad of lanes reads 64 contiguous bytes of one token row (neighbouring lanes
    // on different rows would cost three times the cycles in the address path) and a wave
    // instruction writes one k-step - 4 slots x 16 tokens, 1 KB contiguous - to LDS, where slot s,
    // token t sits at byte s*256 + t*16: the 16 tokens of a slot are one B-fragment row.
    // 64 * steps_per_split pieces, at most 8 per thread.  Rows past n: clamped loads, zeros stored.
    const int x_steps = a.steps_per_split;
    const unsigned char *xsl = reinterpret_cast<const unsigned char *>(a.x) + ((size_t)tok0 * a.k + (size_t)sb * 32) * 2;
    const int n_rel = a.n - 1 - tok0;  // last valid token row of this tile, relative
    const int x_row = lane >> 2, x_grp = lane & 3;
    const bool x_row_ok = x_row <= n_rel;
    const uint32_t x_lane_off = (uint32_t)min(x_row, n_rel) * ((uint32_t)a.k * 2u) + (uint32_t)x_grp * 16u;  // (k < 2^23)
    const int x_wv0 = wave, x_dwv = nthreads >> 6;  // this wave's first k-step and the stride between its pieces
    u32x4 xv[8];
    const bool x_long = x_steps > 4 * x_dwv;  // uniform: more than 4 pieces per thread
#pragma unroll
    for (int b = 0; b < 4; ++b)  // (clamped: a short slice has fewer than 4 pieces per thread)
        xv[b] = *reinterpret_cast<const u32x4 *>(xsl + (size_t)min(x_wv0 + b * x_dwv, x_steps - 1) * 64 + x_lane_off);
    if (x_long) {
#pragma unroll
        for (int b = 4; b < 8; ++b)
            xv[b] = *reinterpret_cast<const u32x4 *>(xsl + (size_t)min(x_wv0 + b * x_dwv, x_steps - 1) * 64 + x_lane_off);
    }

    // the weights last: x and the scales come from L2 and are needed first, the first ring turn
    // comes from HBM and is needed once x is staged
    const uint32_t kb_total = (uint32_t)a.k >> 3;
    const uint32_t lb = ((uint32_t)(row0 >> 3) + (uint32_t)(i16 >> 1)) * kb_total * 32u + (uint32_t)(i16 & 1) * 16u +
                        (uint32_t)g * 32u;
    const unsigned char *qp = a.q + (size_t)(sb + wk) * 128;  // uniform; advances one ring turn per group
    u32x4 wq[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
        wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qp + (size_t)u * (WK * 128) + lb));
    qp += (size_t)U * (WK * 128);
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
    f16x2 sc16[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const f16 h = (f16)sc32[j];
        sc16[j] = f16x2{h, h};
    }
    // ---- x into LDS; one barrier publishes the table and the slice ---------------------------
    unsigned char *x_dst = work + x_grp * 256 + x_row * 16;
#pragma unroll
    for (int b = 0; b < 4; ++b)
        if (x_wv0 + b * x_dwv < x_steps)
            *reinterpret_cast<u32x4 *>(x_dst + (size_t)(x_wv0 + b * x_dwv) * 1024) = x_row_ok ? xv[b] : u32x4{0u, 0u, 0u, 0u};
    if (x_long) {
#pragma unroll
        for (int b = 4; b < 8; ++b)
            if (x_wv0 + b * x_dwv < x_steps)
                *reinterpret_cast<u32x4 *>(x_dst + (size_t)(x_wv0 + b * x_dwv) * 1024) = x_row_ok ? xv[b] : u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    // ---- main loop: n_it / U ring turns, the last one without refills ------------------------
    f32x4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const unsigned char *xb = work + g * 256 + i16 * 16 + wk * 1024;  // B fragment of this wave's step 0
    constexpr int wstep = WK * 1024;                                   // LDS bytes between its consecutive steps
#define TUNA_LEAN_CONSUME(u)                                                                    \
    {                                                                                          \
        const f16x8 b_ = *reinterpret_cast<const f16x8 *>(xb + (u) * wstep);                   \
        _Pragma("unroll") for (int j = 0; j < 4; ++j)                                          \
        {                                                                                      \
            const f16x8 av_ = decode_dword<TUNA_DECODE_GEMM>(wq[u][j], lut, lane4, sc16[j], 0.f); \
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_, acc[j], 0, 0, 0);         \
        }                                                                                      \
    }
    for (int it = U; it < n_it; it += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            TUNA_LEAN_CONSUME(u)
            wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qp + (size_t)u * (WK * 128) + lb));
            // keep the refill right behind its consume (see TUNA_GROUP in gemm_kernel.hpp)
            __builtin_amdgcn_sched_barrier(0);
        }
        qp += (size_t)U * (WK * 128);
        xb += U * wstep;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) TUNA_LEAN_CONSUME(u)
#undef TUNA_LEAN_CONSUME

    // ---- reduction and store (layouts of gemm_kernel) ----------------------------------------
    f16 *outp = reinterpret_cast<f16 *>(a.out);
    const f16 *resp = reinterpret_cast<const f16 *>(a.residual);
    const int out_ld = a.m;
    const bool partial = a.split_k > 1;
    if (WK == 1 && !partial) {
        const int tok = tok0 + i16;
        const int rb = row0 + g * 16;
        if (tok < a.n) {
            if (a.epilogue == TUNA_EPILOGUE_NONE) {
                f16x8 lo, hi;
#pragma unroll
                for (int v = 0; v < 2; ++v)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        lo[v * 4 + j] = (f16)acc[j][v];
                        hi[v * 4 + j] = (f16)acc[j][v + 2];
                    }
                f16 *dst = outp + (size_t)tok * out_ld + rb;
                *reinterpret_cast<f16x8 *>(dst) = lo;
                *reinterpret_cast<f16x8 *>(dst + 8) = hi;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, rb + v * 4, acc[0][v], acc[1][v], acc[2][v],
                                    acc[3][v]);
            }
        }
        return;
    }
    const size_t plane_floats = (size_t)(nthreads >> 6) * 256;
    float *redf = reinterpret_cast<float *>(work);
    __syncthreads();  // every wave is done reading x: the work area is free
#pragma unroll
    for (int j = 0; j < 4; ++j)
        reinterpret_cast<f32x4 *>(redf + j * plane_floats)[(size_t)(wm * WK + wk) * 64 + lane] = acc[j];
    __syncthreads();
    float o[4][4];
    sum_planes<WK, 4, 32>(redf, plane_floats, wm, wk, lane, o, 0);

    const size_t seg_floats = (size_t)a.waves_m * 1024;  // partial sums of one workgroup: [wm][f][j]
    const size_t tile_id = (size_t)blockIdx.y * a.row_tiles + row_tile;
    float *wst = a.ws + tile_id * a.split_k * seg_floats;
    constexpr int NI = WK >= 4 ? 1 : 4 / WK;
    const bool owner = WK <= 4 || wk < 4;  // threads that hold sums (f < 256)
    if (!partial) {
        if (owner) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int f = (i * WK + wk) * 64 + lane;
                const int l = f >> 2, v = f & 3;
                const int tok = tok0 + (l & 15);
                if (tok < a.n)
                    store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, row0 + (l >> 4) * 16 + v * 4, o[i][0], o[i][1],
                                    o[i][2], o[i][3]);
            }
        }
        return;
    }
    if (owner) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int f = (i * WK + wk) * 64 + lane;
            store_partial(wst + (size_t)part * seg_floats + (size_t)wm * 1024 + (size_t)f * 4,
                          f32x4{o[i][0], o[i][1], o[i][2], o[i][3]});
        }
    }
    // hand-over (see gemm_kernel): stores complete, barrier, arrival ticket, last one sums
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(work);
    if (tid == 0) *ticket = __hip_atomic_fetch_add(a.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket != (unsigned)a.split_k - 1u) {
        return;
    }
    if (tid == 0) __hip_atomic_store(a.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!owner) {
        return;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int f = (i * WK + wk) * 64 + lane;
        const float *src = wst + (size_t)wm * 1024 + (size_t)f * 4;
        f32x4 s4 = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int sp0 = 0; sp0 < a.split_k; sp0 += 4) {  // four contributors per round trip, summed in k order
            f32x4 p[4];
            const float *ps[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) ps[b] = src + (size_t)min(sp0 + b, a.split_k - 1) * seg_floats;
            load_partials4(ps[0], ps[1], ps[2], ps[3], p[0], p[1], p[2], p[3]);
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (sp0 + b < a.split_k) s4 += p[b];
        }
        const int l = f >> 2, v = f & 3;
        const int tok = tok0 + (l & 15);
        if (tok < a.n)
            store_features4(outp, resp, a.epilogue, (size_t)tok, out_ld, row0 + (l >> 4) * 16 + v * 4, s4[0], s4[1], s4[2],
                            s4[3]);
    }
}

}  // namespace tuna
