// Instantiations and launcher of the 17..128-token streaming kernel (gemm_mid.hpp).
#include <atomic>
#include <cstdio>

#include "gemm_mid.hpp"

namespace tuna {

typedef void (*MidKernelFn)(const uint8_t *, const void *, const float *, const float *, int, int, int, int, void *,
                            const void *, int, int, int, float *, unsigned *, int, int);
struct MidVariant {
    int u, tt, xb, maxt;
    MidKernelFn fn;
    MidKernelFn fn_shared;  // twin without the nontemporal hint on the weight loads (token chunks side by side), or null
    MidKernelFn fn_lds;     // twin with the packed weights staged through LDS (lds_tile_rows = -1 or the diagnostic switch), or null
    MidKernelFn fn_lds_shared;  // ... without the nontemporal hint, or null
    MidKernelFn fn_split;      // twin for k split across workgroups, or null
    MidKernelFn fn_split_lds;  // ... with the packed weights staged through LDS, or null
};
#define M5(U, TT, XB) {U, TT, XB, 512, gemm_mid_kernel<U, TT, XB, 512, 2>, nullptr, nullptr, nullptr}
#define M5L(U, TT, XB) {U, TT, XB, 512, gemm_mid_kernel<U, TT, XB, 512, 2>, nullptr, gemm_mid_kernel<U, TT, XB, 512, 2, true, true>, nullptr}
#define M5LS(U, TT, XB)                                                                                             \
    {U, TT, XB, 512, gemm_mid_kernel<U, TT, XB, 512, 2>, nullptr, gemm_mid_kernel<U, TT, XB, 512, 2, true, true>, nullptr, \
     gemm_mid_kernel<U, TT, XB, 512, 2, true, false, true>, gemm_mid_kernel<U, TT, XB, 512, 2, true, true, true>}
#define M5SL(U, TT, XB)                                                                                             \
    {U, TT, XB, 512, gemm_mid_kernel<U, TT, XB, 512, 2>, gemm_mid_kernel<U, TT, XB, 512, 2, false>,                \
     gemm_mid_kernel<U, TT, XB, 512, 2, true, true>, gemm_mid_kernel<U, TT, XB, 512, 2, false, true>}
#define M10(U, TT, XB) {U, TT, XB, 1024, gemm_mid_kernel<U, TT, XB, 1024, 4>, nullptr, nullptr, nullptr}
#define M10L(U, TT, XB) {U, TT, XB, 1024, gemm_mid_kernel<U, TT, XB, 1024, 4>, nullptr, gemm_mid_kernel<U, TT, XB, 1024, 4, true, true>, nullptr}
#define M10LS(U, TT, XB)                                                                                            \
    {U, TT, XB, 1024, gemm_mid_kernel<U, TT, XB, 1024, 4>, nullptr, gemm_mid_kernel<U, TT, XB, 1024, 4, true, true>, nullptr, \
     gemm_mid_kernel<U, TT, XB, 1024, 4, true, false, true>, gemm_mid_kernel<U, TT, XB, 1024, 4, true, true, true>}
static const MidVariant kMid[] = {
    // (the ...S entries also have twins for k split across workgroups)
    M5LS(2, 2, 4), M5LS(4, 2, 4), M5(8, 2, 4), M5(2, 2, 8), M5(4, 2, 8), M5(8, 2, 8),
    M5LS(2, 4, 4), M5LS(4, 4, 4), M5(8, 4, 4), M5LS(2, 4, 8), M5LS(4, 4, 8), M5(8, 4, 8),
    M5SL(2, 8, 4), M5SL(2, 8, 8),  // (deeper rings with eight token tiles spill inside the loop)
    M10LS(2, 2, 4), M10LS(4, 2, 4),
    // one token tile: the large shapes at up to 16 tokens (small launches take gemm_lean.hpp first)
    M5(2, 1, 4), M5(4, 1, 4), M5(8, 1, 4), M5(2, 1, 8), M5(4, 1, 8), M5(8, 1, 8), M10L(2, 1, 4), M10L(4, 1, 4), M10(8, 1, 4),
};
#undef M5
#undef M5L
#undef M5LS
#undef M10LS
#undef M5SL
#undef M10
#undef M10L
static constexpr int kNumMid = sizeof(kMid) / sizeof(kMid[0]);

static bool lds_path(const GemmPlan &plan)
{
    return (plan.lds_weights || diag::weight_path() != 0) && (plan.threads == 512 || plan.threads == 1024) &&
           (plan.prefetch == 2 || plan.prefetch == 4);
}

// x chunk the kernel uses: the config's, capped so that two buffers fit beside the decode table
// (and, for the LDS-staged twin, the waves' weight rings).
static int mid_x_chunk(const GemmPlan &plan)
{
    int xc = plan.args.chunk_steps * kStepK;
    const int ring = lds_path(plan) ? (plan.threads / 64) * plan.prefetch * 1024 : 0;  // (twins without an LDS variant: a smaller chunk than they need, harmless)
    const int cap = (kLdsLimit - kLutBytes - ring) / (2 * plan.token_tiles * 32);  // k per buffer
    while (xc > cap) xc >>= 1;
    return xc;
}

static const MidVariant *mid_variant(const GemmPlan &plan, int *xc_out)
{
    const GemmArgs &a = plan.args;
    if (a.group_rows || a.balanced || plan.rw != 1 || plan.decode != TUNA_DECODE_GEMM) return nullptr;
    if (plan.token_tiles != 1 && plan.token_tiles != 2 && plan.token_tiles != 4 && plan.token_tiles != 8) return nullptr;
    if (a.k_stagger < 0 || a.k_stagger > 4096 || a.waves_k > 16 || (a.waves_k & (a.waves_k - 1)) != 0) return nullptr;
    // k split across workgroups: a power of two of equal parts, two or more token tiles (one token tile: the lean
    // kernel's launches), no stagger
    if (a.split_k != 1 && (a.split_log2 < 1 || a.split_log2 > 8 || plan.token_tiles < 2 || a.k_stagger != 0)) return nullptr;
    if (a.k != a.steps_total * kStepK || a.k >= (1 << 23)) return nullptr;
    if (a.m % (a.waves_m * kRowsPerLoad) != 0 || a.waves_m * a.waves_k > 16) return nullptr;
    const int xc = mid_x_chunk(plan);
    // a chunk is whole ring turns of the workgroup: xc / 32 steps, waves_k * prefetch per turn
    if (xc < a.waves_k * plan.prefetch * kStepK || (xc & (xc - 1)) != 0 || a.k % (xc * a.split_k) != 0) return nullptr;
    const int pieces = plan.token_tiles * 2 * xc;  // 16-byte pieces per chunk
    const int per_thread = (pieces + plan.threads - 1) / plan.threads;
    if (per_thread > 8) return nullptr;
    const int xb = per_thread <= 4 ? 4 : 8;
    const int maxt = plan.threads <= 512 ? 512 : 1024;
    for (int i = 0; i < kNumMid; ++i)
        if (kMid[i].u == plan.prefetch && kMid[i].tt == plan.token_tiles && kMid[i].xb == xb && kMid[i].maxt == maxt) {
            if (a.split_k != 1 && !kMid[i].fn_split) return nullptr;
            *xc_out = xc;
            return &kMid[i];
        }
    return nullptr;
}

bool mid_applies(const GemmPlan &plan)
{
    int xc;
    return mid_variant(plan, &xc) != nullptr;
}

bool mid_lds_applies(const GemmPlan &plan)
{
    int xc;
    const MidVariant *v = mid_variant(plan, &xc);
    if (!v || !v->fn_lds || !lds_path(plan)) return false;
    // (the twin fetches a lane's four scales with one 16-byte global -> LDS load)
    if ((reinterpret_cast<uintptr_t>(plan.args.absmax) & 15u) != 0) return false;
    // x pieces (one wave instruction per k-step and token tile) per wave and chunk: 1, 2 or 4
    const int pieces = (xc / 32) * plan.token_tiles, waves = plan.threads / 64;
    if (pieces % waves != 0 || (pieces / waves != 1 && pieces / waves != 2 && pieces / waves != 4)) return false;
    const size_t x_lds = 2 * (size_t)plan.token_tiles * 32 * (size_t)xc, red_lds = 2 * (size_t)waves * 1024;
    return x_lds >= red_lds && (size_t)kLutBytes + x_lds + (size_t)waves * plan.prefetch * 1024 <= (size_t)kLdsLimit;
}

bool mid_describe(const GemmPlan &plan, char *buf, size_t len)
{
    int xc;
    const MidVariant *v = mid_variant(plan, &xc);
    if (!v) return false;
    int used = snprintf(buf, len, "gemm_mid_kernel<U=%d,TT=%d,XB=%d,%d threads%s> x_chunk=%d", v->u, v->tt, v->xb, v->maxt,
                        mid_lds_applies(plan) ? ",weights through LDS" : "", xc);
    if (plan.args.split_k > 1 && used > 0 && (size_t)used < len) snprintf(buf + used, len - used, " split_k=%d", plan.args.split_k);
    return true;
}

// (the opt-in to more than 64 KB of dynamic LDS, once per variant and device: see ensure_lds_opt_in)
static OptInFlag g_mid_attr_done[16][kNumMid];

hipError_t launch_gemm_mid(const GemmPlan &plan, int dev, int cus, hipStream_t stream)
{
    int xc = 0;
    const MidVariant *v = mid_variant(plan, &xc);
    if (!v) return hipErrorInvalidConfiguration;
    const int vi = (int)(v - kMid);
    if (!g_mid_attr_done[dev][vi].load(std::memory_order_acquire)) {
        for (const MidKernelFn f : {v->fn, v->fn_shared, v->fn_lds, v->fn_lds_shared, v->fn_split, v->fn_split_lds}) {
            if (!f) continue;
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(f), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
            if (e != hipSuccess) return e;
        }
        g_mid_attr_done[dev][vi].store(1, std::memory_order_release);
    }
    const GemmArgs &a = plan.args;
    int xc_log2 = 0;
    while ((1 << xc_log2) < xc) ++xc_log2;
    const size_t x_lds = 2 * (size_t)plan.token_tiles * 32 * (size_t)xc;   // two buffers of one chunk
    const size_t red_lds = 2 * (size_t)(plan.threads / 64) * 1024;         // two buffers of one plane per wave
    const bool staged = mid_lds_applies(plan);
    const size_t lds = (size_t)kLutBytes + (staged ? x_lds + (size_t)(plan.threads / 64) * plan.prefetch * 1024
                                                   : (x_lds > red_lds ? x_lds : red_lds));
    // (a config that asks for the LDS-staged twin and cannot have it is an error, except for scales that are only
    // float-aligned: the register twin computes the same bits from them)
    if (plan.lds_weights && !staged && (reinterpret_cast<uintptr_t>(a.absmax) & 15u) == 0) return hipErrorInvalidConfiguration;
    dim3 grid = plan.grid;
    const int split_log2 = a.split_k > 1 ? a.split_log2 : 0;
    const int walk_tiles = a.row_tiles << split_log2;  // (row tile, part of k) pairs
    grid.x = (unsigned)(walk_tiles < cus ? walk_tiles : cus);  // one workgroup per CU (LDS), walking row tiles
    // Several token chunks that do not all fit the device at once: rather than one round of row
    // tile walkers per chunk (every round streams all weights from HBM again), fewer walkers whose
    // token chunks run side by side and share the weights through the caches.  With a multiple of
    // 8 walkers the chunks of a walker can sit on one XCD and share its L2 (the kernel's mapping
    // for chunks > 0); where that would leave more than an eighth of the CUs idle (9 chunks: 24
    // walkers, 216 workgroups) any walker count is used and the chunks of a walker are neighbours
    // in launch order only (chunks < 0), which still shares through the memory-side cache.
    // Mixtral gate+up, eight token tiles: 1024 tokens 1870 -> 1740 us, 2048 tokens 3746 -> 3520 us.
    int chunks = 0, n_wg = (int)grid.x;
    if (grid.y > 1 && (long long)walk_tiles * (long long)grid.y > (long long)cus && grid.y <= 4096) {
        const int c = (int)grid.y;
        const int w8 = (cus / c) & ~7;
        if (w8 >= 8 && (long long)w8 * c * 8 >= 7LL * cus) {
            n_wg = w8;
            chunks = c;
        } else {
            n_wg = cus / c > 0 ? cus / c : 1;
            chunks = -c;
        }
        grid = dim3((unsigned)(n_wg * c), 1, 1);
    }
    const int packed = a.waves_m | a.epilogue << 5 | xc_log2 << 8 | a.wk_log2 << 13 | a.k_stagger << 16;
    // weights that sibling workgroups re-read stay in the caches longer without the nontemporal hint
    // (Mixtral gate+up, 1024 tokens: 1745 -> 1687 us)
    const MidKernelFn fn = split_log2 ? (staged ? v->fn_split_lds : v->fn_split)
                           : staged   ? ((chunks && v->fn_lds_shared) ? v->fn_lds_shared : v->fn_lds)
                                      : (chunks && v->fn_shared) ? v->fn_shared : v->fn;
    hipLaunchKernelGGL(fn, grid, dim3(plan.threads), lds, stream, a.q, a.x, a.code, a.absmax, a.k, a.n, a.m, packed, a.out,
                       a.residual, walk_tiles, n_wg, chunks, a.ws, a.counters, split_log2, 0);
    return hipGetLastError();
}

// ---- scale blocks finer than a row: the BLK twins (one, two or four token tiles, register ring) -------------------------
struct MidBlkVariant {
    int u, tt, maxt;
    MidKernelFn fn;
};
static const MidBlkVariant kMidBlk[] = {
    {2, 1, 512, gemm_mid_kernel<2, 1, 4, 512, 2, true, false, false, true>},
    {4, 1, 512, gemm_mid_kernel<4, 1, 4, 512, 2, true, false, false, true>},
    {2, 1, 1024, gemm_mid_kernel<2, 1, 4, 1024, 4, true, false, false, true>},
    {4, 1, 1024, gemm_mid_kernel<4, 1, 4, 1024, 4, true, false, false, true>},
    {2, 2, 512, gemm_mid_kernel<2, 2, 4, 512, 2, true, false, false, true>},
    {4, 2, 512, gemm_mid_kernel<4, 2, 4, 512, 2, true, false, false, true>},
    {2, 2, 1024, gemm_mid_kernel<2, 2, 4, 1024, 4, true, false, false, true>},
    {4, 2, 1024, gemm_mid_kernel<4, 2, 4, 1024, 4, true, false, false, true>},
    {2, 4, 512, gemm_mid_kernel<2, 4, 4, 512, 2, true, false, false, true>},
    {4, 4, 512, gemm_mid_kernel<4, 4, 4, 512, 2, true, false, false, true>},
};
static constexpr int kNumMidBlk = sizeof(kMidBlk) / sizeof(kMidBlk[0]);
static OptInFlag g_mid_blk_attr_done[16][kNumMidBlk];

// The BLK twin for a planned launch (an unsplit config of one, two or four token tiles the streaming kernel takes, up to four - 1024
// threads: two - scales per thread and chunk), its x chunk and LDS size; null if there is none.
static const MidBlkVariant *mid_blk_variant(const GemmPlan &plan, int blk_shift, int *xc_out, size_t *lds_out)
{
    const GemmArgs &a = plan.args;
    int xc = 0;
    if ((plan.token_tiles != 1 && plan.token_tiles != 2 && plan.token_tiles != 4) || a.split_k != 1 || plan.lds_weights ||
        !mid_variant(plan, &xc))
        return nullptr;
    if (a.n > 16 * plan.token_tiles || a.k % (64 << blk_shift) != 0) return nullptr;  // (one pass over the weights)
    const int pieces = plan.token_tiles * 2 * xc;  // 16-byte x pieces per chunk
    if ((pieces + plan.threads - 1) / plan.threads > 4) return nullptr;
    const int rows_wg = a.waves_m * 64;
    const int nbc = xc >> (6 + blk_shift) > 0 ? xc >> (6 + blk_shift) : 1;  // scale blocks per chunk
    if ((long long)rows_wg * nbc > (plan.threads > 512 ? 2LL : 4LL) * plan.threads) return nullptr;  // scales per thread and chunk
    const size_t x_lds = 2 * (size_t)plan.token_tiles * 32 * (size_t)xc, s_lds = 2 * (size_t)nbc * (size_t)(rows_wg + 4) * 4;
    const size_t red_lds = 2 * (size_t)(plan.threads / 64) * 1024;
    const size_t lds = (size_t)kLutBytes + (x_lds + s_lds > red_lds ? x_lds + s_lds : red_lds);
    if (lds > (size_t)kLdsLimit) return nullptr;
    const int maxt = plan.threads <= 512 ? 512 : 1024;
    for (int i = 0; i < kNumMidBlk; ++i)
        if (kMidBlk[i].u == plan.prefetch && kMidBlk[i].tt == plan.token_tiles && kMidBlk[i].maxt == maxt) {
            *xc_out = xc;
            *lds_out = lds;
            return &kMidBlk[i];
        }
    return nullptr;
}

bool mid_blockwise_applies(const GemmPlan &plan, int blk_shift)
{
    int xc;
    size_t lds;
    return mid_blk_variant(plan, blk_shift, &xc, &lds) != nullptr;
}

hipError_t launch_gemm_mid_blockwise(const GemmPlan &plan, int blk_shift, int dev, int cus, hipStream_t stream)
{
    int xc = 0;
    size_t lds = 0;
    const MidBlkVariant *v = mid_blk_variant(plan, blk_shift, &xc, &lds);
    if (!v) return hipErrorInvalidConfiguration;
    hipError_t e = ensure_lds_opt_in(g_mid_blk_attr_done[dev][(int)(v - kMidBlk)], reinterpret_cast<const void *>(v->fn));
    if (e != hipSuccess) return e;
    const GemmArgs &a = plan.args;
    int xc_log2 = 0;
    while ((1 << xc_log2) < xc) ++xc_log2;
    const int n_wg = a.row_tiles < cus ? a.row_tiles : cus;  // one workgroup per CU, walking row tiles
    const int packed = a.waves_m | a.epilogue << 5 | xc_log2 << 8 | a.wk_log2 << 13 | a.k_stagger << 16;
    hipLaunchKernelGGL(v->fn, dim3((unsigned)n_wg, 1, 1), dim3(plan.threads), lds, stream, a.q, a.x, a.code, a.absmax, a.k, a.n, a.m,
                       packed, a.out, a.residual, a.row_tiles, n_wg, 0, nullptr, nullptr, 0, blk_shift);
    return hipGetLastError();
}

}  // namespace tuna
