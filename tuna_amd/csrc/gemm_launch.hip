// Instantiations of the GEMM kernel and the variant dispatcher.
#include <atomic>
#include <cstdio>

#include "gemm_kernel.hpp"
#include "gemm_lean.hpp"
#include "gemm_narrow.hpp"

namespace tuna {

typedef void (*GemmKernelFn)(const GemmArgs);

struct Variant {
    int rw, u, tt, dec, maxt, minw, mode;  // mode: 0 tile walk, 1 grouped tile walk, 2 one tile per workgroup
    GemmKernelFn fn;
};

#define V(RW, U, TT, DEC, MAXT, MINW) {RW, U, TT, DEC, MAXT, MINW, 0, gemm_kernel<RW, U, TT, DEC, MAXT, MINW, 0>}
#define VG(RW, U, TT, DEC, MAXT, MINW) {RW, U, TT, DEC, MAXT, MINW, 1, gemm_kernel<RW, U, TT, DEC, MAXT, MINW, 1>}
#define V1(RW, U, TT, DEC, MAXT, MINW) {RW, U, TT, DEC, MAXT, MINW, 2, gemm_kernel<RW, U, TT, DEC, MAXT, MINW, 2>}
#define G TUNA_DECODE_GEMM

// Only variants whose main loop compiles without register spills are listed (a spill in the
// loop is a scratch access that drains the prefetch ring); the 4-token-tile variants are the
// exception: they spill a few values and are kept so that 33+ tokens take one pass;
// tuna_amd/make_configs.py mirrors this list.
//   MAXT 512 / MINW 2 : up to 8 waves per workgroup, up to 256 VGPRs
//   MAXT 512 / MINW 4 : up to 8 waves, at most 128 VGPRs, so that two workgroups share a CU
//   MAXT 1024 / MINW 4: 16-wave workgroups
static const Variant kVariants[] = {
    V(1, 2, 1, G, 512, 2), V(1, 2, 2, G, 512, 2), V(1, 2, 4, G, 512, 2),
    V(1, 4, 1, G, 512, 2), V(1, 4, 2, G, 512, 2),
    V(1, 8, 1, G, 512, 2), V(1, 8, 2, G, 512, 2),
    V(2, 2, 1, G, 512, 2), V(2, 4, 1, G, 512, 2),
    V(1, 2, 1, G, 512, 4), V(1, 4, 1, G, 512, 4),
    V(1, 2, 1, G, 1024, 4), V(1, 4, 1, G, 1024, 4),
    // dequant-rounding decode (correctness mode, not tuned)
    V(1, 2, 1, TUNA_DECODE_DEQUANT, 512, 2), V(1, 2, 2, TUNA_DECODE_DEQUANT, 512, 2),
    V(1, 2, 4, TUNA_DECODE_DEQUANT, 512, 2),
    // grouped launches (per-group token lists): 64 rows per wave only
    VG(1, 2, 1, G, 512, 2), VG(1, 2, 2, G, 512, 2), VG(1, 2, 4, G, 512, 2), VG(1, 4, 1, G, 512, 2), VG(1, 4, 2, G, 512, 2),
    VG(1, 2, 1, G, 512, 4), VG(1, 4, 1, G, 512, 4), VG(1, 2, 1, G, 1024, 4), VG(1, 4, 1, G, 1024, 4),
    VG(1, 2, 1, TUNA_DECODE_DEQUANT, 512, 2), VG(1, 2, 2, TUNA_DECODE_DEQUANT, 512, 2),
    VG(1, 2, 4, TUNA_DECODE_DEQUANT, 512, 2),
    // one workgroup per tile (launches that fit the device in one round, fixed split): optional
    // twins of dense variants, picked by launch_gemm when they apply
    V1(1, 2, 1, G, 512, 2), V1(1, 2, 2, G, 512, 2), V1(1, 4, 1, G, 512, 2), V1(1, 4, 2, G, 512, 2),
    V1(1, 8, 1, G, 512, 2), V1(2, 2, 1, G, 512, 2), V1(2, 4, 1, G, 512, 2),
    V1(1, 2, 1, G, 512, 4), V1(1, 4, 1, G, 512, 4), V1(1, 2, 1, G, 1024, 4), V1(1, 4, 1, G, 1024, 4),
};
#undef V
#undef VG
#undef V1
#undef G
static constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

static const Variant *find_variant(int rw, int u, int tt, int dec, int threads, int minw, int mode)
{
    const int maxt = threads <= 512 ? 512 : 1024;
    if (maxt == 1024) minw = 4;
    for (int i = 0; i < kNumVariants; ++i) {
        const Variant &v = kVariants[i];
        if (v.rw == rw && v.u == u && v.tt == tt && v.dec == dec && v.maxt == maxt && v.minw == minw && v.mode == mode)
            return &v;
    }
    return nullptr;
}

bool gemm_variant_exists(int rw, int prefetch, int token_tiles, int decode, int threads, int min_waves, int grouped)
{
    return find_variant(rw, prefetch, token_tiles, decode, threads, min_waves, grouped) != nullptr;
}

// ---- lean twins (gemm_lean.hpp) -------------------------------------------------------------
typedef void (*LeanKernelFn)(const uint8_t *, const void *, const float *, const float *, int, int, int, int, int,
                             void *, const void *, float *, unsigned *, int
);
struct LeanVariant {
    int wk, u, maxt;
    LeanKernelFn fn;
};
#define L5(WK, U) {WK, U, 512, gemm_lean_kernel<WK, U, 512, 2>}
#define L10(WK, U) {WK, U, 1024, gemm_lean_kernel<WK, U, 1024, 4>}
static const LeanVariant kLean[] = {
    L5(1, 2), L5(1, 4), L5(1, 8), L5(2, 2), L5(2, 4), L5(2, 8), L5(4, 2), L5(4, 4), L5(4, 8), L5(8, 2), L5(8, 4), L5(8, 8),
    L10(4, 2), L10(4, 4), L10(8, 2), L10(8, 4), L10(16, 2), L10(16, 4),
};
#undef L5
#undef L10
static constexpr int kNumLean = sizeof(kLean) / sizeof(kLean[0]);

// The lean kernel's LDS: decode table + max(x slice of the split, reduction planes) + ticket.
static size_t lean_lds_bytes(const GemmPlan &plan)
{
    const size_t x_bytes = (size_t)plan.args.steps_per_split * 1024;  // 16 tokens x 32 k x 2 bytes per k-step
    const size_t red_bytes = (size_t)(plan.threads / 64) * 4096;
    return (size_t)kLutBytes + (x_bytes > red_bytes ? x_bytes : red_bytes) + 16;
}

// Launches the lean kernel computes exactly like the general one (conditions in gemm_lean.hpp).
static const LeanVariant *lean_applies(const GemmPlan &plan, int cus)
{
    const GemmArgs &a = plan.args;
    if (!diag::lean_kernels()) return nullptr;
    if (a.group_rows || a.balanced || plan.rw != 1 || plan.token_tiles != 1 || plan.decode != TUNA_DECODE_GEMM) return nullptr;
    if (a.split_log2 < 0 || a.k_stagger != 0) return nullptr;
    if (plan.grid.x != (unsigned)a.tiles_total) return nullptr;
    if (a.k != a.steps_total * kStepK || a.steps_per_split * a.split_k != a.steps_total) return nullptr;
    if (a.steps_per_split % (a.waves_k * plan.prefetch) != 0) return nullptr;
    if (a.m % (a.waves_m * kRowsPerLoad) != 0) return nullptr;
    if (a.steps_per_split * 64 > 8 * plan.threads) return nullptr;  // at most 8 pieces of x per thread
    if (lean_lds_bytes(plan) > (size_t)kLdsLimit) return nullptr;
    if (plan.grid.x >= (1u << 19) || a.split_log2 > 15 || a.epilogue > 3) return nullptr;  // fields of the packed argument
    if (a.k >= (1 << 23)) return nullptr;  // 24-bit row pitch in the x staging
    // all tiles at once: workgroups per CU by LDS and by registers (at most 96 per lane: five
    // waves per SIMD); a launch of several rounds is what the tile walk of gemm_kernel is for
    const int waves = plan.threads / 64;
    const int by_lds = (int)((size_t)kLdsLimit / lean_lds_bytes(plan));
    const int by_regs = 20 / waves > 0 ? 20 / waves : 1;
    if ((long long)plan.grid.x > (long long)cus * (by_lds < by_regs ? by_lds : by_regs)) return nullptr;
    if (((uintptr_t)a.absmax & 15u) != 0) return nullptr;
    const int maxt = plan.threads <= 512 ? 512 : 1024;
    for (int i = 0; i < kNumLean; ++i)
        if (kLean[i].wk == a.waves_k && kLean[i].u == plan.prefetch && kLean[i].maxt == maxt) return &kLean[i];
    return nullptr;
}

// Whether a planned launch would take the lean kernel on a device of `cus` compute units (the host's derivation of
// configs asks: only configs that do are worth proposing for the shapes it proposes them for).
bool launch_is_lean(const GemmPlan &plan, int cus) { return lean_applies(plan, cus) != nullptr; }

// Dynamic LDS above 64 KB needs a one-time opt-in per kernel and device.
static OptInFlag g_attr_done[16][kNumVariants];
static OptInFlag g_lean_attr_done[16][kNumLean];
static std::atomic<int> g_cu_count[16];

hipError_t device_cus(int *dev_out, int *cus_out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    int n = g_cu_count[dev].load(std::memory_order_relaxed);
    if (!n) {
        e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (n <= 0) n = 256;
        g_cu_count[dev].store(n, std::memory_order_relaxed);
    }
    *dev_out = dev;
    *cus_out = n;
    return hipSuccess;
}

hipError_t launch_gemm(const GemmPlan &plan, hipStream_t stream)
{
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return e;
    const unsigned slots = (unsigned)(cus * plan.wgs_per_cu);
    const Variant *v = find_variant(plan.rw, plan.prefetch, plan.token_tiles, plan.decode, plan.threads, plan.min_waves,
                                    plan.args.group_rows ? 1 : 0);
    // (deeper rings with four token tiles exist in the 17..128-token streaming kernel only)
    if ((!v || plan.lds_weights || diag::lean_kernels()) && mid_applies(plan)) {
        e = launch_gemm_mid(plan, dev, cus, stream);
        if (e == hipSuccess) diag::count(diag::kLeanLaunches);
        return e;
    }
    if (!v) return hipErrorInvalidConfiguration;
    if (const LeanVariant *lv = lean_applies(plan, cus)) {
        const int li = (int)(lv - kLean);
        if ((e = ensure_lds_opt_in(g_lean_attr_done[dev][li], reinterpret_cast<const void *>(lv->fn))) != hipSuccess) return e;
        const GemmArgs &a = plan.args;
        const int swz = a.xcd_swizzle && plan.grid.x % 8 == 0;
        const int packed = a.split_log2 | a.waves_m << 4 | a.epilogue << 9 | swz << 11 | (int)(plan.grid.x >> 3) << 12;
        hipLaunchKernelGGL(lv->fn, plan.grid, dim3(plan.threads), lean_lds_bytes(plan), stream, a.q, a.x, a.code, a.absmax,
                           a.k, a.n, a.steps_per_split, packed, a.m, a.out, a.residual, a.ws, a.counters,
                           a.row_tiles
        );
        diag::count(diag::kLeanLaunches);
        return hipGetLastError();
    }
    // a dense launch with a fixed split whose tiles all fit the device at once needs no tile
    // walk: its one-tile-per-workgroup twin, where there is one, computes the same sums
    if (!plan.args.group_rows && !plan.args.balanced && plan.grid.x <= slots &&
        plan.grid.x == (unsigned)plan.args.tiles_total) {
        const Variant *v1 = find_variant(plan.rw, plan.prefetch, plan.token_tiles, plan.decode, plan.threads,
                                         plan.min_waves, 2);
        if (v1) v = v1;
    }
    const int vi = (int)(v - kVariants);
    if ((e = ensure_lds_opt_in(g_attr_done[dev][vi], reinterpret_cast<const void *>(v->fn))) != hipSuccess) return e;
    // persistent workgroups: as many as the device holds at once, each walks tiles with this stride
    dim3 grid = plan.grid;
    if (grid.x > slots) grid.x = slots;
    hipLaunchKernelGGL(v->fn, grid, dim3(plan.threads), plan.lds_bytes, stream, plan.args);
    return hipGetLastError();
}

void describe_gemm_launch(const GemmPlan &plan, int cus, char *buf, size_t len)
{
    const unsigned slots = (unsigned)(cus * plan.wgs_per_cu);
    const Variant *v = find_variant(plan.rw, plan.prefetch, plan.token_tiles, plan.decode, plan.threads, plan.min_waves,
                                    plan.args.group_rows ? 1 : 0);
    if ((!v || diag::lean_kernels()) && mid_describe(plan, buf, len)) return;
    if (!v) {
        snprintf(buf, len, "none");
        return;
    }
    if (const LeanVariant *lv = lean_applies(plan, cus)) {
        snprintf(buf, len, "gemm_lean_kernel<WK=%d,U=%d,%d threads> split_k=%d", lv->wk, lv->u, lv->maxt, plan.args.split_k);
        return;
    }
    int mode = v->mode;
    if (!plan.args.group_rows && !plan.args.balanced && plan.grid.x <= slots && plan.grid.x == (unsigned)plan.args.tiles_total &&
        find_variant(plan.rw, plan.prefetch, plan.token_tiles, plan.decode, plan.threads, plan.min_waves, 2))
        mode = 2;
    snprintf(buf, len, "gemm_kernel<RW=%d,U=%d,TT=%d,DEC=%d,%d threads,%d waves/SIMD,MODE=%d> split_k=%d", v->rw, v->u, v->tt,
             v->dec, v->maxt, v->minw, mode, plan.args.split_k);
}

// ---- narrow-row kernel (gemm_narrow.hpp) ---------------------------------------------------------
typedef void (*NarrowKernelFn)(const uint8_t *, const void *, const float *, const float *, int, int, int, int, void *, int,
                               const void *, int, int, int);
struct NarrowVariant {
    int rows, wk, u, tt;
    NarrowKernelFn fn, fn_perm;  // B fragments loaded per lane (up to 4 tokens) / contiguously and permuted
};
#define N(LW, WK, U) {16 * LW, WK, U, 1, gemm_narrow_kernel<LW, WK, U, false, 1>, gemm_narrow_kernel<LW, WK, U, true, 1>}
#define NT(LW, WK, U, TT) {16 * LW, WK, U, TT, gemm_narrow_kernel<LW, WK, U, true, TT>, gemm_narrow_kernel<LW, WK, U, true, TT>}
#define N24(WK, U) {24, WK, U, 1, gemm_narrow_kernel<2, WK, U, false, 1, false, 24>, gemm_narrow_kernel<2, WK, U, true, 1, false, 24>}
static const NarrowVariant kNarrow[] = {
    N(1, 4, 2),  N(1, 4, 4),  N(1, 4, 8),  N(1, 8, 2),  N(1, 8, 4),  N(1, 8, 8),  N(1, 16, 2), N(1, 16, 4), N(1, 16, 8),
    N(2, 4, 2),  N(2, 4, 4),  N(2, 4, 8),  N(2, 8, 2),  N(2, 8, 4),  N(2, 8, 8),  N(2, 16, 2), N(2, 16, 4), N(2, 16, 8),
    N(1, 1, 2),  N(1, 2, 2),  N(2, 1, 2),  N(2, 2, 2),
    N(4, 4, 2),  N(4, 4, 4),  N(4, 4, 8),  N(4, 8, 2),  N(4, 8, 4),  N(4, 8, 8),  N(4, 16, 2), N(4, 16, 4), N(4, 16, 8),
    // two and four token tiles per workgroup (17..64 tokens per pass over the weights)
    NT(1, 4, 2, 2), NT(1, 4, 4, 2), NT(1, 8, 2, 2), NT(1, 8, 4, 2), NT(1, 16, 2, 2), NT(1, 16, 4, 2),
    NT(2, 4, 2, 2), NT(2, 4, 4, 2), NT(2, 8, 2, 2), NT(2, 8, 4, 2), NT(2, 16, 2, 2), NT(2, 16, 4, 2),
    NT(4, 4, 2, 2), NT(4, 4, 4, 2), NT(4, 8, 2, 2), NT(4, 8, 4, 2), NT(4, 16, 2, 2), NT(4, 16, 4, 2),
    NT(1, 4, 2, 4), NT(1, 4, 4, 4), NT(1, 8, 2, 4), NT(1, 8, 4, 4),
    NT(2, 4, 2, 4), NT(2, 4, 4, 4), NT(2, 8, 2, 4), NT(2, 8, 4, 4),
    NT(4, 4, 2, 4), NT(4, 8, 2, 4),
    // 24 rows per workgroup (a 32-row tile three quarters full): row counts that are 256 tiles of 24 but 192 of 32
    N24(8, 2), N24(8, 4), N24(8, 8), N24(16, 2), N24(16, 4),
};
#undef N
#undef NT
#undef N24
static constexpr int kNumNarrow = sizeof(kNarrow) / sizeof(kNarrow[0]);
static OptInFlag g_narrow_attr_done[16][kNumNarrow][2];

static const NarrowVariant *find_narrow(int rows, int wk, int u, int tt)
{
    for (int i = 0; i < kNumNarrow; ++i)
        if (kNarrow[i].rows == rows && kNarrow[i].wk == wk && kNarrow[i].u == u && kNarrow[i].tt == tt) return &kNarrow[i];
    return nullptr;
}

bool narrow_variant_exists(int rows, int waves_k, int prefetch, int token_tiles)
{
    return find_narrow(rows, waves_k, prefetch, token_tiles) != nullptr;
}

void describe_narrow_launch(int rows, int waves_k, int prefetch, int token_tiles, int n, char *buf, size_t len)
{
    snprintf(buf, len, "gemm_narrow_kernel<LW=%d,WK=%d,U=%d,PERM=%d,TT=%d%s>", (rows + 15) / 16, waves_k, prefetch,
             (n > 4 || token_tiles > 1) ? 1 : 0, token_tiles, rows == 24 ? ",ROWS=24" : "");
}

hipError_t launch_gemm_narrow(const NarrowArgs &args, int rows, int waves_k, int prefetch, int token_tiles, hipStream_t stream)
{
    const NarrowVariant *v = find_narrow(rows, waves_k, prefetch, token_tiles);
    if (!v) return hipErrorInvalidConfiguration;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    const int vi = (int)(v - kNarrow);
    const int perm = args.n > 4;
    const NarrowKernelFn fn = perm ? v->fn_perm : v->fn;
    if ((e = ensure_lds_opt_in(g_narrow_attr_done[dev][vi][perm], reinterpret_cast<const void *>(fn))) != hipSuccess) return e;
    const size_t lds = (size_t)kLutBytes + (size_t)waves_k * ((rows + 15) / 16) * token_tiles * 1024;
    const dim3 grid((unsigned)(args.m / rows), (unsigned)((args.n + 16 * token_tiles - 1) / (16 * token_tiles)), 1);
    hipLaunchKernelGGL(fn, grid, dim3(waves_k * 64), lds, stream, args.q, args.x, args.code, args.absmax, args.k, args.n,
                       args.n_it, args.m, args.out, args.epilogue, args.residual, 0, 1, 0);
    return hipGetLastError();
}

// Scale blocks finer than a row: the narrow-row kernel's BLK variants (the scales of a ring slot's block travel
// through the ring with its weights).  block = 64 << blk_shift weights per scale.
struct BlockwiseVariant {
    int rows, wk, u, tt;
    NarrowKernelFn fn, fn_perm;
};
#define B(LW, WK, U) {16 * LW, WK, U, 1, gemm_narrow_kernel<LW, WK, U, false, 1, true>, gemm_narrow_kernel<LW, WK, U, true, 1, true>}
#define B2(LW, WK, U) {16 * LW, WK, U, 2, gemm_narrow_kernel<LW, WK, U, true, 2, true>, gemm_narrow_kernel<LW, WK, U, true, 2, true>}
static const BlockwiseVariant kBlockwise[] = {
    B(1, 4, 2), B(1, 8, 4), B(1, 16, 2), B(2, 8, 2), B(2, 8, 4), B(2, 16, 2), B(4, 4, 4), B(4, 8, 2), B(4, 8, 4), B(4, 16, 2),
    // two token tiles per workgroup: 17..32 tokens in one pass over the weights
    B2(1, 4, 2), B2(1, 8, 4), B2(2, 8, 2), B2(2, 8, 4), B2(4, 8, 2), B2(4, 8, 4),
};
#undef B
#undef B2
static constexpr int kNumBlockwise = sizeof(kBlockwise) / sizeof(kBlockwise[0]);

static const BlockwiseVariant *find_blockwise(int rows, int waves_k, int prefetch, int tt)
{
    for (int i = 0; i < kNumBlockwise; ++i)
        if (kBlockwise[i].tt == tt && kBlockwise[i].rows == rows && kBlockwise[i].wk == waves_k && kBlockwise[i].u == prefetch)
            return &kBlockwise[i];
    return nullptr;
}

static bool blockwise_fits(const BlockwiseVariant &v, int m, int k) { return m % v.rows == 0 && k % (kStepK * v.wk * v.u) == 0; }

// LDS of a variant's launch without the scales, and the bytes its workgroup's scales take there (rows of nblk + 1 floats)
static size_t blockwise_base_lds(const BlockwiseVariant &v) { return (size_t)kLutBytes + (size_t)v.wk * (v.rows / 16) * v.tt * 1024; }
static size_t blockwise_scale_bytes(const BlockwiseVariant &v, int nblk) { return (size_t)v.rows * (size_t)(nblk + 1) * 4; }

// The library's choice: the widest tile that still gives nine workgroups per sixteen compute units and whose scales
// fit in LDS (measured on the benchmark shapes and three 2560-wide ones with a scale per 64 weights: one round of
// 144 to 256 wide workgroups beats two rounds of narrower ones, and scales read from memory cost 1.4 to 2x).
static const BlockwiseVariant *choose_blockwise(int m, int k, int nblk, int cus, int tt)
{
    static const int pref[][3] = {{64, 8, 4}, {64, 8, 2}, {32, 8, 4}, {32, 8, 2}, {16, 8, 4}, {16, 4, 2}};
    for (int need_lds = 1; need_lds >= 0; --need_lds) {
        const BlockwiseVariant *fallback = nullptr;
        for (const auto &p : pref)
            for (int i = 0; i < kNumBlockwise; ++i) {
                const BlockwiseVariant &v = kBlockwise[i];
                if (v.tt != tt || v.rows != p[0] || v.wk != p[1] || v.u != p[2] || !blockwise_fits(v, m, k)) continue;
                if (need_lds && blockwise_base_lds(v) + blockwise_scale_bytes(v, nblk) > (size_t)kLdsLimit) continue;
                if (m / v.rows >= cus * 9 / 16) return &v;
                // fewer row tiles than that at every height: the narrowest tile that fits, the deeper ring first
                if (!fallback || v.rows < fallback->rows) fallback = &v;
            }
        if (fallback) return fallback;
    }
    return tt > 1 ? choose_blockwise(m, k, nblk, cus, 1) : nullptr;  // (shapes only the 16-row, 4-wave tile of one token tile fits)
}

// The narrow-row scale-block variant the library derives for a shape (token_tiles 1 or 2: what one pass should cover).
bool derive_blockwise_narrow(int m, int k, int blk_shift, int cus, int token_tiles, int *rows, int *waves_k, int *prefetch, int *tt)
{
    const BlockwiseVariant *v = choose_blockwise(m, k, k >> (6 + blk_shift), cus, token_tiles);
    if (!v) return false;
    *rows = v->rows, *waves_k = v->wk, *prefetch = v->u, *tt = v->tt;
    return true;
}

// Whether the variant (rows per workgroup, waves along k, ring, token tiles) is built and fits the shape.
bool blockwise_narrow_runs(int m, int k, int rows, int waves_k, int prefetch, int tt)
{
    const BlockwiseVariant *v = find_blockwise(rows, waves_k, prefetch, tt);
    return v && blockwise_fits(*v, m, k);
}

// Whether the variant keeps its workgroup's scales in LDS for this k and block size (else it reads them from memory
// in the loop, at 1.4 to 2 x the time).
bool blockwise_narrow_scales_in_lds(int k, int blk_shift, int rows, int waves_k, int prefetch, int tt)
{
    const BlockwiseVariant *v = find_blockwise(rows, waves_k, prefetch, tt);
    return v && blockwise_base_lds(*v) + blockwise_scale_bytes(*v, k >> (6 + blk_shift)) <= (size_t)kLdsLimit;
}

hipError_t launch_gemm_blockwise(const NarrowArgs &args, int blk_shift, int rows, int waves_k, int prefetch, int tt, hipStream_t stream)
{
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    const int nblk = args.k >> (6 + blk_shift);
    const BlockwiseVariant *v = find_blockwise(rows, waves_k, prefetch, tt);
    if (!v || !blockwise_fits(*v, args.m, args.k)) return hipErrorInvalidConfiguration;
    const int vi = (int)(v - kBlockwise);
    const int perm = args.n > 4;
    const NarrowKernelFn fn = perm ? v->fn_perm : v->fn;
    static OptInFlag done[16][kNumBlockwise][2];
    if ((e = ensure_lds_opt_in(done[dev][vi][perm], reinterpret_cast<const void *>(fn))) != hipSuccess) return e;
    size_t lds = blockwise_base_lds(*v);
    const dim3 grid((unsigned)(args.m / v->rows), (unsigned)((args.n + 16 * v->tt - 1) / (16 * v->tt)), 1);
    // the workgroup's scales in LDS when they fit beside the table and the reduction planes
    const size_t scale_bytes = blockwise_scale_bytes(*v, nblk);
    const int slds = diag::blockwise_scales_lds() && lds + scale_bytes <= (size_t)kLdsLimit;
    if (slds) lds += scale_bytes;
    hipLaunchKernelGGL(fn, grid, dim3(v->wk * 64), lds, stream, args.q, args.x, args.code, args.absmax, args.k, args.n,
                       args.k / kStepK / v->wk, args.m, args.out, TUNA_EPILOGUE_NONE, nullptr, blk_shift, nblk, slds);
    return hipGetLastError();
}

}  // namespace tuna
