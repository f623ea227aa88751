// Host side of the C ABI: argument checking, shape -> config, launch planning, the
// library-owned split-K workspace, and the HIP-event timing helpers.
//
// Replaces the reference's host dispatcher (kernel.cu:2962-3156: requiredSmem,
// LAUNCH_KERNEL_IF_CONDITION and the 122-arm if-chain in wrapper) and
// dequantize_wrapper (kernel.cu:3243-3253).
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "gemm_multi.hpp"
#include "tuna_internal.h"

namespace tuna {

static thread_local std::string g_error;

int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

int hip_fail(hipError_t e, const char *what)
{
    return fail(TUNA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------------------
// config validation and launch planning
// ---------------------------------------------------------------------------------------

static int check_shape(int m, int n, int k)
{
    if (m <= 0 || n <= 0 || k <= 0) return fail(TUNA_ERR_INVALID_ARG, "m, n, k must be positive (m=%d n=%d k=%d)", m, n, k);
    if ((m & 7) || (k & 7))
        return fail(TUNA_ERR_INVALID_ARG, "m and k must be multiples of 8, the packed block size (m=%d k=%d)", m, k);
    return TUNA_OK;
}

static inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
static inline int log2i(int v)
{
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

static int plan_gemm(int m, int n, int k, const tuna_gemm_config &c, int decode, GemmPlan *plan, int grouped = 0)
{
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    if ((unsigned long long)m * (unsigned long long)k / 2 >= (1ull << 32))
        return fail(TUNA_ERR_UNSUPPORTED, "packed weights of %llu bytes exceed the kernel's 32-bit offsets",
                    (unsigned long long)m * (unsigned long long)k / 2);
    if (decode != TUNA_DECODE_GEMM && decode != TUNA_DECODE_DEQUANT)
        return fail(TUNA_ERR_INVALID_ARG, "decode_mode %d is neither TUNA_DECODE_GEMM nor TUNA_DECODE_DEQUANT", decode);
    if (c.lds_tile_rows > 0) return fail(TUNA_ERR_INVALID_ARG, "plan_gemm called with a many-token config");
    if (c.lds_tile_rows < -1) return fail(TUNA_ERR_INVALID_ARG, "lds_tile_rows=%d (0, -1, 64, 128 or 256)", c.lds_tile_rows);
    if (c.rows_per_wave != 64 && c.rows_per_wave != 128 && c.rows_per_wave != 256)
        return fail(TUNA_ERR_UNSUPPORTED, "rows_per_wave=%d (64, 128 or 256)", c.rows_per_wave);
    if (c.prefetch != 2 && c.prefetch != 4 && c.prefetch != 8)
        return fail(TUNA_ERR_UNSUPPORTED, "prefetch=%d (2, 4 or 8)", c.prefetch);
    if (c.token_tiles != 1 && c.token_tiles != 2 && c.token_tiles != 4 && c.token_tiles != 8)
        return fail(TUNA_ERR_UNSUPPORTED, "token_tiles=%d (1, 2, 4 or 8)", c.token_tiles);
    if (c.waves_m < 1 || !is_pow2(c.waves_k) || c.waves_m * c.waves_k * 64 > kMaxThreads)
        return fail(TUNA_ERR_UNSUPPORTED, "waves_m=%d must be at least 1 and waves_k=%d a power of two, with at most 16 waves",
                    c.waves_m, c.waves_k);
    const int steps_total = ceil_div(k, kStepK);
    if (c.split_k < 0 || c.split_k > steps_total)
        return fail(TUNA_ERR_UNSUPPORTED, "split_k=%d must be in 0..%d for k=%d (0 = balanced)", c.split_k, steps_total, k);
    if (!is_pow2(c.x_chunk) || c.x_chunk < kStepK * c.waves_k * c.prefetch)
        return fail(TUNA_ERR_UNSUPPORTED, "x_chunk=%d must be a power of two >= 32*waves_k*prefetch=%d", c.x_chunk,
                    kStepK * c.waves_k * c.prefetch);
    if (c.k_stagger < 0 || c.k_stagger > 4096) return fail(TUNA_ERR_UNSUPPORTED, "k_stagger=%d must be in 0..4096", c.k_stagger);
    if (k >= (1 << 23)) return fail(TUNA_ERR_UNSUPPORTED, "k=%d exceeds the 24-bit row pitch of the x staging", k);
    const int rw = c.rows_per_wave / kRowsPerLoad;
    const int threads = c.waves_m * c.waves_k * 64;
    const int rows_wg = c.rows_per_wave * c.waves_m;
    // a chunk of x is staged as at most 4 (prefetch 8: 8) pieces of 16 bytes per thread
    const int x_cap = (c.prefetch == 8 ? 4 : 2) * threads;
    if (c.x_chunk * c.token_tiles > x_cap)
        return fail(TUNA_ERR_UNSUPPORTED, "x_chunk=%d x token_tiles=%d exceeds %d for %d threads and prefetch %d", c.x_chunk,
                    c.token_tiles, x_cap, threads, c.prefetch);

    // LDS = decode table + work area; the work area holds the x chunk in the main loop and, in
    // the epilogue, two alternating buffers of one accumulator plane (1 KB) of every wave.
    const int nacc = rw * 4 * c.token_tiles;
    const int lut = decode == TUNA_DECODE_GEMM ? kLutBytes : 64;
    const size_t x_lds = (size_t)c.token_tiles * 16 * (size_t)c.x_chunk * 2;
    // Two buffers of four planes (one barrier per 64-row group instead of four) are used when
    // they cost no occupancy: the x chunk leaves that much room anyway, or the config cannot
    // put two workgroups on a CU in the first place.
    const size_t plane_lds = (size_t)c.waves_k * c.waves_m * 1024;
    const size_t lds_small = (size_t)lut + (x_lds > 2 * plane_lds ? x_lds : 2 * plane_lds);
    // (a wave with a single 64-row group and token tile has nothing to alternate with: one buffer)
    const size_t big_planes = nacc == 4 ? 4 : 8;
    const size_t lds_big = (size_t)lut + (x_lds > big_planes * plane_lds ? x_lds : big_planes * plane_lds);
    const bool two_wgs_possible = threads <= 512 && 2 * lds_small <= (size_t)kLdsLimit;
    const int planes_log2 = (lds_big <= (size_t)kLdsLimit && (lds_big == lds_small || !two_wgs_possible)) ? 2 : 0;
    const size_t red_lds = planes_log2 ? big_planes * plane_lds : 2 * plane_lds;
    const size_t lds = planes_log2 ? lds_big : lds_small;
    if (lds > (size_t)kLdsLimit)
        return fail(TUNA_ERR_UNSUPPORTED, "config needs %zu bytes of LDS, the CU has %d", lds, kLdsLimit);

    // Two workgroups per CU need <= 128 VGPRs each: take that variant when both fit in LDS.
    int min_waves = threads > 512 ? 4 : 2;
    int wgs_per_cu = 1;
    if (threads <= 512 && 2 * lds <= (size_t)kLdsLimit &&
        gemm_variant_exists(rw, c.prefetch, c.token_tiles, decode, threads, 4, grouped)) {
        min_waves = 4;
        wgs_per_cu = 2;
    }
    // (a launch without a variant of the general kernel may still be one the 17..64-token streaming
    // kernel takes: decided below, when the launch arguments are known)
    const bool have_general = gemm_variant_exists(rw, c.prefetch, c.token_tiles, decode, threads, min_waves, grouped);

    const int row_tiles = ceil_div(m, rows_wg);
    const int tok_chunks = ceil_div(n, 16 * c.token_tiles);
    if (tok_chunks > 65535) return fail(TUNA_ERR_UNSUPPORTED, "n=%d needs %d token chunks (max 65535)", n, tok_chunks);
    if ((long long)row_tiles * c.split_k > 0x7fffffffLL) return fail(TUNA_ERR_UNSUPPORTED, "grid too large");

    // Balanced split (split_k == 0): the k ranges of all row tiles, cut into units of one ring
    // turn of the workgroup (coarser if the unit count would overflow the kernel's 32-bit
    // arithmetic), are divided evenly over the workgroups the device holds at once.
    const bool balanced = c.split_k == 0;
    const int slots = kMaxCus * wgs_per_cu;
    int unit_log2 = log2i(c.waves_k) + log2i(c.prefetch);
    int units_per_tile = 0;
    long long units_total = 0;
    if (balanced) {
        for (;; ++unit_log2) {
            units_per_tile = ceil_div(steps_total, 1 << unit_log2);
            units_total = (long long)row_tiles * units_per_tile;
            if ((units_total + 1) * slots < 0x7fffffffLL) break;
            if (units_per_tile == 1) return fail(TUNA_ERR_UNSUPPORTED, "too many row tiles (%d) for a balanced split", row_tiles);
        }
    }
    const unsigned grid_x = balanced ? (unsigned)(units_total < slots ? units_total : slots) : (unsigned)(row_tiles * c.split_k);

    GemmPlan &p = *plan;
    memset(&p, 0, sizeof(p));
    p.rw = rw;
    p.prefetch = c.prefetch;
    p.token_tiles = c.token_tiles;
    p.decode = decode;
    p.min_waves = min_waves;
    p.wgs_per_cu = wgs_per_cu;
    p.lds_weights = c.lds_tile_rows == -1 ? 1 : 0;
    p.threads = threads;
    p.lds_bytes = lds;
    p.grid = dim3(grid_x, (unsigned)tok_chunks, 1);
    // partial sums: one segment is waves_m * nacc planes of 1 KB; two slots per workgroup when balanced
    if (balanced) p.ws_bytes = (size_t)tok_chunks * grid_x * 2 * c.waves_m * nacc * 1024;
    else p.ws_bytes = c.split_k > 1 ? (size_t)tok_chunks * row_tiles * c.split_k * c.waves_m * nacc * 1024 : 0;
    p.n_counters = c.split_k != 1 ? (size_t)tok_chunks * row_tiles : 0;
    GemmArgs &a = p.args;
    a.m = m;
    a.n = n;
    a.k = k;
    a.waves_m = c.waves_m;
    a.waves_k = c.waves_k;
    a.wk_log2 = log2i(c.waves_k);
    a.split_k = c.split_k;
    a.split_log2 = (c.split_k > 0 && (c.split_k & (c.split_k - 1)) == 0) ? log2i(c.split_k) : -1;
    a.steps_total = steps_total;
    a.steps_per_split = balanced ? steps_total : ceil_div(steps_total, c.split_k);
    a.balanced = balanced ? 1 : 0;
    a.unit_log2 = unit_log2;
    a.units_per_tile = units_per_tile;
    a.units_total = (int)units_total;
    a.chunk_steps = c.x_chunk / kStepK;
    a.chunk_log2 = log2i(a.chunk_steps);
    a.row_tiles = row_tiles;
    a.xcd_swizzle = c.xcd_swizzle ? 1 : 0;
    a.k_stagger = c.k_stagger;
    a.lds_bytes = (int)lds;
    a.red_bytes = (int)red_lds;
    a.planes_log2 = planes_log2;
    a.tiles_total = row_tiles * c.split_k;
    if (!have_general && (grouped || !mid_applies(*plan)))
        return fail(TUNA_ERR_UNSUPPORTED,
                    "no %skernel variant for rows_per_wave=%d prefetch=%d token_tiles=%d decode=%d threads=%d",
                    grouped ? "grouped " : "", c.rows_per_wave, c.prefetch, c.token_tiles, decode, threads);
    if (p.lds_weights && (grouped || !mid_lds_applies(*plan)))
        return fail(TUNA_ERR_UNSUPPORTED,
                    "lds_tile_rows=-1 (packed weights through LDS) needs a dense launch of 8 or 16 waves, 64 rows per wave, prefetch 2 "
                    "or 4 (2 with eight token tiles), the GEMM's own decode, m a multiple of 64*waves_m, x chunks that divide k "
                    "(k/split_k for a power-of-two split with two or four token tiles; no other split) and leave room for the rings");
    return TUNA_OK;
}

// Many-token kernel: checks and launch arguments for a config with lds_tile_rows != 0.
struct TiledPlan {
    TiledArgs args;
    int tile_rows, tile_tokens;
    bool mfma32;  // rows_per_wave == 32 in a many-token config: 32 x 32 x 16 MFMAs instead of 16 x 16 x 32
    size_t lds_bytes, ws_bytes, n_counters;
};

static int plan_tiled(int m, int n, int k, const tuna_gemm_config &c, int decode, TiledPlan *plan)
{
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    if (decode != TUNA_DECODE_GEMM)
        return fail(TUNA_ERR_UNSUPPORTED, "the many-token kernel implements TUNA_DECODE_GEMM only");
    const int tile_tokens = 16 * c.token_tiles;
    const bool mfma32 = c.rows_per_wave == 32;
    if (!tiled_variant_exists(c.lds_tile_rows, tile_tokens, mfma32))
        return fail(TUNA_ERR_UNSUPPORTED, "no many-token kernel for a %d x %d tile (rows x tokens)%s", c.lds_tile_rows, tile_tokens,
                    mfma32 ? " with 32 x 32 MFMA tiles" : "");
    const int steps = ceil_div(k, 64);
    if (c.split_k < 1 || c.split_k > steps)
        return fail(TUNA_ERR_UNSUPPORTED, "split_k=%d must be in 1..%d for the many-token kernel", c.split_k, steps);
    if (c.split_k > 65535 || ceil_div(n, tile_tokens) > 65535) return fail(TUNA_ERR_UNSUPPORTED, "grid too large");
    memset(plan, 0, sizeof(*plan));
    plan->tile_rows = c.lds_tile_rows;
    plan->tile_tokens = tile_tokens;
    plan->mfma32 = mfma32;
    plan->lds_bytes = tiled_lds_bytes(c.lds_tile_rows, tile_tokens);
    const size_t tiles = (size_t)ceil_div(m, c.lds_tile_rows) * ceil_div(n, tile_tokens);
    plan->ws_bytes = c.split_k > 1 ? tiles * c.split_k * (size_t)c.lds_tile_rows * tile_tokens * 4 : 0;
    plan->n_counters = c.split_k > 1 ? tiles : 0;
    TiledArgs &a = plan->args;
    a.m = m;
    a.n = n;
    a.k = k;
    a.steps_total = steps;
    a.split_k = c.split_k;
    a.steps_per_split = ceil_div(steps, c.split_k);
    return TUNA_OK;
}

// Narrow-row kernel: checks and launch arguments for a config with rows_per_wave 16 or 32.
struct NarrowPlan {
    NarrowArgs args;
    int rows, waves_k, prefetch, token_tiles;
    size_t lds_bytes;
};

// rows_per_wave 16 or 32, or 64 with waves_m = 0 (64 rows with waves_m >= 1 is the streaming kernel)
static inline bool is_narrow(const tuna_gemm_config &c)
{
    return !c.lds_tile_rows &&
           (c.rows_per_wave == 16 || c.rows_per_wave == 24 || c.rows_per_wave == 32 || (c.rows_per_wave == 64 && c.waves_m == 0));
}

static int plan_narrow(int m, int n, int k, const tuna_gemm_config &c, int decode, NarrowPlan *plan)
{
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    if (decode != TUNA_DECODE_GEMM)
        return fail(TUNA_ERR_UNSUPPORTED, "the narrow-row kernel (rows_per_wave 16, 32) implements TUNA_DECODE_GEMM only");
    if ((unsigned long long)m * (unsigned long long)k / 2 >= (1ull << 32) || (unsigned long long)k * 32 >= (1ull << 32))
        return fail(TUNA_ERR_UNSUPPORTED, "operands exceed the kernel's 32-bit offsets");
    if (c.waves_m != (c.rows_per_wave == 64 ? 0 : 1) || c.split_k != 1 || c.k_stagger != 0)
        return fail(TUNA_ERR_UNSUPPORTED,
                    "the narrow-row kernel needs waves_m=1 (0 with rows_per_wave=64), split_k=1, k_stagger=0 (got %d, %d, %d)",
                    c.waves_m, c.split_k, c.k_stagger);
    if (!is_pow2(c.waves_k) || c.waves_k > 16 || !narrow_variant_exists(c.rows_per_wave, c.waves_k, c.prefetch, c.token_tiles))
        return fail(TUNA_ERR_UNSUPPORTED, "no narrow-row kernel for rows_per_wave=%d waves_k=%d prefetch=%d token_tiles=%d",
                    c.rows_per_wave, c.waves_k, c.prefetch, c.token_tiles);
    if (c.x_chunk != kStepK * c.waves_k * c.prefetch)
        return fail(TUNA_ERR_UNSUPPORTED, "the narrow-row kernel stages no x: x_chunk=%d must be 32*waves_k*prefetch=%d", c.x_chunk,
                    kStepK * c.waves_k * c.prefetch);
    if (m % c.rows_per_wave)
        return fail(TUNA_ERR_UNSUPPORTED, "rows_per_wave=%d needs m=%d to be a multiple of it", c.rows_per_wave, m);
    if (k % (kStepK * c.waves_k * c.prefetch))
        return fail(TUNA_ERR_UNSUPPORTED, "rows_per_wave=%d needs k=%d to be a multiple of 32*waves_k*prefetch=%d",
                    c.rows_per_wave, k, kStepK * c.waves_k * c.prefetch);
    if (ceil_div(n, 16 * c.token_tiles) > 65535) return fail(TUNA_ERR_UNSUPPORTED, "n=%d needs more than 65535 token chunks", n);
    memset(plan, 0, sizeof(*plan));
    plan->token_tiles = c.token_tiles;
    plan->rows = c.rows_per_wave;
    plan->waves_k = c.waves_k;
    plan->prefetch = c.prefetch;
    plan->lds_bytes = (size_t)kLutBytes + (size_t)c.waves_k * ((c.rows_per_wave + 15) / 16) * c.token_tiles * 1024;
    if (plan->lds_bytes > (size_t)kLdsLimit)
        return fail(TUNA_ERR_UNSUPPORTED, "config needs %zu bytes of LDS, the CU has %d", plan->lds_bytes, kLdsLimit);
    plan->args.m = m;
    plan->args.n = n;
    plan->args.k = k;
    plan->args.n_it = k / kStepK / c.waves_k;
    return TUNA_OK;
}

// The streaming-kernel branch of the derivation: 64 rows per wave, rings of 2 k-steps (those
// variants never spill), one or two token tiles.  Many rows -> wide row tiles without any k split
// (accumulators stored straight from registers); few rows -> one 64-row group per workgroup, 8
// waves along k and enough workgroups along k to occupy the CUs.  The dequant-rounding variants
// exist for up to 8 waves only.
static tuna_gemm_config derive_streaming(int m, int n, int k, int decode)
{
    tuna_gemm_config c;
    c.token_tiles = n <= 16 ? 1 : 2;  // more tokens loop over gridDim.y (the 4-tile variants spill)
    c.rows_per_wave = 64;
    c.prefetch = 2;
    c.xcd_swizzle = 1;
    c.k_stagger = 1;
    c.lds_tile_rows = 0;
    const int steps = ceil_div(k, kStepK);
    const int groups64 = ceil_div(m, kRowsPerLoad);
    if (groups64 >= 2048) {
        c.waves_m = 8, c.waves_k = 1;
    } else if (groups64 >= 512) {
        c.waves_m = 4, c.waves_k = 4;
    } else if (groups64 >= 256) {
        c.waves_m = 2, c.waves_k = 8;
    } else {
        c.waves_m = 1, c.waves_k = 8;
    }
    // 16-wave variants exist for one token tile and the GEMM's own decode only
    if ((c.token_tiles > 1 || decode != TUNA_DECODE_GEMM) && c.waves_m * c.waves_k > 8) c.waves_k /= 2;
    const int row_tiles = ceil_div(m, c.rows_per_wave * c.waves_m);
    const int group = c.waves_k * c.prefetch;  // k-steps one workgroup consumes per ring turn
    const int threads = c.waves_m * c.waves_k * 64;
    auto set_chunk = [&](int sps) {
        // x chunk: as long as the staging allows (4 pieces per thread), at most 1024 k, no longer than the split
        // ... and, with more row tiles than CUs, short enough (16 KB) for two workgroups to share a CU
        const int cap_k = (row_tiles > kMaxCus && threads <= 512) ? 512 / c.token_tiles : 1024;
        int chunk_steps = group;  // power of two
        while (chunk_steps < sps && chunk_steps * 2 * kStepK * c.token_tiles <= 2 * threads && chunk_steps * 2 * kStepK <= cap_k)
            chunk_steps *= 2;
        c.x_chunk = chunk_steps * kStepK;
    };
    // k split.  More row tiles than workgroup slots: none.  Otherwise the largest split that still
    // fits one round of tiles, if that fills at least half of the slots (measured: a half-empty
    // round of whole tiles beats the alternative); if no such split exists the k ranges are divided
    // evenly instead (balanced split), which costs a partial-sum epilogue in every workgroup but
    // leaves no CU idle.
    const int max_split = steps / (2 * group) > 0 ? steps / (2 * group) : 1;  // at least two ring turns per workgroup
    c.split_k = 1;
    set_chunk(steps);
    GemmPlan plan;
    if (plan_gemm(m, n, k, c, decode, &plan) != TUNA_OK) return c;
    const int slots = kMaxCus * plan.wgs_per_cu;
    // (an unsplit launch takes the streaming twin only with chunks that divide k: 3584 = 7 x 512, not 3.5 x 1024)
    auto dividing_chunk = [&]() {
        while (c.x_chunk > group * kStepK && k % c.x_chunk != 0) c.x_chunk /= 2;
    };
    if (row_tiles >= slots) {
        dividing_chunk();
        return c;
    }
    int split = slots / row_tiles;
    if (split > max_split) split = max_split;
    if (split < 1) split = 1;
    if ((double)row_tiles * split >= 0.5 * slots) {
        c.split_k = split;
        set_chunk(ceil_div(steps, split));
        if (split == 1) dividing_chunk();
    } else if (steps >= 2 * group) {
        c.split_k = 0;
    }
    return c;
}

// A config for shapes the tuned table does not cover, following what the tuner finds on the
// tuned shapes: many rows -> wide row tiles without any k split (accumulators stored straight
// from registers); few rows -> one 64-row group per workgroup, 8 waves along k and enough
// workgroups along k to occupy the CUs.  Rings of 2 k-steps: those variants never spill.
static bool config_runs(int m, int n, int k, const tuna_gemm_config &c);

// One round of narrow-row workgroups for the shape, if some tile height and tokens per pass give one (the rule is
// described where derive_config uses it).
static bool narrow_round(int m, int n, int k, tuna_gemm_config *out)
{
    tuna_gemm_config c;
    static const int kRows[4] = {64, 32, 24, 16};
    static const int kRing[5][2] = {{8, 4}, {4, 8}, {8, 2}, {4, 4}, {4, 2}};  // waves along k, ring depth
    // 17 tokens and more, first: passes of ONE token tile wherever some tile height puts 128..256 workgroups (from 64
    // for shapes of up to 8 MB) on the device, the height that gives the most; else passes of two, likewise.  Against
    // what the loops below pick (the tallest tile that fits their bounds, passes of two first for an even count of
    // token tiles): 1024 x 8192 at 64 tokens as 64 x 4 workgroups of 16 rows 8.2 us against 12.8 (16 x 4 of 64 rows),
    // 2048 x 8192 at 20 tokens 8.3 against 12.7, 1536 x 6144 at 40 tokens as 64 x 3 of 24 rows 7.9 against 10.5,
    // 3072 x 8192 at 40 tokens as 48 x 3 of 64 rows 13.0 against 16.1 (96 x 2 of 32 rows, two token tiles).
    if (n > 16) {
        const bool small = (long long)m * k <= (8ll << 21);  // 8 MB of packed weights
        for (int tt = 1; tt <= (k > 16384 ? 1 : 2); ++tt) {  // (two token tiles with k beyond 16384: 5120 x 27648 at 64 tokens 67 us, a split many-token tile 48)
            long long best_wgs = 0;
            static const int kOrder[4] = {64, 32, 16, 24};  // (24-row tiles only where no other height fits: they run 2..7 % behind 32-row tiles of fewer workgroups)
            for (int ri = 0; ri < 4; ++ri) {
                const int r = kOrder[ri];
                if (r == 24 && best_wgs) break;
                // (32-row tiles with k beyond 8192 from 65 tokens, one token tile per pass: below, the lean kernel's split
                // is ahead - 1024 x 14336 at 100 tokens as 32 x 7 workgroups 15.1 us against 20.4 of 16 x 7 of 64 rows,
                // at 40 tokens 15.1 against 11.1 of the lean kernel)
                const bool long_k_ok = r == 32 && tt == 1 && n > 64;
                if (m % r != 0 || (r < 32 && k > (small ? 8192 : 4096)) || (r < 64 && k > 8192 && !long_k_ok)) continue;
                const long long wgs = (long long)(m / r) * ceil_div(n, 16 * tt);
                // (up to 32 tokens on larger shapes from 150 workgroups, as in the loops below: 128 workgroups of 64 rows
                // lose to the lean kernel's split there - 4096 x 12288 at 17..32 tokens 19.8..20.9 us against 13.5..14.6)
                // (likewise up to 64 tokens with k beyond 8192: 2048 x 12288 at 64 tokens as 32 x 4 workgroups 19.8 us, lean 13.3)
                if (wgs < (small ? 64 : (n <= 32 || (n <= 64 && k > 8192)) ? 150 : 128) || wgs > kMaxCus || wgs <= best_wgs) continue;
                for (int gi = 0; gi < 5; ++gi) {
                    if (kRing[gi][0] != 8 || k % (32 * kRing[gi][0] * kRing[gi][1]) != 0 || (tt > 1 && kRing[gi][1] > 4)) continue;
                    memset(&c, 0, sizeof(c));
                    c.rows_per_wave = r, c.waves_m = r == 64 ? 0 : 1, c.waves_k = kRing[gi][0], c.prefetch = kRing[gi][1];
                    c.split_k = 1, c.token_tiles = tt, c.x_chunk = 32 * c.waves_k * c.prefetch;
                    if (config_runs(m, n, k, c)) {
                        *out = c, best_wgs = wgs;
                        break;
                    }
                }
            }
            if (best_wgs) return true;
        }
    }
    for (int pass = 0; pass < 2; ++pass) {
        // (65 tokens and more: three to eight passes side by side must run at once - 3072 x 8192 at 96 tokens as
        // 48 x 6 workgroups 26.8 us, as 48 x 3 of two token tiles 20.8 - so the round is 128..256 workgroups there)
        // (up to 16 tokens the second pass starts at 96 workgroups, at 64 with k below 8192, where the lean kernel is
        // no alternative: 1024 x 1024 as 64 workgroups of 16 rows 2.8..3.2 us against 8.8 of the general kernel,
        // 1024 x 4096 4.9..5.8 against 10.8, 2560 x 5120 as 80 of 32 rows 6.4..8.3 against 10.3; 2048 x 8192 as 64
        // of 32 rows 10.7 against 8.0 of the lean kernel)
        const int lo = n > 64 ? (pass ? 64 : 128) : pass ? (n <= 16 && k >= 8192 ? 96 : 64) : 150, hi = n > 64 ? kMaxCus : pass ? 600 : 300;
        if (pass && (long long)m * k > (8ll << 21)) break;  // 8 MB of packed weights
        // (24- and 16-row tiles also at 17..64 tokens, for the shapes too small for a round of taller ones:
        // 2048 x 2048 at 24 tokens as 128 x 2 workgroups of 16 rows 3.9 us against 6.1 of the lean kernel,
        // 1536 x 1536 at 48 tokens as 64 x 3 of 24 rows 4.4 against 11.6 of the general kernel; an odd number
        // of token tiles goes one tile per pass first where those passes fit the device at once, since passes of
        // two would compute a tile of padding: 5120 x 5120 at 48 tokens 11.0 us against 16.0, 2560 x 5120 at 40
        // tokens 7.5 against 12.0)
        const int tt_first = n <= 16 ? 1 : 2;
        for (int ri = 0; ri < 4; ++ri) {
            // (that second pass up to 16 tokens: the shortest tile first - 2048 x 2048 as 128 workgroups of 16 rows
            // 3.5..3.9 us, as 64 of 32 rows 4.1..4.6; 2560 x 5120 as 160 of 16 rows 5.7..7.1, as 80 of 32 rows 6.4..8.3)
            const int r = kRows[pass && n <= 16 ? 3 - ri : ri];
            if (m % r != 0 || (r < 32 && k > (pass && (n > 16 || k < 8192) ? 8192 : 4096)) || (r < 64 && k > 8192)) continue;
            // (65 tokens and more: one token tile per pass first wherever those passes fit the device at once, also for
            // an even count of token tiles - 1024 x 8192 at 256 tokens as 16 x 16 workgroups 13.7 us, as 16 x 8 of two
            // token tiles 19.8; 1024 x 4096 8.7 against 11.9)
            const int tt_step = (n > 64 || (n > 32 && ceil_div(n, 16) % 2 == 1)) ? 1 : -1;
            for (int tt = tt_step > 0 ? 1 : tt_first; tt >= 1 && tt <= tt_first; tt += tt_step) {
                const long long wgs = (long long)(m / r) * ceil_div(n, 16 * tt);
                if (wgs < lo || wgs > hi || (tt > 1 && k > 16384)) continue;
                if (tt_step > 0 && tt == 1 && wgs > kMaxCus) continue;  // (three passes only where they run at once)
                if (!pass && n <= 16 && r == 64 && wgs > 260) continue;  // (two 64-row tiles on some CUs: the streaming twin below)
                for (int gi = 0; gi < 5; ++gi) {
                    if (k % (32 * kRing[gi][0] * kRing[gi][1]) != 0 || (tt > 1 && kRing[gi][1] > 4)) continue;
                    // (a k that only four waves divide: 4096 x 11008 at 64..72 tokens 37..38 us, a split many-token tile 28;
                    // 8192 x 11008 at 24 tokens 37.9 us, the general kernel 26.9; 8192 x 6912 25.0 against 19.7)
                    if (n > 16 && kRing[gi][0] != 8) continue;
                    memset(&c, 0, sizeof(c));
                    c.rows_per_wave = r, c.waves_m = r == 64 ? 0 : 1, c.waves_k = kRing[gi][0], c.prefetch = kRing[gi][1];
                    c.split_k = 1, c.token_tiles = tt, c.x_chunk = 32 * c.waves_k * c.prefetch;
                    if (config_runs(m, n, k, c)) {
                        *out = c;
                        return true;
                    }
                }
            }
        }
    }
    return false;
}


static tuna_gemm_config derive_config(int m, int n, int k)
{
    tuna_gemm_config c;
    if (n <= 64) {
        // One round of workgroups of the narrow-row kernel (a workgroup owns 64, 32, 24 or 16 rows over the whole
        // k range, all waves along k: no partial sums leave the workgroup) when some tile height gives 150..300
        // of them - what the tuner finds on such shapes (3584 x 3584, 4608 x 3584, 5120 x 5120, 8192 x 4096,
        // 11008 x 4096, 15360 x 5120, 16384 x 4096, 16384 x 8192 at 16 tokens: 6.5..18.2 us, 20-35 % under the
        // streaming derivation below).  A workgroup reads all of x, 64 / rows times its weight bytes, so tiles of
        // fewer than 64 rows are taken up to k = 8192 and of fewer than 32 up to k = 4096 only (5120 x 13824 in
        // 32-row tiles: 20.9 us against 18.4).  17..64 tokens: the same with one or two token tiles per pass, the
        // passes side by side in the grid, so that rows x passes make the round (8192 x 3072 at 64 tokens as
        // 128 x 2 workgroups 11.4 us against 27.6; 64- and 32-row tiles only).
        // (Second pass, shapes of up to 8 MB that no tile height brings into that range: 96..600
        // workgroups - 2048 x 2048 as 128 workgroups of 16 rows 3.9 us against 9.0, 8960 x 1536 as 280 of 32 rows
        // 6.0 against 7.9; at 17..64 tokens from 64 workgroups and with the short tiles up to k = 8192:
        // 1280 x 5120 at 20 tokens as 80 x 2 of 16 rows 5.9 us against 16.7 of the general kernel.)
        if (narrow_round(m, n, k, &c)) {
            // (33..64 tokens with k beyond 16384: the split streaming launch described further down instead, where it
            // puts at least as many workgroups on the device as the round - 4096 x 24576 at 40 tokens 34.5 us against
            // 38.5, 3072 x 32768 at 64 tokens 39.4 against 46.5; 5120 x 27648 at 40 tokens, 160 workgroups against the
            // round's 240: 52.6 against 46.1)
            if (n > 32 && k > 16384 && m % 128 == 0 && m <= 8192) {
                const long long round_wgs = (long long)(m / c.rows_per_wave) * ceil_div(n, 16 * c.token_tiles);
                for (int split = 8; split >= 4; split /= 2) {
                    if ((long long)(m / 128) * split > kMaxCus) continue;
                    if ((long long)(m / 128) * split < round_wgs) break;
                    tuna_gemm_config s4;
                    memset(&s4, 0, sizeof(s4));
                    s4.rows_per_wave = 64, s4.waves_m = 2, s4.waves_k = 4, s4.split_k = split, s4.prefetch = 2, s4.x_chunk = 256;
                    s4.token_tiles = 4, s4.lds_tile_rows = -1;
                    if (config_runs(m, n, k, s4)) return s4;
                }
            }
            return c;
        }
        // Many rows (from 330 groups of 64; from 170 at 17..64 tokens): the streaming kernel, unsplit, with the packed
        // weights staged through LDS, 16 waves as 2 x 8 (4 x 4 from 576 groups), chunks of 512 k, a staggered walk -
        // what the tuner finds from 22016 x 4096 to 49152 x 6144 (16 tokens: 14.3, 15.9, 19.3, 30.5 us against 18.1,
        // 19.4, 22.0, 34.1 of the configs below); 17..64 tokens in passes of 32 side by side (12288 x 4096 at 64
        // tokens 19.3 us against 32.0, 16384 x 8192 31.7 against 57.0), 33..64 tokens on 576 groups or more in one
        // pass of 64 with 4 x 2 waves (37888 x 3584: 41.2 against 57.2).
        const int groups = m / 64;
        if (m % 256 == 0 && groups >= (n <= 16 ? 330 : 170) && k % 512 == 0) {
            memset(&c, 0, sizeof(c));
            c.rows_per_wave = 64, c.split_k = 1, c.token_tiles = n <= 16 ? 1 : 2, c.x_chunk = 512, c.xcd_swizzle = 1, c.k_stagger = 2;
            c.lds_tile_rows = -1;
            // (4 x 4 also where the 128-row tiles of 2 x 8 times the passes would not fit the device at once:
            // 20480 x 5120 at 64 tokens as 160 x 2 workgroups 41.5 us, as 80 x 2 31.7)
            const bool second_round = n > 16 && (long long)(groups / 2) * ceil_div(n, 32) > kMaxCus;
            if (groups >= 576 && n > 32) c.waves_m = 4, c.waves_k = 2, c.prefetch = 2, c.token_tiles = 4, c.x_chunk = 256;
            else if (groups >= 576 || second_round) c.waves_m = 4, c.waves_k = 4, c.prefetch = (n <= 16 && k >= 3072) ? 4 : 2, c.x_chunk = n <= 16 ? 512 : 256;
            else c.waves_m = 2, c.waves_k = 8, c.prefetch = 2;
            if (config_runs(m, n, k, c)) return c;
        }
        // Otherwise one round of 140..260 workgroups (..300 with the 16-token passes of 17..64 tokens side by side)
        // of the lean split-K kernel (one workgroup per row tile and power-of-two k slice, no staggered walk) where k
        // divides that way: the few-row shapes the streaming derivation below gives the general kernel with an odd
        // split (4096 x 8192 and 3072 x 8192 at 16 tokens: 12.2 -> 8.4 us; 4096 x 12288 at 32 tokens 21.0 -> 14.4),
        // and mid-size shapes of many rows (20480 x 5120: 19.1 -> 17.5 us).  The most workgroups win, then the
        // narrower row tile.  Up to four passes (64 tokens): few rows with long k have no narrow-row round there
        // either (2048 x 12288 at 33..48 tokens 30.1 -> 12.8 us, 1536 x 12288 at 56..64 tokens 33 -> 13,
        // 1024 x 14336 at 33..48 tokens 26.6 -> 11.0).
        static const int kLeanShape[9][3] = {{1, 16, 2}, {1, 8, 4}, {1, 8, 2}, {2, 8, 2}, {2, 4, 4}, {2, 4, 2}, {4, 4, 4}, {4, 4, 2}, {4, 2, 4}};
        tuna_gemm_config best;
        long long best_wgs = 0;
        const int passes16 = ceil_div(n, 16);
        for (int li = 0; li < 9 && passes16 <= 4; ++li) {
            const int wm = kLeanShape[li][0], wk = kLeanShape[li][1], pf = kLeanShape[li][2];
            if (m % (64 * wm) != 0 || k % 32 != 0) continue;
            const int steps = k / 32;
            for (int split = 1; split <= 16; split *= 2) {
                const long long wgs = (long long)(m / (64 * wm)) * split * passes16;
                if (wgs < 140 || wgs > (passes16 > 1 ? 300 : 260) || wgs <= best_wgs) continue;
                if (steps % split != 0 || (steps / split) % (wk * pf) != 0) continue;
                memset(&c, 0, sizeof(c));
                c.rows_per_wave = 64, c.waves_m = wm, c.waves_k = wk, c.prefetch = pf, c.split_k = split;
                c.token_tiles = 1, c.xcd_swizzle = 1;
                c.x_chunk = 32 * wk * pf;
                while (c.x_chunk * 2 <= 1024 && (k / split) % (c.x_chunk * 2) == 0) c.x_chunk *= 2;
                GemmPlan plan;
                if (plan_gemm(m, n, k, c, TUNA_DECODE_GEMM, &plan) != TUNA_OK || !launch_is_lean(plan, kMaxCus)) continue;
                best = c, best_wgs = wgs;
            }
        }
        if (best_wgs) return best;
    }
    // 65..512 tokens on small shapes: the narrow-row round of above with its passes of 16 or 32 tokens side by side,
    // where one exists - what the tuner finds there (2048 x 2048 at 72 tokens 5.8 us against 9.2 of the model's pick
    // below, 1536 x 6144 8.1 against 18.0, 3072 x 8192 14.2 against 22.5, 5120 x 5120 15.1 against 16.0; 1024 x 8192
    // at 130..224 tokens 13.4 against 22.5, 1536 x 12288 at 160 tokens 19.1 against 31.9, 3072 x 8192 at 144 tokens
    // 19.4 against 24.7, 1024 x 4096 at 512 tokens 12.4 against 16.2); larger shapes have no such round and go on to
    // the model.
    if (n > 64 && n <= 512 && narrow_round(m, n, k, &c)) return c;
    if (n > 32 && n <= 64 && k > 16384 && m % 128 == 0 && m <= 8192) {
        // 33..64 tokens, k beyond 16384, where no narrow-row round exists: the streaming kernel with four token tiles,
        // 128-row workgroups, the weights through LDS and k split in 4 or 8 across workgroups so that the grid fills
        // one round - the table's entry for Llama-70B's down projection, and what the tuner finds on such shapes
        // (5120 x 27648 at 64 tokens 52.5 us against 66.0 of the model's pick below, 6144 x 24576 48.5 against 60.5,
        // 7168 x 18432 40.2 against 48.5, 8192 x 20480 44.1 against 53.7; 10240 x 17408, split in 2: 61.6 against 57.9)
        for (int split = 8; split >= 4; split /= 2) {
            if ((long long)(m / 128) * split > kMaxCus) continue;
            memset(&c, 0, sizeof(c));
            c.rows_per_wave = 64, c.waves_m = 2, c.waves_k = 4, c.split_k = split, c.prefetch = 2, c.x_chunk = 256;
            c.token_tiles = 4, c.lds_tile_rows = -1;
            if (config_runs(m, n, k, c)) return c;
        }
    }
    if (n > 32) {
        // (from 33 tokens where the rules above found nothing - k that 512 does not divide, row counts between their
        // bounds: the general kernel's two passes ran 1.1..2.0 x the model's pick on 57 such cases, 4096 x 11008 at
        // 48 tokens 37.9 us against 27.6 of the 64 x 128 tile split in 4, 10240 x 6144 1.85 x)
        // 65 tokens and more: the tile whose grid costs least by a model read off
        // the timings of 36 shapes outside the table (1024 x 8192 ... 23040 x 3072) at 65 ... 3000 tokens, each with
        // up to thirty candidate launches.  A workgroup's time is its tile's rows x tokens (tokens beyond n included:
        // a tile is computed whole) times a factor of the kernel - the 256 x 256 tile 0.85, the streaming kernel
        // with eight token tiles on 512 rows 0.95, the 128 x 256 tile 1.00, eight token tiles on 256 rows 1.15,
        // 256 x 128 1.20, 128 x 128 and four token tiles on 256 rows 1.45, two token tiles on 256 rows 1.78, four on
        // 128 rows 1.95, two on 128 rows 2.0, up to 320 tokens one token tile on 256, 128 or 64 rows 2.6, 2.2, 4.0, and
        // the 64 x 128 tile 1.8 (what few rows with long k take, k split in 4 to 8; a 64 x 256 tile gains nothing)
        // - plus a fixed part that counts for short k (about 6 us), and grows by
        // a seventh from 160 to 256 workgroups on the device (clock and memory are shared); a launch is as many
        // rounds as its tiles need on 256 CUs, and a round that is not full takes nearly as long as a full one.
        // What the rules below cost before this one: 12288 x 4096 at 288 tokens 68 us (128 x 256 tiles, half empty)
        // against 46 (four token tiles, 240 workgroups), 20480 x 5120 at 384 tokens 153 against 91, 16384 x 8192 at
        // 640 tokens 249 against 195 (256 x 256), 2048 x 2048 at 384 tokens 27 against 13, 20480 x 5120 at 96 tokens
        // 55 against 36, 1024 x 8192 at 160 tokens 89 against 29.  Grids of fewer than 32 workgroups (64 from 256
        // tokens) are left to the rules below, which split k.
        struct Cand { int rows, tokens, streaming; double factor; };
        static const Cand kCand[14] = {{256, 256, 0, 0.85}, {512, 128, 1, 0.95}, {128, 256, 0, 1.00}, {256, 128, 1, 1.15}, {256, 128, 0, 1.20},
                                       {128, 128, 0, 1.45}, {256, 64, 1, 1.45},  {256, 32, 1, 1.78},  {128, 64, 1, 1.95},  {128, 32, 1, 2.00},
                                       {256, 16, 1, 2.60},  {128, 16, 1, 2.20},  {64, 16, 1, 4.00},   {64, 128, 0, 1.80}};
        tuna_gemm_config best;
        double best_cost = 0.0;
        bool found = false;
        static const int kSplit[6] = {1, 2, 3, 4, 6, 8};
        for (int ci = 0; ci < 14 * 6; ++ci) {
            // (the tiles of the many-token kernels also with k split in 2 ... 8 while the grid stays within one
            // round: a split workgroup does its share of the tile's time and the last one to arrive adds the
            // partial tiles, which costs about 0.3 us + 0.05 us per split and 1000 tile elements - what wins on
            // few rows with long k: 4096 x 11008 at 128 tokens 30 us as 32 tiles x 8 against 67 of the best
            // unsplit launch, 5120 x 13824 at 1000 tokens 154 us as 80 tiles of 256 x 256 x 3 against 200)
            const Cand &cd = kCand[ci / 6];
            const int split = kSplit[ci % 6];
            if ((cd.streaming && m % cd.rows != 0) || (cd.tokens == 16 && n > 320)) continue;
            if (split > 1 && (cd.streaming || ceil_div(k, 64) / split < 8)) continue;
            const long long tiles = (long long)ceil_div(m, cd.rows) * ceil_div(n, cd.tokens) * split;
            if (tiles < (n >= 256 ? 64 : 32) || (split > 1 && tiles > kMaxCus)) continue;
            const long long full = tiles / kMaxCus, rest = tiles % kMaxCus;
            const double rounds = 1.15 * (double)full + (rest ? 0.7 + 0.45 * (double)rest / kMaxCus : 0.0);
            const double area = (double)cd.rows * cd.tokens;
            double cost = rounds * (area * cd.factor / split + 1.2e7 / k) + (split > 1 ? (100.0 * split + 600.0) * area / k : 0.0);
            if (found && cost >= best_cost) continue;
            memset(&c, 0, sizeof(c));
            c.rows_per_wave = 64, c.split_k = split, c.prefetch = 2;
            if (!cd.streaming) {
                c.waves_m = 1, c.waves_k = 1, c.x_chunk = 64, c.token_tiles = cd.tokens / 16, c.lds_tile_rows = cd.rows;
            } else {
                c.token_tiles = cd.tokens / 16, c.waves_m = cd.rows / 64, c.waves_k = (c.token_tiles <= 2 ? 16 : 8) / c.waves_m;
                c.x_chunk = c.token_tiles == 8 ? 128 : c.token_tiles == 4 ? 256 : 512;
                // (a k that the chunk does not divide takes shorter chunks and loses the twin with the weights
                // through LDS: the factors above were not measured on that launch - 4096 x 11008 at 72 tokens runs
                // 62 us that way against 46 of 128 x 128 tiles with k split in 4 - so it is priced a third higher)
                const int want_chunk = c.x_chunk;
                while (c.x_chunk > 64 && k % c.x_chunk != 0) c.x_chunk /= 2;
                if (c.x_chunk != want_chunk) cost *= 1.35;
                c.xcd_swizzle = 1, c.lds_tile_rows = cd.rows == 512 ? 0 : -1;
            }
            if (!config_runs(m, n, k, c)) {
                if (c.lds_tile_rows != -1) continue;
                c.lds_tile_rows = 0;  // (no twin with the weights through LDS for this k)
                if (!config_runs(m, n, k, c)) continue;
            }
            if (found && cost >= best_cost) continue;
            best = c, best_cost = cost, found = true;
        }
        if (found) return best;
    }
    if (n > 64 && n <= 256 && k % 512 == 0) {
        // (what the model above leaves: grids too small for it)
        // 65..256 tokens: the streaming kernel with the weights through LDS, 16 waves (8 with four token tiles), the
        // passes of 16, 32 or 64 tokens side by side in the grid (they share the weights through the L2), the tile
        // height and the tokens per pass chosen so that row tiles x passes make one round of 150..256 workgroups -
        // what the tuner finds on 3072 x 8192, 4096 x 12288, 5120 x 5120, 12288 x 4096 and 16384 x 8192 (128 tokens:
        // 22.8, 32.9, 21.1, 27.3, 53.2 us against 60.3, 49.8, 37.2, 33.2, 57.3 of the rules below, which split k for
        // the many-token kernel there).
        static const int kTokWm[6][2] = {{4, 2}, {4, 4}, {2, 2}, {2, 4}, {1, 2}, {1, 4}};  // token tiles per pass, waves along the rows
        for (int ci = 0; ci < 6; ++ci) {
            const int tt = kTokWm[ci][0], wm = kTokWm[ci][1];
            if (m % (64 * wm) != 0) continue;
            const long long wgs = (long long)(m / (64 * wm)) * ceil_div(n, 16 * tt);
            if (wgs < 150 || wgs > kMaxCus) continue;  // (one round: 18432 x 6144 at 256 tokens as 288 workgroups 125 us, as 144 tiles of 128 x 256 89)
            for (int lds = -1; lds <= 0; ++lds) {
                memset(&c, 0, sizeof(c));
                c.rows_per_wave = 64, c.waves_m = wm, c.waves_k = (tt == 4 ? 8 : 16) / wm, c.prefetch = 2, c.split_k = 1;
                c.token_tiles = tt, c.x_chunk = tt == 4 ? 256 : 512, c.xcd_swizzle = 1, c.lds_tile_rows = lds;
                if (config_runs(m, n, k, c)) return c;
            }
        }
    }
    // (The rules from here on serve what the model above leaves: grids too small for it, and launches it cannot run.)
    if (n >= 256 && m >= 24576 && m % 512 == 0 && k % 128 == 0) {
        // many rows, several passes of 128 tokens: the streaming kernel with eight token tiles
        // (64 rows per wave, no split), whose token chunks run side by side and share the
        // weights - what the tuned entries of every shape from 28672 rows choose there.  8 waves
        // along the rows, or 4 x 2 where 512-row tiles times token chunks would not fill the CUs.
        // (Measured on 65536 x 4096, 24576 x 8192 and 40960 x 5120: 7-25 % faster than the
        // many-token kernel from 300 tokens, slower up to 128 tokens, where it stays.)
        memset(&c, 0, sizeof(c));
        const long long chunks = ceil_div(n, 128);
        c.rows_per_wave = 64, c.split_k = 1, c.prefetch = 2, c.x_chunk = 128, c.token_tiles = 8;
        c.waves_m = (m / 512) * chunks >= 200 ? 8 : 4;
        c.waves_k = 8 / c.waves_m;
        if (config_runs(m, n, k, c)) return c;
    }
    if (n > 32 && n < 256 && m >= 24576 && k % 128 == 0) {
        // many rows, 33..255 tokens: one pass of 64 (up to 64 tokens) or passes of 128 tokens
        // through the streaming kernel, with the largest row tile (8, 4 or 2 waves along the rows,
        // the others along k) that still gives 150 workgroups.  Measured on 65536 x 4096,
        // 24576 x 8192 and 40960 x 5120 at 40..200 tokens: 6-32 % faster than passes of 32 tokens
        // through the general kernel or the many-token kernel; where no such tile runs (eight token
        // tiles need at most two waves along k) the derivation below stays.
        const long long chunks = n <= 64 ? 1 : ceil_div(n, 128);
        for (int wm = 8; wm >= 2; wm /= 2) {
            if (m % (64 * wm) != 0 || (long long)(m / (64 * wm)) * chunks < 150) continue;
            memset(&c, 0, sizeof(c));
            c.rows_per_wave = 64, c.waves_m = wm, c.waves_k = 8 / wm, c.split_k = 1, c.prefetch = 2;
            c.x_chunk = c.waves_k <= 2 ? 128 : 256;
            c.token_tiles = n <= 64 ? 4 : 8;
            if (k % c.x_chunk == 0 && config_runs(m, n, k, c)) return c;
            break;
        }
    }
    if (n > 32 && n <= 128 && m >= 12288 && m < 24576 && m % 128 == 0 && k % 256 == 0 &&
        (long long)(m / 128) * ceil_div(n, 64) <= kMaxCus) {
        // 12288..24575 rows, 33..128 tokens: passes of 64 tokens through the streaming kernel with
        // 128-row tiles (2 waves along the rows, 4 along k) when all passes fit the device at once
        // (they then share the weights).  Measured on 12288 x 4096, 16384 x 8192 and 20480 x 5120: equal
        // to 38 % faster than passes of 32 tokens through the general kernel or the many-token
        // kernel (16384 x 8192 at 100 tokens 122 -> 57 us); with more passes than fit it loses.
        memset(&c, 0, sizeof(c));
        c.rows_per_wave = 64, c.waves_m = 2, c.waves_k = 4, c.split_k = 1, c.prefetch = 2, c.x_chunk = 256;
        c.token_tiles = 4;
        if (config_runs(m, n, k, c)) return c;
    }
    if (n >= 768) {
        // very many tokens: the 256 x 256 tile (one wave per SIMD) where it fills the device - from about 150
        // tiles, or from 90 with the k range split in two when k is 8192 or more (with k = 4096 the split loses:
        // 6144 x 4096 at 800 tokens 103 us against 63 of the 128-token tiles).  Measured on
        // 12288 x 6144, 5120 x 5120, 16384 x 8192, 3072 x 9216 and 20480 x 5120 at 1024..8192 tokens: 5-38 %
        // faster than the 128-token tiles below from 150 tiles (12288 x 6144 at 4096 tokens 842 -> 526 us),
        // 10 % with the split at 96 tiles, slower at 80.
        const long long tiles = (long long)ceil_div(m, 256) * ceil_div(n, 256);
        const int split = tiles >= 150 ? 1 : (tiles >= 90 && k >= 8192) ? 2 : 0;
        if (split) {
            memset(&c, 0, sizeof(c));
            c.rows_per_wave = 64, c.waves_m = 1, c.waves_k = 1, c.prefetch = 2, c.x_chunk = 64;
            c.token_tiles = 16, c.lds_tile_rows = 256, c.split_k = split;
            return c;
        }
    }
    if (n >= 128) {
        // many tokens: the kernel that decodes each weight tile once into LDS; 128-token tiles,
        // 256 rows (128 for few rows), k split until about one workgroup per CU
        memset(&c, 0, sizeof(c));
        c.rows_per_wave = 64, c.waves_m = 1, c.waves_k = 1, c.prefetch = 2, c.x_chunk = 64;
        c.token_tiles = 8;
        c.lds_tile_rows = m >= 16384 ? 256 : 128;
        // (from 257 tokens 128 x 256 tiles when they fill the device: 12288 x 4096 at 512 tokens 62.7 us against 82.9)
        if (n > 256 && (long long)ceil_div(m, 128) * ceil_div(n, 256) >= 150) c.lds_tile_rows = 128, c.token_tiles = 16;
        const long long tiles = (long long)ceil_div(m, c.lds_tile_rows) * ceil_div(n, 16 * c.token_tiles);
        const int steps64 = ceil_div(k, 64);
        long long split = tiles >= 150 ? 1 : kMaxCus / tiles;
        if (split > steps64 / 8) split = steps64 / 8;
        if (split < 1) split = 1;
        c.split_k = (int)split;
        return c;
    }
    return derive_streaming(m, n, k, TUNA_DECODE_GEMM);
}

// Whether config c can run the shape (the checks of the three planners).
static bool config_runs(int m, int n, int k, const tuna_gemm_config &c)
{
    if (c.lds_tile_rows > 0) {
        TiledPlan tp;
        return plan_tiled(m, n, k, c, TUNA_DECODE_GEMM, &tp) == TUNA_OK;
    }
    if (is_narrow(c)) {
        NarrowPlan np;
        return plan_narrow(m, n, k, c, TUNA_DECODE_GEMM, &np) == TUNA_OK;
    }
    GemmPlan plan;
    return plan_gemm(m, n, k, c, TUNA_DECODE_GEMM, &plan) == TUNA_OK;
}

// The table's buckets are the reference dispatcher's (kernel.cu:3022-3155) and every entry is tuned at the lower edge
// of its bucket.  A token count inside a bucket often runs faster with the entry of the NEXT bucket, which is tuned for
// more tokens per pass over the weights (8192 x 28672 at 17 tokens 79 -> 40 us, 8192 x 8192 at 20 tokens 23.8 -> 14.8,
// 229376 x 4096 at 100 tokens 297 -> 237) - but not always (2560 x 2560 at 65..96 tokens: 6.7 us with its own entry,
// 10.7 with the next).  Where the hand-over lies is therefore a field of the entry, next_from: the tuner times both
// entries at several counts inside the bucket and writes the count from which the next one wins; entries without
// a tuned value get make_configs.default_next_from.
static int select_config(int m, int n, int k, tuna_gemm_config *cfg, int *from_table)
{
    const TableEntry *own = nullptr;
    for (int i = 0; i < kConfigTableSize && !own; ++i) {
        const TableEntry &e = kConfigTable[i];
        if (e.m == m && e.k == k && n >= e.n_lo && n <= e.n_hi) own = &e;
    }
    const TableEntry *bucket = own;
    if (own && n >= own->next_from) {
        for (int i = 0; i < kConfigTableSize; ++i) {
            const TableEntry &e = kConfigTable[i];
            if (e.m == m && e.k == k && e.n_lo == own->n_hi + 1) {
                if (config_runs(m, n, k, e.cfg)) own = &e;
                break;
            }
        }
    }
    if (own) {
        *cfg = own->cfg;
        // The entries of the three upper buckets are tuned at 512, 1024 and 2048 tokens, and between those counts
        // the best grid changes with every token tile that n gains.  Shapes of fewer than 24576 rows therefore take
        // the pick of the derivation's cost model there (the same tiles the tuner chooses among in these buckets):
        // on the twelve such shapes of the table at 600 ... 2304 tokens the entries are 1.10 x the best of thirty
        // timed launches on average (up to 1.56: 6144 x 4096 at 1200 tokens 106 us against 68; 10240 x 8192 at 1536
        // tokens 289 against 217), the model's picks 1.02 x.  The entry stays where it was tuned: counts with as
        // many 128-token tiles as its tuning count.
        if (n > 512 && m < 24576) {
            const int tuned = own->n_lo <= 512 ? 512 : own->n_lo <= 769 ? 1024 : 2048;
            if (ceil_div(n, 128) != ceil_div(tuned, 128)) *cfg = derive_config(m, n, k);
        }
        // Inside a bucket too an entry can fall behind the derivation, which sizes its grid for n itself where the
        // entry's was sized for the tuning count (6144 x 4096 at 288..300 tokens: 41 us with the entry tuned at 256
        // tokens, 160 workgroups of 384 rows; 30 us derived, 240 of 256 rows) - and as often it does not (7680 x
        // 2560 at 72 tokens: 11.9 us against 14.8).  So this too is measured: the tuner times both at the sampled
        // counts of the bucket and writes the one stretch, if any, where the derived config wins into the entry.
        if (n >= bucket->derived_from && n < bucket->derived_to) *cfg = derive_config(m, n, k);
        if (from_table) *from_table = 1;
        return TUNA_OK;
    }
    *cfg = derive_config(m, n, k);
    if (from_table) *from_table = 0;
    return TUNA_OK;
}

// The config a launch without an explicit one runs.  The tuned table is for the GEMM's own decode;
// the dequant rounding (a correctness mode) has variants of the general kernel only - 64 rows per
// wave, rings of 2, up to 8 waves - so it always takes the derived streaming config.
static int select_config_for(int m, int n, int k, int decode, tuna_gemm_config *cfg, int *from_table)
{
    if (decode == TUNA_DECODE_GEMM) return select_config(m, n, k, cfg, from_table);
    *cfg = derive_streaming(m, n, k, decode);
    if (from_table) *from_table = 0;
    return TUNA_OK;
}

// The checks of the planner `c` belongs to, for a decode mode.
static int validate_for(int m, int n, int k, const tuna_gemm_config &c, int decode)
{
    if (c.lds_tile_rows > 0) {
        TiledPlan tp;
        return plan_tiled(m, n, k, c, decode, &tp);
    }
    if (is_narrow(c)) {
        NarrowPlan np;
        return plan_narrow(m, n, k, c, decode, &np);
    }
    GemmPlan plan;
    return plan_gemm(m, n, k, c, decode, &plan);
}

// ---------------------------------------------------------------------------------------
// split-K workspace: owned by the library, one per (device, stream)
//
// A buffer that has been handed to a launch is never freed or moved before
// tuna_release_workspaces: a HIP graph captured on the stream keeps the pointers in its kernel
// nodes and may be replayed at any later time.  The first request allocates generously (64 MB of
// partial sums and 64 K counters cover every entry of the tuned table); a larger request adds a
// new buffer and retires the old one, which stays allocated for the graphs that know it.
// ---------------------------------------------------------------------------------------

struct Workspace {
    float *ws = nullptr;
    size_t ws_bytes = 0;
    unsigned *counters = nullptr;
    size_t n_counters = 0;
    std::vector<void *> retired;  // outgrown buffers, kept for graphs captured while they were current
};

// First allocation for a (device, stream) pair: what the launch asks for, but at least this much, so that a process
// with many streams does not pay for the largest request of the table (48 MB) on each of them.
constexpr size_t kWsFirstBytes = (size_t)8 << 20;
constexpr size_t kWsFirstCounters = (size_t)64 << 10;

static std::mutex g_ws_mutex;
static std::map<std::pair<int, hipStream_t>, Workspace> g_workspaces;

// Size of the buffer that serves a request of `want` when `have` is current: unchanged if it
// fits, otherwise at least the first-allocation size and at least twice the current one.
static size_t grown_size(size_t have, size_t want, size_t first)
{
    if (want <= have) return have;
    size_t s = have ? 2 * have : first;
    return s > want ? s : want;
}

static int get_workspace(hipStream_t stream, size_t ws_bytes, size_t n_counters, Workspace *out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &w = g_workspaces[std::make_pair(dev, stream)];
    if (w.ws_bytes < ws_bytes || w.n_counters < n_counters) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
            return fail(TUNA_ERR_WORKSPACE,
                        "split-K workspace must grow (%zu bytes) while the stream is capturing; run the shape once before capture",
                        ws_bytes);
        if (w.ws_bytes < ws_bytes) {
            const size_t want = grown_size(w.ws_bytes, ws_bytes, kWsFirstBytes);
            float *fresh = nullptr;
            e = hipMalloc(reinterpret_cast<void **>(&fresh), want);
            if (e != hipSuccess) return fail(TUNA_ERR_WORKSPACE, "hipMalloc(%zu) for the split-K workspace: %s", want, hipGetErrorString(e));
            if (w.ws) w.retired.push_back(w.ws);
            w.ws = fresh;
            w.ws_bytes = want;
        }
        if (w.n_counters < n_counters) {
            const size_t want = grown_size(w.n_counters, n_counters, kWsFirstCounters);
            unsigned *fresh = nullptr;
            e = hipMalloc(reinterpret_cast<void **>(&fresh), want * sizeof(unsigned));
            if (e != hipSuccess) return fail(TUNA_ERR_WORKSPACE, "hipMalloc for the split-K counters: %s", hipGetErrorString(e));
            // zeroed on the launch stream (it is not capturing: checked above) and waited for there: a device-wide
            // synchronisation would disturb other threads' streams and captures.  Kernels leave the counters at zero.
            e = hipMemsetAsync(fresh, 0, want * sizeof(unsigned), stream);
            if (e == hipSuccess) e = hipStreamSynchronize(stream);
            if (e != hipSuccess) {
                (void)hipFree(fresh);
                return hip_fail(e, "clearing the split-K counters");
            }
            if (w.counters) w.retired.push_back(w.counters);
            w.counters = fresh;
            w.n_counters = want;
        }
    }
    *out = w;
    out->retired.clear();
    return TUNA_OK;
}

static void free_workspace(Workspace &w)
{
    if (w.ws) (void)hipFree(w.ws);
    if (w.counters) (void)hipFree(w.counters);
    for (void *p : w.retired) (void)hipFree(p);
    w = Workspace();
}

void drop_workspace(hipStream_t stream)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_workspaces.find(std::make_pair(dev, stream));
    if (it == g_workspaces.end()) return;
    free_workspace(it->second);
    g_workspaces.erase(it);
}

// ---------------------------------------------------------------------------------------
// Static scratch for tuna_matmul_static: the split-K partial sums and arrival counters of a
// launch in device memory that exists from module load on, so that the call allocates nothing.
// Every device the library runs on holds its own copy of the array at its own address until the
// process ends; the host-side name is a stand-in, the address comes from hipGetSymbolAddress
// (once per device, with that device current).
// ---------------------------------------------------------------------------------------
constexpr size_t kStaticCounters = (size_t)64 << 10;                       // arrival counters (4 bytes each) in front
constexpr size_t kStaticWsBytes = (size_t)TUNA_STATIC_WORKSPACE_BYTES;     // partial sums behind them
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticCounters * sizeof(unsigned) + kStaticWsBytes];

static std::mutex g_scratch_mutex;
static unsigned char *g_scratch_ptr[16];  // per device: address of that device's copy of `scratch`

static int static_scratch(unsigned char **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= 16) return fail(TUNA_ERR_NO_DEVICE, "device index %d outside 0..15", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!p) return fail(TUNA_ERR_WORKSPACE, "hipGetSymbolAddress returned no address for the static scratch");
        // The array is zero when the module is loaded and every launch returns the counters it
        // used to zero, so nothing needs clearing here or between calls.
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    *out = g_scratch_ptr[dev];
    return TUNA_OK;
}

// Where a launch gets its partial-sum buffer and counters from.
static int provide_workspace(bool use_static, hipStream_t stream, size_t ws_bytes, size_t n_counters, float **ws, unsigned **counters)
{
    if (!use_static) {
        Workspace w;
        int rc = get_workspace(stream, ws_bytes, n_counters, &w);
        if (rc) return rc;
        *ws = w.ws;
        *counters = w.counters;
        return TUNA_OK;
    }
    if (ws_bytes > kStaticWsBytes || n_counters > kStaticCounters)
        return fail(TUNA_ERR_WORKSPACE,
                    "this launch needs %zu bytes of partial sums and %zu counters; the static scratch holds %zu bytes and %zu counters "
                    "(use tuna_matmul_ex, whose workspace grows)",
                    ws_bytes, n_counters, kStaticWsBytes, kStaticCounters);
    unsigned char *base = nullptr;
    int rc = static_scratch(&base);
    if (rc) return rc;
    *counters = reinterpret_cast<unsigned *>(base);
    *ws = reinterpret_cast<float *>(base + kStaticCounters * sizeof(unsigned));
    return TUNA_OK;
}

int check_ptr(const void *p, const char *name, size_t align)
{
    if (!p) return fail(TUNA_ERR_INVALID_ARG, "%s is null", name);
    if (reinterpret_cast<uintptr_t>(p) % align) return fail(TUNA_ERR_INVALID_ARG, "%s must be %zu-byte aligned", name, align);
    return TUNA_OK;
}

// ---------------------------------------------------------------------------------------
// Several independent GEMMs in one call: batches of up to kMaxMultiProblems problems that the
// batched persistent kernel can run (gemm_multi.hpp) are one launch each; anything else is
// launched problem by problem on the same stream.
// ---------------------------------------------------------------------------------------

struct MultiPlan {
    MultiArgs args;
    int prefetch;
    size_t ws_bytes, n_counters;
};

// Whether problems[0..count) can run as one launch on a device of `cus` compute units; fills `plan`.
// waves_m / prefetch: 0 = chosen here.
// blk_shift >= 0: every problem's absmax is [m, k / (64 << blk_shift)], one scale per block of a row (the BLK variants).
// epilogues / residuals: per problem, or null (the fused-epilogue variants run when any problem has one).
static bool plan_multi(const tuna_gemm_problem *problems, int count, int cus, MultiPlan *plan, int waves_m = 0, int prefetch = 0,
                       int blk_shift = -1, const int32_t *epilogues = nullptr, const void *const *residuals = nullptr)
{
    if (count < 1 || count > kMaxMultiProblems || cus < 1) return false;
    const bool blk = blk_shift >= 0;
    bool epi = false;
    for (int i = 0; epilogues && i < count; ++i) epi = epi || epilogues[i] != TUNA_EPILOGUE_NONE;
    if (epi && blk) return false;
    if (!waves_m) waves_m = diag::multi_waves_m();
    if (!prefetch) prefetch = diag::multi_prefetch();
    // (a ring of two: with every wait of the ring exact it streams as fast as a ring of four on the longest
    // batches and faster on the others - fewer bytes requested ahead at a segment switch)
    if (!prefetch) prefetch = 2;
    if (!multi_variant_exists(blk ? 10 + prefetch : epi ? 20 + prefetch : prefetch)) return false;
    if (!waves_m) {
        // 256-row tiles (4 x 4 waves) when every problem allows, else narrower tiles and more waves along k
        waves_m = 4;
        for (int i = 0; i < count; ++i)
            while (waves_m > 1 && problems[i].m % (64 * waves_m)) waves_m >>= 1;
        // fewer 256-row tiles than workgroups: every tile would be shared by several workgroups and handed
        // over through memory; 128-row tiles (2 x 8 waves) give a workgroup whole tiles more often
        if (waves_m == 4) {
            long long tiles = 0;
            bool k_ok = true;
            for (int i = 0; i < count; ++i) {
                tiles += problems[i].m / 256;
                k_ok = k_ok && problems[i].k % (kStepK * 8 * prefetch) == 0;
            }
            if (tiles < cus && k_ok) waves_m = 2;
        }
    }
    if (waves_m != 1 && waves_m != 2 && waves_m != 4 && waves_m != 8 && waves_m != 16) return false;
    if (blk && waves_m > 4) return false;  // the scale buffers hold 256 rows
    const int waves_k = 16 / waves_m;
    // an x chunk of 32 k-steps (16 with scale blocks) is whole ring turns of every wave
    if (((blk ? 16 : 32) / waves_k) % prefetch || (blk ? 16 : 32) < waves_k * prefetch) return false;
    const int unit_steps = waves_k * prefetch;
    MultiArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    long long units = 0, tiles = 0;
    for (int i = 0; i < count; ++i) {
        const tuna_gemm_problem &p = problems[i];
        if (p.n > 16 || p.m % (64 * waves_m) || p.k % (kStepK * unit_steps)) return false;
        if ((unsigned long long)p.m * (unsigned long long)p.k / 2 >= (1ull << 32) || p.k >= (1 << 23)) return false;
        if (reinterpret_cast<uintptr_t>(p.absmax) % (blk ? 4 : 16)) return false;
        if (blk && (p.k % (64 << blk_shift) || p.k / (64 << blk_shift) < 2)) return false;
        if (p.code != problems[0].code) return false;  // one decode table per launch
        MultiProblem &mp = a.prob[i];
        mp.q = static_cast<const uint8_t *>(p.q);
        mp.x = p.x;
        mp.absmax = static_cast<const float *>(p.absmax);
        mp.out = p.out;
        mp.epilogue = epi ? epilogues[i] : TUNA_EPILOGUE_NONE;
        mp.residual = (epi && residuals && epilogues[i] == TUNA_EPILOGUE_RESIDUAL) ? residuals[i] : nullptr;
        mp.m = p.m, mp.n = p.n, mp.k = p.k;
        mp.units_per_tile = p.k / (kStepK * unit_steps);
        a.unit_begin[i] = (int)units;
        mp.tile_begin = (int)tiles;
        const long long row_tiles = p.m / (64 * waves_m);
        units += row_tiles * mp.units_per_tile;
        tiles += row_tiles;
        if ((units + 1) * cus >= 0x7fffffffLL) return false;
    }
    for (int i = count; i < kMaxMultiProblems; ++i) a.unit_begin[i] = 0x7fffffff;
    int n_wg = units < cus ? (int)units : cus;
    if (n_wg > kMaxCus) n_wg = kMaxCus;
    for (int w = 0, p = 0; w < n_wg; ++w) {
        const long long first = (long long)w * units / n_wg;  // balanced_begin
        while (p + 1 < count && first >= a.unit_begin[p + 1]) ++p;
        a.first_problem[w] = (unsigned char)p;
    }
    a.code = static_cast<const float *>(problems[0].code);
    a.n_problems = count;
    a.units_total = (int)units;
    a.waves_m = waves_m;
    a.wk_log2 = log2i(waves_k);
    a.n_wg = n_wg;
    a.swizzle = (n_wg % 8 == 0) ? 1 : 0;
    a.blk_shift = blk ? blk_shift : 0;
    // variant -2: ring of 2 with weights and x staged through LDS (x chunks of 512 k: every wave needs a whole
    // number of ring turns per chunk, so at most 8 waves along k)
    const bool lds = !blk && !epi && diag::multi_lds() != 0 && prefetch == 2 && waves_k <= 8 && multi_variant_exists(-2);
    plan->prefetch = blk ? 10 + prefetch : epi ? 20 + prefetch : lds ? -2 : prefetch;
    plan->ws_bytes = (size_t)n_wg * 2 * waves_m * 4096;
    plan->n_counters = (size_t)tiles;
    return true;
}

// A dense launch the batched kernel (gemm_multi.hpp) takes as a batch of one: balanced split, 64 rows
// per wave, 16 waves, one token tile, the GEMM's own decode, no fused epilogue.  (plan_multi checks
// the shape's alignment.)  A diagnostic build can turn it off together with the other twins (diag.h).
static bool stream_applies(const tuna_gemm_config &c, int n, int decode, int epilogue)
{
    return c.split_k == 0 && !c.lds_tile_rows && c.rows_per_wave == kRowsPerLoad && c.waves_m >= 1 && c.waves_m * c.waves_k == 16 &&
           c.token_tiles == 1 && n <= 16 && decode == TUNA_DECODE_GEMM && epilogue == TUNA_EPILOGUE_NONE &&
           (c.prefetch == 2 || c.prefetch == 4) && diag::lean_kernels() != 0;
}

static int matmul_impl(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n, int k,
                       const tuna_gemm_config *cfg, int decode, hipStream_t stream, int epilogue = TUNA_EPILOGUE_NONE,
                       const void *residual = nullptr, bool static_ws = false)
{
    int rc;
    if ((rc = check_shape(m, n, k))) return rc;
    if (epilogue != TUNA_EPILOGUE_NONE && epilogue != TUNA_EPILOGUE_RESIDUAL && epilogue != TUNA_EPILOGUE_SILU_MUL)
        return fail(TUNA_ERR_INVALID_ARG, "epilogue %d is not a TUNA_EPILOGUE_* value", epilogue);
    if (epilogue == TUNA_EPILOGUE_RESIDUAL && (rc = check_ptr(residual, "residual", 8))) return rc;
    if ((rc = check_ptr(q, "q", 16)) || (rc = check_ptr(x, "x", 16)) || (rc = check_ptr(code, "code", 4)) ||
        (rc = check_ptr(absmax, "absmax", 4)) || (rc = check_ptr(out, "out", 16)))
        return rc;
    tuna_gemm_config c;
    if (cfg) c = *cfg;
    else select_config_for(m, n, k, decode, &c, nullptr);
    if (c.lds_tile_rows > 0) {
        TiledPlan tp;
        if ((rc = plan_tiled(m, n, k, c, decode, &tp))) return rc;
        // the library's own pick may split k further than the static scratch has room for partial tiles (a split
        // by 8 of 256 tiles of 128 x 256 needs 32 MB): the split is then reduced until it fits - slower, but the
        // call that cannot allocate still runs; a config the caller names is taken as it is
        while (static_ws && !cfg && c.split_k > 1 && (tp.ws_bytes > kStaticWsBytes || tp.n_counters > kStaticCounters)) {
            c.split_k -= 1;
            if ((rc = plan_tiled(m, n, k, c, decode, &tp))) return rc;
        }
        tp.args.q = static_cast<const uint8_t *>(q);
        tp.args.x = x;
        tp.args.code = static_cast<const float *>(code);
        tp.args.absmax = static_cast<const float *>(absmax);
        tp.args.out = out;
        tp.args.epilogue = epilogue;
        tp.args.residual = residual;
        if (tp.ws_bytes && (rc = provide_workspace(static_ws, stream, tp.ws_bytes, tp.n_counters, &tp.args.ws, &tp.args.counters)))
            return rc;
        hipError_t e = launch_gemm_tiled(tp.args, tp.tile_rows, tp.tile_tokens, tp.mfma32, stream);
        if (e != hipSuccess) return hip_fail(e, "many-token gemm launch");
        return TUNA_OK;
    }
    // The narrow-row kernel reads a lane's scales 2 or 4 rows at a time.  A caller that names such a config must align
    // absmax for it; when the library picked the config itself it takes the streaming kernel's derived config for a
    // pointer that is only float-aligned (every other kernel checks the alignment where it chooses its variant).
    if (is_narrow(c) && !cfg) {
        NarrowPlan probe;
        if (plan_narrow(m, n, k, c, decode, &probe) == TUNA_OK && reinterpret_cast<uintptr_t>(absmax) % (probe.rows == 64 ? 16 : 8))
            c = derive_streaming(m, n, k, decode);
    }
    if (is_narrow(c)) {
        NarrowPlan np;
        if ((rc = plan_narrow(m, n, k, c, decode, &np))) return rc;
        if ((rc = check_ptr(absmax, "absmax", np.rows == 64 ? 16 : 8))) return rc;  // scales are read 2 or 4 rows at a time
        np.args.q = static_cast<const uint8_t *>(q);
        np.args.x = x;
        np.args.code = static_cast<const float *>(code);
        np.args.absmax = static_cast<const float *>(absmax);
        np.args.out = out;
        np.args.epilogue = epilogue;
        np.args.residual = residual;
        hipError_t e = launch_gemm_narrow(np.args, np.rows, np.waves_k, np.prefetch, np.token_tiles, stream);
        if (e != hipSuccess) return hip_fail(e, "narrow-row gemm launch");
        return TUNA_OK;
    }
    GemmPlan plan;
    if ((rc = plan_gemm(m, n, k, c, decode, &plan))) return rc;
    if (stream_applies(c, n, decode, epilogue)) {
        // a balanced split over 16-wave workgroups: the batched kernel with a batch of one walks the same
        // segments as gemm_kernel's balanced split and keeps its weight ring full across them
        int dev = 0, cus = 0;
        hipError_t e = device_cus(&dev, &cus);
        if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
        const tuna_gemm_problem one = {q, x, code, absmax, out, m, n, k};
        MultiPlan mp;
        if (plan_multi(&one, 1, cus, &mp, c.waves_m, c.prefetch)) {
            if ((rc = provide_workspace(static_ws, stream, mp.ws_bytes, mp.n_counters, &mp.args.ws, &mp.args.counters))) return rc;
            e = launch_gemm_multi(mp.args, mp.prefetch, dev, stream);
            if (e != hipSuccess) return hip_fail(e, "gemm launch");
            diag::count(diag::kMultiLaunches);
            return TUNA_OK;
        }
    }
    plan.args.q = static_cast<const uint8_t *>(q);
    plan.args.x = x;
    plan.args.code = static_cast<const float *>(code);
    plan.args.absmax = static_cast<const float *>(absmax);
    plan.args.out = out;
    plan.args.epilogue = epilogue;
    plan.args.residual = residual;
    if (plan.ws_bytes && (rc = provide_workspace(static_ws, stream, plan.ws_bytes, plan.n_counters, &plan.args.ws, &plan.args.counters)))
        return rc;
    hipError_t e = launch_gemm(plan, stream);
    if (e != hipSuccess) return hip_fail(e, "gemm launch");
    return TUNA_OK;
}

// Config of a grouped launch chosen by the library.  Candidates, in order: the tuned entry for the
// active rows if it is a streaming config the grouped variants can run as it stands; the derived
// streaming config with its row tile shrunk until it divides m_group; one 64-row group per
// workgroup with 8 waves along k, which runs any shape.  Table entries are never patched: a
// narrow-row, many-token or deep-ring entry has no grouped counterpart.
static int grouped_config(int m_group, int m_active, int max_tok, int k, int decode, tuna_gemm_config *out, GemmPlan *plan)
{
    auto runs = [&](const tuna_gemm_config &c) {
        if (c.lds_tile_rows || is_narrow(c) || c.waves_m < 1 || c.rows_per_wave != kRowsPerLoad) return false;
        if (m_group % (c.rows_per_wave * c.waves_m)) return false;
        return plan_gemm(m_active, max_tok, k, c, decode, plan, 1) == TUNA_OK;
    };
    tuna_gemm_config c;
    if (decode == TUNA_DECODE_GEMM) {
        select_config(m_active, max_tok, k, &c, nullptr);
        if (runs(c)) {
            *out = c;
            return TUNA_OK;
        }
    }
    c = derive_streaming(m_active, max_tok < 64 ? max_tok : 64, k, decode);
    while (c.waves_m > 1 && m_group % (c.rows_per_wave * c.waves_m)) --c.waves_m;
    {
        const int x_cap = 2 * c.waves_m * c.waves_k * 64;
        while (c.x_chunk * c.token_tiles > x_cap && c.x_chunk / 2 >= kStepK * c.waves_k * c.prefetch) c.x_chunk /= 2;
    }
    // 33 to 64 tokens in the largest group: four token tiles take them in one pass over the weights (the derivation
    // stops at two, whose second pass streams every group's weights again: Mixtral gate+up with 48 tokens per expert
    // 288 -> 170 us, down 160 -> 110), with the largest x chunk that still fits beside the table
    if (max_tok > 32) {
        tuna_gemm_config c4 = c;
        c4.token_tiles = 4;
        while (!runs(c4) && c4.x_chunk / 2 >= kStepK * c4.waves_k * c4.prefetch) c4.x_chunk /= 2;
        if (runs(c4)) {
            *out = c4;
            return TUNA_OK;
        }
    }
    if (runs(c)) {
        *out = c;
        return TUNA_OK;
    }
    memset(&c, 0, sizeof(c));
    c.rows_per_wave = kRowsPerLoad, c.waves_m = 1, c.waves_k = 8, c.split_k = 1, c.prefetch = 2, c.x_chunk = 512;
    c.token_tiles = max_tok <= 16 ? 1 : 2;
    c.xcd_swizzle = 1;
    if (runs(c)) {
        *out = c;
        return TUNA_OK;
    }
    return fail(TUNA_ERR_UNSUPPORTED, "no grouped config for m_group=%d, %d active rows, %d tokens, k=%d: %s", m_group, m_active,
                max_tok, k, std::string(g_error).c_str());
}

// Grouped GEMM: n_groups stacked weight matrices of m_group rows, group e applied to the
// activation rows offsets[e] .. offsets[e+1]-1 only.  The offsets are a host array: they are
// validated here and travel to the kernel as launch arguments (no device buffer, no copy).
static int matmul_grouped_impl(const void *q, const void *x, const void *code, const void *absmax, void *out, int m_group,
                               int n_groups, int k, const int32_t *offsets, const tuna_gemm_config *cfg, int decode,
                               hipStream_t stream)
{
    int rc;
    if (n_groups < 1 || n_groups > kMaxGroups)
        return fail(TUNA_ERR_INVALID_ARG, "n_groups=%d must be in 1..%d", n_groups, kMaxGroups);
    if (!offsets) return fail(TUNA_ERR_INVALID_ARG, "token_offsets is null");
    if (m_group <= 0 || (long long)m_group * n_groups > 0x7fffffffLL)
        return fail(TUNA_ERR_INVALID_ARG, "m_group=%d x n_groups=%d out of range", m_group, n_groups);
    if (offsets[0] < 0) return fail(TUNA_ERR_INVALID_ARG, "token_offsets[0]=%d is negative", offsets[0]);
    int max_tok = 0;
    for (int e = 0; e < n_groups; ++e) {
        const int cnt = offsets[e + 1] - offsets[e];
        if (cnt < 0) return fail(TUNA_ERR_INVALID_ARG, "token_offsets must not decrease (group %d)", e);
        if (cnt > max_tok) max_tok = cnt;
    }
    const int n_total = offsets[n_groups];
    const int m = m_group * n_groups;
    if ((rc = check_shape(m, n_total > 0 ? n_total : 1, k))) return rc;
    if (m_group % kRowsPerLoad) return fail(TUNA_ERR_UNSUPPORTED, "m_group=%d must be a multiple of %d", m_group, kRowsPerLoad);
    if ((unsigned long long)m * (unsigned long long)k / 2 >= (1ull << 32))
        return fail(TUNA_ERR_UNSUPPORTED, "packed weights of %llu bytes exceed the kernel's 32-bit offsets",
                    (unsigned long long)m * (unsigned long long)k / 2);
    if (max_tok == 0) return TUNA_OK;  // no group has a token: nothing to compute, nothing to write
    if ((rc = check_ptr(q, "q", 16)) || (rc = check_ptr(x, "x", 16)) || (rc = check_ptr(code, "code", 4)) ||
        (rc = check_ptr(absmax, "absmax", 4)) || (rc = check_ptr(out, "out", 16)))
        return rc;
    // Groups with more tokens than one pass of the grouped kernel takes (64: it would stream their weights once per 64
    // tokens) run as dense GEMMs of their own, each with the table's config for its token count - from 128 tokens a
    // group that is the many-token kernel at two to three times the rate, and a launch per group is nothing beside
    // hundreds of microseconds of matrix work.  (With an explicit config every group goes through the grouped kernel.)
    constexpr int kGroupedPassTokens = 64;
    const size_t group_q_bytes = (size_t)m_group * (size_t)k / 2;
    if (!cfg) {
        // (checked before anything is enqueued: a group that cannot run must not leave the others' rows written)
        for (int e = 0; e < n_groups; ++e) {
            const int cnt = offsets[e + 1] - offsets[e];
            if (cnt <= kGroupedPassTokens) continue;
            tuna_gemm_config dc;
            select_config_for(m_group, cnt, k, decode, &dc, nullptr);
            if ((rc = validate_for(m_group, cnt, k, dc, decode))) return rc;
        }
        for (int e = 0; e < n_groups; ++e) {
            const int cnt = offsets[e + 1] - offsets[e];
            if (cnt <= kGroupedPassTokens) continue;
            // (x rows are k fp16 values and out rows m_group: both multiples of 16 bytes, so the slices stay aligned)
            rc = matmul_impl(static_cast<const uint8_t *>(q) + (size_t)e * group_q_bytes,
                             static_cast<const uint8_t *>(x) + (size_t)offsets[e] * (size_t)k * 2, code,
                             static_cast<const float *>(absmax) + (size_t)e * (size_t)m_group,
                             static_cast<uint8_t *>(out) + (size_t)offsets[e] * (size_t)m_group * 2, m_group, cnt, k, nullptr, decode,
                             stream);
            if (rc) return rc;
        }
    }
    // Only the remaining groups with tokens are walked: the launch is planned for their rows alone.
    int n_active = 0;
    unsigned char act[kMaxGroups];
    max_tok = 0;
    for (int e = 0; e < n_groups; ++e) {
        const int cnt = offsets[e + 1] - offsets[e];
        if (cnt <= 0 || (!cfg && cnt > kGroupedPassTokens)) continue;
        act[n_active++] = (unsigned char)e;
        if (cnt > max_tok) max_tok = cnt;
    }
    if (n_active == 0) return TUNA_OK;  // every group with tokens ran as a dense GEMM
    const int m_active = m_group * n_active;
    tuna_gemm_config c;
    GemmPlan plan;
    if (cfg) {
        c = *cfg;
        if (c.lds_tile_rows || is_narrow(c) || c.waves_m < 1)
            return fail(TUNA_ERR_UNSUPPORTED, "grouped launches run the streaming kernel: rows_per_wave 64, waves_m >= 1, no lds_tile_rows");
        if (m_group % (c.rows_per_wave * c.waves_m))
            return fail(TUNA_ERR_UNSUPPORTED, "rows per workgroup (%d) must divide m_group=%d", c.rows_per_wave * c.waves_m, m_group);
        if ((rc = plan_gemm(m_active, max_tok, k, c, decode, &plan, 1))) return rc;
    } else if ((rc = grouped_config(m_group, m_active, max_tok, k, decode, &c, &plan))) {
        return rc;
    }
    GemmArgs &a = plan.args;
    a.q = static_cast<const uint8_t *>(q);
    a.x = x;
    a.code = static_cast<const float *>(code);
    a.absmax = static_cast<const float *>(absmax);
    a.out = out;
    a.m = m;  // bounds of q and absmax: all groups
    a.n = n_total;
    a.group_rows = m_group;
    a.n_groups = n_groups;
    a.tiles_per_group = m_group / (c.rows_per_wave * c.waves_m);
    for (int e = 0; e <= n_groups; ++e) a.tok_off[e] = offsets[e];
    for (int e = 0; e < n_active; ++e) a.act[e] = act[e];
    if (plan.ws_bytes) {
        Workspace w;
        if ((rc = get_workspace(stream, plan.ws_bytes, plan.n_counters, &w))) return rc;
        a.ws = w.ws;
        a.counters = w.counters;
    }
    hipError_t e = launch_gemm(plan, stream);
    if (e != hipSuccess) return hip_fail(e, "grouped gemm launch");
    return TUNA_OK;
}

extern "C" int tuna_matmul_blockwise(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                                     int k, int block_size, void *stream);

static int matmul_multi_impl(const tuna_gemm_problem *problems, int count, hipStream_t stream, const int32_t *epilogues = nullptr,
                             const void *const *residuals = nullptr)
{
    if (count < 0 || (count > 0 && !problems)) return fail(TUNA_ERR_INVALID_ARG, "problems is null or count=%d negative", count);
    if (count == 0) return TUNA_OK;
    int rc;
    for (int i = 0; epilogues && i < count; ++i) {
        const int ep = epilogues[i];
        if (ep != TUNA_EPILOGUE_NONE && ep != TUNA_EPILOGUE_RESIDUAL && ep != TUNA_EPILOGUE_SILU_MUL)
            return fail(TUNA_ERR_INVALID_ARG, "epilogues[%d]=%d is not a TUNA_EPILOGUE_* value", i, ep);
        if (ep == TUNA_EPILOGUE_RESIDUAL && (!residuals || (rc = check_ptr(residuals[i], "residual", 8))))
            return residuals ? rc : fail(TUNA_ERR_INVALID_ARG, "epilogues[%d] adds a residual but residuals is null", i);
    }
    // every problem is checked before anything is enqueued: a bad one must not leave half a batch behind
    for (int i = 0; i < count; ++i) {
        const tuna_gemm_problem &p = problems[i];
        if ((rc = check_shape(p.m, p.n, p.k))) return rc;
        if ((rc = check_ptr(p.q, "q", 16)) || (rc = check_ptr(p.x, "x", 16)) || (rc = check_ptr(p.code, "code", 4)) ||
            (rc = check_ptr(p.absmax, "absmax", 4)) || (rc = check_ptr(p.out, "out", 16)))
            return rc;
        tuna_gemm_config c;
        select_config(p.m, p.n, p.k, &c, nullptr);
        if ((rc = validate_for(p.m, p.n, p.k, c, TUNA_DECODE_GEMM))) return rc;
    }
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    for (int first = 0; first < count;) {
        // the longest run of problems from `first` that one launch can take
        MultiPlan plan;
        int take = count - first < kMaxMultiProblems ? count - first : kMaxMultiProblems;
        const int min_batch = diag::multi_min_batch();
        while (take >= min_batch && !plan_multi(problems + first, take, cus, &plan, 0, 0, -1, epilogues ? epilogues + first : nullptr,
                                                residuals ? residuals + first : nullptr))
            --take;
        if (take >= min_batch) {
            if ((rc = provide_workspace(false, stream, plan.ws_bytes, plan.n_counters, &plan.args.ws, &plan.args.counters))) return rc;
            e = launch_gemm_multi(plan.args, plan.prefetch, dev, stream);
            if (e != hipSuccess) return hip_fail(e, "batched gemm launch");
            diag::count(diag::kMultiLaunches);
            first += take;
            continue;
        }
        const tuna_gemm_problem &p = problems[first];
        const int ep = epilogues ? epilogues[first] : TUNA_EPILOGUE_NONE;
        if ((rc = matmul_impl(p.q, p.x, p.code, p.absmax, p.out, p.m, p.n, p.k, nullptr, TUNA_DECODE_GEMM, stream, ep,
                              ep == TUNA_EPILOGUE_RESIDUAL ? residuals[first] : nullptr)))
            return rc;
        ++first;
    }
    return TUNA_OK;
}

// Scale blocks: one absmax per block_size consecutive weights of a row (absmax [m, k/block_size], the
// layout of the reference's quantizer for block_size < k, test.py:15-17); block_size == k is one per row.
static int check_block_size(int k, int bs, bool pow2_up_to_256)
{
    if (bs == k) return TUNA_OK;
    if (bs < 8 || (bs & 7) || k % bs) return fail(TUNA_ERR_INVALID_ARG, "block_size=%d must be a multiple of 8 that divides k=%d", bs, k);
    if (pow2_up_to_256 && (!is_pow2(bs) || bs > 256))
        return fail(TUNA_ERR_UNSUPPORTED, "block_size=%d: the quantizer takes 8, 16, 32, 64, 128, 256 or k", bs);
    return TUNA_OK;
}

static int dequant_impl(const void *q, const void *absmax, const void *code, void *out, int m, int k, int bs, int decode,
                        hipStream_t stream)
{
    int rc;
    if ((rc = check_shape(m, 1, k))) return rc;
    if (decode != TUNA_DECODE_GEMM && decode != TUNA_DECODE_DEQUANT)
        return fail(TUNA_ERR_INVALID_ARG, "decode_mode %d is neither TUNA_DECODE_GEMM nor TUNA_DECODE_DEQUANT", decode);
    if ((rc = check_block_size(k, bs, false))) return rc;
    if ((rc = check_ptr(q, "q", 16)) || (rc = check_ptr(absmax, "absmax", 4)) || (rc = check_ptr(code, "code", 4)) ||
        (rc = check_ptr(out, "out", 16)))
        return rc;
    hipError_t e = launch_dequant(static_cast<const uint8_t *>(q), static_cast<const float *>(absmax),
                                  static_cast<const float *>(code), out, m, k, bs, decode, stream);
    if (e != hipSuccess) return hip_fail(e, "dequant launch");
    return TUNA_OK;
}

static int quantize_impl(const void *w, const void *code, void *q, void *absmax, int m, int k, int bs, hipStream_t stream)
{
    int rc;
    if ((rc = check_shape(m, 1, k))) return rc;
    if ((rc = check_block_size(k, bs, true))) return rc;
    if ((rc = check_ptr(w, "w", 16)) || (rc = check_ptr(code, "code", 4)) || (rc = check_ptr(q, "q", 16)) ||
        (rc = check_ptr(absmax, "absmax", 4)))
        return rc;
    hipError_t e = launch_quantize(w, static_cast<const float *>(code), q, static_cast<float *>(absmax), m, k, bs, stream);
    if (e != hipSuccess) return hip_fail(e, "quantize launch");
    return TUNA_OK;
}

}  // namespace tuna

using namespace tuna;

extern "C" {


TUNA_EXPORT int tuna_version(void) { return TUNA_AMD_VERSION; }

TUNA_EXPORT const char *tuna_status_string(int status)
{
    switch (status) {
    case TUNA_OK: return "ok";
    case TUNA_ERR_INVALID_ARG: return "invalid argument";
    case TUNA_ERR_UNSUPPORTED: return "unsupported shape or config";
    case TUNA_ERR_HIP: return "HIP runtime error";
    case TUNA_ERR_NO_DEVICE: return "no usable device";
    case TUNA_ERR_WORKSPACE: return "split-K workspace unavailable";
    default: return "unknown status";
    }
}

TUNA_EXPORT const char *tuna_last_error(void) { return g_error.c_str(); }

TUNA_EXPORT int tuna_matmul(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                            int k, void *stream)
{
    return matmul_impl(q, x, code, absmax, out, m, n, k, nullptr, TUNA_DECODE_GEMM, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_matmul_ex(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                               int k, const tuna_gemm_config *cfg, int decode_mode, void *stream)
{
    return matmul_impl(q, x, code, absmax, out, m, n, k, cfg, decode_mode, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_init(void)
{
    unsigned char *p = nullptr;
    return static_scratch(&p);
}

TUNA_EXPORT int tuna_matmul_static(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                                   int k, const tuna_gemm_config *cfg, int decode_mode, void *stream)
{
    return matmul_impl(q, x, code, absmax, out, m, n, k, cfg, decode_mode, static_cast<hipStream_t>(stream), TUNA_EPILOGUE_NONE,
                       nullptr, true);
}

TUNA_EXPORT int tuna_matmul_fused(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                                  int k, const tuna_gemm_config *cfg, int decode_mode, int epilogue, const void *residual,
                                  void *stream)
{
    return matmul_impl(q, x, code, absmax, out, m, n, k, cfg, decode_mode, static_cast<hipStream_t>(stream), epilogue, residual);
}

TUNA_EXPORT int tuna_matmul_multi(const tuna_gemm_problem *problems, int count, void *stream)
{
    return matmul_multi_impl(problems, count, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_matmul_multi_fused(const tuna_gemm_problem *problems, const int32_t *epilogues, const void *const *residuals,
                                        int count, void *stream)
{
    return matmul_multi_impl(problems, count, static_cast<hipStream_t>(stream), epilogues, residuals);
}

TUNA_EXPORT int tuna_matmul_multi_blockwise(const tuna_gemm_problem *problems, int count, int block_size, void *stream)
{
    if (count < 0 || (count > 0 && !problems)) return fail(TUNA_ERR_INVALID_ARG, "problems is null or count=%d negative", count);
    if (count == 0) return TUNA_OK;
    if (block_size < 64 || !is_pow2(block_size))
        return fail(TUNA_ERR_UNSUPPORTED, "block_size=%d: the batched blockwise GEMM takes 64, 128, 256, ...", block_size);
    int rc;
    // every problem is checked before anything is enqueued: a bad one must not leave half a batch behind
    for (int i = 0; i < count; ++i) {
        const tuna_gemm_problem &p = problems[i];
        if ((rc = check_shape(p.m, p.n, p.k))) return rc;
        if (p.k % block_size || p.k / block_size < 2 || p.m % 16 || p.k % 256)
            return fail(TUNA_ERR_UNSUPPORTED, "problem %d: scale blocks of %d need k=%d a multiple of them (at least two), m=%d of 16, k of 256",
                        i, block_size, p.k, p.m);
        if ((unsigned long long)p.m * (unsigned long long)p.k / 2 >= (1ull << 32) || (unsigned long long)p.k * 32 >= (1ull << 32))
            return fail(TUNA_ERR_UNSUPPORTED, "problem %d: operands exceed the kernel's 32-bit offsets", i);
        if ((p.n + 15) / 16 > 65535) return fail(TUNA_ERR_UNSUPPORTED, "problem %d: n=%d needs more than 65535 token chunks", i, p.n);
        if ((rc = check_ptr(p.q, "q", 16)) || (rc = check_ptr(p.x, "x", 16)) || (rc = check_ptr(p.code, "code", 4)) ||
            (rc = check_ptr(p.absmax, "absmax", 4)) || (rc = check_ptr(p.out, "out", 16)))
            return rc;
    }
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int shift = log2i(block_size) - 6;
    for (int first = 0; first < count;) {
        MultiPlan plan;
        int take = count - first < kMaxMultiProblems ? count - first : kMaxMultiProblems;
        const int min_batch = diag::multi_min_batch();
        while (take >= min_batch && !plan_multi(problems + first, take, cus, &plan, 0, 0, shift)) --take;
        if (take >= min_batch) {
            if ((rc = provide_workspace(false, st, plan.ws_bytes, plan.n_counters, &plan.args.ws, &plan.args.counters))) return rc;
            e = launch_gemm_multi(plan.args, plan.prefetch, dev, st);
            if (e != hipSuccess) return hip_fail(e, "batched blockwise gemm launch");
            diag::count(diag::kMultiLaunches);
            first += take;
            continue;
        }
        const tuna_gemm_problem &p = problems[first];
        if ((rc = tuna_matmul_blockwise(p.q, p.x, p.code, p.absmax, p.out, p.m, p.n, p.k, block_size, stream))) return rc;
        ++first;
    }
    return TUNA_OK;
}

TUNA_EXPORT int tuna_matmul_grouped(const void *q, const void *x, const void *code, const void *absmax, void *out,
                                    int m_group, int n_groups, int k, const int32_t *token_offsets,
                                    const tuna_gemm_config *cfg, int decode_mode, void *stream)
{
    return matmul_grouped_impl(q, x, code, absmax, out, m_group, n_groups, k, token_offsets, cfg, decode_mode,
                               static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_dequant(const void *q, const void *absmax, const void *code, void *out, int m, int k, void *stream)
{
    return dequant_impl(q, absmax, code, out, m, k, k, TUNA_DECODE_DEQUANT, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_quantize(const void *w, const void *code, void *q, void *absmax, int m, int k, void *stream)
{
    return quantize_impl(w, code, q, absmax, m, k, k, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_quantize_blockwise(const void *w, const void *code, void *q, void *absmax, int m, int k, int block_size,
                                        void *stream)
{
    return quantize_impl(w, code, q, absmax, m, k, block_size, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------------------
// GEMM with scale blocks finer than a row (absmax [m, k / block_size]).
//
// A launch is described by a tuna_gemm_config, like a per-row one, and what the config names decides the kernel:
//   lds_tile_rows > 0                     the many-token kernel's scale-block variants: tile lds_tile_rows x 16 * token_tiles,
//                                         k split split_k ways (16 x 16 x 32 MFMA tiles; no 256 x 256 tile)
//   rows_per_wave 16 / 32, or 64 with     the narrow-row kernel's scale-block variants: that many rows per workgroup,
//   waves_m = 0                           waves_k waves along k, ring `prefetch`, one or two token tiles per pass
//   split_k == 0                          the batched streaming kernel as a batch of one (or of the token chunks):
//                                         waves_m x 16 / waves_m waves, ring `prefetch`, balanced split
//   anything else                         the streaming kernel's scale-block twin: unsplit row-tile walkers with the
//                                         config's workgroup shape, ring, x chunk and stagger, 1 / 2 / 4 token tiles
// A config comes from the caller (tuna_matmul_blockwise_ex), from the table of tuned entries keyed by (m, token bucket,
// k, block_size) (config_table.cpp, written by the tuner), or from the rules of derive_blockwise below.
// ---------------------------------------------------------------------------------------
enum BlockwiseFamily { kBlkNarrow = 0, kBlkMulti = 1, kBlkTiled = 2, kBlkMid = 3 };

static BlockwiseFamily blockwise_family(const tuna_gemm_config &c)
{
    if (c.lds_tile_rows > 0) return kBlkTiled;
    if (is_narrow(c)) return kBlkNarrow;
    if (c.split_k == 0) return kBlkMulti;
    return kBlkMid;
}

struct BlockwiseCall {
    const void *q, *x, *code, *absmax;
    void *out;
    int m, n, k, block_size;
};

// Runs `c` on the call (dry: checks only that it could, launches nothing, needs no device).
static int run_blockwise(const BlockwiseCall &b, const tuna_gemm_config &c, hipStream_t st, bool dry)
{
    const int m = b.m, n = b.n, k = b.k, shift = log2i(b.block_size) - 6;
    int rc, dev = 0, cus = kMaxCus;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) {
        if (!dry) return hip_fail(e, "hipGetDevice");
        (void)hipGetLastError();
        dev = 0, cus = kMaxCus;
    }
    switch (blockwise_family(c)) {
    case kBlkNarrow: {
        if (c.token_tiles != 1 && c.token_tiles != 2) return fail(TUNA_ERR_UNSUPPORTED, "narrow-row scale-block kernel: one or two token tiles");
        if (!blockwise_narrow_runs(m, k, c.rows_per_wave, c.waves_k, c.prefetch, c.token_tiles))
            return fail(TUNA_ERR_UNSUPPORTED, "no narrow-row scale-block variant with %d rows, %d waves, ring %d, %d token tiles fits m=%d k=%d",
                        c.rows_per_wave, c.waves_k, c.prefetch, c.token_tiles, m, k);
        if (dry) return TUNA_OK;
        NarrowArgs a;
        memset(&a, 0, sizeof(a));
        a.q = static_cast<const uint8_t *>(b.q);
        a.x = b.x;
        a.code = static_cast<const float *>(b.code);
        a.absmax = static_cast<const float *>(b.absmax);
        a.out = b.out;
        a.m = m, a.n = n, a.k = k;
        e = launch_gemm_blockwise(a, shift, c.rows_per_wave, c.waves_k, c.prefetch, c.token_tiles, st);
        if (e != hipSuccess) return hip_fail(e, "blockwise gemm launch");
        diag::count(diag::kBlockwiseNarrow);
        return TUNA_OK;
    }
    case kBlkMulti: {
        // a batch of one for up to 16 tokens; the token chunks of 16 as the problems of a batch beyond that (every chunk
        // streams the weights again, in one launch per 32 chunks)
        const int chunks = (n + 15) / 16;
        auto plan_batch = [&](int c0, MultiPlan *plan) {
            const int cnt = chunks - c0 < kMaxMultiProblems ? chunks - c0 : kMaxMultiProblems;
            tuna_gemm_problem probs[kMaxMultiProblems];
            for (int ch = 0; ch < cnt; ++ch) {
                const int t0 = (c0 + ch) * 16;
                probs[ch] = {b.q, static_cast<const char *>(b.x) + (size_t)t0 * k * 2, b.code, b.absmax,
                             static_cast<char *>(b.out) + (size_t)t0 * m * 2, m, n - t0 < 16 ? n - t0 : 16, k};
            }
            return plan_multi(probs, cnt, cus, plan, c.waves_m, c.prefetch, shift);
        };
        if (c.waves_m < 1 || c.waves_m * c.waves_k != 16) return fail(TUNA_ERR_UNSUPPORTED, "batched scale-block kernel: waves_m x waves_k must be 16 waves");
        for (int c0 = 0; c0 < chunks; c0 += kMaxMultiProblems) {  // (nothing is enqueued unless every batch of chunks can run)
            MultiPlan plan;
            if (!plan_batch(c0, &plan)) return fail(TUNA_ERR_UNSUPPORTED, "the batched scale-block kernel cannot take m=%d n=%d k=%d with %d x %d waves, ring %d", m, n, k, c.waves_m, c.waves_k, c.prefetch);
        }
        if (dry) return TUNA_OK;
        for (int c0 = 0; c0 < chunks; c0 += kMaxMultiProblems) {
            MultiPlan plan;
            if (!plan_batch(c0, &plan)) return fail(TUNA_ERR_UNSUPPORTED, "blockwise gemm: a batch of token chunks stopped planning");
            if ((rc = provide_workspace(false, st, plan.ws_bytes, plan.n_counters, &plan.args.ws, &plan.args.counters))) return rc;
            e = launch_gemm_multi(plan.args, plan.prefetch, dev, st);
            if (e != hipSuccess) return hip_fail(e, "blockwise gemm launch");
            diag::count(diag::kMultiLaunches);
            diag::count(diag::kBlockwiseMulti);
        }
        return TUNA_OK;
    }
    case kBlkTiled: {
        tuna_gemm_config t = c;
        t.rows_per_wave = 64;  // (16 x 16 x 32 MFMA tiles: the scale-block variants exist for those)
        // (the 256 x 256 tile has no scale-block variant: its threads have no registers left for eight more scales)
        if (!tiled_variant_exists(t.lds_tile_rows, 16 * t.token_tiles, false) || (t.lds_tile_rows == 256 && t.token_tiles == 16))
            return fail(TUNA_ERR_UNSUPPORTED, "no many-token scale-block variant with a %d x %d tile", t.lds_tile_rows, 16 * t.token_tiles);
        TiledPlan tp;
        if ((rc = plan_tiled(m, n, k, t, TUNA_DECODE_GEMM, &tp))) return rc;
        if (dry) return TUNA_OK;
        tp.args.q = static_cast<const uint8_t *>(b.q);
        tp.args.x = b.x;
        tp.args.code = static_cast<const float *>(b.code);
        tp.args.absmax = static_cast<const float *>(b.absmax);
        tp.args.out = b.out;
        tp.args.epilogue = TUNA_EPILOGUE_NONE;
        tp.args.residual = nullptr;
        tp.args.blk_shift = shift;
        if (tp.ws_bytes && (rc = provide_workspace(false, st, tp.ws_bytes, tp.n_counters, &tp.args.ws, &tp.args.counters))) return rc;
        e = launch_gemm_tiled(tp.args, tp.tile_rows, tp.tile_tokens, false, st, true);
        if (e != hipSuccess) return hip_fail(e, "many-token blockwise gemm launch");
        diag::count(diag::kBlockwiseTiled);
        return TUNA_OK;
    }
    case kBlkMid: {
        tuna_gemm_config t = c;
        t.lds_tile_rows = 0;  // (register ring: the twins have no LDS-staged form)
        const int tiles = n > 32 ? 4 : n > 16 ? 2 : 1;  // token tiles: one pass over the weights
        GemmPlan plan;
        if (n > 64 || t.token_tiles != tiles || t.split_k != 1 || t.rows_per_wave != 64 || t.waves_m < 1 || m % (64 * t.waves_m) != 0)
            return fail(TUNA_ERR_UNSUPPORTED, "streaming scale-block twin: up to 64 tokens in one pass (%d token tiles), unsplit, m=%d a multiple of 64 x waves_m", tiles, m);
        if ((rc = plan_gemm(m, n, k, t, TUNA_DECODE_GEMM, &plan))) return rc;
        if (!mid_blockwise_applies(plan, shift)) return fail(TUNA_ERR_UNSUPPORTED, "no streaming scale-block twin for this workgroup shape, ring and x chunk");
        if (dry) return TUNA_OK;
        plan.args.q = static_cast<const uint8_t *>(b.q);
        plan.args.x = b.x;
        plan.args.code = static_cast<const float *>(b.code);
        plan.args.absmax = static_cast<const float *>(b.absmax);
        plan.args.out = b.out;
        plan.args.epilogue = TUNA_EPILOGUE_NONE;
        plan.args.residual = nullptr;
        e = launch_gemm_mid_blockwise(plan, shift, dev, cus, st);
        if (e != hipSuccess) return hip_fail(e, "streaming blockwise gemm launch");
        diag::count(diag::kBlockwiseMid);
        return TUNA_OK;
    }
    }
    return fail(TUNA_ERR_UNSUPPORTED, "unknown blockwise kernel family");
}

// The config for a shape that has no tuned entry, from what the tuner found on the benchmark shapes (a scale per 64
// weights, us).  The streaming kernel's twin where the per-row table has an unsplit streaming entry for the shape and
// it has many rows and at least 48 MB of packed weights (up to 16 tokens: less than 400 MB; from 33 tokens: at least
// 100 MB) - twin / narrow-row / batched at 16 tokens: 62-64 / 77 / 68-69 on 57344 x 8192, 21.5-22.2 / 23.3 / 24.6 on
// 28672 x 4096, 64-65 / 71 / 64 on 32768 x 14336, but 132 / 148 / 114 on 229376 x 4096; at 32 tokens 80 / 131 / 117,
// 30.7 / 31.5 / 40.6, 78 / 134 / 112 and 169 / 205 / 210; at 64 tokens twin / many-token kernel 103 / 130, 49.9 / 47.5,
// 111 / 125 and 182 / 252.  From 33 tokens otherwise the many-token kernel: the per-row entry's tile if it is one, else
// 256 x 64 up to 64 tokens, 128 x 128 up to 128, 128 x 256 beyond, k split until the launch fills the device.  The
// batched kernel for large aligned shapes - narrow / batched at 16 tokens: 8.7 / 15.5 on 6144 x 4096, 14.1 / 16.3 on
// 8192 x 8192, 19.4 / 20.9 on 10240 x 8192, 22.4 / 24.2 on 28672 x 4096, but 18.5 / 16.5 on 4096 x 14336, 44 / 35 on
// 8192 x 28672, 75 / 66 on 57344 x 8192; at one token the narrow kernel wins up to 57344 x 8192 (63 / 65) and loses on
// 229376 x 4096 (117 / 102); at 32 tokens 11.9 / 16.9 on 6144 x 4096, 20.3 / 24.6 on 8192 x 8192, 30.9 / 38.7 on
// 28672 x 4096, but 37.2 / 30.4 on 10240 x 8192, 29.6 / 22.7 on 4096 x 14336, 134 / 106 on 32768 x 14336.  Everything
// else: the narrow-row kernel, the widest tile that gives nine workgroups per sixteen compute units.
static int derive_blockwise(const BlockwiseCall &b, tuna_gemm_config *out)
{
    const int m = b.m, n = b.n, k = b.k, shift = log2i(b.block_size) - 6;
    const long long packed_bytes = (long long)m * k / 2;
    int dev = 0, cus = kMaxCus;
    if (device_cus(&dev, &cus) != hipSuccess) {
        (void)hipGetLastError();
        cus = kMaxCus;
    }
    tuna_gemm_config row;  // the per-row GEMM's config for the shape
    select_config(m, n, k, &row, nullptr);
    const bool mid_wins = n > 32 ? m >= 16384 && packed_bytes >= (100ll << 20)
                                 : m >= 16384 && packed_bytes >= (48ll << 20) && (n > 16 || packed_bytes < (400ll << 20));
    if (n <= 64 && mid_wins) {
        const int tiles = n > 32 ? 4 : n > 16 ? 2 : 1;
        tuna_gemm_config c = row;
        c.lds_tile_rows = 0;
        if (row.lds_tile_rows <= 0 && row.rows_per_wave == 64 && row.token_tiles == tiles && row.split_k == 1 && row.waves_m >= 1 &&
            row.waves_m * row.waves_k >= 8 && (row.prefetch == 2 || row.prefetch == 4) && run_blockwise(b, c, nullptr, true) == TUNA_OK) {
            *out = c;
            return TUNA_OK;
        }
    }
    const bool stream_wins = n > 16  ? packed_bytes >= (100ll << 20) || (k > 8192 && packed_bytes >= (12ll << 20)) ||
                                           (k > 4096 && packed_bytes >= (40ll << 20))
                             : n > 4 ? packed_bytes >= (100ll << 20) || (n > 8 && k >= 12288 && packed_bytes >= (20ll << 20))
                                     : packed_bytes >= (256ll << 20);
    if ((n > 32 || (n > 16 && !stream_wins)) && n <= 512) {
        // (17..32 tokens too, where the batched kernel's rule below does not claim the shape: passes of one token tile
        // on more workgroups against one pass of two - 1024 x 8192 at 20 tokens 11.4 us against 13.0, 2560 x 5120 9.5
        // against 10.6, 4096 x 4096 8.4 against 9.1)
        // 33..512 tokens on small shapes: one round of narrow-row workgroups with the token passes side by side, as in
        // derive_config, where some tile height and tokens per pass give 128..256 of them (32-row tiles from 64 for shapes
        // of up to 8 MB) and the workgroup's scales stay in LDS - 32-row tiles first, one token tile per pass first (blocks of
        // 64, narrow round against the model's many-token tile below: 1024 x 4096 at 72..100 tokens 7.9 us against
        // 14.2, 1536 x 6144 at 72 tokens 10.2 against 16.4, 2048 x 2048 at 100 tokens 7.3 against 12.2 and at 256
        // tokens 10.6 against 13.4, 3072 x 3072 at 130 tokens 12.4 against 19.6, 3072 x 8192 at 72 tokens 17.8
        // against 23.9; with the scales read from memory - 64-row tiles of two token tiles at k = 8192 - 42 us
        // against 19..33; at 33..64 tokens against the 256 x 64 tile with k split to fill the device, the rule below:
        // 2048 x 2048 6.1..6.3 us against 18.0..18.8, 1024 x 8192 11.6..12.4 against 28.2..28.9, 2560 x 5120
        // 9.6..13.9 against 25.6..26.4, 5120 x 5120 13.6..20.1 against 26.6..27.3, 8192 x 1024 8.5..9.2 against 17).
        static const int kTry[4][2] = {{32, 1}, {32, 2}, {64, 1}, {64, 2}};
        static const int kRing[4][2] = {{8, 4}, {8, 2}, {4, 4}, {4, 2}};
        // (32-row tiles whatever k, unlike the per-row kernel's round: 2560 x 10240 at 36..48 tokens as 80 x 3 workgroups
        // of 32 rows 15.5..17.2 us, the model's many-token tile 22.8; 1024 x 14336 at 100 tokens as 32 x 7 18.7, as
        // 16 x 7 of 64 rows 26.4)
        for (const auto &t : kTry) {
            const int r = t[0], tt = t[1];
            if (m % r != 0 || (r < 64 && tt > 1 && k > 8192)) continue;  // (two token tiles on 32 rows with long k: 1024 x 14336 at 200 tokens 31.2 us, a split 64 x 128 tile 24.4)
            const long long wgs = (long long)(m / r) * ceil_div(n, 16 * tt);
            // (1024 x 14336 at 64 tokens as 64 workgroups of 64 rows: 28.2 us, a split 64 x 128 tile 23.3; 1024 x 8192 at
            // 24 tokens as 64 workgroups of 32 rows: 11.4 us, one pass of two token tiles 14.1)
            if (wgs > kMaxCus || wgs < (packed_bytes <= (8ll << 20) && r < 64 ? 64 : 128)) continue;
            for (const auto &g : kRing) {
                if (!blockwise_narrow_scales_in_lds(k, shift, r, g[0], g[1], tt)) continue;
                tuna_gemm_config c;
                memset(&c, 0, sizeof(c));
                c.rows_per_wave = r, c.waves_m = r == 64 ? 0 : 1, c.waves_k = g[0], c.prefetch = g[1];
                c.split_k = 1, c.token_tiles = tt, c.x_chunk = 512;
                if (run_blockwise(b, c, nullptr, true) == TUNA_OK) {
                    *out = c;
                    return TUNA_OK;
                }
            }
        }
    }
    if (n > 32) {
        // 33 tokens and more: the many-token tile and k split whose grid costs least by the model of derive_config,
        // with the factors of the scale-block variants (128 x 256 tile 1.0, 256 x 128, 128 x 128 and 64 x 256 1.2,
        // 256 x 64 and 64 x 128 1.6; split in 2 ... 8 while the grid stays near one round), read off sixteen
        // shapes x ten counts from 72 to 2048 tokens with blocks of 64, each timed with every tile and split: the
        // model's pick is within 7 % of the best on all 160 cases (the rule below, which this one precedes: 1.23 x
        // on average, up to 2.8 x where it split k by 8 or 10 - 4096 x 4096 at 200 tokens 74 us against 26).
        struct Tile { int rows, tokens; double factor; };
        static const Tile kTiles[6] = {{128, 256, 1.0}, {256, 128, 1.2}, {128, 128, 1.2}, {64, 256, 1.2}, {256, 64, 1.6}, {64, 128, 1.6}};
        static const int kSplits[6] = {1, 2, 3, 4, 6, 8};
        tuna_gemm_config best;
        double best_cost = 0.0;
        bool found = false;
        for (const Tile &t : kTiles)
            for (int split : kSplits) {
                const long long tiles = (long long)ceil_div(m, t.rows) * ceil_div(n, t.tokens) * split;
                if (split > 1 && (tiles > 300 || ceil_div(k, 64) / split < 8)) continue;
                if (tiles < 32) continue;
                const long long full = tiles / kMaxCus, rest = tiles % kMaxCus;
                const double rounds = 1.15 * (double)full + (rest ? 0.7 + 0.45 * (double)rest / kMaxCus : 0.0);
                const double area = (double)t.rows * t.tokens;
                const double cost = rounds * (area * t.factor / split + 0.6e7 / k) + (split > 1 ? (100.0 * split + 300.0) * area / k : 0.0);
                if (found && cost >= best_cost) continue;
                tuna_gemm_config c;
                memset(&c, 0, sizeof(c));
                c.rows_per_wave = 64, c.waves_m = 1, c.waves_k = 1, c.prefetch = 2, c.x_chunk = 64;
                c.token_tiles = t.tokens / 16, c.lds_tile_rows = t.rows, c.split_k = split;
                if (run_blockwise(b, c, nullptr, true) != TUNA_OK) continue;
                best = c, best_cost = cost, found = true;
            }
        if (found) {
            *out = best;
            return TUNA_OK;
        }
    }
    if (n > 32) {
        tuna_gemm_config c = row;
        if (c.lds_tile_rows <= 0 || !tiled_variant_exists(c.lds_tile_rows, 16 * c.token_tiles, false) ||
            (c.lds_tile_rows == 256 && c.token_tiles == 16)) {
            c.lds_tile_rows = n > 64 ? 128 : 256;
            c.token_tiles = n > 128 ? 16 : n > 64 ? 8 : 4;
            c.waves_m = c.waves_k = 1, c.prefetch = 2, c.x_chunk = 64, c.xcd_swizzle = 0, c.k_stagger = 0;
            // fewer tiles than compute units: split k until the launch fills them (at least eight k-steps per workgroup)
            const long long tiles = (long long)ceil_div(m, c.lds_tile_rows) * ceil_div(n, 16 * c.token_tiles);
            const int steps = ceil_div(k, 64);
            long long split = tiles > 0 ? cus / tiles : 1;
            if (split > steps / 8) split = steps / 8;
            c.split_k = split < 1 ? 1 : (int)split;
        }
        c.rows_per_wave = 64;
        if (run_blockwise(b, c, nullptr, true) == TUNA_OK) {
            *out = c;
            return TUNA_OK;
        }
    }
    if (stream_wins) {
        // the batched kernel's own choice of tile height (256 rows, 128 where those are fewer than workgroups), ring of
        // two; then whatever height the row count allows
        tuna_gemm_problem one = {b.q ? b.q : b.out, b.x, b.code, nullptr, b.out, m, n < 16 ? n : 16, k};
        MultiPlan plan;
        tuna_gemm_config c;
        memset(&c, 0, sizeof(c));
        c.rows_per_wave = 64, c.split_k = 0, c.x_chunk = 512, c.token_tiles = 1;
        if (plan_multi(&one, 1, cus, &plan, 0, 0, shift)) {
            c.waves_m = plan.args.waves_m, c.waves_k = 16 / c.waves_m, c.prefetch = plan.prefetch - 10;
            if (run_blockwise(b, c, nullptr, true) == TUNA_OK) {
                *out = c;
                return TUNA_OK;
            }
        }
        for (int wm = 4; wm >= 1; wm >>= 1) {
            c.waves_m = wm, c.waves_k = 16 / wm, c.prefetch = 2;
            if (run_blockwise(b, c, nullptr, true) == TUNA_OK) {
                *out = c;
                return TUNA_OK;
            }
        }
    }
    tuna_gemm_config c;
    memset(&c, 0, sizeof(c));
    int rows = 0, wk = 0, u = 0, tt = 0;
    if (!derive_blockwise_narrow(m, k, shift, cus, n > 16 ? 2 : 1, &rows, &wk, &u, &tt))
        return fail(TUNA_ERR_UNSUPPORTED, "no scale-block kernel takes m=%d n=%d k=%d block_size=%d", m, n, k, b.block_size);
    c.rows_per_wave = rows, c.waves_m = rows == 64 ? 0 : 1, c.waves_k = wk, c.split_k = 1, c.prefetch = u, c.x_chunk = 512, c.token_tiles = tt;
    *out = c;
    return TUNA_OK;
}

// Tuned entry for (m, n, k, block_size) if the table has one that can run the call, else the derived config.
static int select_blockwise(const BlockwiseCall &b, tuna_gemm_config *cfg, int *from_table)
{
    if (from_table) *from_table = 0;
    for (int i = 0; i < kBlockwiseTableSize; ++i) {
        const BlockwiseTableEntry &e = kBlockwiseTable[i];
        // (from 33 tokens an entry holds at the count it was tuned at, its bucket's lower edge: further into the bucket
        // the derivation knows the token tiles that n has gained - 8192 x 8192 at 100 tokens with blocks of 64 runs
        // 68 us with the entry of the bucket 64..127 and 41 with the model's pick, 8192 x 28672 at 56 tokens 115 us
        // with the entry of the bucket 32..63 and 69 derived)
        if (e.m == b.m && e.k == b.k && e.block_size == b.block_size && b.n >= e.n_lo && b.n <= e.n_hi &&
            (b.n <= 32 || b.n == e.n_lo) && run_blockwise(b, e.cfg, nullptr, true) == TUNA_OK) {
            *cfg = e.cfg;
            if (from_table) *from_table = 1;
            return TUNA_OK;
        }
    }
    return derive_blockwise(b, cfg);
}

static int check_blockwise_call(const BlockwiseCall &b, bool pointers)
{
    int rc;
    if ((rc = check_shape(b.m, b.n, b.k))) return rc;
    if (b.block_size < 64 || !is_pow2(b.block_size) || b.k % b.block_size || b.block_size >= b.k)
        return fail(TUNA_ERR_UNSUPPORTED, "block_size=%d: the GEMM takes 64, 128, 256, ... (a power of two that divides k=%d) or k",
                    b.block_size, b.k);
    if (b.m % 16 || b.k % 256)
        return fail(TUNA_ERR_UNSUPPORTED, "scale blocks need m a multiple of 16 and k of 256 (m=%d, k=%d)", b.m, b.k);
    if ((unsigned long long)b.m * (unsigned long long)b.k / 2 >= (1ull << 32) || (unsigned long long)b.k * 32 >= (1ull << 32))
        return fail(TUNA_ERR_UNSUPPORTED, "operands exceed the kernel's 32-bit offsets");
    if ((b.n + 15) / 16 > 65535) return fail(TUNA_ERR_UNSUPPORTED, "n=%d needs more than 65535 token chunks", b.n);
    if (pointers && ((rc = check_ptr(b.q, "q", 16)) || (rc = check_ptr(b.x, "x", 16)) || (rc = check_ptr(b.code, "code", 4)) ||
                     (rc = check_ptr(b.absmax, "absmax", 4)) || (rc = check_ptr(b.out, "out", 16))))
        return rc;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_matmul_blockwise_ex(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                                         int k, int block_size, const tuna_gemm_config *cfg, void *stream)
{
    if (block_size == k) return matmul_impl(q, x, code, absmax, out, m, n, k, cfg, TUNA_DECODE_GEMM, static_cast<hipStream_t>(stream));
    const BlockwiseCall b = {q, x, code, absmax, out, m, n, k, block_size};
    int rc;
    if ((rc = check_blockwise_call(b, true))) return rc;
    tuna_gemm_config c;
    if (cfg) c = *cfg;
    else if ((rc = select_blockwise(b, &c, nullptr))) return rc;
    return run_blockwise(b, c, static_cast<hipStream_t>(stream), false);
}

TUNA_EXPORT int tuna_matmul_blockwise(const void *q, const void *x, const void *code, const void *absmax, void *out, int m, int n,
                                      int k, int block_size, void *stream)
{
    return tuna_matmul_blockwise_ex(q, x, code, absmax, out, m, n, k, block_size, nullptr, stream);
}

TUNA_EXPORT int tuna_select_config_blockwise(int m, int n, int k, int block_size, tuna_gemm_config *cfg, int *from_table)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    const BlockwiseCall b = {nullptr, nullptr, nullptr, nullptr, nullptr, m, n, k, block_size};
    int rc;
    if ((rc = check_blockwise_call(b, false))) return rc;
    return select_blockwise(b, cfg, from_table);
}

TUNA_EXPORT int tuna_validate_config_blockwise(int m, int n, int k, int block_size, const tuna_gemm_config *cfg)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    const BlockwiseCall b = {nullptr, nullptr, nullptr, nullptr, nullptr, m, n, k, block_size};
    int rc;
    if ((rc = check_blockwise_call(b, false))) return rc;
    return run_blockwise(b, *cfg, nullptr, true);
}

TUNA_EXPORT int tuna_blockwise_table_size(void) { return kBlockwiseTableSize; }

TUNA_EXPORT int tuna_blockwise_table_entry(int i, int *m, int *n_lo, int *n_hi, int *k, int *block_size, tuna_gemm_config *cfg)
{
    if (i < 0 || i >= kBlockwiseTableSize) return fail(TUNA_ERR_INVALID_ARG, "table index %d out of range", i);
    const BlockwiseTableEntry &e = kBlockwiseTable[i];
    if (m) *m = e.m;
    if (n_lo) *n_lo = e.n_lo;
    if (n_hi) *n_hi = e.n_hi;
    if (k) *k = e.k;
    if (block_size) *block_size = e.block_size;
    if (cfg) *cfg = e.cfg;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_dequant_blockwise(const void *q, const void *absmax, const void *code, void *out, int m, int k,
                                       int block_size, int decode_mode, void *stream)
{
    return dequant_impl(q, absmax, code, out, m, k, block_size, decode_mode, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_dequant_ex(const void *q, const void *absmax, const void *code, void *out, int m, int k,
                                int decode_mode, void *stream)
{
    return dequant_impl(q, absmax, code, out, m, k, k, decode_mode, static_cast<hipStream_t>(stream));
}

TUNA_EXPORT int tuna_select_config(int m, int n, int k, tuna_gemm_config *cfg, int *from_table)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    return select_config(m, n, k, cfg, from_table);
}

TUNA_EXPORT int tuna_derive_config(int m, int n, int k, tuna_gemm_config *cfg)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    *cfg = derive_config(m, n, k);
    return TUNA_OK;
}

TUNA_EXPORT int tuna_select_config_ex(int m, int n, int k, int decode_mode, tuna_gemm_config *cfg, int *from_table)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    if (decode_mode != TUNA_DECODE_GEMM && decode_mode != TUNA_DECODE_DEQUANT)
        return fail(TUNA_ERR_INVALID_ARG, "decode_mode %d is neither TUNA_DECODE_GEMM nor TUNA_DECODE_DEQUANT", decode_mode);
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    return select_config_for(m, n, k, decode_mode, cfg, from_table);
}

TUNA_EXPORT int tuna_select_config_grouped(int m_group, int n_active, int max_tokens, int k, int decode_mode,
                                           tuna_gemm_config *cfg)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    if (m_group <= 0 || n_active < 1 || n_active > kMaxGroups || max_tokens < 1 || m_group % kRowsPerLoad ||
        (long long)m_group * n_active > 0x7fffffffLL)
        return fail(TUNA_ERR_INVALID_ARG, "m_group=%d (a positive multiple of %d), n_active=%d (1..%d), max_tokens=%d (>= 1)",
                    m_group, kRowsPerLoad, n_active, kMaxGroups, max_tokens);
    int rc = check_shape(m_group * n_active, max_tokens, k);
    if (rc) return rc;
    GemmPlan plan;
    return grouped_config(m_group, m_group * n_active, max_tokens, k, decode_mode, cfg, &plan);
}

TUNA_EXPORT int tuna_validate_config(int m, int n, int k, const tuna_gemm_config *cfg)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    return validate_for(m, n, k, *cfg, TUNA_DECODE_GEMM);
}

TUNA_EXPORT int tuna_validate_config_ex(int m, int n, int k, const tuna_gemm_config *cfg, int decode_mode)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    return validate_for(m, n, k, *cfg, decode_mode);
}

TUNA_EXPORT int tuna_config_footprint(int m, int n, int k, const tuna_gemm_config *cfg, size_t *lds_bytes,
                                      size_t *workspace_bytes)
{
    if (!cfg) return fail(TUNA_ERR_INVALID_ARG, "cfg is null");
    if (cfg->lds_tile_rows > 0) {
        TiledPlan tp;
        int rc = plan_tiled(m, n, k, *cfg, TUNA_DECODE_GEMM, &tp);
        if (rc) return rc;
        if (lds_bytes) *lds_bytes = tp.lds_bytes;
        if (workspace_bytes) *workspace_bytes = tp.ws_bytes;
        return TUNA_OK;
    }
    if (is_narrow(*cfg)) {
        NarrowPlan np;
        int rc = plan_narrow(m, n, k, *cfg, TUNA_DECODE_GEMM, &np);
        if (rc) return rc;
        if (lds_bytes) *lds_bytes = np.lds_bytes;
        if (workspace_bytes) *workspace_bytes = 0;
        return TUNA_OK;
    }
    GemmPlan plan;
    int rc = plan_gemm(m, n, k, *cfg, TUNA_DECODE_GEMM, &plan);
    if (rc) return rc;
    if (lds_bytes) *lds_bytes = plan.lds_bytes;
    if (workspace_bytes) *workspace_bytes = plan.ws_bytes;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_config_segments(int m, int n, int k, const tuna_gemm_config *cfg, int n_workgroups, int workgroup,
                                     int *segments, int max_segments, int *n_segments)
{
    if (!cfg || !n_segments) return fail(TUNA_ERR_INVALID_ARG, "cfg or n_segments is null");
    if (is_narrow(*cfg)) {  // one workgroup per row tile, the whole k range
        NarrowPlan np;
        int rc = plan_narrow(m, n, k, *cfg, TUNA_DECODE_GEMM, &np);
        if (rc) return rc;
        const int tiles = m / np.rows;
        if (workgroup < 0 || workgroup >= tiles) return fail(TUNA_ERR_INVALID_ARG, "workgroup %d outside 0..%d", workgroup, tiles - 1);
        if (segments && max_segments > 0) {
            segments[0] = workgroup;
            segments[1] = 0;
            segments[2] = k / kStepK;
            segments[3] = -1;
        }
        *n_segments = 1;
        return TUNA_OK;
    }
    GemmPlan plan;
    int rc = plan_gemm(m, n, k, *cfg, TUNA_DECODE_GEMM, &plan);
    if (rc) return rc;
    const GemmArgs &a = plan.args;
    int nw = n_workgroups > 0 ? n_workgroups : (int)plan.grid.x;
    const int cap = kMaxCus * plan.wgs_per_cu;
    if (nw > cap) nw = cap;
    if (nw > (int)plan.grid.x) nw = (int)plan.grid.x;
    if (workgroup < 0 || workgroup >= nw) return fail(TUNA_ERR_INVALID_ARG, "workgroup %d outside 0..%d", workgroup, nw - 1);
    int count = 0;
    auto emit = [&](int row_tile, int sb, int nsteps, int part) {
        if (segments && count < max_segments) {
            segments[4 * count + 0] = row_tile;
            segments[4 * count + 1] = sb;
            segments[4 * count + 2] = nsteps;
            segments[4 * count + 3] = part;
        }
        ++count;
    };
    if (a.balanced) {
        const int t_begin = balanced_begin((unsigned)workgroup, (unsigned)nw, (unsigned)a.units_total);
        const int t_end = balanced_begin((unsigned)workgroup + 1u, (unsigned)nw, (unsigned)a.units_total);
        for (int t = t_begin; t < t_end;) {
            const Segment sg = balanced_segment(t, t_begin, t_end, a.units_per_tile, a.unit_log2, a.steps_total);
            emit(sg.row_tile, sg.sb, sg.nsteps, sg.part);
            t = sg.next;
        }
    } else {
        for (int t = workgroup; t < a.tiles_total; t += nw) {
            const int row_tile = t / a.split_k, ks = t - row_tile * a.split_k;
            const int sb = ks * a.steps_per_split;
            int nsteps = (a.steps_total < sb + a.steps_per_split ? a.steps_total : sb + a.steps_per_split) - sb;
            if (nsteps < 0) nsteps = 0;
            emit(row_tile, sb, nsteps, a.split_k == 1 ? -1 : ks);
        }
    }
    *n_segments = count;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_config_contributors(int m, int n, int k, const tuna_gemm_config *cfg, int n_workgroups, int row_tile,
                                         int *first_workgroup, int *count, int *first_slot)
{
    if (!cfg || !first_workgroup || !count || !first_slot) return fail(TUNA_ERR_INVALID_ARG, "null argument");
    if (is_narrow(*cfg)) {
        NarrowPlan np;
        int rc = plan_narrow(m, n, k, *cfg, TUNA_DECODE_GEMM, &np);
        if (rc) return rc;
        if (row_tile < 0 || row_tile >= m / np.rows) return fail(TUNA_ERR_INVALID_ARG, "row_tile %d out of range", row_tile);
        *first_workgroup = -1;
        *count = 1;
        *first_slot = 0;
        return TUNA_OK;
    }
    GemmPlan plan;
    int rc = plan_gemm(m, n, k, *cfg, TUNA_DECODE_GEMM, &plan);
    if (rc) return rc;
    const GemmArgs &a = plan.args;
    if (row_tile < 0 || row_tile >= a.row_tiles) return fail(TUNA_ERR_INVALID_ARG, "row_tile %d outside 0..%d", row_tile, a.row_tiles - 1);
    if (!a.balanced) {
        *first_workgroup = -1;
        *count = a.split_k;
        *first_slot = 0;
        return TUNA_OK;
    }
    int nw = n_workgroups > 0 ? n_workgroups : (int)plan.grid.x;
    const int cap = kMaxCus * plan.wgs_per_cu;
    if (nw > cap) nw = cap;
    if (nw > (int)plan.grid.x) nw = (int)plan.grid.x;
    unsigned lo, cnt, slot;
    balanced_contributors((unsigned)row_tile, (unsigned)a.units_per_tile, (unsigned)a.units_total, (unsigned)nw, &lo, &cnt, &slot);
    *first_workgroup = (int)lo;
    *count = (int)cnt;
    *first_slot = (int)slot;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_config_table_size(void) { return kConfigTableSize; }

TUNA_EXPORT int tuna_config_table_entry(int i, int *m, int *n_lo, int *n_hi, int *k, tuna_gemm_config *cfg)
{
    if (i < 0 || i >= kConfigTableSize) return fail(TUNA_ERR_INVALID_ARG, "table index %d out of range", i);
    const TableEntry &e = kConfigTable[i];
    if (m) *m = e.m;
    if (n_lo) *n_lo = e.n_lo;
    if (n_hi) *n_hi = e.n_hi;
    if (k) *k = e.k;
    if (cfg) *cfg = e.cfg;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_config_table_next_from(int i)
{
    if (i < 0 || i >= kConfigTableSize) {
        fail(TUNA_ERR_INVALID_ARG, "table index %d out of range", i);
        return -1;
    }
    return kConfigTable[i].next_from;
}

TUNA_EXPORT int tuna_config_table_derived_range(int i, int *from, int *to)
{
    if (i < 0 || i >= kConfigTableSize) return fail(TUNA_ERR_INVALID_ARG, "table index %d out of range", i);
    if (from) *from = kConfigTable[i].derived_from;
    if (to) *to = kConfigTable[i].derived_to;
    return TUNA_OK;
}

TUNA_EXPORT int tuna_describe_launch(int m, int n, int k, const tuna_gemm_config *cfg, int decode_mode, char *buf, size_t len)
{
    if (!buf || len < 16) return fail(TUNA_ERR_INVALID_ARG, "buf is null or shorter than 16 bytes");
    int rc = check_shape(m, n, k);
    if (rc) return rc;
    tuna_gemm_config c;
    if (cfg) c = *cfg;
    else select_config_for(m, n, k, decode_mode, &c, nullptr);
    if (c.lds_tile_rows > 0) {
        TiledPlan tp;
        if ((rc = plan_tiled(m, n, k, c, decode_mode, &tp))) return rc;
        const bool wide = tp.tile_rows == 256 && tp.tile_tokens == 256;  // gemm_wide.hip: one wave per SIMD
        snprintf(buf, len, "%s<%d rows x %d tokens%s> split_k=%d", wide ? "gemm_wide_kernel" : "gemm_tiled_kernel", tp.tile_rows,
                 tp.tile_tokens, tp.mfma32 ? ",mfma 32x32x16" : "", c.split_k);
        return TUNA_OK;
    }
    if (is_narrow(c)) {
        NarrowPlan np;
        if ((rc = plan_narrow(m, n, k, c, decode_mode, &np))) return rc;
        describe_narrow_launch(np.rows, np.waves_k, np.prefetch, np.token_tiles, n, buf, len);
        return TUNA_OK;
    }
    GemmPlan plan;
    if ((rc = plan_gemm(m, n, k, c, decode_mode, &plan))) return rc;
    if (stream_applies(c, n, decode_mode, TUNA_EPILOGUE_NONE)) {
        const tuna_gemm_problem one = {buf, buf, buf, nullptr, buf, m, n, k};  // (only sizes and alignment are looked at)
        MultiPlan mp;
        if (plan_multi(&one, 1, kMaxCus, &mp, c.waves_m, c.prefetch)) {
            snprintf(buf, len, "gemm_multi_kernel<U=%d> waves_m=%d waves_k=%d", mp.prefetch, c.waves_m, c.waves_k);
            return TUNA_OK;
        }
    }
    int cus = kMaxCus, dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        cus = v;
    else
        (void)hipGetLastError();
    describe_gemm_launch(plan, cus, buf, len);
    return TUNA_OK;
}

TUNA_EXPORT int tuna_release_workspaces(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    e = hipDeviceSynchronize();
    if (e != hipSuccess) return hip_fail(e, "hipDeviceSynchronize");
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (auto it = g_workspaces.begin(); it != g_workspaces.end();) {
        if (it->first.first == dev) {
            free_workspace(it->second);
            it = g_workspaces.erase(it);
        } else {
            ++it;
        }
    }
    return TUNA_OK;
}

}  // extern "C"
