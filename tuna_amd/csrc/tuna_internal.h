// Internal declarations shared by the host API and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "../../include/tuna_amd.h"
#include "diag.h"

#define TUNA_EXPORT __attribute__((visibility("default")))

namespace tuna {

// LDS byte-pair lookup table: 256 rows (one per packed byte value) x 64 copies
// (one per lane) of a half2 {code[byte >> 4], code[byte & 15]}.  Row stride is 256
// bytes so a lane's address is (byte << 8) | (lane << 2): every lane of a wave reads
// its own bank column, whatever the data.
constexpr int kLutBytes = 256 * 64 * 4;
constexpr int kLdsLimit = 160 * 1024;

// Dynamic LDS above 64 KB needs a one-time opt-in per kernel and device.  `done` is read without a
// lock on every launch; the attribute call is idempotent, so threads racing on a kernel's first
// launch may both make it.
typedef std::atomic<unsigned char> OptInFlag;
inline hipError_t ensure_lds_opt_in(OptInFlag &done, const void *kernel)
{
    if (done.load(std::memory_order_acquire)) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
    if (e == hipSuccess) done.store(1, std::memory_order_release);
    return e;
}
constexpr int kStepK = 32;          // k per MFMA step (v_mfma_f32_16x16x32_f16)
constexpr int kRowsPerLoad = 64;    // weight rows covered by one 128-bit load per lane
constexpr int kMaxThreads = 1024;
constexpr int kMaxGroups = 64;      // experts per grouped launch (their token offsets travel as kernel arguments)
constexpr int kMaxCus = 256;        // compute units of the largest gfx950 part: bounds the persistent grid

// Everything a GEMM launch needs, filled by the host from a tuna_gemm_config.
struct GemmArgs {
    const uint8_t *q;
    const void *x;
    const float *code;
    const float *absmax;
    void *out;
    const void *residual;  // fp16, layout of out: added before the final rounding (TUNA_EPILOGUE_RESIDUAL)
    int epilogue;          // TUNA_EPILOGUE_*
    float *ws;           // split-K partial sums (library owned), may be null if split_k == 1
    unsigned *counters;  // one arrival counter per (token chunk, row tile), zero between launches
    int m, n, k;
    int waves_m, waves_k, split_k;  // waves_k is a power of two, waves_m any count
    int split_log2;                 // log2(split_k) if it is a power of two, else -1
    int wk_log2;
    int steps_total;      // ceil(k / 32)
    int steps_per_split;  // k-steps owned by one workgroup
    int chunk_steps;      // k-steps of x staged in LDS at a time (power of two)
    int chunk_log2;
    int row_tiles;        // workgroups along m
    int xcd_swizzle;
    int k_stagger;        // k-steps by which consecutive row tiles start later in their k range (0: none)
    int lds_bytes;        // dynamic LDS size of the launch (last 16 bytes: arrival ticket)
    int red_bytes;        // bytes of the reduction buffers in the LDS work area
    int planes_log2;      // log2(accumulator planes reduced per epilogue pass)
    int tiles_total;      // row_tiles * split_k: tiles walked by the persistent workgroups
    int balanced;         // 1: balanced split (config split_k == 0), the fields below apply
    int unit_log2;        // log2(k-steps per unit), a unit being what the split is made of
    int units_per_tile;   // ceil(steps_total / unit)
    int units_total;      // row_tiles * units_per_tile; (units_total + 1) * gridDim.x < 2^31
    // grouped (mixture-of-experts) launches: the weight rows are n_groups stacked matrices of
    // group_rows rows each; group e multiplies only the activation rows tok_off[e] ..
    // tok_off[e+1]-1 and writes out[token, row - e*group_rows] (leading dimension group_rows).
    // group_rows == 0: one dense GEMM.  Row tiles never straddle groups.
    // Row tiles count over the groups that have tokens: row tile r belongs to group
    // act[r / tiles_per_group].
    int group_rows;
    int n_groups;
    int tiles_per_group;
    int tok_off[kMaxGroups + 1];
    unsigned char act[kMaxGroups];
};

// ---------------------------------------------------------------------------------------
// Balanced split: arithmetic shared by the kernel and the host (tuna_config_segments).
// The k range of every row tile is cut into units of 2^unit_log2 k-steps; the T units of all
// row tiles form one sequence; workgroup w of nw owns units [floor(w*T/nw), floor((w+1)*T/nw))
// and walks them as segments that end at row tile boundaries.  (T + 1) * nw < 2^31.
// ---------------------------------------------------------------------------------------
struct Segment {
    int row_tile;  // row tile of the segment
    int sb;        // first k-step
    int nsteps;    // k-steps (the last unit of a row tile may be short)
    int part;      // -1: the whole row tile (sums are final); 0 / 1: the workgroup's partial-sum slot
    int next;      // cursor of the workgroup's next segment
};

__host__ __device__ inline int balanced_begin(unsigned w, unsigned nw, unsigned T) { return (int)((w * T) / nw); }

// Segment that starts at unit u of the workgroup owning units [t_begin, t_end).
__host__ __device__ inline Segment balanced_segment(int u, int t_begin, int t_end, int units_per_tile, int unit_log2,
                                                    int steps_total)
{
    Segment s;
    s.row_tile = (int)((unsigned)u / (unsigned)units_per_tile);
    const int u_in = u - s.row_tile * units_per_tile;
    const int left_tile = units_per_tile - u_in, left_wg = t_end - u;
    const int seg = left_wg < left_tile ? left_wg : left_tile;
    s.sb = u_in << unit_log2;
    const int want = seg << unit_log2, have = steps_total - s.sb;
    s.nsteps = want < have ? want : have;
    s.part = seg == units_per_tile ? -1 : (u == t_begin ? 0 : 1);
    s.next = u + seg;
    return s;
}

// Contributors of a row tile: workgroups w_lo .. w_lo + n - 1, in k order; first_slot is the
// slot contributor 0 used (every later contributor starts the row tile's share at its own
// first unit, so it used slot 0).
__host__ __device__ inline void balanced_contributors(unsigned row_tile, unsigned units_per_tile, unsigned T, unsigned nw,
                                                      unsigned *w_lo, unsigned *n, unsigned *first_slot)
{
    const unsigned u0 = row_tile * units_per_tile, u1 = u0 + units_per_tile - 1u;
    // the workgroup that owns unit u is the largest w with floor(w*T/nw) <= u
    const unsigned lo = ((u0 + 1u) * nw - 1u) / T;
    const unsigned hi = ((u1 + 1u) * nw - 1u) / T;
    *w_lo = lo;
    *n = hi - lo + 1u;
    *first_slot = (lo * T) / nw < u0 ? 1u : 0u;
}

// Launch arguments of the many-token kernel (gemm_tiled.hip): weights decoded once per
// workgroup tile into LDS.  k-steps are 64 long here.
struct TiledArgs {
    const uint8_t *q;
    const void *x;
    const float *code;
    const float *absmax;
    void *out;
    const void *residual;  // as in GemmArgs
    int epilogue;
    float *ws;           // split-K partial tiles (library owned), unused if split_k == 1
    unsigned *counters;  // one arrival counter per tile, zero between launches
    int m, n, k;
    int steps_total;      // ceil(k / 64)
    int split_k;          // gridDim.z
    int steps_per_split;
    int row_tiles, tok_tiles;  // gridDim.x = row_tiles * tok_tiles: token tiles of a row tile are launched together
    int blk_shift;        // scale-block variants: absmax is [m, k / (64 << blk_shift)], one scale per block of a row
};

inline int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

struct GemmPlan {
    GemmArgs args;
    dim3 grid;
    int threads;
    int rw, prefetch, token_tiles, decode;
    int min_waves;  // waves per SIMD the variant is compiled for (2: <=256 VGPRs, 4: <=128)
    int wgs_per_cu; // workgroups of this launch that fit on one CU (LDS and registers)
    int lds_weights; // the config asks for the packed weights staged through LDS (lds_tile_rows == -1)
    size_t lds_bytes;
    size_t ws_bytes;
    size_t n_counters;
};

// gemm_kernel.hip
hipError_t launch_gemm(const GemmPlan &plan, hipStream_t stream);
// 17..128-token streaming twin of the general kernel (gemm_mid.hpp) for the launches it applies to.
bool mid_applies(const GemmPlan &plan);
bool mid_lds_applies(const GemmPlan &plan);
// The streaming kernel's twins for scale blocks finer than a row (64 << blk_shift weights per scale): whether one takes
// the planned launch (one token tile, unsplit, no stagger), and the launch.
bool mid_blockwise_applies(const GemmPlan &plan, int blk_shift);
hipError_t launch_gemm_mid_blockwise(const GemmPlan &plan, int blk_shift, int dev, int cus, hipStream_t stream);  // ... with the packed weights staged through LDS
hipError_t launch_gemm_mid(const GemmPlan &plan, int dev, int cus, hipStream_t stream);
bool mid_describe(const GemmPlan &plan, char *buf, size_t len);
// Name and template arguments of the kernel launch_gemm would start for `plan` on a device of `cus` CUs.
void describe_gemm_launch(const GemmPlan &plan, int cus, char *buf, size_t len);
void describe_narrow_launch(int rows, int waves_k, int prefetch, int token_tiles, int n, char *buf, size_t len);
// Narrow-row kernel (gemm_narrow.hpp): 16 or 32 rows per workgroup, all waves along k.
struct NarrowArgs {
    const uint8_t *q;
    const void *x;
    const float *code;
    const float *absmax;
    void *out;
    const void *residual;
    int epilogue;
    int m, n, k;
    int n_it;  // k-steps per wave: k / 32 / waves
};
bool narrow_variant_exists(int rows, int waves_k, int prefetch, int token_tiles);
hipError_t launch_gemm_narrow(const NarrowArgs &args, int rows, int waves_k, int prefetch, int token_tiles, hipStream_t stream);
// the narrow-row kernel's scale-block variants (a scale per 64 << blk_shift weights of a row)
hipError_t launch_gemm_blockwise(const NarrowArgs &args, int blk_shift, int rows, int waves_k, int prefetch, int token_tiles,
                                 hipStream_t stream);
bool derive_blockwise_narrow(int m, int k, int blk_shift, int cus, int token_tiles, int *rows, int *waves_k, int *prefetch, int *tt);
bool blockwise_narrow_scales_in_lds(int k, int blk_shift, int rows, int waves_k, int prefetch, int tt);
bool blockwise_narrow_runs(int m, int k, int rows, int waves_k, int prefetch, int token_tiles);
bool launch_is_lean(const GemmPlan &plan, int cus);  // the planned launch would take the lean kernel
bool gemm_variant_exists(int rw, int prefetch, int token_tiles, int decode, int threads, int min_waves, int grouped);

// gemm_multi.hip: several 1..16-token GEMMs in one launch of persistent workgroups (gemm_multi.hpp)
struct MultiArgs;
bool multi_variant_exists(int prefetch);
size_t multi_lds_bytes();
hipError_t launch_gemm_multi(const MultiArgs &args, int prefetch, int dev, hipStream_t stream);
// Compute units of the current device (cached); *dev receives its index.
hipError_t device_cus(int *dev, int *cus);

// gemm_tiled.hip
hipError_t launch_gemm_tiled(const TiledArgs &args, int tile_rows, int tile_tokens, bool mfma32, hipStream_t stream,
                             bool scale_blocks = false);
// 256 x 256 tile, one wave per SIMD (gemm_wide.hip): reached through launch_gemm_tiled
size_t wide_lds_bytes();
hipError_t launch_gemm_wide(const TiledArgs &args, bool mfma32, hipStream_t stream);
bool tiled_variant_exists(int tile_rows, int tile_tokens, bool mfma32);
size_t tiled_lds_bytes(int tile_rows, int tile_tokens);

// dequant_kernel.hip
hipError_t launch_dequant(const uint8_t *q, const float *absmax, const float *code, void *out,
                          int m, int k, int block_size, int decode, hipStream_t stream);
hipError_t launch_quantize(const void *w, const float *code, void *q, float *absmax, int m, int k, int block_size,
                           hipStream_t stream);

// api.cpp: error reporting (the message tuna_last_error returns, per thread), argument checks and the per-stream
// workspace, for the other host translation units
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);
int check_ptr(const void *p, const char *name, size_t align);
void drop_workspace(hipStream_t stream);  // frees the split-K workspace of a stream that is about to be destroyed

// config_table.cpp
struct TableEntry {
    int m, n_lo, n_hi, k;
    int next_from;  // token counts from here to n_hi take the next bucket's entry (n_hi + 1: none does)
    tuna_gemm_config cfg;
    // token counts in [derived_from, derived_to), inside n_lo .. n_hi, take the derived config instead: the tuner
    // timed it there at least a twentieth faster than what the table hands out (0, 0: nowhere)
    int derived_from, derived_to;
};
extern const TableEntry kConfigTable[];
extern const int kConfigTableSize;
// tuned entries of the GEMM with scale blocks finer than a row: (m, token bucket, k, block_size) -> config
struct BlockwiseTableEntry {
    int m, n_lo, n_hi, k, block_size;
    tuna_gemm_config cfg;
};
extern const BlockwiseTableEntry kBlockwiseTable[];
extern const int kBlockwiseTableSize;

}  // namespace tuna
