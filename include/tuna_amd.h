/*
 * tuna_amd - C ABI of the MI355X (gfx950) FP16-activation x 4-bit-codebook-weight GEMM.
 *
 * This is the drop-in boundary: plain pointers and sizes, no torch types.  Every
 * device pointer is caller-owned memory on the current HIP device; `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  All entry points are
 * stream-ordered and never synchronise the host with the device, unless stated.
 *
 * Naming follows the reference: m = weight rows (output features), n = activation
 * rows (tokens), k = reduction length.
 *
 * Tensor layouts (identical to the reference's, extension.cpp:26-49):
 *   q       uint8  [m/8, k/8, 32]  one 32-byte record per 8x8 weight block; byte b of
 *                                  block (mb, kb) holds row mb*8 + b/4, column
 *                                  kb*8 + 2*(b%4) in its high nibble and column
 *                                  kb*8 + 2*(b%4) + 1 in its low nibble
 *                                  (test.py:58-65, kernel.cu:3221-3228)
 *   x       fp16   [n, k]          row-major (test.py:76)
 *   code    fp32   [16]            codebook (kernel.cu:3014)
 *   absmax  fp32   [m]             one scale per weight row (kernel.cu:3015)
 *   out     fp16   [n, m]          row-major (kernel.cu:2872, 2957-2959)
 */
#ifndef TUNA_AMD_H
#define TUNA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TUNA_AMD_VERSION 100 /* major*10000 + minor*100 + patch */

/* Status codes.  The reference returns void and silently does nothing for
 * shapes outside its table (kernel.cu:3018-3156); here every call reports. */
enum {
    TUNA_OK = 0,
    TUNA_ERR_INVALID_ARG = 1, /* null pointer, misaligned pointer, bad size          */
    TUNA_ERR_UNSUPPORTED = 2, /* shape or config the kernels cannot run              */
    TUNA_ERR_HIP = 3,         /* a HIP runtime call failed (see tuna_last_error)     */
    TUNA_ERR_NO_DEVICE = 4,   /* no usable gfx950 device                             */
    TUNA_ERR_WORKSPACE = 5    /* split-K workspace could not be provided             */
};

/* Decode rounding of a 4-bit code into an fp16 weight.
 * TUNA_DECODE_GEMM    : fp16(code) * fp16(absmax) as an fp16 multiply - what the
 *                       reference GEMM feeds its tensor cores (kernel.cu:2178-2192
 *                       with the fp16 staging of kernel.cu:2770, 2800).
 * TUNA_DECODE_DEQUANT : fp16(code * absmax) with the product in fp32 - what the
 *                       reference dequant op writes (kernel.cu:3222-3228).        */
enum { TUNA_DECODE_GEMM = 1, TUNA_DECODE_DEQUANT = 2 };

/* What happens to the fp32 sums before they are stored (tuna_matmul_fused).
 * TUNA_EPILOGUE_RESIDUAL : out = fp16(sum + residual), residual fp16 [n, m] (may be `out` itself).
 * TUNA_EPILOGUE_SILU_MUL : for a combined gate+up projection whose weight rows are interleaved
 *                          (row 2i = gate_i, row 2i+1 = up_i): out [n, m/2] with
 *                          out[t, i] = fp16(silu(sum[t, 2i]) * sum[t, 2i+1]).               */
enum { TUNA_EPILOGUE_NONE = 0, TUNA_EPILOGUE_RESIDUAL = 1, TUNA_EPILOGUE_SILU_MUL = 2 };

/* Tile configuration of one GEMM launch: the CDNA4 counterpart of the reference's
 * KernelConfig (configs.cu:12-54).  A workgroup is waves_m x waves_k wave64s; a wave
 * owns rows_per_wave weight rows and walks k in steps of 32; the workgroup owns
 * rows_per_wave*waves_m rows and a 1/split_k share of k.                          */
typedef struct tuna_gemm_config {
    int32_t rows_per_wave; /* 64, 128 or 256: 128-bit loads per lane per k-step x 64.  16, 24 or 32 (with
                              waves_m 1), or 64 with waves_m 0: the narrow-row kernel - that many rows per
                              workgroup, every wave along k, no split (m a multiple of it; 24 is a 32-row
                              tile three quarters full, for row counts that make 256 tiles of 24) */
    int32_t waves_m;       /* waves along the weight rows (any count; waves_m*waves_k <= 16) */
    int32_t waves_k;       /* waves along k inside the workgroup, a power of two (reduced in LDS) */
    int32_t split_k;       /* workgroups along k (reduced through the workspace); 0 = balanced:
                              the k ranges of all row tiles, laid end to end, are divided
                              evenly over the workgroups the device holds at once      */
    int32_t prefetch;      /* 2, 4 or 8: k-steps of packed weights in flight per wave */
    int32_t x_chunk;       /* k elements of x staged in LDS at a time: a power of two, at least
                              32*waves_k*prefetch, and x_chunk*token_tiles at most 2x the workgroup's
                              threads (4x with prefetch 8)                            */
    int32_t token_tiles;   /* 1, 2 or 4: 16-token MFMA tiles per pass over the weights */
    int32_t xcd_swizzle;   /* 1: remap workgroup ids so neighbours share an XCD       */
    int32_t k_stagger;     /* row tile r starts r*k_stagger k-steps into its k range and wraps
                              around (0: every row tile starts at the front).  When k*4 bytes,
                              the distance between block rows, is a large power of two, tiles
                              walking in lockstep keep hitting the same memory channels  */
    int32_t lds_tile_rows; /* 0: streaming kernel (all fields above).  -1: the same, with the packed
                              weights, x and scales staged through LDS by global -> LDS loads
                              (the reference's weight path, kernel.cu:1997-2042) instead of
                              registers: same results bit for bit; for launches of 8 or 16 waves
                              with prefetch 2 or 4 (2 with eight token tiles), k unsplit or, with
                              two or four token tiles, split into a power of two of equal parts.  64, 128 or 256: the
                              many-token kernel, which decodes a tile of this many weight rows
                              once into LDS for token_tiles*16 (64, 128 or 256) tokens; only
                              token_tiles, split_k (>= 1) and rows_per_wave are read besides:
                              rows_per_wave == 32 multiplies with 32 x 32 x 16 MFMA tiles
                              (tiles of at least 32 tokens), any other value with 16 x 16 x 32
                              (the reference's counterpart: its MMA shapes, kernel.cu:411-465).
                              256 rows x 256 tokens is a kernel of its own (one wave per SIMD, a
                              wave owns 128 x 128) */
} tuna_gemm_config;

int tuna_version(void);
const char *tuna_status_string(int status);
/* Message of the last failing call on this host thread ("" if none). */
const char *tuna_last_error(void);

/* out[n, m] = x[n, k] . decode(q, code, absmax)[m, k]^T, fp32 accumulate, fp16 output.
 * Replaces  void wrapper(void *q, void *x, void *c, void *s, void *o, int m, int n,
 * int k, cudaStream_t)  (kernel.cu:3009, declared extension.cpp:22); same argument
 * order.  `out` is overwritten (it need not be zeroed, unlike kernel.cu:2739-2745).
 * Uses TUNA_DECODE_GEMM and the built-in shape->config table (any m % 8 == 0,
 * k % 8 == 0, n >= 1 is accepted; shapes outside the table get a derived config). */
int tuna_matmul(const void *q, const void *x, const void *code, const void *absmax,
                void *out, int m, int n, int k, void *stream);

/* Same, with an explicit config (NULL = table lookup) and decode mode. */
int tuna_matmul_ex(const void *q, const void *x, const void *code, const void *absmax,
                   void *out, int m, int n, int k, const tuna_gemm_config *cfg,
                   int decode_mode, void *stream);

/* Bytes of split-K partial sums the static scratch of tuna_matmul_static holds (plus 65536
 * arrival counters). */
#define TUNA_STATIC_WORKSPACE_BYTES (16u << 20)

/* Optional one-time set-up on the current device: resolves the device address of the static
 * scratch that tuna_matmul_static uses.  tuna_matmul_static does the same on its first call on
 * a device; calling this first keeps even that step out of the caller's critical section. */
int tuna_init(void);

/* tuna_matmul_ex for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Where
 * tuna_matmul_ex takes the split-K partial sums and arrival counters of a launch from a
 * library-owned workspace that is allocated on first use, this entry point takes them from a
 * fixed array in device memory that is part of the loaded library (16 MB + 256 KB, held on
 * every GPU the library runs on until the process ends) and calls no allocating routine.  A
 * launch that needs more than TUNA_STATIC_WORKSPACE_BYTES of partial sums or more than 65536
 * counters fails with TUNA_ERR_WORKSPACE (where the library picks the config - cfg NULL - and its
 * pick splits k of a many-token tile further than that, it reduces the split until it fits).  All calls on one GPU share that GPU's array: calls
 * that may overlap (different streams) race; calls on one stream are ordered and safe.  The
 * kernels return the counters they used to zero, so nothing is cleared between calls.  Results
 * are those of tuna_matmul_ex, bit for bit. */
int tuna_matmul_static(const void *q, const void *x, const void *code, const void *absmax,
                       void *out, int m, int n, int k, const tuna_gemm_config *cfg,
                       int decode_mode, void *stream);

/* tuna_matmul_ex with a fused epilogue (the step after the GEMM in a decoder layer: the
 * residual add after the attention-out / down projections, SiLU(gate) * up after the combined
 * gate+up projection), saving a launch and a round trip of the activations through HBM.
 * `residual` is read only with TUNA_EPILOGUE_RESIDUAL.  No counterpart in the reference. */
int tuna_matmul_fused(const void *q, const void *x, const void *code, const void *absmax,
                      void *out, int m, int n, int k, const tuna_gemm_config *cfg,
                      int decode_mode, int epilogue, const void *residual, void *stream);

/* One GEMM of a batch: the arguments of tuna_matmul. */
typedef struct tuna_gemm_problem {
    const void *q;      /* uint8 [m/8, k/8, 32] */
    const void *x;      /* fp16  [n, k]         */
    const void *code;   /* fp32  [16]           */
    const void *absmax; /* fp32  [m]            */
    void *out;          /* fp16  [n, m]         */
    int32_t m, n, k;
} tuna_gemm_problem;

/* `count` independent GEMMs in one call - the projections of a decoder layer that do not feed
 * one another (Q, K and V kept separate; gate and up), the experts of a mixture, the layers of
 * a benchmark sweep (README.md:25-27 totals are layers x four GEMMs).  `problems` is a host
 * array read during the call.  Runs of up to 32 consecutive problems with at most 16 tokens
 * each, rows in multiples of 64, k in multiples of 256 or more, 16-byte aligned scales and one
 * shared codebook become ONE launch of persistent workgroups: the k ranges of all row tiles of
 * all problems are laid end to end and divided evenly over the compute units, a workgroup
 * streams its share without a gap between problems, and the per-launch fixed time (about 2.5
 * us kernel-to-kernel, the ramp of the memory system, the uneven finish) is paid once per batch
 * instead of once per GEMM.  Results are deterministic and within the GEMM's tolerance of
 * tuna_matmul's (the summation order differs where tuna_matmul uses another kernel).  Problems
 * that do not qualify are launched one by one, exactly as tuna_matmul would.  Ordering is that
 * of one call on `stream`; no problem may read what another one writes.  All problems are
 * checked before anything is enqueued.  No counterpart in the reference. */
int tuna_matmul_multi(const tuna_gemm_problem *problems, int count, void *stream);
/* tuna_matmul_multi with a fused epilogue per problem (those of tuna_matmul_fused): epilogues[i] is the
 * TUNA_EPILOGUE_* of problem i and residuals[i] its residual (fp16 [n, m], 8-byte aligned, may be the problem's
 * own output; ignored unless the epilogue is TUNA_EPILOGUE_RESIDUAL).  For TUNA_EPILOGUE_SILU_MUL the problem's
 * weight rows are interleaved (2i: gate, 2i+1: up) and its out is fp16 [n, m/2].  Either array may be NULL
 * (no epilogues / no residuals).  A decoder layer's projections launched together - SiLU-mul on the combined
 * gate+up GEMM, the residual add on the out and down projections - cost one launch instead of four GEMMs and
 * two element-wise kernels; as in tuna_matmul_multi no problem may read what another one writes.  No
 * counterpart in the reference (README.md:25-27 counts a layer as four separate GEMMs). */
int tuna_matmul_multi_fused(const tuna_gemm_problem *problems, const int32_t *epilogues,
                            const void *const *residuals, int count, void *stream);
/* The same for weights with one scale per block_size (64, 128, 256, ...) consecutive weights of a row: every
 * problem's absmax is fp32 [m, k / block_size] (the layout tuna_quantize_blockwise writes, the reference
 * quantizer's for block_size < k, test.py:7-17), 4-byte aligned.  Problems that do not qualify for the batched
 * launch are run one by one as tuna_matmul_blockwise would.  No counterpart in the reference's kernels. */
int tuna_matmul_multi_blockwise(const tuna_gemm_problem *problems, int count, int block_size, void *stream);

/* Grouped GEMM (mixture of experts with per-expert token lists) in one launch.  The weights
 * are n_groups (<= 64) matrices of m_group rows stacked along m - q [n_groups*m_group/8, k/8,
 * 32], absmax [n_groups*m_group] - exactly the layout of the dense stacked call.  x [n_total,
 * k] holds the activation rows sorted by group: group e owns rows token_offsets[e] ..
 * token_offsets[e+1]-1 (token_offsets: HOST array of n_groups+1 non-decreasing ints, read
 * during the call; n_total = token_offsets[n_groups]).  out [n_total, m_group]:
 *   out[t, r] = x[t, :] . decode(W_e)[r, :]   for t in group e.
 * Groups without tokens are skipped: their weights are not read.  m_group must be a multiple
 * of 64 (of the config's rows per workgroup if cfg is given; NULL = table lookup on
 * (n_groups*m_group, largest group, k)).  With cfg NULL a group of more than 64 tokens (prefill
 * sizes) runs as a dense GEMM of its own on the same stream - tuna_matmul on the group's slices
 * of q, absmax, x and out, bit-identical to that call - and only the smaller groups share the
 * grouped launch: the grouped kernel would stream such a group's weights once per 64 tokens, the
 * many-token kernels decode them once per 128 to 256.  No counterpart in the reference, whose 8-expert
 * benchmark applies every expert to every token (README.md:16-18); this is the op a
 * router-driven Mixtral layer needs. */
int tuna_matmul_grouped(const void *q, const void *x, const void *code, const void *absmax,
                        void *out, int m_group, int n_groups, int k,
                        const int32_t *token_offsets, const tuna_gemm_config *cfg,
                        int decode_mode, void *stream);

/* out[m, k] fp16 row-major = decode(q, code, absmax), TUNA_DECODE_DEQUANT rounding.
 * Replaces  void dequantize_wrapper(void *q, void *a, void *c, void *o, const int m,
 * const int k, cudaStream_t)  (kernel.cu:3243, declared extension.cpp:24). */
int tuna_dequant(const void *q, const void *absmax, const void *code, void *out,
                 int m, int k, void *stream);

/* Same with the decode rounding selectable (TUNA_DECODE_GEMM gives the image of the
 * weights the GEMM multiplies with). */
int tuna_dequant_ex(const void *q, const void *absmax, const void *code, void *out,
                    int m, int k, int decode_mode, void *stream);

/* Quantizer and packer on the device: fp16 weights w [m, k] row-major -> q [m/8, k/8, 32] and
 * absmax fp32 [m] (one scale per weight row) for the 16-entry codebook `code`.  The
 * arithmetic of the reference harness's quantize_blockwise_dynamic_4bit with block_size == k
 * and preprocess=True (test.py:7-68): absmax = max |w|; index = argmin |fp32(w) / absmax -
 * code[j]| in fp32, first index on ties; packing of test.py:55-65.  An all-zero row gets index
 * 0 throughout (0/0 makes every candidate NaN and torch.argmin then returns 0).  The reference
 * has this only as Python on torch tensors. */
int tuna_quantize(const void *w, const void *code, void *q, void *absmax, int m, int k, void *stream);

/* Scale blocks finer than a row.  The reference's quantizer takes a block_size (test.py:7-17): the
 * weights, flattened row-major, are cut into blocks of block_size elements with one absmax each,
 * so for k a multiple of block_size element (r, c) uses absmax[r * (k/block_size) + c/block_size];
 * its kernels only ever run block_size == k (test.py:81, kernel.cu:2904).  The three entry points
 * below take absmax fp32 [m, k/block_size] in that layout; block_size == k is the plain op.
 *   tuna_quantize_blockwise : block_size 8, 16, 32, 64, 128, 256 or k.
 *   tuna_dequant_blockwise  : any multiple of 8 that divides k.
 *   tuna_matmul_blockwise   : block_size 64, 128, 256, ... (a multiple of 64 that divides k) with m
 *                             a multiple of 16 and k of 256; TUNA_DECODE_GEMM rounding,
 *                             fp16(code) * fp16(absmax of the block), as in tuna_matmul.       */
int tuna_quantize_blockwise(const void *w, const void *code, void *q, void *absmax, int m, int k,
                            int block_size, void *stream);
int tuna_dequant_blockwise(const void *q, const void *absmax, const void *code, void *out, int m, int k,
                           int block_size, int decode_mode, void *stream);
int tuna_matmul_blockwise(const void *q, const void *x, const void *code, const void *absmax,
                          void *out, int m, int n, int k, int block_size, void *stream);
/* tuna_matmul_blockwise with an explicit config (NULL: the library's choice, as tuna_matmul_blockwise).  The
 * reference makes the scale block a field of every kernel config (deq_block_size, configs.cu:31); here a blockwise
 * launch is described by the same tuna_gemm_config as a per-row one and what the config names decides the kernel:
 * lds_tile_rows > 0 the many-token kernel (tile lds_tile_rows x 16 * token_tiles, k split split_k ways);
 * rows_per_wave 16 / 32, or 64 with waves_m = 0, the narrow-row kernel (that many rows per workgroup, waves_k waves
 * along k, ring `prefetch`, one or two token tiles); split_k == 0 the batched streaming kernel (waves_m x 16 / waves_m
 * waves, ring `prefetch`); anything else the streaming kernel's scale-block twin (up to 64 tokens: unsplit row-tile
 * walkers of waves_m x waves_k waves, ring, x chunk and stagger as named).  TUNA_ERR_UNSUPPORTED if the config cannot
 * run the call. */
int tuna_matmul_blockwise_ex(const void *q, const void *x, const void *code, const void *absmax,
                             void *out, int m, int n, int k, int block_size,
                             const tuna_gemm_config *cfg, void *stream);
/* The config tuna_matmul_blockwise runs for (m, n, k, block_size): the tuned entry of the blockwise table, keyed by
 * (m, token bucket, k, block_size), if there is one (*from_table = 1), else a config derived from the shape.  Host only. */
int tuna_select_config_blockwise(int m, int n, int k, int block_size, tuna_gemm_config *cfg, int *from_table);
/* TUNA_OK if `cfg` can run the blockwise GEMM (m, n, k, block_size).  Host only. */
int tuna_validate_config_blockwise(int m, int n, int k, int block_size, const tuna_gemm_config *cfg);
/* The blockwise table (generated from tuna_amd/configs/param_map_blockwise.json). */
int tuna_blockwise_table_size(void);
int tuna_blockwise_table_entry(int i, int *m, int *n_lo, int *n_hi, int *k, int *block_size, tuna_gemm_config *cfg);

/* Shape -> config.  Replaces the if-chain of kernel.cu:3018-3156 over the constants of
 * configs.cu:56-3331 by a table lookup on (m, n-bucket, k) with a derived fallback.
 * Runs on the host only (no device needed).  Returns 1 in *from_table when the shape
 * hit a tuned entry. */
int tuna_select_config(int m, int n, int k, tuna_gemm_config *cfg, int *from_table);
/* The config tuna_matmul_ex(cfg = NULL, decode_mode) runs: the table lookup above for
 * TUNA_DECODE_GEMM; for TUNA_DECODE_DEQUANT, whose kernel variants the table is not tuned for,
 * always a derived config.  Host only. */
int tuna_select_config_ex(int m, int n, int k, int decode_mode, tuna_gemm_config *cfg, int *from_table);
/* The config tuna_matmul_grouped(cfg = NULL) runs for n_active groups with tokens, the largest
 * of them with max_tokens.  Host only. */
int tuna_select_config_grouped(int m_group, int n_active, int max_tokens, int k, int decode_mode,
                               tuna_gemm_config *cfg);
/* The config the library derives for a shape when its table has no entry for it - also for shapes that have
 * one: what the tuner seeds its search with, and what a table entry has to beat.  Host only. */
int tuna_derive_config(int m, int n, int k, tuna_gemm_config *cfg);

/* Name and template arguments of the kernel a GEMM launch would start (cfg NULL = the library's
 * choice), e.g. "gemm_narrow_kernel<LW=2,WK=8,U=4,PERM=1,TT=1>": for logs, and for matching a timing
 * with a profile.  Host only; with a device present the
 * device's CU count decides between twins, otherwise 256 CUs are assumed. */
int tuna_describe_launch(int m, int n, int k, const tuna_gemm_config *cfg, int decode_mode,
                         char *buf, size_t len);

/* TUNA_OK if `cfg` can run shape (m, n, k); otherwise an error and tuna_last_error(). */
int tuna_validate_config(int m, int n, int k, const tuna_gemm_config *cfg);
/* Same for a decode mode (tuna_validate_config checks TUNA_DECODE_GEMM). */
int tuna_validate_config_ex(int m, int n, int k, const tuna_gemm_config *cfg, int decode_mode);
/* Dynamic LDS bytes and workspace bytes a launch of `cfg` needs. */
int tuna_config_footprint(int m, int n, int k, const tuna_gemm_config *cfg,
                          size_t *lds_bytes, size_t *workspace_bytes);
/* How a launch of `cfg` divides the work (host only, no device needed): the segments
 * workgroup `workgroup` of `n_workgroups` walks (0 = as many as the launch would start on
 * a 256-CU device), four ints each: row tile, first k-step (32 k each), k-steps, and the
 * slot of its partial sums (-1: the segment is a whole row tile and writes the output
 * itself).  At most max_segments are written; *n_segments is the full count.  No counterpart
 * in the reference, whose grid is one threadblock per tile (kernel.cu:2962-3007). */
int tuna_config_segments(int m, int n, int k, const tuna_gemm_config *cfg, int n_workgroups,
                         int workgroup, int *segments, int max_segments, int *n_segments);
/* Balanced split only (split_k == 0): the workgroups whose partial sums make up row tile
 * `row_tile`, first_workgroup .. first_workgroup + count - 1 in k order, and the slot the
 * first of them used (all later ones use slot 0).  With a fixed split: -1, split_k, 0. */
int tuna_config_contributors(int m, int n, int k, const tuna_gemm_config *cfg, int n_workgroups,
                             int row_tile, int *first_workgroup, int *count, int *first_slot);
/* Enumerate the built-in table: entry i -> its shape key and config. */
int tuna_config_table_size(void);
int tuna_config_table_entry(int i, int *m, int *n_lo, int *n_hi, int *k, tuna_gemm_config *cfg);
/* Entries are tuned at the lower edge n_lo of their token bucket; token counts from this value to n_hi get the next
 * bucket's entry from tuna_select_config instead, where that entry can run them (n_hi + 1: none does; -1: bad
 * index).  Written by the tuner, which times both entries inside the bucket. */
int tuna_config_table_next_from(int i);
/* Token counts in [*from, *to), inside the entry's n_lo .. n_hi, get the derived config from tuna_select_config
 * instead of the table's (0, 0: none do).  Written by the tuner, which times both at several counts inside the
 * bucket: the derivation sizes its grid for n itself, an entry's grid was sized for n_lo.  No counterpart in the
 * reference, whose buckets hand out one config each (kernel.cu:3022-3155). */
int tuna_config_table_derived_range(int i, int *from, int *to);

/* Releases the library-owned split-K workspaces of the current device (synchronises
 * the device first).  Until then a workspace that a launch has used is never freed or moved -
 * HIP graphs captured earlier keep working when later launches need a larger one - so call this
 * only when no captured graph that contains GEMMs of this library will be replayed again. */
int tuna_release_workspaces(void);

#ifdef __cplusplus
}
#endif
#endif /* TUNA_AMD_H */
