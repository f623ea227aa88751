/*
 * tuna_amd - measurement and diagnostic entry points of libtuna_amd_bench.so, the diagnostic build.
 *
 * libtuna_amd_bench.so holds everything libtuna_amd.so holds (the same object files; it exports
 * every entry point of tuna_amd.h too) plus the tools declared here for bench.py, the tuner and the
 * tests: timing loops with HIP events on the launch stream, known-traffic yardstick kernels, and
 * process-wide switches between kernels that compute identical results, with counters that tell which
 * kernel ran.  The product library has none of these: its routing choices are constants.  None of
 * them replaces an interface of the reference; the product's C ABI is tuna_amd.h.
 */
#ifndef TUNA_AMD_BENCH_H
#define TUNA_AMD_BENCH_H

#include "tuna_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Timing helper for the bench and the tuner: enqueues `warmup` untimed and `iters`
 * timed GEMMs on `stream`, launch i using weight set (i mod n_sets) of q_list /
 * absmax_list (rotating over distinct weights defeats the L2 / MALL caches), and
 * returns the elapsed milliseconds of the timed launches measured with HIP events
 * recorded on `stream`.  use_graph != 0 captures one rotation into a HIP graph and
 * replays it iters / n_sets times, followed by one replay of a graph of the first
 * iters % n_sets launches: the events bracket exactly `iters` launches either way.
 * This call synchronises the host with `stream`. */
int tuna_time_matmul(const void *const *q_list, const void *const *absmax_list, int n_sets,
                     const void *x, const void *code, void *out, int m, int n, int k,
                     const tuna_gemm_config *cfg, int decode_mode, int warmup, int iters,
                     int use_graph, void *stream, float *elapsed_ms);
/* The same GEMMs dealt round-robin to `n_streams` (1..16) streams of the default priority that the
 * call creates and destroys: launch i goes to stream i mod n_streams, writes out_list[i mod n_streams]
 * (n_streams distinct output buffers) and uses weight set i mod n_sets.  All streams start behind one
 * event and the end event waits for all of them; the time is that of `iters` launches in all.
 * use_graph != 0: up to 256 launches are recorded, with that fork and join, into one HIP graph of
 * n_streams parallel branches and the graph is replayed, which takes the host's enqueue time out of
 * the picture.  It answers one question: do independent GEMMs on different streams overlap on the
 * device. */
int tuna_time_matmul_streams(const void *const *q_list, const void *const *absmax_list, int n_sets,
                             const void *x, const void *code, void *const *out_list, int n_streams,
                             int m, int n, int k, const tuna_gemm_config *cfg, int decode_mode,
                             int use_graph, int warmup, int iters, float *elapsed_ms);
/* Launches of a kernel that does nothing (`blocks` workgroups of `threads` threads, one pointer
 * argument), on one stream of the call's own - use_graph != 0: recorded into a HIP graph of 64 launches
 * and replayed, which takes the host's enqueue time out of the cadence - or dealt to n_streams > 1
 * streams as above: the time any launch costs on this device.  `sink`: 4 writable bytes. */
int tuna_time_empty_launches(void *sink, int blocks, int threads, int n_streams, int use_graph,
                             int warmup, int iters, float *elapsed_ms);
/* Yardstick of the split-K hand-over: `pairs` (1..64) producer / consumer workgroup pairs, one workgroup per compute
 * unit, partners on one XCD (same_xcd != 0: workgroups 8 apart in launch order) or on neighbouring XCDs, run `iters`
 * rounds of: producer stores 1 KB and waits for the acknowledgement, bumps a flag with a returning device-scope atomic;
 * consumer sees the flag, loads the 1 KB and checks it.  store_sc1 / load_sc1: the accesses carry the sc1 bit (what the
 * kernels' hand-over uses: coherent across the eight L2s) or stay in the XCD's own L2; reuse != 0: the same 1 KB every
 * round, so that a stale line in the consumer's caches shows as a mismatch.  out6 receives: nanoseconds per round for
 * the acknowledged store, the atomic's round trip and the load; mismatching 16-byte pieces; rounds given up (every wait
 * is bounded); pairs whose workgroups did share an XCD (read back from the hardware).  Allocates its own buffers and
 * synchronises `stream`. */
int tuna_measure_handover(int same_xcd, int store_sc1, int load_sc1, int reuse, int pairs, int iters,
                          void *stream, double *out6);
/* Same protocol for the blockwise GEMM with an explicit config, as tuna_matmul_blockwise_ex runs it: every absmax_list
 * entry is fp32 [m, k / block_size]; cfg NULL = the library's choice.  What the tuner times the blockwise candidates
 * with. */
int tuna_time_matmul_blockwise(const void *const *q_list, const void *const *absmax_list, int n_sets,
                               const void *x, const void *code, void *out, int m, int n, int k, int block_size,
                               const tuna_gemm_config *cfg, int warmup, int iters, int use_graph,
                               void *stream, float *elapsed_ms);
/* Same protocol for tuna_matmul_multi: `problems` holds n_sets batches of `count` problems each,
 * iteration i is one call with batch (i mod n_sets); the time is that of `iters` calls. */
int tuna_time_matmul_multi(const tuna_gemm_problem *problems, int n_sets, int count, int warmup,
                           int iters, int use_graph, void *stream, float *elapsed_ms);
/* Same protocol for the grouped GEMM. */
int tuna_time_matmul_grouped(const void *const *q_list, const void *const *absmax_list, int n_sets,
                             const void *x, const void *code, void *out, int m_group, int n_groups,
                             int k, const int32_t *token_offsets, const tuna_gemm_config *cfg,
                             int decode_mode, int warmup, int iters, int use_graph, void *stream,
                             float *elapsed_ms);
/* Same protocol for the dequant kernel. */
int tuna_time_dequant(const void *const *q_list, const void *const *absmax_list, int n_sets,
                      const void *code, void *out, int m, int k, int warmup, int iters,
                      void *stream, float *elapsed_ms);
/* Plain device-to-device copy kernel of `bytes` bytes (16-byte multiples), timed the
 * same way: the known-traffic yardstick the HBM counters are scaled against. */
int tuna_time_copy(const void *src, void *dst, size_t bytes, int warmup, int iters,
                   void *stream, float *elapsed_ms);

/* Read-only streaming kernel over `bytes` bytes of `src` (16-byte multiples), `blocks`
 * workgroups of 256 threads (0 = 2048): the ceiling a pure HBM reader reaches on the device,
 * reported beside the GEMM's rate.  `variant`: 0 nontemporal loads, 8 in flight per lane;
 * 1 plain loads, 8; 2 nontemporal, 16; 3 plain, 16; 4 nontemporal, 4; 5 plain, 4.  `sink` is
 * 4 writable bytes. */
int tuna_time_read(const void *src, void *sink, size_t bytes, int blocks, int variant, int warmup,
                   int iters, void *stream, float *elapsed_ms);

/* What the matrix cores and the LDS deliver on this device, the yardsticks of the many-token kernels as the
 * read kernel is that of the streaming ones.  unit 0 / 1: independent v_mfma_f32_16x16x32_f16 back to back from
 * one / two waves per SIMD (16 accumulators each); 2: v_mfma_f32_32x32x16_f16 from one wave per SIMD (4
 * accumulators); 3: 16-byte LDS reads in the pattern of an MFMA fragment read from a tile of 128-byte rows; 4:
 * 4-byte LDS reads in the pattern of the byte-pair decode table; 5: 16-byte LDS writes in the pattern of the
 * decoded weight tile; 6: the same bytes as pairs of 8-byte writes; 7: 16-byte writes at consecutive addresses;
 * 8 / 9: the table reads of 4 with one copy of the table per 32 / 16 lanes instead of per 64, a pseudo-random byte
 * per lane (3..9 with 8 waves per compute unit); 10 / 13: v_mfma_f32_32x32x16_f16 from one / two waves per SIMD and
 * 12 / 11: v_mfma_f32_16x16x32_f16 from one / two waves per SIMD, 16 accumulators, with four + four operand
 * registers of pseudo-random fp16 values in (-1, 1) - the rate the matrix cores sustain on real data, which is
 * well below the rate on the regular operands of units 0..2; 14 / 15 / 16: units 4 / 3 / 5 with 16 waves per
 * compute unit (8 waves do not keep enough reads in flight to saturate the LDS); 17..21: the k-step of a 64-token
 * streaming launch without its memory side, eight waves per compute unit, per wave and iteration sixteen table reads
 * + four fragment reads and sixteen 16x16x32 MFMAs on pseudo-random operands - 17 the MFMAs only, 18 the LDS reads
 * only, 19 both in every wave (reads requested ahead of the MFMAs, used behind them), 20 four waves (one per SIMD)
 * with the MFMAs of two and four with the reads of two, 21 both in every wave with the reads requested between the
 * MFMAs and used an iteration later: whether 19..21 take the longer of 17 and 18 or their sum says whether a compute
 * unit overlaps the two.  One
 * workgroup per compute unit (two for units 1, 11, 13).  *work_per_launch receives the flops (0..2, 10..13, 17..21:
 * the MFMAs' of 17, also for 18) or LDS bytes (3..9, 14..16) of one launch; `sink`: 8 writable bytes. */
int tuna_time_unit_rate(int unit, void *sink, int warmup, int iters, void *stream, float *elapsed_ms,
                        double *work_per_launch);

/* Self-test of the quantizer's division: the kernel divides by a block's maximum with a refined
 * reciprocal and one fused correction instead of the general IEEE sequence; this runs that
 * division for every pair of fp16 values (w, a) with a > 0 finite and |w| <= a - all the quotients
 * the quantizer can form - against the IEEE division on the device (zeros of either sign count as
 * equal: the quotient is only ever compared or subtracted from).  `counts`: two zeroed device
 * uint64; counts[0] receives the pairs checked, counts[1] the mismatches. */
int tuna_selftest_quantizer_division(void *counts, void *stream);

/* Diagnostic override of the batched kernel's workgroup shape (tuna_matmul_multi): waves along the
 * rows (1, 2, 4, 8 or 16 of the workgroup's 16 waves; 0 = the library's choice) and ring depth
 * (2 or 4; 0 = the library's choice).  For A/B timing. */
int tuna_set_multi_shape(int waves_m, int prefetch);
/* Switch, process-wide: batches that run with a ring of 2 stage the packed weights and x through LDS
 * (global -> LDS loads, as the LDS-staged twins of the streaming kernel do) instead of registers.
 * Bit-identical results; for A/B timing.  Returns the previous setting. */
int tuna_set_multi_weight_path(int through_lds);
/* Diagnostic: tuna_matmul_blockwise calls so far in this process that ran the narrow-row kernel (kernel 0), launches of
 * the batched streaming kernel (1), calls that ran the many-token kernel (2) and calls that ran the streaming kernel's
 * scale-block twin (3) on their behalf. */
unsigned long long tuna_blockwise_launches(int kernel);
/* A/B switch of the narrow-row blockwise GEMM, process-wide: 1 (default) copies a workgroup's scales into LDS once and
 * reads them from there (when they fit beside the decode table), 0 reads them from memory with every ring slot.
 * Bit-identical results.  Returns the previous setting. */
int tuna_set_blockwise_scales_lds(int enabled);

/* Diagnostic: the shortest run of problems tuna_matmul_multi hands to the batched kernel
 * (default 2; 1 sends single problems through it as well).  Returns the previous value. */
int tuna_set_multi_min_batch(int count);
/* Diagnostic: launches of the batched kernel so far in this process. */
unsigned long long tuna_multi_launches(void);

/* Diagnostic switch, process-wide, default on: dense launches that qualify run one of two
 * kernels stripped of everything else the general one carries - small launches (one workgroup
 * per tile, power-of-two split, aligned shapes, up to 16 tokens per tile) and launches with 2, 4
 * or 8 token tiles and no split of k across workgroups (x chunks double-buffered in LDS).  Both
 * compute the general kernel's results bit for bit; turning them off is for A/B timing and for
 * the tests that check exactly that.  A config whose ring depth or token tile count only the
 * second kernel has (prefetch 4 or 8 with 4 token tiles, 8 token tiles, 16 waves with 2 or more
 * token tiles) runs it regardless of the switch.  Returns the previous setting.  No counterpart
 * in the reference. */
int tuna_set_lean_kernels(int enabled);

/* Diagnostic: how many GEMM launches of this process took one of those kernels so far. */
unsigned long long tuna_lean_launches(void);

/* Diagnostic switch, process-wide, default 0: with 1, unsplit 16-wave launches of up to 16 tokens
 * and 8- or 16-wave launches with more token tiles (the streaming kernel of gemm_mid.hpp, ring depth 2 or 4) stage the packed weights through
 * LDS (global_load_lds_dwordx4 into a per-wave ring, ds_read_b128 when a slot is consumed) instead
 * of loading them into registers.  Same access pattern, ring depth, arithmetic and results; it
 * exists so that the two weight paths can be timed against each other on one box (the reference
 * stages its packed weights through shared memory, kernel.cu:1997-2042).  Returns the previous
 * setting.  tuna_describe_launch names the path a launch would take. */
int tuna_set_weight_path(int through_lds);

#ifdef __cplusplus
}
#endif
#endif /* TUNA_AMD_BENCH_H */
