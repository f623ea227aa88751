// Internal declarations shared by the host API and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/tuna_amd.h"

namespace tuna {

// LDS byte-pair lookup table: 256 rows (one per packed byte value) x 64 copies
// (one per lane) of a half2 {code[byte >> 4], code[byte & 15]}.  Row stride is 256
// bytes so a lane's address is (byte << 8) | (lane << 2): every lane of a wave reads
// its own bank column, whatever the data.
constexpr int kLutBytes = 256 * 64 * 4;
constexpr int kLdsLimit = 160 * 1024;
constexpr int kStepK = 32;          // k per MFMA step (v_mfma_f32_16x16x32_f16)
constexpr int kRowsPerLoad = 64;    // weight rows covered by one 128-bit load per lane
constexpr int kMaxThreads = 1024;

// Everything a GEMM launch needs, filled by the host from a tuna_gemm_config.
struct GemmArgs {
    const uint8_t *q;
    const void *x;
    const float *code;
    const float *absmax;
    void *out;
    float *ws;           // split-K partial sums (library owned), may be null if split_k == 1
    unsigned *counters;  // one arrival counter per (token chunk, row tile), zero between launches
    int m, n, k;
    int waves_m, waves_k, split_k;  // waves_m and waves_k are powers of two
    int wm_log2, wk_log2;
    int steps_total;      // ceil(k / 32)
    int steps_per_split;  // k-steps owned by one workgroup
    int chunk_steps;      // k-steps of x staged in LDS at a time (power of two)
    int chunk_log2;
    int row_tiles;        // workgroups along m
    int xcd_swizzle;
    int lds_bytes;        // dynamic LDS size of the launch (last 16 bytes: arrival ticket)
    int red_bytes;        // bytes of the reduction buffers in the LDS work area
    int planes_log2;      // log2(accumulator planes reduced per epilogue pass)
    int tiles_total;      // row_tiles * split_k: tiles walked by the persistent workgroups
#ifdef TUNA_TRACE
    unsigned long long *trace;  // development builds only: 16 timestamps per workgroup
#endif
};

struct GemmPlan {
    GemmArgs args;
    dim3 grid;
    int threads;
    int rw, prefetch, token_tiles, decode;
    int min_waves;  // waves per SIMD the variant is compiled for (2: <=256 VGPRs, 4: <=128)
    int wgs_per_cu; // workgroups of this launch that fit on one CU (LDS and registers)
    size_t lds_bytes;
    size_t ws_bytes;
    size_t n_counters;
};

// gemm_kernel.hip
hipError_t launch_gemm(const GemmPlan &plan, hipStream_t stream);
bool gemm_variant_exists(int rw, int prefetch, int token_tiles, int decode, int threads, int min_waves);

// dequant_kernel.hip
hipError_t launch_dequant(const uint8_t *q, const float *absmax, const float *code, void *out,
                          int m, int k, int decode, hipStream_t stream);
hipError_t launch_copy(const void *src, void *dst, size_t bytes, hipStream_t stream);
hipError_t launch_read(const void *src, void *sink, size_t bytes, int blocks, hipStream_t stream);

// config_table.cpp
struct TableEntry {
    int m, n_lo, n_hi, k;
    tuna_gemm_config cfg;
};
extern const TableEntry kConfigTable[];
extern const int kConfigTableSize;

}  // namespace tuna
