// Yardstick and self-test kernels of the diagnostic build (libtuna_amd_bench.so): a plain copy (the known-traffic
// launch the HBM counters are scaled by), a read-only stream (the ceiling a pure HBM reader reaches), the matrix-core
// and LDS unit rates, and the exhaustive check of the quantizer's division.  None of them is part of the product
// library.
#include "tuna_internal.h"
#include "bench_internal.h"
#include "quantize_div.hpp"

namespace tuna {

typedef _Float16 f16;
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Plain copy: the known-traffic yardstick for the HBM counters.
__global__ __launch_bounds__(256) void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Read-only stream: the ceiling a pure HBM reader reaches on this device.  UNROLL loads of 16
// bytes in flight per lane (UNROLL * 4 KB per workgroup and step), blocks walk the buffer in
// lockstep; NT selects nontemporal (streaming) or plain loads.
template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void read_kernel(const u32x4 *__restrict__ src, uint32_t *__restrict__ sink, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    u32x4 acc = u32x4{0u, 0u, 0u, 0u};
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = NT ? __builtin_nontemporal_load(src + i + u * stride) : src[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
    }
    for (; i < n16; i += stride) acc ^= NT ? __builtin_nontemporal_load(src + i) : src[i];
    const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (r == 0x9e3779b9u) sink[0] = r;  // practically never: keeps the loads alive
}

// A kernel that does nothing (one pointer argument, as every real kernel has at least one): what a launch costs by
// itself.
__global__ void empty_kernel(uint32_t *sink)
{
    if (sink == reinterpret_cast<uint32_t *>(1)) *sink = 0u;
}

hipError_t launch_empty(void *sink, int blocks, int threads, hipStream_t stream)
{
    hipLaunchKernelGGL(empty_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0, stream, static_cast<uint32_t *>(sink));
    return hipGetLastError();
}

// ---- hand-over yardstick: what one producer -> consumer step of a split-K hand-over costs between two workgroups --------
// Workgroup pairs (producer b, consumer b + stride; one workgroup per compute unit): the producer stores 1 KB, waits for
// the stores to be acknowledged, bumps a flag with a returning atomic; the consumer polls the flag, loads the 1 KB and
// checks it, then acknowledges; `iters` rounds in lock step, every wait bounded.  store_sc1 / load_sc1: the accesses
// carry the sc1 bit (coherent across the device's eight L2s: write-through stores, loads that do not hit in a
// neighbouring compute unit's stale lines) or not (they stay in the XCD's own L2).  reuse: the same 1 KB every round
// (a stale line in the consumer's caches then shows as a mismatch) or a fresh one.  Times in units of the 100 MHz
// constant clock, summed over rounds.
struct HandoverResult {
    unsigned long long store_ack, atomic_rtt, load_lat, mismatches, timeouts, xcc_prod, xcc_cons;
};

__global__ __launch_bounds__(64) void handover_kernel(int stride, int npairs, int store_sc1, int load_sc1, int reuse, int iters,
                                                      u32x4 *data, unsigned *flags, unsigned *acks, HandoverResult *res)
{
    extern __shared__ unsigned char occupy_the_cu[];
    const int wg = blockIdx.x, lane = threadIdx.x;
    // pairs tile the grid in groups of 2 * stride workgroups: the first `stride` produce, the next `stride` consume
    const int grp = wg / (2 * stride), in = wg % (2 * stride);
    const int p = grp * stride + (in % stride);
    if (p >= npairs) return;
    const bool producer = in < stride;
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(xcc));
    unsigned *flag = flags + p * 64, *ack = acks + p * 64;
    unsigned long long t_st = 0, t_at = 0, t_ld = 0, mism = 0, tmo = 0;
    for (int it = 1; it <= iters; ++it) {
        u32x4 *d = data + ((size_t)p * (reuse ? 1 : iters) + (reuse ? 0 : it - 1)) * 64 + lane;
        const unsigned want = (unsigned)it * 2654435761u + (unsigned)p;
        if (producer) {
            const u32x4 v = u32x4{want, want ^ 1u, want ^ 2u, want + (unsigned)lane};
            const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
            if (store_sc1) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" ::"v"(d), "v"(v) : "memory");
            else asm volatile("global_store_dwordx4 %0, %1, off\n\ts_waitcnt vmcnt(0)" ::"v"(d), "v"(v) : "memory");
            const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
            if (lane == 0) (void)__hip_atomic_fetch_add(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const unsigned long long t2 = __builtin_amdgcn_s_memrealtime();
            t_st += t1 - t0;
            t_at += t2 - t1;
            int spins = 0;
            unsigned a = 0;
            do {
                a = lane == 0 ? __hip_atomic_load(ack, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
                a = __shfl(a, 0);
            } while (a < (unsigned)it && ++spins < 1000000);
            if (a < (unsigned)it) { ++tmo; break; }
        } else {
            int spins = 0;
            unsigned f = 0;
            do {
                f = lane == 0 ? __hip_atomic_fetch_add(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
                f = __shfl(f, 0);
            } while (f < (unsigned)it && ++spins < 1000000);
            if (f < (unsigned)it) { ++tmo; break; }
            u32x4 v;
            const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
            if (load_sc1) asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(d) : "memory");
            else asm volatile("global_load_dwordx4 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(d) : "memory");
            const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
            t_ld += t1 - t0;
            if (v[0] != want || v[1] != (want ^ 1u) || v[2] != (want ^ 2u) || v[3] != want + (unsigned)lane) ++mism;
            if (lane == 0) __hip_atomic_store(ack, (unsigned)it, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    unsigned long long m_all = mism;
    for (int o = 32; o; o >>= 1) m_all += __shfl_xor(m_all, o);
    if (lane == 0) {
        HandoverResult *r = res + p;
        if (producer) { r->store_ack = t_st; r->atomic_rtt = t_at; r->xcc_prod = xcc; }
        else { r->load_lat = t_ld; r->mismatches = m_all; r->xcc_cons = xcc; }
        if (tmo) atomicAdd(&r->timeouts, tmo);
    }
}

// out[0..5]: mean store-acknowledge, atomic round trip and load latency in nanoseconds per round, mismatching 16-byte
// pieces, rounds given up, pairs whose two workgroups ran on one XCD.  Allocates and frees its own buffers; synchronises.
hipError_t run_handover_yardstick(int stride, int npairs, int store_sc1, int load_sc1, int reuse, int iters, hipStream_t stream, double *out)
{
    const int groups = (npairs + stride - 1) / stride, grid = groups * 2 * stride;
    u32x4 *data = nullptr;
    unsigned *flags = nullptr, *acks = nullptr;
    HandoverResult *res = nullptr;
    const size_t data_bytes = (size_t)npairs * (reuse ? 1 : iters) * 1024;
    hipError_t e;
    if ((e = hipMalloc(&data, data_bytes)) != hipSuccess) return e;
    if ((e = hipMalloc(&flags, (size_t)npairs * 256)) == hipSuccess && (e = hipMalloc(&acks, (size_t)npairs * 256)) == hipSuccess &&
        (e = hipMalloc(&res, (size_t)npairs * sizeof(HandoverResult))) == hipSuccess &&
        (e = hipMemsetAsync(data, 0, data_bytes, stream)) == hipSuccess && (e = hipMemsetAsync(flags, 0, (size_t)npairs * 256, stream)) == hipSuccess &&
        (e = hipMemsetAsync(acks, 0, (size_t)npairs * 256, stream)) == hipSuccess &&
        (e = hipMemsetAsync(res, 0, (size_t)npairs * sizeof(HandoverResult), stream)) == hipSuccess &&
        (e = hipFuncSetAttribute(reinterpret_cast<const void *>(handover_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024)) == hipSuccess) {
        // 100 KB of LDS per workgroup: one workgroup per compute unit, so that all pairs are resident together
        hipLaunchKernelGGL(handover_kernel, dim3((unsigned)grid), dim3(64), 100 * 1024, stream, stride, npairs, store_sc1, load_sc1, reuse, iters,
                           data, flags, acks, res);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(stream);
        if (e == hipSuccess) {
            HandoverResult *h = new HandoverResult[npairs];
            e = hipMemcpy(h, res, (size_t)npairs * sizeof(HandoverResult), hipMemcpyDeviceToHost);
            double st = 0, at = 0, ld = 0, mm = 0, to = 0, same = 0;
            for (int i = 0; i < npairs; ++i) {
                st += (double)h[i].store_ack; at += (double)h[i].atomic_rtt; ld += (double)h[i].load_lat;
                mm += (double)h[i].mismatches; to += (double)h[i].timeouts; same += h[i].xcc_prod == h[i].xcc_cons ? 1.0 : 0.0;
            }
            const double den = (double)npairs * iters;
            out[0] = st / den * 10.0; out[1] = at / den * 10.0; out[2] = ld / den * 10.0; out[3] = mm; out[4] = to; out[5] = same;
            delete[] h;
        }
    }
    (void)hipFree(data);
    if (flags) (void)hipFree(flags);
    if (acks) (void)hipFree(acks);
    if (res) (void)hipFree(res);
    return e;
}

// variant: 0 nontemporal x8 (default), 1 plain x8, 2 nontemporal x16, 3 plain x16, 4 nontemporal x4, 5 plain x4
hipError_t launch_read(const void *src, void *sink, size_t bytes, int blocks, int variant, hipStream_t stream)
{
    const size_t n16 = bytes / 16;
    if (blocks <= 0) blocks = 256 * 8;
    const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
    uint32_t *k = reinterpret_cast<uint32_t *>(sink);
    const dim3 grid((unsigned)blocks), block(256);
    switch (variant) {
    case 0: hipLaunchKernelGGL((read_kernel<8, true>), grid, block, 0, stream, s, k, n16); break;
    case 1: hipLaunchKernelGGL((read_kernel<8, false>), grid, block, 0, stream, s, k, n16); break;
    case 2: hipLaunchKernelGGL((read_kernel<16, true>), grid, block, 0, stream, s, k, n16); break;
    case 3: hipLaunchKernelGGL((read_kernel<16, false>), grid, block, 0, stream, s, k, n16); break;
    case 4: hipLaunchKernelGGL((read_kernel<4, true>), grid, block, 0, stream, s, k, n16); break;
    case 5: hipLaunchKernelGGL((read_kernel<4, false>), grid, block, 0, stream, s, k, n16); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---- unit rates: what the matrix cores and the LDS of this device deliver to the access patterns the
// many-token kernel uses, measured the way the read kernel measures HBM --------------------------------
typedef float rate_f32x16 __attribute__((ext_vector_type(16)));
typedef float rate_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t rate_u32x2 __attribute__((ext_vector_type(2)));
constexpr int kRateIters = 4096;

// Independent MFMAs back to back, nothing else: NACC accumulators per wave, 4 waves per workgroup.  RANDOM: the
// operands are four + four registers of pseudo-random fp16 values in (-1, 1) instead of one pair of small
// regular numbers - what the matrix cores draw, and the clock they are then given, depends on the bits that toggle.
template <bool M32, int NACC, bool RANDOM = false>
__global__ __launch_bounds__(256) void mfma_rate_kernel(uint32_t *sink)
{
    constexpr int NOP = RANDOM ? 4 : 1;
    f16x8 a[NOP], b[NOP];
#pragma unroll
    for (int o = 0; o < NOP; ++o)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if constexpr (RANDOM) {
                uint32_t h = (threadIdx.x * 8u + e + o * 4099u + blockIdx.x * 131071u) * 2654435761u;
                h ^= h >> 15, h *= 2246822519u, h ^= h >> 13;
                a[o][e] = (f16)((float)(int)(h & 0xffffu) * (1.0f / 32768.0f) - 1.0f);
                b[o][e] = (f16)((float)(int)(h >> 16) * (1.0f / 32768.0f) - 1.0f);
            } else {
                a[o][e] = (f16)(0.001f * (float)threadIdx.x + (float)e);
                b[o][e] = (f16)(0.5f * (float)e);
            }
        }
    float s = 0.f;
    if constexpr (M32) {
        rate_f32x16 acc[NACC];
#pragma unroll
        for (int i = 0; i < NACC; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < kRateIters; ++it)
#pragma unroll
            for (int i = 0; i < NACC; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(i >> 2) % NOP], b[i % NOP], acc[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < NACC; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][e];
    } else {
        rate_f32x4 acc[NACC];
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] = rate_f32x4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < kRateIters; ++it)
#pragma unroll
            for (int i = 0; i < NACC; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(i >> 2) % NOP], b[i % NOP], acc[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < NACC; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    }
    if (s == 12345.678f) sink[0] = 1u;  // practically never: keeps the chain alive
}

// LDS traffic of 8 (THREADS = 1024: 16) waves per CU, eight accesses per wave and iteration, addresses opaque to
// the compiler.
// MODE 0: 16-byte reads the way a wave reads an MFMA fragment from a tile of 128-byte rows (lane = row 0..15 x
// k-group, slot ^ (row & 7)); 1: 4-byte reads the way the decode reads the byte-pair table ((byte << 8) | (lane
// << 2), byte from a counter); 2: 16-byte writes the way the decoded weights are stored (4 rows x 8 k-blocks
// per 32 lanes); 3: the same bytes as two 8-byte writes each; 4: 16-byte writes at consecutive addresses; 5 / 6:
// the table reads of 1 with one copy of the table per 32 / 16 lanes and a pseudo-random byte per lane.
template <int MODE, int THREADS = 512>
__global__ __launch_bounds__(THREADS) void lds_rate_kernel(uint32_t *sink)
{
    extern __shared__ __align__(16) unsigned char smem[];
    for (int i = threadIdx.x; i < 65536 / 4; i += THREADS) reinterpret_cast<uint32_t *>(smem)[i] = (uint32_t)i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t s = 0;
    if constexpr (MODE == 0) {
        const int row = lane & 15, g = lane >> 4;
        const uint32_t base = (uint32_t)(row * 128 + ((g ^ (row & 7)) << 4) + wave * 4096);
        for (int it = 0; it < kRateIters; ++it)
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                uint32_t off = (base + r * 2048 + (it & 1) * 32768) & 65535u;
                asm volatile("" : "+v"(off));
                const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + off);
                s += v[0] ^ v[1] ^ v[2] ^ v[3];
            }
    } else if constexpr (MODE == 1) {
        for (int it = 0; it < kRateIters; ++it)
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                uint32_t off = ((uint32_t)((it * 8 + r + wave * 31) & 255) << 8) | ((uint32_t)lane << 2);
                asm volatile("" : "+v"(off));
                s += *reinterpret_cast<const uint32_t *>(smem + off);
            }
    } else if constexpr (MODE == 5 || MODE == 6) {
        constexpr int REP = MODE == 5 ? 32 : 16;  // lanes that have a copy of the table of their own
        for (int it = 0; it < kRateIters; ++it)
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                uint32_t off = ((uint32_t)(((it * 8 + r) * 37 + wave * 31 + lane * lane * 13 + (lane >> 3)) & 255) * (REP * 4)) | ((uint32_t)(lane % REP) << 2);
                asm volatile("" : "+v"(off));
                s += *reinterpret_cast<const uint32_t *>(smem + off);
            }
    } else if constexpr (MODE == 3) {
        const int half = lane & 1, kb = (lane >> 1) & 7, mbl = lane >> 4;
        rate_u32x2 v = {(uint32_t)threadIdx.x, 1u};
        for (int it = 0; it < kRateIters; ++it) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = mbl * 8 + half * 4 + ((r >> 1) & 3);
                uint32_t off = (uint32_t)(row * 128 + ((kb ^ (row & 7)) << 4) + (r & 1) * 8 + wave * 4096 + ((it + (r >> 3)) & 1) * 32768) & 65535u;
                asm volatile("" : "+v"(off));
                *reinterpret_cast<rate_u32x2 *>(smem + off) = v;
            }
            v[0] += 1u;
        }
        __syncthreads();
        s = smem[threadIdx.x];
    } else if constexpr (MODE == 4) {
        u32x4 v = {(uint32_t)threadIdx.x, 1u, 2u, 3u};
        for (int it = 0; it < kRateIters; ++it) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                uint32_t off = (uint32_t)(lane * 16 + r * 1024 + wave * 8192) & 65535u;
                asm volatile("" : "+v"(off));
                *reinterpret_cast<u32x4 *>(smem + off) = v;
            }
            v[0] += 1u;
        }
        __syncthreads();
        s = smem[threadIdx.x];
    } else {
        const int half = lane & 1, kb = (lane >> 1) & 7, mbl = lane >> 4;
        u32x4 v = {(uint32_t)threadIdx.x, 1u, 2u, 3u};
        for (int it = 0; it < kRateIters; ++it) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int row = mbl * 8 + half * 4 + (r & 3);
                uint32_t off = (uint32_t)(row * 128 + ((kb ^ (row & 7)) << 4) + wave * 4096 + ((it + (r >> 2)) & 1) * 32768) & 65535u;
                asm volatile("" : "+v"(off));
                *reinterpret_cast<u32x4 *>(smem + off) = v;
            }
            v[0] += 1u;
        }
        __syncthreads();
        s = smem[threadIdx.x];
    }
    if (s == 0x9e3779b9u && sink[1] == 77u) sink[0] = s;  // practically never
}

// The k-step of a 64-token streaming launch without its memory side, eight waves per CU: per wave and iteration
// sixteen table reads and four fragment reads from LDS and sixteen independent 16x16x32 MFMAs on pseudo-random
// operands.  MODE 0: the MFMAs only; 1: the LDS reads only; 2: both in every wave, the reads requested ahead of the
// MFMAs and used behind them; 3: waves 0-3 (one per SIMD) do the MFMAs of two waves, waves 4-7 the reads of two;
// 4: both in every wave, one or two reads requested behind each MFMA and used two iterations later.
// Whether 2 and 3 take the longer of 0 and 1 or their sum says whether a CU overlaps the two kinds of work.
constexpr int kMixedIters = 1024;
template <int MODE>
__global__ __launch_bounds__(512) void mixed_rate_kernel(uint32_t *sink)
{
    extern __shared__ __align__(16) unsigned char smem[];
    for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<uint32_t *>(smem)[i] = (uint32_t)i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    f16x8 a[4], b[4];
#pragma unroll
    for (int o = 0; o < 4; ++o)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            uint32_t h = (threadIdx.x * 8u + e + o * 4099u + blockIdx.x * 131071u) * 2654435761u;
            h ^= h >> 15, h *= 2246822519u, h ^= h >> 13;
            a[o][e] = (f16)((float)(int)(h & 0xffffu) * (1.0f / 32768.0f) - 1.0f);
            b[o][e] = (f16)((float)(int)(h >> 16) * (1.0f / 32768.0f) - 1.0f);
        }
    rate_f32x4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = rate_f32x4{0.f, 0.f, 0.f, 0.f};
    uint32_t s = 0;
    const bool do_mfma = MODE == 0 || MODE == 2 || (MODE == 3 && wave < 4);
    const bool do_lds = MODE == 1 || MODE == 2 || (MODE == 3 && wave >= 4);
    const int reps = MODE == 3 ? 2 : 1;
    for (int it = 0; it < (MODE == 4 ? 0 : kMixedIters); ++it)
        for (int rep = 0; rep < reps; ++rep) {
            uint32_t t[16];
            u32x4 f[4];
            if (do_lds) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    uint32_t off = ((uint32_t)((it * 16 + r + wave * 31 + rep * 7) & 255) << 8) | ((uint32_t)lane << 2);
                    asm volatile("" : "+v"(off));
                    t[r] = *reinterpret_cast<const uint32_t *>(smem + off);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    uint32_t off = (uint32_t)(lane * 16 + r * 1024 + wave * 4096 + ((it + rep) & 1) * 32768) & 65535u;
                    asm volatile("" : "+v"(off));
                    f[r] = *reinterpret_cast<const u32x4 *>(smem + off);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (do_mfma) {
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i >> 2], b[i & 3], acc[i], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (do_lds) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s += t[r];
#pragma unroll
                for (int r = 0; r < 4; ++r) s += f[r][0] ^ f[r][1] ^ f[r][2] ^ f[r][3];
            }
        }
    if constexpr (MODE == 4) {
        // the reads of an iteration are requested between its MFMAs, one or two behind each, and used at the end of
        // the next iteration (two register sets take turns: a copy would wait for the reads it copies)
        uint32_t t[2][16];
        u32x4 f[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int r = 0; r < 16; ++r) t[h][r] = 0u;
#pragma unroll
            for (int r = 0; r < 4; ++r) f[h][r] = u32x4{0u, 0u, 0u, 0u};
        }
        for (int it = 0; it < kMixedIters; it += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s += t[h][r];  // (requested an iteration ago... or two, for h = 0 of the first turn: zeros)
#pragma unroll
                for (int r = 0; r < 4; ++r) s += f[h][r][0] ^ f[h][r][1] ^ f[h][r][2] ^ f[h][r][3];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i >> 2], b[i & 3], acc[i], 0, 0, 0);
                    uint32_t off = ((uint32_t)(((it + h) * 16 + i + wave * 31) & 255) << 8) | ((uint32_t)lane << 2);
                    asm volatile("" : "+v"(off));
                    t[h][i] = *reinterpret_cast<const uint32_t *>(smem + off);
                    if (i < 4) {
                        uint32_t off2 = (uint32_t)(lane * 16 + i * 1024 + wave * 4096 + h * 32768) & 65535u;
                        asm volatile("" : "+v"(off2));
                        f[h][i] = *reinterpret_cast<const u32x4 *>(smem + off2);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // a table read and a fragment read
                }
#pragma unroll
                for (int i = 4; i < 16; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += t[h][r];
    }
    float fs = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) fs += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if ((s == 0x9e3779b9u && sink[1] == 77u) || fs == 12345.678f) sink[0] = s;  // practically never
}

// unit: 0 / 1 v_mfma_f32_16x16x32_f16 with one / two waves per SIMD (16 accumulators), 2 v_mfma_f32_32x32x16_f16
// (one wave per SIMD, 4 accumulators); 3 LDS fragment reads, 4 LDS table reads, 5 LDS tile writes, 6 the tile
// writes as 8-byte halves, 7 16-byte writes at consecutive addresses, 8 / 9 table reads with a copy of the table
// per 32 / 16 lanes; 10 / 13 32x32x16 and 12 / 11 16x16x32 MFMAs on pseudo-random operands from one / two waves per
// SIMD; 14 / 15 / 16: units 4 / 3 / 5 from 16 waves per compute unit; 17..21: mixed_rate_kernel<0..4>.  *work = flops
// (0..2, 10..13, 17..21: those of the MFMAs of modes 0, 2 and 3, also for mode 1, which has none - the four times
// are what is compared) or bytes (3..9, 14..16) of one launch on `cus` compute units.
hipError_t launch_unit_rate(int unit, int cus, uint32_t *sink, double *work, hipStream_t stream)
{
    static OptInFlag attr[16][15];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    switch (unit) {
    case 0: hipLaunchKernelGGL((mfma_rate_kernel<false, 16>), dim3(cus), dim3(256), 0, stream, sink); *work = (double)cus * 4 * kRateIters * 16 * 16384.0; break;
    case 1: hipLaunchKernelGGL((mfma_rate_kernel<false, 16>), dim3(2 * cus), dim3(256), 0, stream, sink); *work = (double)cus * 8 * kRateIters * 16 * 16384.0; break;
    case 2: hipLaunchKernelGGL((mfma_rate_kernel<true, 4>), dim3(cus), dim3(256), 0, stream, sink); *work = (double)cus * 4 * kRateIters * 4 * 32768.0; break;
    case 3:
        if ((e = ensure_lds_opt_in(attr[dev][0], reinterpret_cast<const void *>(lds_rate_kernel<0>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<0>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 16.0; break;
    case 4:
        if ((e = ensure_lds_opt_in(attr[dev][1], reinterpret_cast<const void *>(lds_rate_kernel<1>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<1>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 4.0; break;
    case 5:
        if ((e = ensure_lds_opt_in(attr[dev][2], reinterpret_cast<const void *>(lds_rate_kernel<2>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<2>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 16.0; break;
    case 6:
        if ((e = ensure_lds_opt_in(attr[dev][3], reinterpret_cast<const void *>(lds_rate_kernel<3>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<3>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 16.0; break;
    case 7:
        if ((e = ensure_lds_opt_in(attr[dev][4], reinterpret_cast<const void *>(lds_rate_kernel<4>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<4>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 16.0; break;
    case 10: hipLaunchKernelGGL((mfma_rate_kernel<true, 16, true>), dim3(cus), dim3(256), 0, stream, sink); *work = (double)cus * 4 * kRateIters * 16 * 32768.0; break;
    case 11: hipLaunchKernelGGL((mfma_rate_kernel<false, 16, true>), dim3(2 * cus), dim3(256), 0, stream, sink); *work = (double)cus * 8 * kRateIters * 16 * 16384.0; break;
    case 12: hipLaunchKernelGGL((mfma_rate_kernel<false, 16, true>), dim3(cus), dim3(256), 0, stream, sink); *work = (double)cus * 4 * kRateIters * 16 * 16384.0; break;
    case 13: hipLaunchKernelGGL((mfma_rate_kernel<true, 16, true>), dim3(2 * cus), dim3(256), 0, stream, sink); *work = (double)cus * 8 * kRateIters * 16 * 32768.0; break;
    case 14:
        if ((e = ensure_lds_opt_in(attr[dev][7], reinterpret_cast<const void *>(lds_rate_kernel<1, 1024>))) != hipSuccess) return e;
        hipLaunchKernelGGL((lds_rate_kernel<1, 1024>), dim3(cus), dim3(1024), 65536, stream, sink); *work = (double)cus * 1024 * kRateIters * 8 * 4.0; break;
    case 15:
        if ((e = ensure_lds_opt_in(attr[dev][8], reinterpret_cast<const void *>(lds_rate_kernel<0, 1024>))) != hipSuccess) return e;
        hipLaunchKernelGGL((lds_rate_kernel<0, 1024>), dim3(cus), dim3(1024), 65536, stream, sink); *work = (double)cus * 1024 * kRateIters * 8 * 16.0; break;
    case 16:
        if ((e = ensure_lds_opt_in(attr[dev][9], reinterpret_cast<const void *>(lds_rate_kernel<2, 1024>))) != hipSuccess) return e;
        hipLaunchKernelGGL((lds_rate_kernel<2, 1024>), dim3(cus), dim3(1024), 65536, stream, sink); *work = (double)cus * 1024 * kRateIters * 8 * 16.0; break;
    case 17:
        if ((e = ensure_lds_opt_in(attr[dev][10], reinterpret_cast<const void *>(mixed_rate_kernel<0>))) != hipSuccess) return e;
        hipLaunchKernelGGL(mixed_rate_kernel<0>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 8 * kMixedIters * 16 * 16384.0; break;
    case 18:
        if ((e = ensure_lds_opt_in(attr[dev][11], reinterpret_cast<const void *>(mixed_rate_kernel<1>))) != hipSuccess) return e;
        hipLaunchKernelGGL(mixed_rate_kernel<1>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 8 * kMixedIters * 16 * 16384.0; break;
    case 19:
        if ((e = ensure_lds_opt_in(attr[dev][12], reinterpret_cast<const void *>(mixed_rate_kernel<2>))) != hipSuccess) return e;
        hipLaunchKernelGGL(mixed_rate_kernel<2>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 8 * kMixedIters * 16 * 16384.0; break;
    case 20:
        if ((e = ensure_lds_opt_in(attr[dev][13], reinterpret_cast<const void *>(mixed_rate_kernel<3>))) != hipSuccess) return e;
        hipLaunchKernelGGL(mixed_rate_kernel<3>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 8 * kMixedIters * 16 * 16384.0; break;
    case 21:
        if ((e = ensure_lds_opt_in(attr[dev][14], reinterpret_cast<const void *>(mixed_rate_kernel<4>))) != hipSuccess) return e;
        hipLaunchKernelGGL(mixed_rate_kernel<4>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 8 * kMixedIters * 16 * 16384.0; break;
    case 8:
        if ((e = ensure_lds_opt_in(attr[dev][5], reinterpret_cast<const void *>(lds_rate_kernel<5>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<5>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 4.0; break;
    case 9:
        if ((e = ensure_lds_opt_in(attr[dev][6], reinterpret_cast<const void *>(lds_rate_kernel<6>))) != hipSuccess) return e;
        hipLaunchKernelGGL(lds_rate_kernel<6>, dim3(cus), dim3(512), 65536, stream, sink); *work = (double)cus * 512 * kRateIters * 8 * 4.0; break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_copy(const void *src, void *dst, size_t bytes, hipStream_t stream)
{
    const size_t n16 = bytes / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4 *>(src), reinterpret_cast<u32x4 *>(dst), n16);
    return hipGetLastError();
}

// Self-test of div_by_block_max: every pair of fp16 values (w, a) with a > 0 finite and |w| <= a,
// against the IEEE division (zeros of either sign count as equal).  One workgroup per value of a;
// counts[0] += pairs, counts[1] += mismatches.
__global__ __launch_bounds__(256) void division_selftest_kernel(unsigned long long *counts)
{
    const uint16_t abits = (uint16_t)(blockIdx.x + 1);  // 0x0001 .. 0x7bff: every positive finite fp16
    const float a = (float)__builtin_bit_cast(f16, abits);
    const float y = refined_rcp(a);
    unsigned long long n = 0, bad = 0;
    for (uint32_t wb = threadIdx.x; wb < 65536u; wb += 256u) {
        const uint16_t mag = (uint16_t)(wb & 0x7fffu);
        if (mag > abits) continue;  // |w| > a, infinities, NaNs
        const float w = (float)__builtin_bit_cast(f16, (uint16_t)wb);
        const float got = div_by_block_max(w, a, y), want = __fdiv_rn(w, a);
        ++n;
        // (a zero quotient may come out with the other sign: -0 / a is -0, the correction step gives +0;
        // every later use of the quotient is a comparison or a difference, where the two are one value)
        const bool same = __builtin_bit_cast(uint32_t, got) == __builtin_bit_cast(uint32_t, want) || (got == 0.f && want == 0.f);
        bad += same ? 0u : 1u;
    }
    atomicAdd(counts, n);
    if (bad) atomicAdd(counts + 1, bad);
}

hipError_t launch_division_selftest(unsigned long long *counts, hipStream_t stream)
{
    hipLaunchKernelGGL(division_selftest_kernel, dim3(0x7bff), dim3(256), 0, stream, counts);
    return hipGetLastError();
}

}  // namespace tuna
