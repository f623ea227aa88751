// Packed 4-bit weights -> fp16 [m, k] row-major, for gfx950.
//
// Replaces dequantize_4bit / dequantize_wrapper (kernel.cu:3158-3253).  The op is a
// pure stream (k*m/2 bytes in, 2*k*m bytes out), so the design is about HBM
// transactions only:
//   * a wave reads 1 KB of one block row with one global_load_dwordx4 per lane
//     (lane l: block column kb0 + l/2, rows 4*(l%2) .. +3), nontemporal;
//   * a dword is one weight row x 8 consecutive k, i.e. 16 bytes of output; lanes of
//     equal parity write 512 contiguous bytes per output row, nontemporal.  No LDS
//     transpose is needed (the reference needs one because its lanes own single bytes,
//     kernel.cu:3218-3240);
//   * decode: 16-entry fp32 (or fp16) table in LDS - all lanes hit 16 dwords in 16
//     distinct banks, equal addresses broadcast, so it is conflict free - then
//     fp32 multiply + round (TUNA_DECODE_DEQUANT, kernel.cu:3222-3228) or an fp16
//     multiply (TUNA_DECODE_GEMM, kernel.cu:2178-2192).
#include "tuna_internal.h"
#include "quantize_div.hpp"

#include <type_traits>

namespace tuna {

typedef _Float16 f16;
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kDqUnroll = 4;  // 1 KB chunks per wave

// BLK: one scale per `bs` consecutive weights of a row, absmax [m, k/bs] (the layout the reference's
// quantizer writes for block_size < k, test.py:15-17); otherwise one scale per row.
template <int DEC, bool BLK>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ q,
                                                      const float *__restrict__ absmax,
                                                      const float *__restrict__ code,
                                                      f16 *__restrict__ out, int m, int k, int bs)
{
    __shared__ float cf[16];
    __shared__ f16 ch[16];
    const int tid = threadIdx.x;
    if (tid < 16) {
        cf[tid] = code[tid];
        ch[tid] = (f16)code[tid];
    }
    __syncthreads();
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int kb_total = k >> 3;
    const int mb = blockIdx.y * 4 + wave;
    if (mb >= (m >> 3)) return;
    const int half = lane & 1;
    const int kb_lane = blockIdx.x * (32 * kDqUnroll) + (lane >> 1);
    const int nblk = BLK ? k / bs : 1;

    float s32[4];
    f16 s16[4];
    if constexpr (!BLK) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s32[j] = absmax[mb * 8 + half * 4 + j];
            s16[j] = (f16)s32[j];
        }
    }
    const uint8_t *src = q + ((size_t)mb * kb_total) * 32 + half * 16;
    u32x4 w[kDqUnroll];
#pragma unroll
    for (int u = 0; u < kDqUnroll; ++u) {
        const int kb = kb_lane + u * 32;
        if (kb < kb_total) w[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (size_t)kb * 32));
    }
#pragma unroll
    for (int u = 0; u < kDqUnroll; ++u) {
        const int kb = kb_lane + u * 32;
        if (kb >= kb_total) continue;
        if constexpr (BLK) {
            const int blk = (kb * 8) / bs;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                s32[j] = absmax[(size_t)(mb * 8 + half * 4 + j) * nblk + blk];
                s16[j] = (f16)s32[j];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t d = w[u][j];
            f16x8 r;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                // column e of the row sits at bit 8*(e/2) + 4*(1 - e%2)  (test.py:58-65)
                const uint32_t nib = (d >> (8 * (e >> 1) + 4 * (1 - (e & 1)))) & 15u;
                if constexpr (DEC == TUNA_DECODE_DEQUANT) r[e] = (f16)(cf[nib] * s32[j]);
                else r[e] = ch[nib] * s16[j];
            }
            f16 *dst = out + (size_t)(mb * 8 + half * 4 + j) * k + (size_t)kb * 8;
            __builtin_nontemporal_store(r, reinterpret_cast<f16x8 *>(dst));
        }
    }
}

hipError_t launch_dequant(const uint8_t *q, const float *absmax, const float *code, void *out,
                          int m, int k, int bs, int decode, hipStream_t stream)
{
    const int kb_total = k >> 3;
    dim3 grid((kb_total + 32 * kDqUnroll - 1) / (32 * kDqUnroll), ((m >> 3) + 3) / 4, 1);
    f16 *o = reinterpret_cast<f16 *>(out);
    if (bs == k) {
        if (decode == TUNA_DECODE_DEQUANT)
            hipLaunchKernelGGL((dequant_kernel<TUNA_DECODE_DEQUANT, false>), grid, dim3(256), 0, stream, q, absmax, code, o, m, k, bs);
        else
            hipLaunchKernelGGL((dequant_kernel<TUNA_DECODE_GEMM, false>), grid, dim3(256), 0, stream, q, absmax, code, o, m, k, bs);
    } else {
        if (decode == TUNA_DECODE_DEQUANT)
            hipLaunchKernelGGL((dequant_kernel<TUNA_DECODE_DEQUANT, true>), grid, dim3(256), 0, stream, q, absmax, code, o, m, k, bs);
        else
            hipLaunchKernelGGL((dequant_kernel<TUNA_DECODE_GEMM, true>), grid, dim3(256), 0, stream, q, absmax, code, o, m, k, bs);
    }
    return hipGetLastError();
}

// fp16 weights [m, k] -> packed 4-bit codes + absmax: the device form of the reference harness's
// quantize_blockwise_dynamic_4bit (test.py:7-68).  Same arithmetic: absmax = max |w| over a block of
// `bs` consecutive weights of a row as fp32 (bs == k: one scale per row, what the kernels of the
// reference run); normalized = fp32(w) / absmax with an fp32 division (test.py:41, fp16 / fp32
// promotes to fp32); index = argmin_j |normalized - code[j]| in fp32, first index on ties
// (torch.argmin, test.py:50-53); nibble packing of test.py:55-65.  A block of zeros gets index 0: the
// reference divides by zero there, every candidate distance is NaN, and torch.argmin over an all-NaN
// column returns index 0.
//
// One workgroup per block row (8 weight rows), 64 threads per row, 16-byte reads (a row's threads
// read 1 KB contiguous).  NP > 0: the whole row (k <= 512*NP) is read once into registers, all
// loads in flight together, so the op streams the weights exactly once; NP == 0: two passes (the
// second mostly from cache).  Block maxima come from shuffles inside the row's 64 threads.  For a
// codebook that is sorted with gaps wide enough that fp32 rounding cannot reorder distances, the
// nearest entry is found by a 4-step binary search over the 15 decision boundaries between
// neighbouring entries (each the smallest fp32 value the argmin gives to the upper entry, found by
// bisection with the argmin's own arithmetic once per workgroup) - the argmin's result, since
// |nv - c| is monotonic in c on either side of nv; any other codebook takes the 16 comparisons.
// The division by the block maximum is a multiply by its refined reciprocal and one fused correction.  A thread's dword (one row, 8
// consecutive k) is written through a 2 KB LDS tile so that the stores are 16 bytes per lane and
// contiguous (the records of 64 block columns), not 4 bytes at a stride of 32.
// Nearest entry of a sorted codebook: bnd[i] (i = 0..14) is the smallest binary32 value that the
// argmin assigns to entry i + 1 rather than entry i, so the index is the number of boundaries <= nv:
// a 4-step binary search, as a tree of selects over the 15 values (uniform, held in registers).
__device__ __forceinline__ uint32_t nearest_sorted(float nv, const float (&b)[16])
{
    const bool b3 = nv >= b[7];
    const float t2 = b3 ? b[11] : b[3];
    const float u3 = b3 ? b[13] : b[5], v3 = b3 ? b[9] : b[1];
    const float p4 = b3 ? b[14] : b[6], q4 = b3 ? b[12] : b[4], r4 = b3 ? b[10] : b[2], s4 = b3 ? b[8] : b[0];
    const bool b2 = nv >= t2;
    const float t3 = b2 ? u3 : v3;
    const float x4 = b2 ? p4 : r4, y4 = b2 ? q4 : s4;
    const bool b1 = nv >= t3;
    const float t4 = b1 ? x4 : y4;
    const bool b0 = nv >= t4;
    return (b3 ? 8u : 0u) + (b2 ? 4u : 0u) + (b1 ? 2u : 0u) + (b0 ? 1u : 0u);  // a NaN nv ends at 0 like the argmin
}

// The same count of boundaries <= nv without the search: the quotients lie in [-1, 1], cut into 64 buckets
// of 1/32; when no two boundaries share a bucket, a bucket knows how many boundaries lie below it and the one
// boundary (if any) inside it, and the index is that count plus one comparison.  bucket_of is monotonic in
// nv (a fused multiply-add, a clamp, a truncation), so every value of a lower bucket is below the boundary
// of a higher one and vice versa: the result is the binary search's for every nv, NaN included (bucket 0, the
// comparison false, index 0).  One LDS table of {boundary, count} pairs in the lane-private layout of the
// GEMM's decode table (entry e of lane l at (e << 9) | (l << 3): one 8-byte read, no bank conflicts whatever
// the data).
constexpr int kQuantBuckets = 65;
constexpr int kQuantTabBytes = kQuantBuckets * 512;  // per bucket and lane: fp32 boundary (+inf if none), boundaries below it
typedef __attribute__((address_space(3))) unsigned char lds_u8;
typedef uint32_t quant_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) quant_u32x2 lds_pair;

__device__ __forceinline__ uint32_t bucket_of(float nv)
{
    return (uint32_t)__builtin_amdgcn_fmed3f(__builtin_fmaf(nv, 32.0f, 32.0f), 0.0f, 64.0f);
}

__device__ __forceinline__ uint32_t nearest_bucketed(float nv, uint32_t tab_lane)
{
    const uint32_t e = bucket_of(nv);
    const quant_u32x2 t = *reinterpret_cast<const lds_pair *>((uintptr_t)((e << 9) + tab_lane));
    const uint32_t bnd_bits = t[0], below = t[1];
    return below + (nv >= __builtin_bit_cast(float, bnd_bits) ? 1u : 0u);
}

__device__ __forceinline__ uint32_t nearest_any(float nv, const float (&c)[16])
{
    float bd = fabsf(__fsub_rn(nv, c[0]));
    uint32_t best = 0;
#pragma unroll
    for (int i = 1; i < 16; ++i) {
        const float dd = fabsf(__fsub_rn(nv, c[i]));
        if (dd < bd) {
            bd = dd;
            best = i;
        }
    }
    return best;
}

// Smallest binary32 v in [lo, hi] for which the argmin prefers hi: |v - hi| < |v - lo| in fp32
// arithmetic (ties keep the lower index).  The predicate is monotonic in v (both rounded differences
// are), so a bisection over the bit patterns finds it; lo < hi finite, and it holds at v = hi.  Two probes
// 64 patterns either side of the rounded midpoint come first: the boundary lies between them unless the
// midpoint is tiny against the gap, and the bisection then takes 7 steps instead of 31.
__device__ inline float decision_boundary(float lo, float hi)
{
    auto key = [](float f) {  // order-preserving map of finite floats to integers (both zeros -> 0)
        const int32_t i = __builtin_bit_cast(int32_t, f);
        return i < 0 ? -(i & 0x7fffffff) : i;
    };
    auto unkey = [](int32_t k) {
        const uint32_t i = k < 0 ? (uint32_t)(-k) | 0x80000000u : (uint32_t)k;
        return __builtin_bit_cast(float, i);
    };
    auto prefers_hi = [&](int32_t kv) {
        const float v = unkey(kv);
        return fabsf(__fsub_rn(v, hi)) < fabsf(__fsub_rn(v, lo));
    };
    int32_t a = key(lo), b = key(hi);  // predicate false at a (distance 0 to lo), true at b; b - a < 2^32
    const int32_t mid0 = key(0.5f * lo + 0.5f * hi);
#pragma unroll
    for (int side = -1; side <= 1; side += 2) {
        const int64_t want = (int64_t)mid0 + side * 64;
        if (want > (int64_t)a && want < (int64_t)b) {
            const int32_t p = (int32_t)want;
            if (prefers_hi(p)) b = p;
            else a = p;
        }
    }
    while ((uint32_t)b - (uint32_t)a > 1u) {
        const int32_t mid = (int32_t)((uint32_t)a + (((uint32_t)b - (uint32_t)a) >> 1));
        if (prefers_hi(mid)) b = mid;
        else a = mid;
    }
    return unkey(b);
}

// max(acc, |t|) over eight fp16 values, two at a time: the magnitudes are the bit patterns with the sign
// cleared, packed maxima never round, and the conversion to fp32 at the end is exact - the maximum the
// reference forms in fp32, at one instruction per weight.  (NaN is skipped by either form of the maximum.)
typedef f16 quant_f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ quant_f16x2 pk_absmax8(quant_f16x2 acc, f16x8 t)
{
    const u32x4 b = __builtin_bit_cast(u32x4, t) & 0x7fff7fffu;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t pair = b[i];  // (a bit_cast of the vector element itself reads element 0)
        acc = __builtin_elementwise_max(acc, __builtin_bit_cast(quant_f16x2, pair));
    }
    return acc;
}
__device__ __forceinline__ float pk_absmax_value(quant_f16x2 acc) { return fmaxf((float)acc[0], (float)acc[1]); }

template <int NP>
__global__ __launch_bounds__(512, NP == 16 ? 2 : 4) void quantize_kernel(const f16 *__restrict__ w, const float *__restrict__ code,
                                                       uint32_t *__restrict__ q32, float *__restrict__ absmax, int m, int k,
                                                       int bs)
{
    __shared__ float cs[16], bs_[15];
    __shared__ int fast_s, tab_s, jb_s[15];
    __shared__ uint32_t pair_s[kQuantBuckets][2];
    extern __shared__ __align__(16) unsigned char qtab[];  // bucket table
    constexpr int TPR = 64;  // threads per weight row: a row's threads read 1 KB contiguous
    // records of the block row being assembled: [step][block column of the step (64)][row (8)] - all NP steps
    // of a row held in registers (one barrier per block row), or two buffers of one step each (NP == 0)
    __shared__ __align__(16) uint32_t tile[NP > 0 ? NP : 2][TPR * 8];
    const int tid = threadIdx.x;
    if (tid < 16) cs[tid] = code[tid];
    __syncthreads();
    if (tid == 0) {
        // sorted, and every gap far above the rounding of a difference (|nv| <= 1, so a difference is
        // at most 1 + max|c| and its rounding error below 2^-23 of that)
        float cmax = fmaxf(fabsf(cs[0]), fabsf(cs[15]));
        const float thr = (1.0f + cmax) * 9.5367431640625e-7f;  // 2^-20
        int ok = 1;
        for (int i = 0; i < 15; ++i) ok &= (cs[i + 1] - cs[i] >= thr) ? 1 : 0;
        fast_s = ok && cmax < 3.0e38f;
    }
    __syncthreads();
    const bool fast = fast_s != 0;
    if (fast && tid < 15) bs_[tid] = decision_boundary(cs[tid], cs[tid + 1]);
    __syncthreads();
    // bucket tables, if every boundary is finite and has a bucket of its own
    if (tid == 0) {
        int ok = fast ? 1 : 0;
        for (int i = 0; i < 15 && ok; ++i) {
            jb_s[i] = (int)bucket_of(bs_[i]);
            ok &= (fabsf(bs_[i]) < 3.0e38f) && (i == 0 || jb_s[i] > jb_s[i - 1]) ? 1 : 0;
        }
        tab_s = ok;
    }
    __syncthreads();
    const bool tabled = tab_s != 0;
    const uint32_t tab0 = (uint32_t)(uintptr_t)(lds_u8 *)qtab;
    const uint32_t tab_lane = tab0 + ((uint32_t)(tid & 63) << 3);
    if (tabled) {
        if (tid < kQuantBuckets) {  // a bucket's pair: its boundary (+inf: none) and the boundaries below it
            float b = __builtin_inff();
            uint32_t n = 0;
#pragma unroll
            for (int i = 0; i < 15; ++i) {
                b = jb_s[i] == tid ? bs_[i] : b;
                n += jb_s[i] < tid ? 1u : 0u;
            }
            pair_s[tid][0] = __builtin_bit_cast(uint32_t, b);
            pair_s[tid][1] = n;
        }
        __syncthreads();
        for (int p = tid; p < kQuantTabBytes / 16; p += 512) {  // 32 stores of 16 bytes (two lanes' pairs) per bucket
            const uint32_t u = pair_s[p >> 5][0], n = pair_s[p >> 5][1];
            reinterpret_cast<u32x4 *>(qtab)[p] = u32x4{u, n, u, n};
        }
    }
    __syncthreads();

    // The block rows, with the nearest-entry rule as a compile-time choice (the three loops share nothing
    // but their registers: the table path must not carry the 15 boundaries of the search).  MODE 0: bucket
    // tables; 1: binary search over the boundaries; 2: the 16 comparisons.
    auto run = [&](auto mode_tag) {
    constexpr int MODE = decltype(mode_tag)::value;
    float c[16];  // MODE 1: the boundaries; MODE 2: the codebook
#pragma unroll
    for (int i = 0; i < 16; ++i) c[i] = MODE == 1 ? (i < 15 ? bs_[i] : 0.f) : MODE == 2 ? cs[i] : 0.f;
    constexpr bool AHEAD = NP > 0 && NP <= 8;
    f16x8 v[NP > 0 ? NP : 1];
    for (int mb = blockIdx.x; mb < (m >> 3); mb += gridDim.x) {
    const int r8 = tid / TPR, j = tid % TPR;
    const int row = mb * 8 + r8;
    const int kb_total = k >> 3;
    const int n_steps = (kb_total + TPR - 1) / TPR;  // steps of 64 block columns
    const f16 *src = w + (size_t)row * k;
    const bool by_row = bs == k;
    const int lanes_blk = by_row ? TPR : bs >> 3;  // threads that share a scale (a power of two <= 32)
    const int nblk = k / bs;

    float row_max = 0.f;
    if constexpr (NP > 0) {
        if (!AHEAD || mb == (int)blockIdx.x) {
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int kb = i * TPR + j;
                v[i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                if (kb < kb_total) v[i] = *reinterpret_cast<const f16x8 *>(src + (size_t)kb * 8);
            }
        }
    }
    // the next block row's weights are requested before this one's arithmetic (registers for both up to NP = 8)
    f16x8 vn[AHEAD ? NP : 1];
    if constexpr (AHEAD) {
        if (mb + (int)gridDim.x < (m >> 3)) {
            const f16 *srcn = src + (size_t)gridDim.x * 8 * k;
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int kb = i * TPR + j;
                vn[i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                if (kb < kb_total) vn[i] = *reinterpret_cast<const f16x8 *>(srcn + (size_t)kb * 8);
            }
        }
    }
    if (by_row) {
        quant_f16x2 pm = quant_f16x2{(f16)0.f, (f16)0.f};
        if constexpr (NP > 0) {
#pragma unroll
            for (int i = 0; i < NP; ++i) pm = pk_absmax8(pm, v[i]);
        } else {
            for (int kb = j; kb < kb_total; kb += TPR) pm = pk_absmax8(pm, *reinterpret_cast<const f16x8 *>(src + (size_t)kb * 8));
        }
        row_max = pk_absmax_value(pm);
#pragma unroll
        for (int off = TPR / 2; off >= 1; off >>= 1) row_max = fmaxf(row_max, __shfl_xor(row_max, off, TPR));
        if (j == 0) absmax[row] = row_max;
    }

    // one step: 64 block columns of the 8 rows -> 2 KB of packed records
    auto step = [&](int st, f16x8 t) {
        const int kb = st * TPR + j;
        float amax = row_max;
        if (!by_row) {
            amax = pk_absmax_value(pk_absmax8(quant_f16x2{(f16)0.f, (f16)0.f}, t));
            for (int off = 1; off < lanes_blk; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, TPR));
            if (kb < kb_total && (j & (lanes_blk - 1)) == 0) absmax[(size_t)row * nblk + (kb * 8) / bs] = amax;
        }
        uint32_t d = 0;
        if (amax > 0.f) {  // (a block of zeros: every index 0)
            const float y = refined_rcp(amax);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float nv = div_by_block_max((float)t[e], amax, y);
                uint32_t best;
                if constexpr (MODE == 0) best = nearest_bucketed(nv, tab_lane);
                else if constexpr (MODE == 1) best = nearest_sorted(nv, c);
                else best = nearest_any(nv, c);
                d |= best << (8 * (e >> 1) + 4 * (1 - (e & 1)));  // byte e/2 of the dword; even column = high nibble
            }
        }
        if constexpr (NP > 0) {
            tile[st][j * 8 + r8] = d;  // (stored after the block row's last step)
        } else {
            uint32_t *tb = tile[st & 1];
            tb[j * 8 + r8] = d;
            __syncthreads();  // (the other buffer was read before the previous step's barrier)
            if (tid < 2 * TPR) {
                const int kb0 = st * TPR;
                const int kbw = kb0 + (tid >> 1);  // block column of the 16 bytes this thread writes
                if (kbw < kb_total)
                    *reinterpret_cast<u32x4 *>(q32 + ((size_t)mb * kb_total + kb0) * 8 + tid * 4) = *reinterpret_cast<const u32x4 *>(tb + tid * 4);
            }
        }
    };
    if constexpr (NP > 0) {
        // (fully unrolled: an array indexed by a loop counter would live in scratch memory)
#pragma unroll
        for (int st = 0; st < NP; ++st)
            if (st < n_steps) step(st, v[st]);  // (uniform: every thread of the workgroup takes the same steps)
        __syncthreads();  // the block row's records are complete
        // 16 bytes per thread and pass: the records of NP * 64 block columns, contiguous in the packed layout
#pragma unroll
        for (int p = tid; p < NP * 2 * TPR; p += 512) {
            const int kbw = p >> 1;  // block column of the 16 bytes this thread writes
            if (kbw < kb_total)
                *reinterpret_cast<u32x4 *>(q32 + (size_t)mb * kb_total * 8 + (size_t)p * 4) =
                    *reinterpret_cast<const u32x4 *>(&tile[0][0] + p * 4);
        }
        if constexpr (AHEAD) {
#pragma unroll
            for (int i = 0; i < NP; ++i) v[i] = vn[i];
        }
    } else {
        for (int st = 0; st < n_steps; ++st) {
            const int kb = st * TPR + j;
            f16x8 t = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (kb < kb_total) t = *reinterpret_cast<const f16x8 *>(src + (size_t)kb * 8);
            step(st, t);
        }
    }
    __syncthreads();  // (the next block row writes the tile buffers this one's stores read)
    }
    };
    if (tabled) run(std::integral_constant<int, 0>{});
    else if (fast) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, 2>{});
}

hipError_t launch_quantize(const void *w, const float *code, void *q, float *absmax, int m, int k, int bs, hipStream_t stream)
{
    const f16 *wp = static_cast<const f16 *>(w);
    uint32_t *qp = static_cast<uint32_t *>(q);
    // one workgroup per block row up to three per compute unit (what fits beside the bucket tables), which then
    // walk the block rows: the tables are built once per workgroup
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return e;
    const int rows8 = m / 8;
    const dim3 grid((unsigned)(rows8 < 3 * cus ? rows8 : 3 * cus)), block(512);
    const size_t lds = (size_t)kQuantTabBytes;
    if (k <= 512 * 4) hipLaunchKernelGGL(quantize_kernel<4>, grid, block, lds, stream, wp, code, qp, absmax, m, k, bs);
    else if (k <= 512 * 8) hipLaunchKernelGGL(quantize_kernel<8>, grid, block, lds, stream, wp, code, qp, absmax, m, k, bs);
    else if (k <= 512 * 16) hipLaunchKernelGGL(quantize_kernel<16>, grid, block, lds, stream, wp, code, qp, absmax, m, k, bs);
    else hipLaunchKernelGGL(quantize_kernel<0>, grid, block, lds, stream, wp, code, qp, absmax, m, k, bs);
    return hipGetLastError();
}

}  // namespace tuna
