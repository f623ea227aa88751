/*
 * CPU oracle for the FP16-activation x 4-bit-codebook-weight GEMM path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * reference's algorithm, used only as the checker by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  The product
 * path (tuna_amd/csrc) never links, loads or calls anything in here.
 *
 * Every function cites the reference file:line it restates.  All fp16 values are
 * carried as raw uint16_t bit patterns and all fp16 arithmetic is done in
 * software so that results do not depend on the host's F16C / compiler flags.
 *
 * Parity pins (what each function is checked against, in tests/test_oracle.py):
 *   orc_f32_to_f16 / orc_f16_to_f32 / orc_f64_to_f16 : exhaustive / dense sweeps
 *       against numpy's IEEE-754 float16 conversions (independent implementation)
 *   orc_nf4_codebook  : the literal constants of test.py:19-37 as fp32 bit patterns
 *   orc_pack / orc_unpack : test.py:58-65 (forward) and kernel.cu:3221-3228
 *       (inverse) are independent statements in the reference that must be mutual
 *       inverses; closed-form bit positions, brute force on 8x8 and 16x24
 *   orc_decode_d1 / orc_decode_d2 : exhaustive 16 codes x 65536 scales against
 *       numpy fp16 / fp32 arithmetic; known-answer rows for scale 0x211f
 *   orc_dequant : unpack + decode, checked against a numpy gather
 *   orc_quantize : per-row absmax + nearest codebook entry + packing (test.py:7-68),
 *       checked against numpy float32 division / |difference| / argmin (first index on
 *       ties) incl. exact midpoints between codes, and against the round trip through
 *       orc_dequant.  All-zero rows: the reference divides by zero, every candidate
 *       distance is NaN and torch.argmin over an all-NaN column returns index 0;
 *       pinned by running that torch expression (CPU torch) in the test.
 *   *_blk       : the same functions with one scale per block of block_size consecutive weights
 *       of a row (test.py:7-17 layout); block_size == k is the plain function.  Checked against
 *       numpy gathers / matmul with the scales expanded per element, and the quantizer against
 *       the torch expressions of test.py:15-53 run on the CPU with block_size < k.
 *   orc_gemm*   : textbook contraction; checked against numpy float64 matmul,
 *       linearity, one-hot read-out of the decoded weights, row permutation
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* IEEE-754 binary16 <-> binary32/binary64, round-to-nearest-even             */
/* (kernel.cu:2770, 2800, 3227 use the CUDA default RN conversions)           */
/* ------------------------------------------------------------------------- */

ORC_API float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* shared core: round a 64-bit significand-carrying double to binary16 */
ORC_API uint16_t orc_f64_to_f16(double d)
{
    uint64_t b;
    memcpy(&b, &d, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int exp = (int)((b >> 52) & 0x7ff);
    uint64_t man = b & 0xfffffffffffffull;
    if (exp == 0x7ff) { /* inf / nan */
        if (man) return (uint16_t)(sign | 0x7e00u | (uint16_t)(man >> 42));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (exp == 0) return sign; /* double subnormals are far below half range */
    int e = exp - 1023;        /* unbiased */
    man |= 1ull << 52;         /* 53-bit significand, value = man * 2^(e-52) */
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    int shift;                 /* bits to drop so the result has the half's lsb */
    if (e >= -14) shift = 42;  /* normal half: 10 fraction bits */
    else shift = 42 + (-14 - e);
    if (shift > 63) return sign; /* below half of the smallest subnormal */
    uint64_t q = man >> shift;
    uint64_t rem = man & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    uint16_t out;
    if (e >= -14) {
        /* q has 11 bits (implicit one at bit 10), may have carried to bit 11 */
        uint32_t he = (uint32_t)(e + 15);
        uint32_t v = (he << 10) + (uint32_t)(q - 0x400u); /* carry propagates into exponent */
        if (v >= 0x7c00u) v = 0x7c00u;
        out = (uint16_t)v;
    } else {
        out = (uint16_t)q; /* subnormal, q <= 0x400 (0x400 == smallest normal) */
    }
    return (uint16_t)(sign | out);
}

ORC_API uint16_t orc_f32_to_f16(float f)
{
    /* float -> double is exact, so one rounding happens, in orc_f64_to_f16 */
    return orc_f64_to_f16((double)f);
}

/* ------------------------------------------------------------------------- */
/* Codebook: the 16 NF4 constants the reference's harness builds              */
/* (test.py:19-37); stored as float32 like the `code` tensor (kernel.cu:3014)  */
/* ------------------------------------------------------------------------- */

ORC_API void orc_nf4_codebook(float out[16])
{
    static const float c[16] = {
        -1.0f,
        -0.6961928009986877f,
        -0.5250730514526367f,
        -0.39491748809814453f,
        -0.28444138169288635f,
        -0.18477343022823334f,
        -0.09105003625154495f,
        0.0f,
        0.07958029955625534f,
        0.16093020141124725f,
        0.24611230194568634f,
        0.33791524171829224f,
        0.44070982933044434f,
        0.5626170039176941f,
        0.7229568362236023f,
        1.0f,
    };
    memcpy(out, c, sizeof(c));
}

/* ------------------------------------------------------------------------- */
/* Packed layout  q : uint8 [m/8, k/8, 32]                                     */
/* forward  (test.py:58-65): reshape [m/8, 8, k/8, 4, 2] -> permute to         */
/*          [m/8, k/8, 8, 4, 2] -> byte = first*16 + second                    */
/* inverse  (kernel.cu:3171, 3211, 3221-3228): byte `lid` of block (mb, kb)    */
/*          is row mb*8 + lid/4, columns kb*8 + (lid%4)*2 (+0 high, +1 low)    */
/* ------------------------------------------------------------------------- */

static inline size_t q_offset(int row, int col, int k)
{
    /* byte that holds weight (row, col) */
    size_t mb = (size_t)(row >> 3), kb = (size_t)(col >> 3);
    size_t byte = (size_t)((row & 7) * 4 + ((col & 7) >> 1));
    return (mb * (size_t)(k >> 3) + kb) * 32 + byte;
}

ORC_API int orc_pack(const uint8_t *codes, uint8_t *q, int m, int k)
{
    if (m <= 0 || k <= 0 || (m & 7) || (k & 7)) return 1;
    memset(q, 0, (size_t)m * (size_t)k / 2);
    for (int r = 0; r < m; r++)
        for (int c = 0; c < k; c++) {
            uint8_t v = codes[(size_t)r * k + c] & 15u;
            size_t o = q_offset(r, c, k);
            if ((c & 1) == 0) q[o] |= (uint8_t)(v << 4); /* even column: high nibble */
            else q[o] |= v;                              /* odd column : low nibble  */
        }
    return 0;
}

ORC_API int orc_unpack(const uint8_t *q, uint8_t *codes, int m, int k)
{
    if (m <= 0 || k <= 0 || (m & 7) || (k & 7)) return 1;
    for (int r = 0; r < m; r++)
        for (int c = 0; c < k; c++) {
            uint8_t b = q[q_offset(r, c, k)];
            codes[(size_t)r * k + c] = (c & 1) ? (b & 15u) : (uint8_t)(b >> 4);
        }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* The two decode roundings of the reference                                   */
/* ------------------------------------------------------------------------- */

/* D1 - the GEMM's in-register decode (kernel.cu:2178-2192): codebook and scale
 * are rounded to fp16 when staged (kernel.cu:2800, 2770), then multiplied as
 * fp16 x fp16 with one RN rounding.  The product of two 11-bit significands is
 * exact in binary32, so rounding that float once to fp16 is the fp16 product. */
ORC_API uint16_t orc_decode_d1(float code, float absmax)
{
    float c = orc_f16_to_f32(orc_f32_to_f16(code));
    float s = orc_f16_to_f32(orc_f32_to_f16(absmax));
    volatile float p = c * s; /* exact */
    return orc_f32_to_f16(p);
}

/* D2 - the standalone dequant op (kernel.cu:3222-3228): float multiply (one
 * RN rounding to binary32) followed by the float -> half RN conversion. */
ORC_API uint16_t orc_decode_d2(float code, float absmax)
{
    volatile float p = code * absmax;
    return orc_f32_to_f16(p);
}

#define ORC_D1 1
#define ORC_D2 2

static void build_row_lut(uint16_t lut[16], const float *code, float absmax, int mode)
{
    for (int i = 0; i < 16; i++)
        lut[i] = (mode == ORC_D1) ? orc_decode_d1(code[i], absmax) : orc_decode_d2(code[i], absmax);
}

/* Scale blocks.  The reference's quantizer takes a block_size (test.py:7-9): the weights, flattened
 * row-major, are cut into blocks of block_size elements and every block gets its own absmax
 * (test.py:15-17), i.e. element (r, c) of an [m, k] matrix with k a multiple of block_size uses
 * absmax[(r*k + c) / block_size] = absmax[r * (k/block_size) + c / block_size].  The reference's
 * kernels only ever run block_size == k (one scale per row: kernel.cu:2904 indexes absmax by row,
 * test.py:81); the *_blk functions below restate the same arithmetic for finer blocks and the
 * plain functions are their block_size == k case. */
static inline float blk_scale(const float *absmax, int r, int c, int k, int bs)
{
    return absmax[(size_t)r * (size_t)(k / bs) + (size_t)(c / bs)];
}

/* out[m, k] fp16 row-major (kernel.cu:3238); mode selects D1 or D2 */
ORC_API int orc_dequant_blk(const uint8_t *q, const float *absmax, const float *code,
                            uint16_t *out, int m, int k, int mode, int bs)
{
    if (m <= 0 || k <= 0 || (m & 7) || (k & 7)) return 1;
    if (mode != ORC_D1 && mode != ORC_D2) return 2;
    if (bs <= 0 || k % bs) return 5;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < m; r++) {
        uint16_t lut[16];
        for (int c = 0; c < k; c++) {
            if (c % bs == 0) build_row_lut(lut, code, blk_scale(absmax, r, c, k, bs), mode);
            uint8_t b = q[q_offset(r, c, k)];
            uint8_t nib = (c & 1) ? (b & 15u) : (uint8_t)(b >> 4);
            out[(size_t)r * k + c] = lut[nib];
        }
    }
    return 0;
}

ORC_API int orc_dequant(const uint8_t *q, const float *absmax, const float *code,
                        uint16_t *out, int m, int k, int mode)
{
    return orc_dequant_blk(q, absmax, code, out, m, k, mode, k);
}

/* ------------------------------------------------------------------------- */
/* Quantizer (test.py:7-68 with block_size == k): absmax[r] = max |w[r, :]| as   */
/* fp32; normalized = fp32(w) / absmax (fp32 division, test.py:41: fp16 / fp32   */
/* promotes to fp32); code index = argmin_j |normalized - code[j]| in fp32 with  */
/* the first index on ties (torch.argmin, test.py:50-53); packed as test.py:55-65 */
/* ------------------------------------------------------------------------- */
ORC_API int orc_quantize_blk(const uint16_t *w, const float *code, uint8_t *q, float *absmax, int m, int k, int bs)
{
    if (m <= 0 || k <= 0 || (m & 7) || (k & 7)) return 1;
    if (bs <= 0 || k % bs) return 5;
    const int nb = k / bs;
    memset(q, 0, (size_t)m * k / 2);
#pragma omp parallel for schedule(static)
    for (int mb = 0; mb < m / 8; mb++) {
        for (int r8 = 0; r8 < 8; r8++) {
            const int r = mb * 8 + r8;
            for (int b0 = 0; b0 < nb; b0++) {
                float amax = 0.f;
                for (int c = b0 * bs; c < (b0 + 1) * bs; c++) {
                    const float v = fabsf(orc_f16_to_f32(w[(size_t)r * k + c]));
                    if (v > amax) amax = v;
                }
                absmax[(size_t)r * nb + b0] = amax;
                for (int c = b0 * bs; c < (b0 + 1) * bs; c++) {
                    int best = 0; /* all-NaN candidates: torch.argmin returns index 0 */
                    if (amax > 0.f) {
                        const volatile float nv = orc_f16_to_f32(w[(size_t)r * k + c]) / amax; /* fp32, no excess precision */
                        float bd = 0.f;
                        for (int j = 0; j < 16; j++) {
                            const volatile float d = fabsf(nv - code[j]);
                            if (j == 0 || d < bd) {
                                bd = d;
                                best = j;
                            }
                        }
                    }
                    uint8_t *b = &q[q_offset(r, c, k)];
                    *b |= (c & 1) ? (uint8_t)best : (uint8_t)(best << 4);
                }
            }
        }
    }
    return 0;
}

ORC_API int orc_quantize(const uint16_t *w, const float *code, uint8_t *q, float *absmax, int m, int k)
{
    return orc_quantize_blk(w, code, q, absmax, m, k, k);
}

/* ------------------------------------------------------------------------- */
/* GEMM: out[n, m] = X[n, k] . Wdeq[m, k]^T, stored [n, m] row-major           */
/* (kernel.cu:2872 leadingDims {k,k,m}; kernel.cu:2957-2959 transposed store)  */
/* Weights are decoded to fp16 first (mode D1 = what the reference GEMM feeds  */
/* its tensor cores, D2 = dequantize-then-matmul); accumulation is binary64    */
/* (acc64 != 0; products of two halves are exact, the sum is rounded once to   */
/* fp16) or binary32 in plain k order (acc64 == 0).                            */
/* `rows`/`n_rows` optionally restrict the computation to a subset of weight   */
/* rows; out is then [n, n_rows].                                              */
/* ------------------------------------------------------------------------- */

ORC_API int orc_gemm_rows(const uint8_t *q, const uint16_t *x, const float *code,
                          const float *absmax, uint16_t *out, int m, int n, int k,
                          int mode, int acc64, const int32_t *rows, int n_rows)
{
    if (m <= 0 || k <= 0 || n < 0 || (m & 7) || (k & 7)) return 1;
    if (mode != ORC_D1 && mode != ORC_D2) return 2;
    int nr = rows ? n_rows : m;
    float *xf = (float *)malloc((size_t)n * k * sizeof(float) + 4);
    if (!xf) return 3;
    for (size_t i = 0; i < (size_t)n * k; i++) xf[i] = orc_f16_to_f32(x[i]);
    int bad = 0;
#pragma omp parallel for schedule(static)
    for (int ri = 0; ri < nr; ri++) {
        int r = rows ? rows[ri] : ri;
        if (r < 0 || r >= m) { bad = 1; continue; }
        uint16_t lut[16];
        float lutf[16];
        build_row_lut(lut, code, absmax[r], mode);
        for (int i = 0; i < 16; i++) lutf[i] = orc_f16_to_f32(lut[i]);
        float *w = (float *)malloc((size_t)k * sizeof(float));
        for (int c = 0; c < k; c++) {
            uint8_t b = q[q_offset(r, c, k)];
            w[c] = lutf[(c & 1) ? (b & 15u) : (b >> 4)];
        }
        for (int t = 0; t < n; t++) {
            const float *xr = xf + (size_t)t * k;
            uint16_t h;
            if (acc64) {
                double s = 0.0;
                for (int c = 0; c < k; c++) s += (double)xr[c] * (double)w[c];
                h = orc_f64_to_f16(s);
            } else {
                float s = 0.0f;
                for (int c = 0; c < k; c++) s = fmaf(xr[c], w[c], s);
                h = orc_f32_to_f16(s);
            }
            out[(size_t)t * nr + ri] = h;
        }
        free(w);
    }
    free(xf);
    return bad ? 4 : 0;
}

ORC_API int orc_gemm(const uint8_t *q, const uint16_t *x, const float *code,
                     const float *absmax, uint16_t *out, int m, int n, int k,
                     int mode, int acc64)
{
    return orc_gemm_rows(q, x, code, absmax, out, m, n, k, mode, acc64, NULL, 0);
}

/* Same contraction with the exact double sums returned (no final rounding):
 * lets tests measure the GPU's error against the un-rounded value. */
ORC_API int orc_gemm_rows_f64_blk(const uint8_t *q, const uint16_t *x, const float *code,
                                  const float *absmax, double *out, int m, int n, int k,
                                  int mode, int bs, const int32_t *rows, int n_rows)
{
    if (m <= 0 || k <= 0 || n < 0 || (m & 7) || (k & 7)) return 1;
    if (mode != ORC_D1 && mode != ORC_D2) return 2;
    if (bs <= 0 || k % bs) return 5;
    int nr = rows ? n_rows : m;
    int bad = 0;
#pragma omp parallel for schedule(static)
    for (int ri = 0; ri < nr; ri++) {
        int r = rows ? rows[ri] : ri;
        if (r < 0 || r >= m) { bad = 1; continue; }
        double *w = (double *)malloc((size_t)k * sizeof(double));
        uint16_t lut[16];
        for (int c = 0; c < k; c++) {
            if (c % bs == 0) build_row_lut(lut, code, blk_scale(absmax, r, c, k, bs), mode);
            uint8_t b = q[q_offset(r, c, k)];
            w[c] = (double)orc_f16_to_f32(lut[(c & 1) ? (b & 15u) : (b >> 4)]);
        }
        for (int t = 0; t < n; t++) {
            double s = 0.0;
            for (int c = 0; c < k; c++) s += (double)orc_f16_to_f32(x[(size_t)t * k + c]) * w[c];
            out[(size_t)t * nr + ri] = s;
        }
        free(w);
    }
    return bad ? 4 : 0;
}

ORC_API int orc_gemm_rows_f64(const uint8_t *q, const uint16_t *x, const float *code,
                              const float *absmax, double *out, int m, int n, int k,
                              int mode, const int32_t *rows, int n_rows)
{
    return orc_gemm_rows_f64_blk(q, x, code, absmax, out, m, n, k, mode, k, rows, n_rows);
}

/* ------------------------------------------------------------------------- */
/* CPU baseline: "dequantize, then matmul" on the host cores.                  */
/* decode D2 to an fp16 [m, k] image (kernel.cu:3158-3241), then               */
/* Y[n, m] = X . W^T with binary32 accumulation and fp16 output.               */
/* Timed in two legs; seconds are returned through t_decode / t_matmul.        */
/* ------------------------------------------------------------------------- */

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

ORC_API int orc_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORC_API int orc_cpu_baseline(const uint8_t *q, const uint16_t *x, const float *code,
                             const float *absmax, uint16_t *out, uint16_t *wbuf,
                             int m, int n, int k, int threads,
                             double *t_decode, double *t_matmul)
{
    if (m <= 0 || k <= 0 || n <= 0 || (m & 7) || (k & 7)) return 1;
    if (threads < 1) threads = 1;
#ifdef _OPENMP
    omp_set_num_threads(threads);
#endif
    static float h2f[65536];
    static int h2f_ready = 0;
    if (!h2f_ready) {
        for (int i = 0; i < 65536; i++) h2f[i] = orc_f16_to_f32((uint16_t)i);
        h2f_ready = 1;
    }
    double t0 = now_s();
    /* leg 1: dequantize into wbuf[m, k] (fp16), block by block like the packed layout */
#pragma omp parallel for schedule(static)
    for (int mb = 0; mb < m / 8; mb++) {
        uint16_t lut[8][16];
        for (int r = 0; r < 8; r++) build_row_lut(lut[r], code, absmax[mb * 8 + r], ORC_D2);
        for (int kb = 0; kb < k / 8; kb++) {
            const uint8_t *blk = q + ((size_t)mb * (k / 8) + kb) * 32;
            for (int r = 0; r < 8; r++) {
                uint16_t *o = wbuf + (size_t)(mb * 8 + r) * k + kb * 8;
                for (int j = 0; j < 4; j++) {
                    uint8_t b = blk[r * 4 + j];
                    o[2 * j] = lut[r][b >> 4];
                    o[2 * j + 1] = lut[r][b & 15u];
                }
            }
        }
    }
    double t1 = now_s();
    /* leg 2: Y = X . W^T, fp32 accumulate */
    float *xf = (float *)malloc((size_t)n * k * sizeof(float));
    if (!xf) return 3;
    for (size_t i = 0; i < (size_t)n * k; i++) xf[i] = h2f[x[i]];
#pragma omp parallel
    {
        float *wrow = (float *)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(static)
        for (int r = 0; r < m; r++) {
            const uint16_t *wr = wbuf + (size_t)r * k;
            for (int c = 0; c < k; c++) wrow[c] = h2f[wr[c]];
            for (int t = 0; t < n; t++) {
                const float *xr = xf + (size_t)t * k;
                float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f, s4 = 0.f, s5 = 0.f, s6 = 0.f, s7 = 0.f;
                int c = 0;
                for (; c + 8 <= k; c += 8) {
                    s0 += xr[c] * wrow[c];
                    s1 += xr[c + 1] * wrow[c + 1];
                    s2 += xr[c + 2] * wrow[c + 2];
                    s3 += xr[c + 3] * wrow[c + 3];
                    s4 += xr[c + 4] * wrow[c + 4];
                    s5 += xr[c + 5] * wrow[c + 5];
                    s6 += xr[c + 6] * wrow[c + 6];
                    s7 += xr[c + 7] * wrow[c + 7];
                }
                float s = ((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7));
                for (; c < k; c++) s += xr[c] * wrow[c];
                out[(size_t)t * m + r] = orc_f32_to_f16(s);
            }
        }
        free(wrow);
    }
    free(xf);
    double t2 = now_s();
    if (t_decode) *t_decode = t1 - t0;
    if (t_matmul) *t_matmul = t2 - t1;
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Array forms of the scalar functions (so tests can sweep millions of cases)  */
/* ------------------------------------------------------------------------- */

ORC_API void orc_f32_to_f16_many(const float *in, uint16_t *out, size_t n)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(in[i]);
}

ORC_API void orc_f64_to_f16_many(const double *in, uint16_t *out, size_t n)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_f64_to_f16(in[i]);
}

ORC_API void orc_f16_to_f32_many(const uint16_t *in, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(in[i]);
}

/* out[i] = decode(code[i], absmax[i]) */
ORC_API void orc_decode_many(const float *code, const float *absmax, uint16_t *out, size_t n, int mode)
{
    for (size_t i = 0; i < n; i++)
        out[i] = (mode == ORC_D1) ? orc_decode_d1(code[i], absmax[i]) : orc_decode_d2(code[i], absmax[i]);
}
