// Streaming GEMM kernel for shapes with many rows, up to 128 tokens per pass (gfx950, wave64).
//
// With two, four or eight 16-token tiles per wave every decoded weight fragment feeds as many
// MFMAs and the launch sits between the bandwidth and the matrix-core bound: what counts is how
// many weight loads a wave keeps in flight and how little else it does.  (With one token tile it
// is the general kernel without a split across workgroups, a tile walk to pay for or a stagger.)
// This kernel computes exactly what gemm_kernel computes for one class of launches:
//   * dense, m a multiple of the workgroup's rows, k a multiple of the x chunk, chunks of whole
//     ring turns of the workgroup: no clamped or conditional weight loads, no tails; with all
//     waves along m the accumulators are final and stored from registers, with waves along k they
//     are summed through LDS in wave order as in gemm_kernel;
//   * k unsplit, or (two or more token tiles, no stagger) split into a power of two of equal parts
//     of whole x chunks: a workgroup then walks (row tile, part) pairs, and the parts of a row tile
//     meet through the workspace as in gemm_kernel - partial sums stored, an arrival ticket per
//     tile, the last arrival adds the parts in k order and stores the outputs.  No workgroup
//     waits for another;
//   * x chunks are double-buffered in LDS: chunk c + 1 is requested before chunk c is consumed
//     and written to the other buffer after it, one barrier per chunk, and the weight ring runs
//     on across chunk and tile boundaries' barriers without being emptied;
//   * arguments as separate scalars (preloaded with the wave), persistent workgroups walking row
//     tiles with a fixed stride, the decode table built once per workgroup.
// Same operand mapping, decode and summation order as gemm_kernel (see gemm_kernel.hpp), so the
// results are bit-identical to the general kernel run with the same config.  launch_gemm picks
// it when the launch qualifies (mid_applies in gemm_launch.hip).
#pragma once
#include "gemm_kernel.hpp"

namespace tuna {

template <bool NT>
__device__ __forceinline__ u32x4 load_weights(const u32x4 *p)
{
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}

// Packed weights through LDS instead of registers (LDSW variants): one 16-byte global -> LDS load per
// lane (global_load_lds_dwordx4: the data goes from the memory pipeline into LDS without passing a
// register; lane l's bytes land at the slot's base + 16*l) and, when the slot is consumed, one
// ds_read_b128 of the same bytes.  A pure transit buffer: the same global access pattern, ring depth
// and waits as the register ring, which is what makes the two comparable.
template <bool NT>
__device__ __forceinline__ void load_weights_to_lds(const unsigned char *p, unsigned char *slot)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p),
                                     (__attribute__((address_space(3))) void *)(slot), 16, 0, NT ? 2 : 0);
}

// With global -> LDS loads in flight the compiler makes every LDS store and every workgroup fence
// wait for ALL of them (they are LDS writes it cannot tell apart from the x staging area), which
// would empty the ring at every chunk switch; and it waits for everything, too, before it uses a
// register loaded from global memory while such loads are in flight.  The LDSW variants therefore
// bring x into LDS the same way (lane (token, 8-k group) fetches its own B-fragment piece of a
// k-step, so a wave instruction fills one k-step of the chunk buffer), build the decode table with
// stores the compiler does not look into, and synchronise with a bare barrier behind an explicit
// wait for the wave's own LDS operations; the waits for the loads are written out where a slot or
// a chunk is used.
__device__ __forceinline__ void lds_store16_opaque(unsigned char *p, u32x4 v)
{
    const uint32_t a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)p;
    asm volatile("ds_write_b128 %0, %1" ::"v"(a), "v"(v) : "memory");
}
__device__ __forceinline__ void barrier_lds_only()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS stores have been performed
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
}

// NT: weight loads carry the nontemporal hint (each byte is used once per launch).  Launches whose
// token chunks share the weights through the caches (a_chunks != 0) run the twin without it.
// SPLIT: the twin for launches with k split across workgroups (the unsplit kernels carry none of its code).
// BLK: one scale per block of 64 << a_blk_shift weights of a row (absmax [m, k / block]) instead of one per row:
// beside every x chunk the scales of the workgroup's rows for the chunk's blocks are staged in LDS (rounded to
// fp16, twice in a dword, as [block of the chunk][row]; two buffers, switched with the x buffers), and a lane reads
// its four rows' scales of a k-step's block with one 16-byte LDS read.  Register ring, no split; the stagger of a
// row tile's k walk is t * k_stagger whole x chunks.
template <int U, int TT, int XB, int MAXT, int MINW, bool NT = true, bool LDSW = false, bool SPLIT = false, bool BLK = false>
__global__ __launch_bounds__(MAXT, MINW) void gemm_mid_kernel(const uint8_t *a_q, const void *a_x, const float *a_code,
                                                              const float *a_absmax, int a_k, int a_n, int a_m, int a_packed,
                                                              void *a_out, const void *a_residual, int a_row_tiles,
                                                              int a_n_wg, int a_chunks, float *a_ws, unsigned *a_counters,
                                                              int a_split_log2, int a_blk_shift)
{
    static_assert(!BLK || (!LDSW && !SPLIT), "scale blocks: register ring, unsplit");
    // a_packed = waves_m | epilogue << 5 | log2(x chunk in k) << 8 | log2(waves_k) << 13 | k_stagger << 16
    const int waves_m = a_packed & 31;
    const int epilogue = (a_packed >> 5) & 7;
    const int xc_log2 = (a_packed >> 8) & 31;
    const int wk_log2 = (a_packed >> 13) & 7;
    const int waves_k = 1 << wk_log2;
    const unsigned k_stagger = (unsigned)a_packed >> 16;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *lut = smem;
    unsigned char *xbuf = smem + kLutBytes;  // two buffers of one x chunk: [slot][token tile][token][16 B]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave & (waves_k - 1);  // wave (wm, wk): rows 64*wm.., k-steps wk, wk + waves_k, ...
    const int wm = wave >> wk_log2;
    const int nthreads = (waves_m * 64) << wk_log2;
    const uint32_t lane4 = (uint32_t)lane << 2;
    // Which row tiles and which chunk of 16*TT tokens this workgroup takes.  a_chunks == 0: row tile
    // walk from blockIdx.x, token chunk blockIdx.y.  Otherwise (launches of several rounds) a
    // one-dimensional grid of a_n_wg walkers x |a_chunks| token chunks in which the token chunks of
    // a walker run side by side: they stream the same weights at about the same time, so the
    // weights come from HBM once per launch instead of once per token chunk.  a_chunks > 1: a_n_wg
    // is a multiple of 8 and the chunks of a walker share an XCD and its L2 (workgroups are dealt to
    // the 8 XCDs in turn, workgroup L sits on XCD L % 8); a_chunks < -1: they are neighbours in
    // launch order.
    int tile = blockIdx.x, tok_chunk = blockIdx.y;
    if (a_chunks > 1) {
        const unsigned slot = blockIdx.x >> 3;
        tok_chunk = (int)(slot % (unsigned)a_chunks);
        tile = (int)(slot / (unsigned)a_chunks) * 8 + (int)(blockIdx.x & 7);
    } else if (a_chunks < -1) {
        tok_chunk = (int)(blockIdx.x % (unsigned)(-a_chunks));
        tile = (int)(blockIdx.x / (unsigned)(-a_chunks));
    }
    const int tok0 = tok_chunk * (16 * TT);
    const int xc = 1 << xc_log2;
    const int chunk_its = (xc >> 5) >> wk_log2;      // k-steps of one wave per chunk, a multiple of U
    // k split across workgroups (a_split_log2 != 0): a_row_tiles counts (row tile, part) pairs, pair t is row tile
    // t >> a_split_log2, part t & (parts - 1); n_steps, n_chunks and k_len are those of one part
    const int split_log2 = SPLIT ? a_split_log2 : 0;
    const int k_len = a_k >> split_log2;
    const int n_chunks = k_len >> xc_log2;
    const int n_steps = k_len >> 5;
    const uint32_t kb_total = (uint32_t)a_k >> 3;
    const uint32_t xbuf_bytes = (uint32_t)(TT * 32) << xc_log2;  // 16*TT tokens x xc k x 2 bytes
    const int x_pieces = (int)(xbuf_bytes >> 4);
    // x staging, global -> registers -> LDS: piece p = tid + b*nthreads of a chunk is (as in
    // gemm_kernel.hpp) token row (p/64 % TT)*16 + lane/4, k-step p/64 / TT, 8-k group lane%4 - every
    // quad of lanes reads 64 contiguous bytes of one token row, a wave instruction writes one k-step
    // of one token tile.  Nothing of it depends on the chunk, so the byte offsets are formed once
    // and a chunk costs XB loads with a uniform base plus XB LDS writes (there are registers to
    // spare here; the general kernel recomputes them per chunk to save some).
    uint32_t x_goff[XB], x_loff[XB], x_kloc[XB];  // (x_kloc: the piece's k within its chunk, for the stagger's wrap)
    uint32_t x_inchunk = 0, x_real = 0;  // bit b: piece b exists in a chunk / its token row exists
    {
        const int row_l = lane >> 2, grp = lane & 3;
#pragma unroll
        for (int b = 0; b < XB; ++b) {
            const int p = tid + b * nthreads;
            const int wv = p >> 6;
            const int row = (wv % TT) * 16 + row_l, ks = wv / TT;
            const bool in = p < x_pieces;
            x_kloc[b] = in ? (uint32_t)(ks * 32 + grp * 8) : 0u;
            x_goff[b] = in ? ((uint32_t)min(row, a_n - 1 - tok0) * (uint32_t)a_k + x_kloc[b]) * 2u : 0u;
            x_loff[b] = (uint32_t)((ks * 4 + grp) * (256 * TT) + row * 16);
            x_inchunk |= in ? 1u << b : 0u;
            x_real |= (in && tok0 + row < a_n) ? 1u << b : 0u;
        }
    }
    // BLK: scale s = tid + i * nthreads (i < SB) of a chunk is row s >> nbc_log2 of the workgroup's, block
    // s & (nbc - 1) of the chunk's nbc (consecutive lanes read consecutive blocks of a row); stored at
    // [block][row] with rows padded by 4 so that the lanes of a store hit different banks
    constexpr int SB = MAXT > 512 ? 2 : 4;  // (the 1024-thread twins have 128 registers per lane)
    const int blk_log2 = BLK ? 6 + a_blk_shift : 0;                       // log2(weights per scale)
    const int nbc_log2 = BLK ? max(xc_log2 - blk_log2, 0) : 0;          // log2(blocks per chunk)
    const int s_pitch = waves_m * 64 + 4;                               // dwords between the blocks of a buffer
    const int s_count = BLK ? (waves_m * 64) << nbc_log2 : 0;           // scales per chunk
    const uint32_t sbuf_bytes = BLK ? ((uint32_t)s_pitch << nbc_log2) * 4u : 0u;
    unsigned char *sbuf = xbuf + 2 * xbuf_bytes;                        // two scale buffers behind the x buffers
    float sv[BLK ? SB : 1];
    const int nblk = BLK ? a_k >> blk_log2 : 1;                         // scales per row
    /* (kbase: the chunk's logical k; rot_k: the tile's stagger, whole chunks here, so a chunk never wraps inside) */ \
#define TUNA_MID_S_LOAD(row0_wg, kbase, rot_k)                                                   \
    if constexpr (BLK) {                                                                       \
        int kp_ = (kbase) + (rot_k);                                                           \
        if (kp_ >= a_k) kp_ -= a_k;                                                            \
        const float *sp_ = a_absmax + (size_t)(row0_wg) * (size_t)nblk + (kp_ >> blk_log2);    \
        _Pragma("unroll") for (int i = 0; i < SB; ++i)                                         \
        {                                                                                      \
            const int s_ = min(tid + i * nthreads, s_count - 1);                               \
            sv[i] = sp_[(size_t)(s_ >> nbc_log2) * (size_t)nblk + (s_ & ((1 << nbc_log2) - 1))]; \
        }                                                                                      \
    }
#define TUNA_MID_S_STORE(buf)                                                                   \
    if constexpr (BLK) {                                                                       \
        _Pragma("unroll") for (int i = 0; i < SB; ++i)                                         \
        {                                                                                      \
            const int s_ = tid + i * nthreads;                                                 \
            const uint32_t h_ = (uint32_t)f16_bits((f16)sv[i]);                                \
            if (s_ < s_count)                                                                  \
                reinterpret_cast<uint32_t *>(buf)[(s_ & ((1 << nbc_log2) - 1)) * s_pitch + (s_ >> nbc_log2)] = h_ | (h_ << 16); \
        }                                                                                      \
    }
    const unsigned char *x_tile = reinterpret_cast<const unsigned char *>(a_x) + (size_t)tok0 * a_k * 2;
    // Chunk at logical k `kbase` of a tile whose walk starts rot_k elements into the k range and
    // wraps around (stagger, as in gemm_kernel.hpp): physical k = logical + rot_k, minus k past the
    // end - a piece is 8 k of one 32-k step and rot_k a multiple of 32, so no piece straddles the wrap.
#define TUNA_MID_X_LOAD(kbase, rot_k, part_k)                                                   \
    {                                                                                          \
        const uint32_t kb_ = (uint32_t)(kbase) + (uint32_t)(rot_k);                            \
        const unsigned char *xc_ = x_tile + (size_t)(kb_ + (uint32_t)(part_k)) * 2;            \
        const uint32_t wrap_at_ = (uint32_t)k_len - kb_; /* pieces at or past it wrap (kb_ < 2k) */ \
        _Pragma("unroll") for (int b = 0; b < XB; ++b) xst.v[b] = *reinterpret_cast<const u32x4 *>( \
            xc_ + x_goff[b] - ((int32_t)(x_kloc[b] - wrap_at_) >= 0 ? (size_t)k_len * 2 : (size_t)0)); \
    }
    // (rows past n are zeroed, as the general kernel does)
#define TUNA_MID_X_STORE(buf)                                                                   \
    {                                                                                          \
        _Pragma("unroll") for (int b = 0; b < XB; ++b) if (x_inchunk >> b & 1u)                \
        {                                                                                      \
            const u32x4 v_ = (x_real >> b & 1u) ? xst.v[b] : u32x4{0u, 0u, 0u, 0u};            \
            *reinterpret_cast<u32x4 *>((buf) + x_loff[b]) = v_;                                \
        }                                                                                      \
    }

    // LDSW: chunk `kbase` of x straight into `buf`, one wave instruction per k-step and token tile: piece
    // i = wave + b*(waves of the workgroup), b < xdma_n (a uniform count of 1, 2 or 4: the explicit waits
    // below count on it), is k-step i / TT, token tile i % TT, and lands at buf + i KB; lane (token i16,
    // 8-k group g) fetches its own B-fragment piece.  Token rows past n are clamped (their output
    // columns are never stored).
    const int xdma_n = LDSW ? max(1, ((xc >> 5) * TT) / (nthreads >> 6)) : 0;
#define TUNA_MID_X_DMA(buf, kbase, rot_steps, part_steps)                                       \
    {                                                                                          \
        _Pragma("unroll 1") for (int b = 0; b < xdma_n; ++b)                                  \
        {                                                                                      \
            const int i_ = min(wave + b * (nthreads >> 6), (xc >> 5) * TT - 1);                \
            const int ks_ = i_ / TT, tt_ = i_ % TT;                                            \
            int s_ = ((kbase) >> 5) + ks_ + (rot_steps);                                       \
            if (s_ >= n_steps) s_ -= n_steps;                                                  \
            s_ += (part_steps);                                                                \
            const uint32_t lane_ = ((uint32_t)min(tt_ * 16 + i16, a_n - 1 - tok0) * (uint32_t)a_k + (uint32_t)g * 8u) * 2u; \
            load_weights_to_lds<false>(x_tile + (size_t)s_ * 64 + lane_, (buf) + i_ * 1024);   \
        }                                                                                      \
    }

    float code_lane;
    if constexpr (LDSW) {
        // through the scalar cache: a vector load here would be one more thing in flight that the
        // compiler waits for by waiting for everything
        // (uniform, read before the kernel's first store; the selection starts from a constant: a
        // select between two loads would be turned back into one vector load)
        const float *__restrict__ code_ptr = a_code;
        float cs[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) cs[j] = code_ptr[j];
        code_lane = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) code_lane = i16 == j ? cs[j] : code_lane;
    } else {
        code_lane = a_code[i16];
    }
    // weights of this wave's rows: lane (i16, g) loads 16 bytes = dword j of row 4*i16 + j's 8 k
    // (block row i16/2, second half of the block for odd i16), block column 4*step + g
    uint32_t lb = 0;
    int rot = 0;
    int ps = 0;  // first k-step of the tile's part
    u32x4 wq[U];
    f32x4 sc32{0.f, 0.f, 0.f, 0.f};
    XStage<XB> xst;
#define TUNA_MID_TILE_FETCH(t)                                                                  \
    {                                                                                          \
        const int row0_ = ((t) >> split_log2) * (waves_m * 64) + wm * 64;                      \
        ps = ((t) & ((1 << split_log2) - 1)) * n_steps;                                        \
        /* stagger: row tile t walks k starting rot steps in, wrapping around (gemm_kernel.hpp) */ \
        rot = (k_stagger && n_steps > 1) ? (int)(((unsigned)(t) * k_stagger) % (unsigned)n_steps) : 0; \
        /* BLK: whole chunks, so that a chunk's scale blocks are contiguous */                 \
        if constexpr (BLK) rot = (k_stagger && n_chunks > 1) ? (int)(((unsigned)(t) * k_stagger) % (unsigned)n_chunks) << (xc_log2 - 5) : 0; \
        lb = ((uint32_t)(row0_ >> 3) + (uint32_t)(i16 >> 1)) * kb_total * 32u + (uint32_t)(i16 & 1) * 16u + (uint32_t)g * 32u; \
        /* x and the scales first: vector loads return in order, and the tile's first barrier */ \
        /* waits for the x pieces only - the first ring turn stays in flight across it */        \
        if constexpr (!LDSW) TUNA_MID_X_LOAD(0, rot << 5, ps << 5)                             \
        if constexpr (BLK) {                                                                   \
            TUNA_MID_S_LOAD(((t) >> split_log2) * (waves_m * 64), 0, rot << 5)                 \
        } else if constexpr (!LDSW) {                                                          \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) sc32[j] = a_absmax[row0_ + i16 * 4 + j]; \
        }                                                                                      \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                          \
        {                                                                                      \
            int s_ = wk + (u << wk_log2) + rot;                                                \
            if (s_ >= n_steps) s_ -= n_steps;                                                  \
            s_ += ps;                                                                          \
            if constexpr (LDSW) load_weights_to_lds<NT>(a_q + (size_t)s_ * 128 + lb, wring + u * 1024); \
            else wq[u] = load_weights<NT>(reinterpret_cast<const u32x4 *>(a_q + (size_t)s_ * 128 + lb)); \
        }                                                                                      \
    }
    // LDSW: this wave's ring of U slots of 1 KB, behind the two x buffers
    unsigned char *wring = xbuf + 2 * ((uint32_t)(TT * 32) << xc_log2) + wave * (U * 1024);
    bool first_tile = true;
    // LDSW: chunk 0 of tile t into buffer 0 and the lane's four scales into this wave's KB of buffer 1
    // (free until chunk 1 is requested; read back at the top of the tile)
#define TUNA_MID_TOP_DMA(t, rot_steps)                                                          \
    {                                                                                          \
        TUNA_MID_X_DMA(xbuf, 0, rot_steps, ((t) & ((1 << split_log2) - 1)) * n_steps)          \
        load_weights_to_lds<false>(reinterpret_cast<const unsigned char *>(a_absmax + ((t) >> split_log2) * (waves_m * 64) + wm * 64 + i16 * 4), \
                                   xbuf + ((uint32_t)(TT * 32) << xc_log2) + wave * 1024);     \
    }
    if constexpr (LDSW) {
        // the first tile's ahead of its ring (later tiles: at the top of the tile, when the
        // reduction has left the x area)
        if (tile < a_row_tiles) {
            const int rot0_ = (k_stagger && n_steps > 1) ? (int)(((unsigned)tile * k_stagger) % (unsigned)n_steps) : 0;
            TUNA_MID_TOP_DMA(tile, rot0_)
        }
    }
    if (tile < a_row_tiles) TUNA_MID_TILE_FETCH(tile)

    // ---- decode table (see gemm_kernel.hpp), built while the first loads are in flight --------
    {
        const int code_bits = (int)f16_bits((f16)code_lane);
        for (int p0 = tid; p0 < kLutBytes / 16; p0 += 4 * nthreads) {
            uint32_t v[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int e = (p0 + b * nthreads) >> 4;
                const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((e >> 4) << 2, code_bits);
                const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((e & 15) << 2, code_bits);
                v[b] = hi | (lo << 16);
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int p = p0 + b * nthreads;
                if (p < kLutBytes / 16) {
                    if constexpr (LDSW) lds_store16_opaque(lut + (size_t)p * 16, u32x4{v[b], v[b], v[b], v[b]});
                    else reinterpret_cast<u32x4 *>(lut)[p] = u32x4{v[b], v[b], v[b], v[b]};
                }
            }
        }
    }

    f16 *outp = reinterpret_cast<f16 *>(a_out);
    const f16 *resp = reinterpret_cast<const f16 *>(a_residual);
    // B fragment of lane (token i16, k-group g), local step sl, token tile tt:
    // slot sl*4 + g, byte slot*(256*TT) + tt*256 + i16*16
    // (LDSW: a KB per k-step and token tile, lane l's piece at 16*l)
    const uint32_t xb_lane = (LDSW ? (uint32_t)lane * 16 : (uint32_t)g * (256 * TT) + (uint32_t)i16 * 16) + (uint32_t)wk * (1024 * TT);
    constexpr uint32_t xb_tile = LDSW ? 1024 : 256;  // bytes between the token tiles of a k-step
    const uint32_t wstep = (uint32_t)(1024 * TT) << wk_log2;  // LDS bytes between this wave's consecutive steps

    // One ring turn: U of this wave's k-steps, each consumed (B fragments from LDS, 4 fragments
    // decoded, 4*TT MFMAs) and refilled with the wave's step U iterations on (the last turn
    // re-reads the tile's last step: in bounds, never consumed).
#define TUNA_MID_GROUP(sl, first)                                                               \
    {                                                                                          \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                          \
        {                                                                                      \
            if constexpr (LDSW) {                                                              \
                /* the slot's load has landed: U - 1 younger ring loads, in a chunk's first turn */ \
                /* also the XB x pieces just requested, may stay in flight */                  \
                if (!(first)) __builtin_amdgcn_s_waitcnt(wait_vmcnt(U - 1));                   \
                else if (xdma_n == 4) __builtin_amdgcn_s_waitcnt(wait_vmcnt(U + 3));           \
                else if (xdma_n == 2) __builtin_amdgcn_s_waitcnt(wait_vmcnt(U + 1));           \
                else __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));                                \
                wq[u] = *reinterpret_cast<const u32x4 *>(wring + u * 1024 + lane * 16);        \
            }                                                                                  \
            f16x8 b_[TT];                                                                      \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) b_[tt] =                         \
                *reinterpret_cast<const f16x8 *>(xb + (size_t)((sl) + u) * wstep + tt * xb_tile); \
            if constexpr (BLK) {                                                               \
                /* the block of this wave's k-step (sl + u) of the chunk, counted from the chunk's first */ \
                const int rel_ = min(((((sl) + u) << wk_log2) + wk) >> (blk_log2 - 5), (1 << nbc_log2) - 1); \
                const u32x4 s4_ = *reinterpret_cast<const u32x4 *>(sb_lane + (size_t)rel_ * (size_t)(s_pitch * 4)); \
                _Pragma("unroll") for (int j = 0; j < 4; ++j)                                  \
                {                                                                              \
                    const uint32_t e_ = s4_[j]; /* (a copy: bit_cast of a vector element reads element 0) */ \
                    sc16[j] = __builtin_bit_cast(f16x2, e_);                                   \
                }                                                                              \
            }                                                                                  \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                      \
            {                                                                                  \
                const f16x8 av_ = decode_dword<TUNA_DECODE_GEMM>(wq[u][j], lut, lane4, sc16[j], 0.f); \
                _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) acc[j][tt] =                 \
                    __builtin_amdgcn_mfma_f32_16x16x32_f16(av_, b_[tt], acc[j][tt], 0, 0, 0);  \
            }                                                                                  \
            int s_ = min(wk + ((it + u + U) << wk_log2), n_steps - 1) + cur_rot;               \
            if (s_ >= n_steps) s_ -= n_steps;                                                  \
            if constexpr (LDSW) {                                                              \
                /* behind the MFMAs that used the slot's bytes: the slot is free */            \
                __builtin_amdgcn_sched_barrier(0);                                             \
                load_weights_to_lds<NT>(qrow + (size_t)s_ * 128, wring + u * 1024);            \
            } else {                                                                           \
                wq[u] = load_weights<NT>(reinterpret_cast<const u32x4 *>(qrow + (size_t)s_ * 128)); \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0); /* keep each refill right behind its consume */ \
        }                                                                                      \
        it += U;                                                                               \
    }

    while (tile < a_row_tiles) {
        if constexpr (LDSW) {
            if (first_tile) {
                __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));  // chunk 0 and the scales are older than the ring's U loads
            } else {
                TUNA_MID_TOP_DMA(tile, rot)
                __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
            }
            first_tile = false;
            sc32 = *reinterpret_cast<const f32x4 *>(xbuf + ((uint32_t)(TT * 32) << xc_log2) + wave * 1024 + lane * 16);
        }
        f16x2 sc16[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f16 h = (f16)sc32[j];
            sc16[j] = f16x2{h, h};
        }
        const int row0 = (tile >> split_log2) * (waves_m * 64) + wm * 64;
        f32x4 acc[4][TT];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) acc[j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

        // chunk 0 of x into buffer 0 (every wave has left the previous tile's last chunk: the
        // barrier that ends a chunk), then the table and the chunk are published together
        if constexpr (LDSW) {
            barrier_lds_only();  // (every wave has waited for its pieces of chunk 0 and read its scales)
        } else {
            TUNA_MID_X_STORE(xbuf)
            TUNA_MID_S_STORE(sbuf)
            // (threads without a piece to store have not waited for theirs, see gemm_kernel.hpp; the U
            // weight loads of the ring are younger than every x piece and may stay in flight)
            __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));
            __syncthreads();
        }

        const unsigned char *qrow = a_q + lb + (size_t)ps * 128;
        const int cur_rot = rot;
        const int cur_ps = ps;
        int it = 0;  // this wave's next iteration (its k-step wk + it*waves_k)
        for (int c = 0; c < n_chunks; ++c) {
            const bool has_next = c + 1 < n_chunks;
            // (unconditional - the last chunk requests itself again and drops it: behind a branch
            // the compiler could not count these loads into the waits of the first ring turn)
            if constexpr (LDSW) {
                // (the other buffer was last read in chunk c - 1, which ended with a barrier)
                TUNA_MID_X_DMA(xbuf + ((c + 1) & 1) * xbuf_bytes, min(c + 1, n_chunks - 1) << xc_log2, cur_rot, cur_ps)
            } else {
                TUNA_MID_X_LOAD(min(c + 1, n_chunks - 1) << xc_log2, cur_rot << 5, cur_ps << 5)
                TUNA_MID_S_LOAD(row0 - wm * 64, min(c + 1, n_chunks - 1) << xc_log2, cur_rot << 5)
            }
            const unsigned char *xb = xbuf + (c & 1) * xbuf_bytes + xb_lane;
            // BLK: this lane's four rows in the chunk's scale buffer
            [[maybe_unused]] const unsigned char *sb_lane = sbuf + (c & 1) * sbuf_bytes + (size_t)(wm * 64 + i16 * 4) * 4;
            // (the first ring turn of a chunk is a copy of its own: there the x pieces just
            // requested are in flight behind the ring, and only straight-line code lets the
            // compiler count them into its waits instead of waiting them out)
            TUNA_MID_GROUP(0, true)
            for (int sl = U; sl < chunk_its; sl += U) TUNA_MID_GROUP(sl, false)
            if constexpr (LDSW) {
                __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));  // this wave's pieces of the next chunk have landed
                barrier_lds_only();
            } else {
                if (has_next) {
                    // the other buffer was last read in chunk c - 1, which ended with a barrier
                    __builtin_amdgcn_s_waitcnt(wait_vmcnt(U));  // exactly the last ring turn's refills are younger
                    TUNA_MID_X_STORE(xbuf + ((c + 1) & 1) * xbuf_bytes)
                    TUNA_MID_S_STORE(sbuf + ((c + 1) & 1) * sbuf_bytes)
                }
                __syncthreads();
            }
        }

        // ---- next tile's loads, then this tile's store ------------------------------------------
        const int cur_row0 = row0;
        const int cur_tile = tile;
        tile += a_n_wg;
        if (tile < a_row_tiles) TUNA_MID_TILE_FETCH(tile)
        if (wk_log2 != 0 || split_log2 != 0) {
            // Waves along k: every wave puts its copy of a plane (one float4 per lane) in LDS - two
            // buffers alternate in the x area, free since the barrier that ended the last chunk -
            // and thread (wk, lane) sums floats f = (i*waves_k + wk)*64 + lane of it in wave order:
            // float f = l*4 + v of plane j is token l%16, weight row 16*(l/16) + 4*v + j of the wave's
            // 64, so after the four planes a thread owns 4 consecutive features of one token.
            float *redf = reinterpret_cast<float *>(xbuf);
            const size_t plane_floats = (size_t)(waves_m << wk_log2) * 256;
            // split: this wave row's partial sums of part p of the tile at wst + p * seg_floats, as [token tile][f] float4s
            const size_t seg_floats = (size_t)waves_m * (TT * 1024);
            const size_t tile_id = (size_t)tok_chunk * (size_t)(a_row_tiles >> split_log2) + (size_t)(cur_tile >> split_log2);
            float *wst = a_ws + (tile_id << split_log2) * seg_floats + (size_t)wm * (TT * 1024);
            const int part = cur_tile & ((1 << split_log2) - 1);
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                float o[4][4];  // [i][j]
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float *buf = redf + (size_t)((tt * 4 + j) & 1) * plane_floats;
                    reinterpret_cast<f32x4 *>(buf)[(size_t)wave * 64 + lane] = acc[j][tt];
                    __syncthreads();
                    sum_planes_any<1, 32>(wk_log2, buf, plane_floats, wm, wk, lane, o, j);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int f = ((i << wk_log2) + wk) * 64 + lane;
                    if (f >= 256) continue;
                    if (split_log2 != 0) {
                        store_partial(wst + (size_t)part * seg_floats + (size_t)(tt * 256 + f) * 4,
                                      f32x4{o[i][0], o[i][1], o[i][2], o[i][3]});
                        continue;
                    }
                    const int l = f >> 2, v = f & 3;
                    const int tok = tok0 + tt * 16 + (l & 15);
                    if (tok < a_n)
                        store_features4(outp, resp, epilogue, (size_t)tok, a_m, cur_row0 + (l >> 4) * 16 + v * 4, o[i][0], o[i][1],
                                        o[i][2], o[i][3]);
                }
            }
            if (split_log2 != 0) {
                // hand-over (see gemm_kernel): stores complete, barrier (also: every read of the reduction
                // buffers is done), arrival ticket, the last arrival adds the parts in k order
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __syncthreads();
                volatile unsigned *ticket = reinterpret_cast<volatile unsigned *>(xbuf);
                if (tid == 0) *ticket = __hip_atomic_fetch_add(a_counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                const int parts = 1 << split_log2;
                if (*ticket == (unsigned)parts - 1u) {
                    if (tid == 0) __hip_atomic_store(a_counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    for (int tt = 0; tt < TT; ++tt)
                        for (int i = 0; i < 4; ++i) {
                            const int f = ((i << wk_log2) + wk) * 64 + lane;
                            if (f >= 256) break;
                            const float *src = wst + (size_t)(tt * 256 + f) * 4;
                            f32x4 s4 = f32x4{0.f, 0.f, 0.f, 0.f};
                            for (int sp0 = 0; sp0 < parts; sp0 += 4) {  // four contributors per round trip
                                f32x4 p[4];
                                const float *psrc[4];
#pragma unroll
                                for (int b = 0; b < 4; ++b) psrc[b] = src + (size_t)min(sp0 + b, parts - 1) * seg_floats;
                                load_partials4(psrc[0], psrc[1], psrc[2], psrc[3], p[0], p[1], p[2], p[3]);
#pragma unroll
                                for (int b = 0; b < 4; ++b)
                                    if (sp0 + b < parts) s4 += p[b];
                            }
                            const int l = f >> 2, v = f & 3;
                            const int tok = tok0 + tt * 16 + (l & 15);
                            if (tok < a_n)
                                store_features4(outp, resp, epilogue, (size_t)tok, a_m, cur_row0 + (l >> 4) * 16 + v * 4, s4[0],
                                                s4[1], s4[2], s4[3]);
                        }
                }
            }
            __syncthreads();  // the x area is written again at the top of the next tile
            continue;
        }
        // Lane (token i16, group g) owns 16 consecutive output features, acc[j][tt][v] being
        // feature 4*v + j of them: two 16-byte stores per token tile.
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const int tok = tok0 + tt * 16 + i16;
            const int rb = cur_row0 + g * 16;
            if (tok >= a_n) continue;
            if (epilogue == TUNA_EPILOGUE_NONE) {
                f16x8 lo, hi;
#pragma unroll
                for (int v = 0; v < 2; ++v)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        lo[v * 4 + j] = (f16)acc[j][tt][v];
                        hi[v * 4 + j] = (f16)acc[j][tt][v + 2];
                    }
                f16 *dst = outp + (size_t)tok * a_m + rb;
                *reinterpret_cast<f16x8 *>(dst) = lo;
                *reinterpret_cast<f16x8 *>(dst + 8) = hi;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    store_features4(outp, resp, epilogue, (size_t)tok, a_m, rb + v * 4, acc[0][tt][v], acc[1][tt][v], acc[2][tt][v],
                                    acc[3][tt][v]);
            }
        }
    }
#undef TUNA_MID_GROUP
#undef TUNA_MID_X_LOAD
#undef TUNA_MID_S_LOAD
#undef TUNA_MID_S_STORE
#undef TUNA_MID_X_STORE
#undef TUNA_MID_X_DMA
#undef TUNA_MID_TOP_DMA
#undef TUNA_MID_TILE_FETCH
}

}  // namespace tuna
