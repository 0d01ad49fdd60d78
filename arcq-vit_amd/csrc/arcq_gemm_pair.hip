// Stages 2+3 on weights reconstructed beforehand, x_hat in the 32-row block layout: the eight-wave weight-stationary
// kernel with TWO row blocks per wave and pass (wave tile 64 rows x 128 columns = 2 x 4 MFMA blocks).
//
//   y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias,   x_hat as 16-byte pieces [M/32][K/8][32 rows][8 values]
//   (a last block of r < 32 rows as [K/8][r][8]),  w_hat [N,K] fp16 row-major.
//
// Operand budget of a CU per MFMA time (32 clocks, four SIMDs): LDS delivers 4 KB, the vector memory path 2 KB.  With
// one row block per wave every w_hat fragment read from LDS (1 KB) feeds a single MFMA, i.e. the LDS runs at its limit;
// with two row blocks it feeds two, and an x_hat fragment (from L2, one coalesced 16-byte load per lane) still feeds
// four.  The pass structure, slab slices copied global -> LDS, k order inside a group and operand roles are those of
// gemm_slab8_kernel, so results are bit-identical to it (every output accumulates its k-steps in the same order).
//
// x_hat fragments live in eight 16-byte slots per lane (k-step x row block): the slot of k-step kk is refilled with
// the next group's k-step kk right after the MFMAs that consumed it, so every load has four k-steps (32 MFMAs) to
// arrive.  Left-over blocks of a workgroup (fewer than sixteen) are dealt as pairs, single blocks and column halves.
#include "arcq_common.h"
#include "arcq_gemm.h"
#include "arcq_act_quant_core.h"

#include <stdlib.h>
#include <type_traits>

namespace arcq {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kSlabN = 128;                 // columns per slab
constexpr int kTJ = kSlabN / 32;            // 4 column blocks
constexpr int kStageRow = 144;              // bytes per staged output row: 128 + 16 pad
constexpr int kStageTile = 32 * kStageRow;  // 4608 B per wave

// WAVES waves per workgroup and SG groups per K slice of the slab.  (8, 6) is one workgroup per CU.  (Two workgroups of
// four waves per CU with three-group slices, 70 KB of LDS each, so that one multiplies while the other copies a slice
// or writes a block out, measured 35-45 % slower on every shape: 466 against 342 us at 50 432 x 3 072 x 1 024.)
// DB: two slab buffers (of SG = 3 groups each, the same LDS as one of six): the next slice is copied while the
// current one is multiplied, one barrier per slice instead of two and no wait for the copy.
template <int WAVES, int SG, bool DB> struct PairCfg {
    static constexpr int kPieces = SG * 8 + 1;            // 16-byte pieces per slab row, one of them padding
    static constexpr int kPitch = kPieces * 16;           // (conflict-free 16-byte fragment reads)
    static constexpr int kSlabBytes = kSlabN * kPitch;
    static constexpr int kSlabs = DB ? 2 : 1;
    static constexpr int kSmem = kSlabs * kSlabBytes + WAVES * kStageTile + kSlabN * static_cast<int>(sizeof(float)) + 64;
};

// s_waitcnt vmcnt(V) with expcnt and lgkmcnt unconstrained (vmcnt is split over bits 3:0 and 15:14).
template <int V> __device__ __forceinline__ void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt((V & 15) | ((V >> 4) << 14) | 0x0F70);
    asm volatile("" ::: "memory");
}

// NQ = 0, or the bits (2 / 3 / 4) of the activation quantizer of the layer that consumes this one's output: y then
// receives that layer's x_hat (stage 1 of the rounded, optionally GELU'd output) in the block layout instead of the
// output itself (arcq_act_quant_core.h, next_quant_chunk); fp16 output and N a multiple of 64 only.
template <typename TOUT, int WAVES, int SG, bool DB, int NQ>
__global__ void __launch_bounds__(64 * WAVES)
gemm_pair_kernel(const __half *__restrict__ xb, const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K,
                 int row_ranges, int blocks_per_range, const __half *__restrict__ w_hat,
                 const TOUT *__restrict__ residual, int gelu, const float *__restrict__ nx_thr, const float *__restrict__ nx_cb)
{
    static_assert(NQ == 0 || sizeof(TOUT) == 2, "the next layer's stage 1 works on fp16 outputs");
    constexpr int kWaves = WAVES;
    constexpr int kSliceGroups = SG;
    constexpr int kPieces = PairCfg<WAVES, SG, DB>::kPieces;
    constexpr int kPitch = PairCfg<WAVES, SG, DB>::kPitch;
    constexpr int kSlabBytes = PairCfg<WAVES, SG, DB>::kSlabBytes;
    constexpr int kAllSlabs = PairCfg<WAVES, SG, DB>::kSlabs * kSlabBytes;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *slab = smem;          // DB: two buffers, slab and slab + kSlabBytes
    float *s_bias = reinterpret_cast<float *>(smem + kAllSlabs + kWaves * kStageTile);      // [128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int lh = lane >> 5;
    const int G = K / 64;

    // Tile = (row range, slab); each XCD (workgroups are dealt to the 8 XCDs round-robin) takes a contiguous run of
    // tiles, ordered as tile_range_slab describes.
    const int n_slabs = (N + kSlabN - 1) / kSlabN;
    const int tiles = n_slabs * row_ranges;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    int tile_range, tile_slab;
    tile_range_slab(tile, n_slabs, row_ranges, slab_group_size(n_slabs, K, M, blocks_per_range, 2 * kWaves), tile_range, tile_slab);
    const int n_base = tile_slab * kSlabN;
    const int total_blocks = (M + 31) / 32;
    const int blk0 = tile_range * blocks_per_range;
    const int blk1 = min(total_blocks, blk0 + blocks_per_range);
    const int nblk = blk1 - blk0;
    const int full_passes = nblk / (2 * kWaves);       // every wave multiplies a pair of blocks
    const int rest = nblk - full_passes * 2 * kWaves;  // 0 .. 15 blocks for one more pass
    const int passes = full_passes + (rest > 0 ? 1 : 0);
    const int slices = (G + kSliceGroups - 1) / kSliceGroups;

    const int lane_off = lr * kPitch + lh * 64;          // this lane's fragment position inside a slab buffer
    unsigned char *stage = smem + kAllSlabs + wave * kStageTile;

    if (tid < kSlabN) s_bias[tid] = (bias && n_base + tid < N) ? bias[n_base + tid] : 0.0f;
    const unsigned char *nq_lds = smem + PairCfg<WAVES, SG, DB>::kSmem;
    if constexpr (NQ != 0)      // (the barriers of the first slab fill publish the tables)
        next_quant_setup<NQ>(nx_thr, nx_cb, smem + PairCfg<WAVES, SG, DB>::kSmem, tid, 64 * WAVES);
    // Direct global -> LDS loads: the slab is filled as one flat run of 16-byte pieces (piece p = row * kPieces +
    // column; the hardware writes lane l's piece at the wave-uniform LDS base + 16 l), 64 pieces per instruction
    // whatever the row length; padding pieces and the columns past a short last slice are skipped.  The caller
    // waits for vmcnt and the barrier.
    auto copy_slice = [&](unsigned char *dst, int g0, int ng) __attribute__((always_inline)) {
        for (int p0 = wave * 64; p0 < kSlabN * kPieces; p0 += kWaves * 64) {
            const int p = p0 + lane;
            const int row = p / kPieces, col = p - row * kPieces;
            const int n = min(n_base + row, N - 1);
            if (col < 8 * ng && row < kSlabN)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(w_hat + static_cast<int64_t>(n) * K + g0 * 64 + col * 8),
                    (__attribute__((address_space(3))) void *)(dst + p0 * 16), 16, 0, 0);
        }
    };

    // The same copy for the places where it runs under other LDS traffic (the write-out of a pass; with two buffers
    // the whole multiplication of the previous slice): issued from inline assembly, because the compiler orders every
    // LDS read behind a pending global -> LDS load it knows of (it cannot tell that the regions are disjoint) and would
    // wait for the slice right away.  The caller waits (vmcnt) and passes a barrier before anybody reads the buffer.
    auto copy_slice_unseen = [&](unsigned char *dst, int g0, int ng) __attribute__((always_inline)) {
        for (int p0 = wave * 64; p0 < kSlabN * kPieces; p0 += kWaves * 64) {
            const int p = p0 + lane;
            const int row = p / kPieces, col = p - row * kPieces;
            const int n = min(n_base + row, N - 1);
            const __half *src = w_hat + static_cast<int64_t>(n) * K + g0 * 64 + col * 8;
            const uint32_t lds = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                (__attribute__((address_space(3))) unsigned char *)(dst + p0 * 16))));      // wave-uniform
            if (col < 8 * ng && row < kSlabN)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
        }
    };

    // x_hat fragments: lane (lr, lh) reads, for k-step kk of group g, piece 8 g + 4 lh + kk of row lr of its block
    // (k = 64 g + 32 lh + 8 kk ... + 7).  A last block of fewer than 32 rows is stored compactly: its pieces are
    // `rows` apart instead of 32, and the lanes past its last row re-read that row (their outputs are not stored).
    // Address of this lane's first piece of block b0 + nb (group 0, k-step 0) and the distance between k-steps.
    auto set_blocks = [&](auto nbc, const int b0, const char *(&xbase)[decltype(nbc)::value], int (&kstep)[decltype(nbc)::value]) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int blk = min(b0 + nb, total_blocks - 1);
            const int rows = min(32, M - blk * 32);
            kstep[nb] = rows * 16;
            xbase[nb] = reinterpret_cast<const char *>(xb) + static_cast<int64_t>(blk) * K * 64 + lh * 4 * kstep[nb] +
                        min(lr, rows - 1) * 16;
        }
    };
    // The first group's fragments, requested in the order in which the group loop refills the slots (the scheduling
    // barriers pin it).  The compiler's wait-count bookkeeping merges this state with the loop's own at the top of the
    // group loop and waits for the stricter of the two: with the loads in any other order here (left alone it
    // reverses them) that is vmcnt(0) in every iteration, i.e. no load is ever left in flight across a group.
    auto first_fragments = [&](auto nbc, u32x4_t (&xs)[4][decltype(nbc)::value], const char *const (&xbase)[decltype(nbc)::value],
                               const int (&kstep)[decltype(nbc)::value]) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                xs[kk][nb] = *reinterpret_cast<const u32x4_t *>(xbase[nb] + kk * kstep[nb]);
                __builtin_amdgcn_sched_barrier(0);
            }
    };
    auto fill_slice = [&](int g0, int ng) __attribute__((always_inline)) {
        __syncthreads();      // every wave is done reading the previous slice
        copy_slice(slab, g0, ng);
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): the slice has landed in LDS
        asm volatile("" ::: "memory");
        __syncthreads();
    };

    // The groups [g0, g0 + ng) of the resident slice times NB row blocks and NJ column tiles from tile jb.  Slot kk is
    // refilled, right after the MFMAs that read it, with k-step kk of the next group; after the last group of the
    // tensor (g == G - 1) with group 0 of the blocks at xnext (the wave's next pass, or any valid address).
    auto multiply_slice = [&](auto nbc, auto njc, float16_t (&acc)[decltype(nbc)::value][decltype(njc)::value],
                              u32x4_t (&xs)[4][decltype(nbc)::value], const char *const (&xbase)[decltype(nbc)::value],
                              const int (&kstep)[decltype(nbc)::value], const char *const (&xnext)[decltype(nbc)::value],
                              const int (&knext)[decltype(nbc)::value], const int g0, const int ng, const int jb,
                              const unsigned char *slab_cur) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
        constexpr int NJ = decltype(njc)::value;
        const unsigned char *slab_wave = slab_cur + lane_off + jb * 32 * kPitch;
        half8_t bf[2][NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) bf[0][j] = *reinterpret_cast<const half8_t *>(slab_wave + j * 32 * kPitch);
        // A wave that multiplies goes before the waves of its SIMD that copy or write out: those wait for memory
        // most of the time anyway, while every issue slot this one loses idles the matrix pipe (measured 2-9 %).
        __builtin_amdgcn_s_setprio(2);
        for (int gl = 0; gl < ng; ++gl) {
            const bool wrap = g0 + gl + 1 >= G;
            const char *rbase[NB];
            int rstep[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                rstep[nb] = wrap ? knext[nb] : kstep[nb];
                rbase[nb] = wrap ? xnext[nb] : xbase[nb] + (g0 + gl + 1) * 8 * kstep[nb];
            }
            const unsigned char *bsrc = slab_wave + gl * 128;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                // w_hat fragments of the next k-step (of the next group after the fourth; past the slice after its
                // last one: read and never used)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    bf[(kk + 1) & 1][j] = *reinterpret_cast<const half8_t *>(bsrc + j * 32 * kPitch + (kk + 1) * 16 + (kk == 3 ? 64 : 0));
                half8_t af[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) __builtin_memcpy(&af[nb], &xs[kk][nb], 16);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        acc[nb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[kk & 1][j], af[nb], acc[nb][j], 0, 0, 0);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    xs[kk][nb] = *reinterpret_cast<const u32x4_t *>(rbase[nb] + kk * rstep[nb]);
#pragma unroll
                for (int q = 0; q < NB * NJ; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                     // 1 MFMA
                    if (q < NJ) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);         // 1 LDS read
                    if (q >= NB * NJ - NB) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // 1 global load
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // The NB blocks from b0 (32 x 32 NJ values each, columns from tile jb) leave in chunks of 128 bytes per row through
    // the wave's private staging tile (LDS operations of one wave execute in order: no wait is needed between them).
    auto write_out = [&](auto nbc, auto njc, const float16_t (&acc)[decltype(nbc)::value][decltype(njc)::value],
                         const int b0, const int jb) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
        constexpr int NJ = decltype(njc)::value;
        constexpr int kChunkCols = 128 / static_cast<int>(sizeof(TOUT));     // 64 (fp16) / 32 (fp32)
        constexpr int kChunks = NJ * 32 / kChunkCols;
        constexpr int kBlocksPerChunk = kChunkCols / 32;
        constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));
        // Whole 16-byte pieces everywhere in this slab (wave-uniform): the common case takes no per-piece branch.
        const bool whole = (N % kVec) == 0 && n_base + kSlabN <= N;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int pblk = b0 + nb;
#pragma unroll
            for (int ch = 0; ch < kChunks; ++ch) {
                // Bias values first: the compiler cannot tell the bias reads from the staging writes (both LDS) and
                // would otherwise wait for each read in turn.
                float4 bv[kBlocksPerChunk][4];
#pragma unroll
                for (int jj = 0; jj < kBlocksPerChunk; ++jj)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        bv[jj][q] = *reinterpret_cast<const float4 *>(s_bias + (jb + ch * kBlocksPerChunk + jj) * 32 + 8 * q + 4 * lh);
#pragma unroll
                for (int jj = 0; jj < kBlocksPerChunk; ++jj) {
                    const int j = ch * kBlocksPerChunk + jj;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int cl = jj * 32 + 8 * q + 4 * lh;            // column inside the chunk
                        const float o0 = acc[nb][j][4 * q] + bv[jj][q].x, o1 = acc[nb][j][4 * q + 1] + bv[jj][q].y;
                        const float o2 = acc[nb][j][4 * q + 2] + bv[jj][q].z, o3 = acc[nb][j][4 * q + 3] + bv[jj][q].w;
                        unsigned char *dst = stage + lr * kStageRow + cl * static_cast<int>(sizeof(TOUT));
                        if constexpr (sizeof(TOUT) == 2) {
                            const __half2 lo = __floats2half2_rn(o0, o1), hi = __floats2half2_rn(o2, o3);
                            u32x2_t pk;
                            pk[0] = *reinterpret_cast<const uint32_t *>(&lo);
                            pk[1] = *reinterpret_cast<const uint32_t *>(&hi);
                            *reinterpret_cast<u32x2_t *>(dst) = pk;
                        } else {
                            u32x4_t pk;
                            pk[0] = __float_as_uint(o0); pk[1] = __float_as_uint(o1);
                            pk[2] = __float_as_uint(o2); pk[3] = __float_as_uint(o3);
                            *reinterpret_cast<u32x4_t *>(dst) = pk;
                        }
                    }
                }
                __builtin_amdgcn_wave_barrier();
                if constexpr (NQ != 0) {
                    const int c0 = n_base + jb * 32 + ch * kChunkCols;          // the chunk is one group of the consumer's rows
                    if (c0 < N)
                        next_quant_chunk<NQ>(nq_lds, kWaves, stage, kStageRow, lane, gelu != 0, 1.0e-6f,
                                             reinterpret_cast<__half *>(y) + static_cast<int64_t>(pblk) * 32 * N,
                                             min(32, M - pblk * 32), c0 / 8);
                    __builtin_amdgcn_wave_barrier();
                    continue;
                }
                const int col = n_base + jb * 32 + ch * kChunkCols + (lane & 7) * kVec;
                const int row0 = pblk * 32 + (lane >> 3);
                TOUT *dst0 = y + static_cast<int64_t>(row0) * N + col;
                u32x4_t v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[i] = *reinterpret_cast<const u32x4_t *>(stage + (i * 8 + (lane >> 3)) * kStageRow + (lane & 7) * 16);
                if (residual || gelu) {          // wave-uniform
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (row0 + i * 8 < M && col < N)
                            post_ops16<TOUT>(v[i], residual ? residual + static_cast<int64_t>(row0 + i * 8) * N + col : nullptr,
                                             gelu != 0, (N % kVec) == 0 ? kVec : N - col);
                }
                if (whole) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (row0 + i * 8 < M)
                            store_streaming16(dst0 + static_cast<int64_t>(i) * 8 * N, v[i][0], v[i][1], v[i][2], v[i][3]);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (row0 + i * 8 < M && col < N) {
                            TOUT *dst = dst0 + static_cast<int64_t>(i) * 8 * N;
                            if ((N % kVec) == 0 && col + kVec <= N) {
                                store_streaming16(dst, v[i][0], v[i][1], v[i][2], v[i][3]);
                            } else {
                                const TOUT *e = reinterpret_cast<const TOUT *>(&v[i]);
#pragma unroll
                                for (int k = 0; k < kVec; ++k)
                                    if (col + k < N) dst[k] = e[k];
                            }
                        }
                    }
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    };

    // ---- slab protocol ----
    // One buffer (DB == false): a slice is copied between two barriers while nobody multiplies; a slab that holds all
    // of K is copied once and stays; the first slice of the next pass is requested before the write-out of this one.
    // Two buffers (DB == true): while slice s is multiplied from one buffer the other receives what is needed next
    // (slice s + 1, or after the last slice the first slice of the pass that follows), requested from inline assembly
    // right after the barrier that freed that buffer.  At the slice's end a wave waits until its own share of the copy
    // has landed -- vmcnt(4 NB): its only younger vector-memory operations are the 4 NB fragment loads of its last
    // group, which may stay in flight -- and one barrier publishes the buffer.  `cur` = buffer of the slice to multiply.
    int cur = 0;
    auto slab_at = [&](int i) { return slab + i * kSlabBytes; };
    // The slices of one pass.  On entry slice 0 is resident (in buffer `cur` when DB); `then_first` = after the last
    // slice, the first slice is made resident again for a pass that follows.  Every wave of the workgroup runs this
    // once per pass with the same `then_first`; the barriers are the same in every instantiation.
    auto run_slices = [&](auto nbc, auto njc, float16_t (&acc)[decltype(nbc)::value][decltype(njc)::value],
                          u32x4_t (&xs)[4][decltype(nbc)::value], const char *const (&xbase)[decltype(nbc)::value],
                          const int (&kstep)[decltype(nbc)::value], const char *const (&xnext)[decltype(nbc)::value],
                          const int (&knext)[decltype(nbc)::value], const int b0, const int jb, const bool live,
                          const bool then_first) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
        for (int sl = 0; sl < slices; ++sl) {
            const int g0 = sl * kSliceGroups;
            const bool last = sl + 1 == slices;
            if constexpr (DB) {
                if (!last) copy_slice_unseen(slab_at(cur ^ 1), g0 + kSliceGroups, min(kSliceGroups, G - g0 - kSliceGroups));
                else if (then_first) copy_slice_unseen(slab_at(cur ^ 1), 0, min(kSliceGroups, G));
                if (live) multiply_slice(nbc, njc, acc, xs, xbase, kstep, xnext, knext, g0, min(kSliceGroups, G - g0), jb, slab_at(cur));
                if (!last) {
                    if (live) wait_vmcnt<4 * NB>(); else wait_vmcnt<0>();
                    __syncthreads();
                    cur ^= 1;
                }
            } else {
                if (live) multiply_slice(nbc, njc, acc, xs, xbase, kstep, xnext, knext, g0, min(kSliceGroups, G - g0), jb, slab);
                if (!last) fill_slice(g0 + kSliceGroups, min(kSliceGroups, G - g0 - kSliceGroups));
            }
        }
        if constexpr (DB) {
            if (live) write_out(nbc, njc, acc, b0, jb);
            if (then_first) {
                if (live) wait_vmcnt<4 * NB>(); else wait_vmcnt<0>();      // (stores are younger still: some of them are waited for too)
                __syncthreads();
                cur ^= 1;
            }
        } else {
            const bool refill = slices > 1 && then_first;
            if (refill) {
                __syncthreads();      // every wave is done reading the last slice
                copy_slice_unseen(slab, 0, min(kSliceGroups, G));
            }
            if (live) write_out(nbc, njc, acc, b0, jb);
            if (refill) {
                wait_vmcnt<0>();
                __syncthreads();
            }
        }
    };

    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I4 = std::integral_constant<int, 4>;

    // ---- full passes: every wave multiplies a pair of blocks.  The fragment slots run on from one pass into the next
    // (the last group of a pass refills them with the first group of the wave's next pair). ----
    if (full_passes > 0) {
        float16_t acc[2][4];
        u32x4_t xs[4][2];
        const char *xcur[2], *xnxt[2];
        int kcur[2], knxt[2];
        set_blocks(I2{}, blk0 + 2 * wave, xcur, kcur);
        first_fragments(I2{}, xs, xcur, kcur);
        fill_slice(0, min(kSliceGroups, G));
        for (int pass = 0; pass < full_passes; ++pass) {
            const bool more = pass + 1 < full_passes;
            const int b0 = blk0 + pass * 2 * kWaves + 2 * wave;
            if (more) {
                set_blocks(I2{}, b0 + 2 * kWaves, xnxt, knxt);
            } else {          // nothing follows: re-read this pair's last group (lines the wave has just read)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    knxt[nb] = kcur[nb];
                    xnxt[nb] = xcur[nb] + (G - 1) * 8 * kcur[nb];
                }
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[nb][j][v] = 0.0f;
            run_slices(I2{}, I4{}, acc, xs, xcur, kcur, xnxt, knxt, b0, 0, true, more || rest > 0);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                xcur[nb] = xnxt[nb];
                kcur[nb] = knxt[nb];
            }
        }
    }

    // ---- the left-over blocks (fewer than sixteen): one more pass, dealt as pairs, single blocks and column halves.
    // Every wave runs it exactly once, whatever its share. ----
    auto last_pass = [&](auto nbc, auto njc, const int b0, const int jb, const bool live) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
        constexpr int NJ = decltype(njc)::value;
        float16_t acc[NB][NJ];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[nb][j][v] = 0.0f;
        const char *xbase[NB], *xlast[NB];
        int kstep[NB];
        set_blocks(nbc, b0, xbase, kstep);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) xlast[nb] = xbase[nb] + (G - 1) * 8 * kstep[nb];
        u32x4_t xs[4][NB];
        if (live) first_fragments(nbc, xs, xbase, kstep);
        if (full_passes == 0) fill_slice(0, min(kSliceGroups, G));      // (else the last full pass left slice 0 resident)
        run_slices(nbc, njc, acc, xs, xbase, kstep, xlast, kstep, b0, jb, live, false);
    };
    if (rest > 0) {
        const int base = blk0 + full_passes * 2 * kWaves;
        if (rest >= kWaves) {
            // rest - 8 pairs in front, single blocks behind them: pairs + (8 - pairs) waves, 2 pairs + 8 - pairs = rest blocks
            const int pairs = rest - kWaves;
            if (wave < pairs) last_pass(I2{}, I4{}, base + 2 * wave, 0, true);
            else last_pass(I1{}, I4{}, base + 2 * pairs + (wave - pairs), 0, true);
        } else {
            // Fewer blocks than waves: as many as there are spare waves are split into two halves of 64 columns (after
            // full passes only while at most two are split: more waves than that fetching the same x_hat at once cost
            // more than the shorter pass gains).  A half keeps the k order of every output it computes.
            int S = min(rest, kWaves - rest);
            if (passes > 1 && S > 2) S = 0;
            const int W = rest - S;
            if (wave < W) {
                last_pass(I1{}, I4{}, base + wave, 0, true);
            } else {
                const int i = (wave - W) >> 1;
                const bool live = i < S;
                last_pass(I1{}, I2{}, live ? base + W + i : base, ((wave - W) & 1) * 2, live);
            }
        }
    }
}

template <typename TOUT, int WAVES, int SG, bool DB, int NQ = 0>
void launch_pair_t(const GemmArgs &g, hipStream_t stream, const void *w_hat, int ranges, int blocks_per_range)
{
    auto kernel = gemm_pair_kernel<TOUT, WAVES, SG, DB, NQ>;
    constexpr int kSmem = PairCfg<WAVES, SG, DB>::kSmem + (NQ ? next_quant_lds_bytes(NQ) : 0);
    allow_dynamic_lds<gemm_pair_kernel<TOUT, WAVES, SG, DB, NQ>>(kSmem);
    const int n_slabs = (g.N + kSlabN - 1) / kSlabN;
    const int tiles = n_slabs * ranges;
    hipLaunchKernelGGL(kernel, dim3(8 * ((tiles + 7) / 8)), dim3(64 * WAVES), kSmem, stream,
                       static_cast<const __half *>(g.x_hat), g.bias, static_cast<TOUT *>(g.y), g.M, g.N, g.K, ranges,
                       blocks_per_range, static_cast<const __half *>(w_hat), static_cast<const TOUT *>(g.residual),
                       g.gelu ? 1 : 0, g.next_thr, g.next_cb);
}

}  // namespace

// Row ranges of the weight-stationary kernels: `slots` workgroups on the chip at once (one or two per CU).
static void pair_ranges(const GemmArgs &g, int slots, int &ranges, int &blocks_per_range)
{
    const int n_slabs = (g.N + kSlabN - 1) / kSlabN;
    const int total_blocks = (g.M + 31) / 32;
    ranges = slots / n_slabs;
    if (ranges < 1) ranges = 1;
    if (ranges > total_blocks) ranges = total_blocks;
    blocks_per_range = (total_blocks + ranges - 1) / ranges;
    ranges = (total_blocks + blocks_per_range - 1) / blocks_per_range;
}

// Whether the two-blocks-per-wave kernel is the one to run for this shape (weights already reconstructed).
// Measured against gemm_slab8_kernel on the twelve DeiT-S / DeiT-B / ViT-L layer shapes: 8-17 % faster wherever K spans
// several slab slices and a workgroup has at least eight row blocks (DeiT-B qkv 65.7 -> 54.1 us, fc1 85.2 -> 73.0,
// ViT-L qkv 358 -> 325, fc2 444 -> 414), equal within 3 % on the single-slice shapes (K = 384), where the eight-wave
// kernel's finer dealing of 15-19 blocks matters as much as the halved LDS traffic, and on five-block workgroups.
bool gemm_pair_pays(const GemmArgs &g)
{
    int ranges, per;
    pair_ranges(g, device_cus(), ranges, per);
    return g.K > 6 * 64 && per >= 8;
}

// g.x_hat is in the 32-row block layout; w_hat [N,K] fp16 holds the reconstructed weights.
void launch_gemm_pair(const GemmArgs &g, const void *w_hat, hipStream_t stream)
{
    int ranges, per;
    pair_ranges(g, device_cus(), ranges, per);
    // Two slab buffers of three groups measured 0-4 % faster than one of six on every multi-slice shape (DeiT-B fc1
    // 72.3 -> 69.7 us, qkv 55.2 -> 53.7, ViT-L qkv 326 -> 324); ARCQ_PAIR=1 pins the single buffer (tuning aid).
    if (g.next_thr) {          // quantize the output for the next layer (fp16 output; the entry point checked the rest)
        if (g.bits == 4) launch_pair_t<__half, 8, 3, true, 4>(g, stream, w_hat, ranges, per);
        else if (g.bits == 3) launch_pair_t<__half, 8, 3, true, 3>(g, stream, w_hat, ranges, per);
        else launch_pair_t<__half, 8, 3, true, 2>(g, stream, w_hat, ranges, per);
        return;
    }
    const char *e = tuning().pair;
    const bool db = e ? e[0] != '1' : true;
    if (db) {
        if (g.y_f16) launch_pair_t<__half, 8, 3, true>(g, stream, w_hat, ranges, per);
        else launch_pair_t<float, 8, 3, true>(g, stream, w_hat, ranges, per);
        return;
    }
    if (g.y_f16) launch_pair_t<__half, 8, 6, false>(g, stream, w_hat, ranges, per);
    else launch_pair_t<float, 8, 6, false>(g, stream, w_hat, ranges, per);
}

}  // namespace arcq
