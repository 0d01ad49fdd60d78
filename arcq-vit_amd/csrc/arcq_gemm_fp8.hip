// Stage 3 of the FP8-operand layer, hand-written for gfx950: y[M,N] = (x8[M,K] * w8[N,K]^T) / w_mult + bias on
// v_mfma_f32_32x32x64_f8f6f4 (OCP E4M3 operands, fp32 accumulation).  The low-precision formulation that
// EXT/arcq_linear_kernel.cu:22-202 points at; no counterpart in the reference.
//
//   x8 as 16-byte pieces [M/32][K/16][32 rows][16 values] (a last block of r < 32 rows as [K/16][r][16]): what
//   arcq_act_quant_fp8_blocked writes;  w8 [N,K] row-major: what arcq_weight_dequant_fp8 writes.
//
// Structure: the weight-stationary kernel with two row blocks per wave and pass (wave tile 64 rows x 128 columns =
// 2 x 4 MFMA blocks, eight waves), as the fp16 kernel of arcq_gemm_pair.hip; byte for byte the same traffic per matrix
// clock: a unit of 128 k-values is 128 bytes of a row (what a group of 64 fp16 values is there) and two MFMAs of 64
// clocks per (row block, column block) where fp16 has four of 32.  A lane (row r = lane % 32, half h = lane / 32)
// holds, for k-step s of unit u, the 32 bytes k = 128 u + 64 s + 32 h ... + 31 of its row, for both operands (the
// instruction pairs the two operands' bytes position by position, so any assignment of k to positions is valid as long
// as both use the same one).  Operand roles are swapped (w8 is the instruction's first operand): accumulator element
// v of lane l is y[m = l % 32][n = 8 (v / 4) + 4 (l / 32) + v % 4].  Every output accumulates its k-steps in ascending
// order in fp32, whatever the pass structure.
#include "arcq_common.h"
#include "arcq_gemm.h"

#include <stdlib.h>
#include <type_traits>

namespace arcq {
namespace {

typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kSlabN = 128;                 // columns per slab
constexpr int kTJ = kSlabN / 32;            // 4 column blocks
constexpr int kStageRow = 144;              // bytes per staged output row: 128 + 16 pad
constexpr int kStageTile = 32 * kStageRow;  // 4608 B per wave

// WAVES waves per workgroup and SG units (of 128 k-values) per K slice of the slab.
// DB: two slab buffers (of SG = 3 units each): the next slice is copied while the current one is multiplied, one
// barrier per slice instead of two and no wait for the copy.
template <int WAVES, int SG, bool DB> struct Fp8Cfg {
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

template <typename TOUT, int WAVES, int SG, bool DB>
__global__ void __launch_bounds__(64 * WAVES)
gemm_fp8_kernel(const uint8_t *__restrict__ xb, const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K,
                int row_ranges, int blocks_per_range, const uint8_t *__restrict__ w_hat, float inv_mult)
{
    constexpr int kWaves = WAVES;
    constexpr int kSliceGroups = SG;
    constexpr int kPieces = Fp8Cfg<WAVES, SG, DB>::kPieces;
    constexpr int kPitch = Fp8Cfg<WAVES, SG, DB>::kPitch;
    constexpr int kSlabBytes = Fp8Cfg<WAVES, SG, DB>::kSlabBytes;
    constexpr int kAllSlabs = Fp8Cfg<WAVES, SG, DB>::kSlabs * kSlabBytes;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *slab = smem;          // DB: two buffers, slab and slab + kSlabBytes
    float *s_bias = reinterpret_cast<float *>(smem + kAllSlabs + kWaves * kStageTile);      // [128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int lh = lane >> 5;
    const int G = K / 128;          // units of 128 k-values (128 bytes of a row)

    // Tile = (row range, slab); each XCD (workgroups are dealt to the 8 XCDs round-robin) takes a contiguous run of
    // tiles, ordered as tile_range_slab describes.
    const int n_slabs = (N + kSlabN - 1) / kSlabN;
    const int tiles = n_slabs * row_ranges;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    int tile_range, tile_slab;
    tile_range_slab(tile, n_slabs, row_ranges, slab_group_size(n_slabs, K / 2, M, blocks_per_range, 2 * kWaves), tile_range, tile_slab);      // (sizes in bytes: K fp8 values = K / 2 fp16 values)
    const int n_base = tile_slab * kSlabN;
    const int total_blocks = (M + 31) / 32;
    const int blk0 = tile_range * blocks_per_range;
    const int blk1 = min(total_blocks, blk0 + blocks_per_range);
    const int nblk = blk1 - blk0;
    const int full_passes = nblk / (2 * kWaves);       // every wave multiplies a pair of blocks
    const int rest = nblk - full_passes * 2 * kWaves;  // 0 .. 15 blocks for one more pass
    const int passes = full_passes + (rest > 0 ? 1 : 0);
    const int slices = (G + kSliceGroups - 1) / kSliceGroups;

    const int lane_off = lr * kPitch + lh * 32;          // this lane's fragment position inside a slab buffer
    unsigned char *stage = smem + kAllSlabs + wave * kStageTile;

    if (tid < kSlabN) s_bias[tid] = (bias && n_base + tid < N) ? bias[n_base + tid] : 0.0f;
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
                    (const __attribute__((address_space(1))) void *)(w_hat + static_cast<int64_t>(n) * K + g0 * 128 + col * 16),
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
            const uint8_t *src = w_hat + static_cast<int64_t>(n) * K + g0 * 128 + col * 16;
            const uint32_t lds = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                (__attribute__((address_space(3))) unsigned char *)(dst + p0 * 16))));      // wave-uniform
            if (col < 8 * ng && row < kSlabN)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
        }
    };

    // x8 fragments: lane (lr, lh) reads, for k-step s of unit u, the pieces 8 u + 4 s + 2 lh and + 1 of row lr of its
    // block (k = 128 u + 64 s + 32 lh ... + 31); slot i = 2 s + e holds piece 8 u + 4 s + 2 lh + e.  A last block of
    // fewer than 32 rows is stored compactly: its pieces are `rows` apart instead of 32, and the lanes past its last
    // row re-read that row (their outputs are not stored).
    // Address of this lane's first piece of block b0 + nb (group 0, k-step 0) and the distance between k-steps.
    auto set_blocks = [&](auto nbc, const int b0, const char *(&xbase)[decltype(nbc)::value], int (&kstep)[decltype(nbc)::value]) __attribute__((always_inline)) {
        constexpr int NB = decltype(nbc)::value;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int blk = min(b0 + nb, total_blocks - 1);
            const int rows = min(32, M - blk * 32);
            kstep[nb] = rows * 16;
            xbase[nb] = reinterpret_cast<const char *>(xb) + static_cast<int64_t>(blk) * K * 32 + lh * 2 * kstep[nb] +
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
                xs[kk][nb] = *reinterpret_cast<const u32x4_t *>(xbase[nb] + (4 * (kk >> 1) + (kk & 1)) * kstep[nb]);
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
        // The w8 fragment of column block j lives in slot j; right after the MFMAs that read it the slot takes the same
        // block's fragment of the next k-step, so every LDS read has the MFMAs of the other blocks (NB (NJ - 1) of 64
        // clocks) to arrive.
        u32x4_t bf[NJ][2];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 2; ++e) bf[j][e] = *reinterpret_cast<const u32x4_t *>(slab_wave + j * 32 * kPitch + e * 16);
        // A wave that multiplies goes before the waves of its SIMD that copy or write out.
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
            for (int s2 = 0; s2 < 2; ++s2) {
                i32x8_t af[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    __builtin_memcpy(&af[nb], &xs[2 * s2][nb], 16);
                    __builtin_memcpy(reinterpret_cast<char *>(&af[nb]) + 16, &xs[2 * s2 + 1][nb], 16);
                }
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    i32x8_t wf;
                    __builtin_memcpy(&wf, &bf[j][0], 16);
                    __builtin_memcpy(reinterpret_cast<char *>(&wf) + 16, &bf[j][1], 16);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        acc[nb][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, af[nb], acc[nb][j], 0, 0, 0, 0, 0, 0);
                    // the next k-step's fragment of this block (of the next unit after the second k-step; past the
                    // slice after its last unit: read and never used)
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        bf[j][e] = *reinterpret_cast<const u32x4_t *>(bsrc + j * 32 * kPitch + (s2 + 1) * 64 + e * 16);
                }
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        xs[2 * s2 + e][nb] = *reinterpret_cast<const u32x4_t *>(rbase[nb] + (4 * s2 + e) * rstep[nb]);
#pragma unroll
                for (int q = 0; q < NB * NJ; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                       // 1 MFMA
                    if ((q + 1) % NB == 0) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                // 2 LDS reads
                    // the x8 refills go behind the last MFMA that reads the slots they overwrite (issued earlier they
                    // would need registers of their own: the kernel is at the limit of 256)
                    if (q == NB * NJ - 1) __builtin_amdgcn_sched_group_barrier(0x020, 2 * NB, 0);
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
                        // (inv_mult is a power of two: the scaling is exact, the sum rounds once)
                        const float o0 = acc[nb][j][4 * q] * inv_mult + bv[jj][q].x, o1 = acc[nb][j][4 * q + 1] * inv_mult + bv[jj][q].y;
                        const float o2 = acc[nb][j][4 * q + 2] * inv_mult + bv[jj][q].z, o3 = acc[nb][j][4 * q + 3] * inv_mult + bv[jj][q].w;
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
                const int col = n_base + jb * 32 + ch * kChunkCols + (lane & 7) * kVec;
                const int row0 = pblk * 32 + (lane >> 3);
                TOUT *dst0 = y + static_cast<int64_t>(row0) * N + col;
                u32x4_t v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[i] = *reinterpret_cast<const u32x4_t *>(stage + (i * 8 + (lane >> 3)) * kStageRow + (lane & 7) * 16);
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

template <typename TOUT, int WAVES, int SG, bool DB>
void launch_fp8_t(const void *x8, const void *w8, const float *bias, float inv_mult, void *y, int M, int N, int K,
                  hipStream_t stream)
{
    auto kernel = gemm_fp8_kernel<TOUT, WAVES, SG, DB>;
    constexpr int kSmem = Fp8Cfg<WAVES, SG, DB>::kSmem;
    allow_dynamic_lds<gemm_fp8_kernel<TOUT, WAVES, SG, DB>>(kSmem);
    // Row ranges: one workgroup per compute unit (tiles = slabs x ranges ~ the number of compute units).
    const int n_slabs = (N + kSlabN - 1) / kSlabN;
    const int total_blocks = (M + 31) / 32;
    int ranges = device_cus() / n_slabs;
    if (ranges < 1) ranges = 1;
    if (ranges > total_blocks) ranges = total_blocks;
    const int blocks_per_range = (total_blocks + ranges - 1) / ranges;
    ranges = (total_blocks + blocks_per_range - 1) / blocks_per_range;
    const int tiles = n_slabs * ranges;
    hipLaunchKernelGGL(kernel, dim3(8 * ((tiles + 7) / 8)), dim3(64 * WAVES), kSmem, stream,
                       static_cast<const uint8_t *>(x8), bias, static_cast<TOUT *>(y), M, N, K, ranges, blocks_per_range,
                       static_cast<const uint8_t *>(w8), inv_mult);
}

}  // namespace
}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_linear_fp8_blocked(const void *x8_blocked, const void *w8, const float *bias, float w_mult, void *y,
                                     int y_dtype, int64_t M, int64_t N, int64_t K, void *stream)
{
    if (M < 0 || N < 0 || K < 0) return fail(ARCQ_ERR_SHAPE, "arcq_linear_fp8_blocked: negative size");
    if (K % 128 != 0)
        return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fp8_blocked: in_features must be a multiple of 128 (got %lld)",
                    static_cast<long long>(K));
    if (y_dtype != ARCQ_F16 && y_dtype != ARCQ_F32) return fail(ARCQ_ERR_DTYPE, "arcq_linear_fp8_blocked: y must be float16 or float32");
    if (!(w_mult > 0.0f)) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fp8_blocked: w_mult must be positive");
    if (M == 0 || N == 0) return ARCQ_OK;
    if (K == 0) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fp8_blocked: in_features must not be 0");
    if (!x8_blocked || !w8 || !y) return fail(ARCQ_ERR_NULL, "arcq_linear_fp8_blocked: NULL tensor pointer");
    if (M >= (int64_t(1) << 31) - 256 || N >= (int64_t(1) << 31) - 256 || M * K >= (int64_t(1) << 32))
        return fail(ARCQ_ERR_SHAPE, "arcq_linear_fp8_blocked: M, N or K too large");
    if (!aligned(x8_blocked, 16) || !aligned(w8, 16) || !aligned(y, 16))
        return fail(ARCQ_ERR_ALIGN, "arcq_linear_fp8_blocked: x8_blocked, w8 and y must be 16-byte aligned");
    const float inv = 1.0f / w_mult;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (y_dtype == ARCQ_F16)
        launch_fp8_t<__half, 8, 3, true>(x8_blocked, w8, bias, inv, y, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), st);
    else
        launch_fp8_t<float, 8, 3, true>(x8_blocked, w8, bias, inv, y, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), st);
    return launch_status("arcq_linear_fp8_blocked");
}
