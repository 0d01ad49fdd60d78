// Stages 2+3 fused, weight-stationary kernel for x_hat in the 32-row block layout:
//   y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias,   x_hat stored as 16-byte pieces [M/32][K/8][32 rows][8 values]
//   (a last block of r < 32 rows as [K/8][r][8]: the tensor takes exactly M*K values).
//
// In that layout the MFMA fragment of a 32-row block and k-step (lane = row, 8 consecutive k) is one fully coalesced
// 16-byte load per lane (512 contiguous bytes per half wave), so x_hat goes from L2 straight into the operand
// registers: no LDS tile, no LDS writes, no wave-level synchronization.  That frees enough registers and LDS
// bandwidth for EIGHT or TWELVE waves per workgroup (two or three per SIMD), each multiplying one 32-row block at a
// time with the resident 128-column slab; the other waves of a SIMD keep the matrix pipe busy while one waits on L2.
// (With x_hat row-major a fragment load touches 32 rows per instruction, which costs the texture path more than the
// MFMAs it feeds; staging through LDS instead saturates LDS bandwidth at two waves per SIMD.)
//
// Slab handling (a slice of up to 6 groups rebuilt from the packed codes once per workgroup, or copied from weights
// reconstructed beforehand), k order inside a group (lane half h covers k = 32h + 8*step ... + 7 in k-step `step`)
// and operand roles (w_hat is the MFMA "A" operand; accumulator element v of lane l is
// y[m = l%32][n = 32j + 8*(v/4) + 4*(l/32) + v%4]) are those of the four-wave kernel; both accumulate in the same
// k order, so their results are bit-identical.
#include "arcq_common.h"
#include "arcq_gemm.h"
#include "arcq_act_quant_core.h"

#include <stdlib.h>
#include <type_traits>

#ifndef ARCQ_SPLIT_DEFAULT
#define ARCQ_SPLIT_DEFAULT 1
#endif

namespace arcq {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kSlabN = 128;                 // columns per slab
constexpr int kSliceGroups = 6;             // groups per K slice
constexpr int kPitch = kSliceGroups * 128 + 16;   // bytes per slab row: 384 halves + 16 B pad (conflict-free 16-B reads)
constexpr int kSlabBytes = kSlabN * kPitch;       // 100352
constexpr int kTJ = kSlabN / 32;            // 4 column blocks
constexpr int kStageRow = 144;              // bytes per staged output row: 128 + 16 pad
constexpr int kStageTile = 32 * kStageRow;  // 4608 B per wave
constexpr int kHalves = 2 * kSliceGroups;   // half groups (32 codes) per slab row and slice

template <int BITS>
__device__ __forceinline__ void load_codes(const uint8_t *__restrict__ p, uint32_t (&w)[BITS])
{
    if constexpr (BITS == 4) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(p);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
    } else if constexpr (BITS == 2) {
        const u32x2_t v = *reinterpret_cast<const u32x2_t *>(p);
        w[0] = v[0]; w[1] = v[1];
    } else {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
        w[0] = q[0]; w[1] = q[1]; w[2] = q[2];
    }
}

template <int BITS>
__device__ __forceinline__ uint32_t code_at(const uint32_t (&w)[BITS], int q)
{
    const int bit = q * BITS;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + BITS > 32) v |= w[d + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}

// PRE = true: the weights were reconstructed beforehand into a fp16 [N,K] buffer; slab slices are copied,
// global -> LDS directly, instead of rebuilt.
// WAVES = 8 or 12 waves per workgroup (two or three per SIMD).
// AHEAD = 1 or 2: how many k-steps the LDS reads of the w_hat fragments run ahead of the MFMAs that use them (two
// where the registers allow it: the LDS round trip under load is longer than one k-step of four MFMAs).
// NQ = 0, or the bits (2 / 3 / 4) of the activation quantizer of the layer that consumes this one's output: y then
// receives that layer's x_hat in the block layout instead of the output itself (arcq_act_quant_core.h,
// next_quant_chunk); fp16 output, N a multiple of 64, copied weights and eight waves only.
template <int BITS, typename TOUT, bool PRE, int WAVES, int AHEAD, int NQ = 0>
__global__ void __launch_bounds__(64 * WAVES)
gemm_slab8_kernel(const __half *__restrict__ xb, const uint8_t *__restrict__ pw, const float *__restrict__ cb,
                  const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                  const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K,
                  int row_ranges, int blocks_per_range, const __half *__restrict__ w_hat,
                  const TOUT *__restrict__ residual, int gelu, const float *__restrict__ nx_thr, const float *__restrict__ nx_cb)
{
    static_assert(NQ == 0 || (sizeof(TOUT) == 2 && PRE), "the next layer's stage 1: fp16 outputs, copied weights");
    constexpr int L = 1 << BITS;
    constexpr int kWaves = WAVES;
    constexpr bool SPLIT = ARCQ_SPLIT_DEFAULT;                   // left-over blocks are dealt in halves
    constexpr int kThreads = 64 * WAVES;
    constexpr int kStageBytes = kWaves * kStageTile;
    constexpr int kRounds = kSlabN * kHalves / kThreads;       // half groups per thread and slice
    static_assert(kSlabN * kHalves % kThreads == 0, "slice work must divide evenly");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *slab = smem;
    float *lut = reinterpret_cast<float *>(smem + kSlabBytes + kStageBytes);      // [L][64]
    float *s_bias = lut + L * 64;                                                   // [128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int lh = lane >> 5;
    const int G = K / 64;
    const int64_t pcols = static_cast<int64_t>(K) * BITS / 8;

    // Tile = (row range, slab), slab fastest; each XCD (workgroups are dealt to the 8 XCDs round-robin) takes a
    // contiguous run of tiles so that the slabs sharing a row range read x_hat through one L2.
    const int n_slabs = (N + kSlabN - 1) / kSlabN;
    const int tiles = n_slabs * row_ranges;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    // (weights copied from the workspace: slabs in groups that fit L2, see tile_range_slab)
    int tile_range, tile_slab;
    tile_range_slab(tile, n_slabs, row_ranges, PRE ? slab_group_size(n_slabs, K, M, blocks_per_range, kWaves) : n_slabs, tile_range, tile_slab);
    const int n_base = tile_slab * kSlabN;
    const int total_blocks = (M + 31) / 32;
    const int blk0 = tile_range * blocks_per_range;
    const int blk1 = min(total_blocks, blk0 + blocks_per_range);
    // Row blocks of this wave: blk0 + wave, + 8, + 16, ... (one per pass).  Dealing them round-robin instead of in
    // contiguous runs keeps the four SIMDs (waves w, w + 4, w + 8 share one) within one block of each other.
    const int passes = (blk1 - blk0 + kWaves - 1) / kWaves;      // same for all waves: barriers stay uniform
    const int slices = (G + kSliceGroups - 1) / kSliceGroups;

    const unsigned char *slab_lane = slab + lr * kPitch + lh * 64;
    unsigned char *stage = smem + kSlabBytes + wave * kStageTile;

    // Codes and metadata of one slice: fetched into registers first (for the first slice at the very top of the
    // kernel, so that this latency, the codebook's and the first x_hat units' all overlap), converted afterwards.
    // Half group number p = round * threads + tid: consecutive lanes read consecutive pieces of a weight row.
    uint32_t codes[kRounds][BITS];
    float c[kRounds], s[kRounds], m[kRounds];
    auto fetch_slice = [&](int g0) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const int p = r * kThreads + tid;
            const int row = p / kHalves, q = p % kHalves;
            const int n = min(n_base + row, N - 1);
            const int g = min(g0 + (q >> 1), G - 1);
            load_codes<BITS>(pw + static_cast<int64_t>(n) * pcols + g * (8 * BITS) + (q & 1) * (4 * BITS), codes[r]);
            const int64_t mi = static_cast<int64_t>(n) * G + g;
            c[r] = wc[mi];
            s[r] = ws[mi];
            m[r] = wcs[mi];
        }
    };
    if constexpr (!PRE) {
        fetch_slice(0);
        if (tid < 64) {
#pragma unroll
            for (int cc = 0; cc < L; ++cc) lut[cc * 64 + lane] = cb[cc];
        }
    }
    if (tid < kSlabN) s_bias[tid] = (bias && n_base + tid < N) ? bias[n_base + tid] : 0.0f;
    const unsigned char *nq_lds = reinterpret_cast<const unsigned char *>(s_bias + kSlabN);
    if constexpr (NQ != 0)      // (the barriers of the first slab fill publish the tables)
        next_quant_setup<NQ>(nx_thr, nx_cb, reinterpret_cast<unsigned char *>(s_bias + kSlabN), tid, kThreads);
    // PRE: one direct global -> LDS load per slab row (lanes 0..47 carry the row's 48 16-byte pieces, the hardware
    // writes lane l's piece at the wave-uniform LDS base + 16 l); the caller waits for vmcnt and the barrier.
    auto copy_slice = [&](int g0, int ng) __attribute__((always_inline)) {
        const bool active = lane < 8 * ng;
        for (int row = wave; row < kSlabN; row += kWaves) {
            const int n = min(n_base + row, N - 1);
            if (active)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(w_hat + static_cast<int64_t>(n) * K + g0 * 64 + lane * 8),
                    (__attribute__((address_space(3))) void *)(slab + row * kPitch), 16, 0, 0);
        }
    };
    auto dequant_slice = [&](int ng) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const int p = r * kThreads + tid;
            const int row = p / kHalves, q = p % kHalves;
            if ((q >> 1) < ng) {
                // All 32 table lookups of this half group are issued before the first is used.
                const float mg = m[r] * 0.015625f;          // S/64, exact
                float v[32];
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    const uint32_t code = code_at<BITS>(codes[r], e);
                    v[e] = *reinterpret_cast<const float *>(
                        reinterpret_cast<const char *>(lut) + ((code << 8) | (static_cast<uint32_t>(lane) << 2)));
                }
                unsigned char *dst = slab + row * kPitch + q * 64;
#pragma unroll
                for (int q8 = 0; q8 < 4; ++q8) {
                    half8_t hv;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        hv[e] = static_cast<_Float16>(fma_f32(v[q8 * 8 + e] - mg, s[r], c[r]));
                    *reinterpret_cast<half8_t *>(dst + q8 * 16) = hv;
                }
            }
        }
    };

    // x_hat load cursor: the next unit (pass, group) to fetch; it runs two units ahead of the MFMA loop.  A unit is
    // one group of the wave's current 32-row block: four fragments (k-steps) of 16 bytes per lane, 512 contiguous
    // bytes per half wave and k-step.  Past the wave's last block the cursor keeps re-reading a valid block.
    // A last block of fewer than 32 rows is stored compactly ([K/8][rows][8]): its pieces are `rows` apart instead
    // of 32, and the lanes past its last row re-read that row (their outputs are not stored).
    int ld_pass = 0, ld_g = 0;
    const char *ld_base;
    int ld_kstep = 512;                // bytes between the pieces of consecutive k-steps of the current block
    // Blocks of a pass.  A full pass gives every wave one block (32 rows x the slab's 128 columns).  A pass with fewer
    // blocks than waves (the last one of a workgroup) splits as many blocks as there are spare waves into two halves
    // of 64 columns: waves 0 .. W-1 take whole blocks, the pairs after them one block each.  A half keeps the k order
    // of every output it computes, so results do not depend on how a block was dealt.  In a workgroup of one pass
    // this always pays (5 blocks on 8 waves: the busiest SIMD multiplies 9 units per slice instead of 12; proj / fc2
    // of DeiT-S 9.2 -> 8.4 and 25.3 -> 22.7 us); after full passes only while at most two blocks are split (10 blocks:
    // 12.6 -> 11.8 us; with three or four, six or eight waves fetch the same x_hat at once: 19 blocks 19.3 -> 21.0).
    auto assign = [&](int pass, int &blk, int &jb, int &nj) {
        const int base = blk0 + pass * kWaves;
        const int nb = min(kWaves, blk1 - base);
        int S = (SPLIT && nb > 0) ? min(nb, kWaves - nb) : 0;
        if (passes > 1 && S > 2) S = 0;          // (measured: see launch_slab8)
        const int W = nb - S;
        if (wave < W || !SPLIT) {
            blk = base + wave;
            jb = 0;
            nj = kTJ;
        } else {
            const int i = (wave - W) >> 1;
            blk = i < S ? base + W + i : blk1;
            jb = ((wave - W) & 1) * (kTJ / 2);
            nj = kTJ / 2;
        }
    };
    auto set_base = [&](int pass) {
        int ablk, ajb, anj;
        assign(pass, ablk, ajb, anj);
        const int blk = min(ablk, total_blocks - 1);
        const int rows = min(32, M - blk * 32);
        ld_kstep = rows * 16;
        ld_base = reinterpret_cast<const char *>(xb) + static_cast<int64_t>(blk) * K * 64 + lh * 4 * ld_kstep +
                  min(lr, rows - 1) * 16;
    };
    auto load_unit = [&](u32x4_t (&r)[4]) {
        const char *p = ld_base + ld_g * (8 * ld_kstep);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) r[kk] = *reinterpret_cast<const u32x4_t *>(p + kk * ld_kstep);
        if (++ld_g == G) {
            ld_g = 0;
            if (ld_pass + 1 < passes) set_base(++ld_pass);
        }
    };

    u32x4_t r0[4], r1[4], r2[4];       // ring: the unit being multiplied, the next one, the one after
    set_base(0);
    load_unit(r0);
    load_unit(r1);

    // One pass of one wave over NJ of the slab's four 32-column tiles, starting at tile jb.  Every wave of the
    // workgroup runs this once per pass, whatever its NJ: the barriers inside are the same in every instantiation.
    auto run_pass = [&](auto njc, const int pass, const int pblk, const int jb, const bool live) __attribute__((always_inline)) {
        constexpr int NJ = decltype(njc)::value;
        const unsigned char *slab_wave = slab_lane + jb * 32 * kPitch;
        float16_t acc[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;

        // One unit = one group = four k-steps of 4 MFMAs.  Every k-step also issues the LDS reads of the w_hat
        // fragments needed AHEAD k-steps later; k-step 1 fetches the unit two ahead into the ring slot the previous
        // unit used.  Slots 0 .. AHEAD - 1 of `bf` hold the fragments of (gl, k-steps 0 .. AHEAD - 1) on entry and of
        // (gl + 1, the same k-steps) on exit.
        constexpr int kSlots = 2 * AHEAD;
        half8_t bf[kSlots][NJ];
        auto unit = [&](const u32x4_t (&cur_set)[4], u32x4_t (&load_set)[4], int gl) {
            const unsigned char *bsrc = slab_wave + gl * 128;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int t = kk + AHEAD;           // the k-step whose fragments are read now; t >= 4: of the next group
                const int off = t < 4 ? t * 16 : 128 + (t - 4) * 16;      // (past the slice on its last unit: unused)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    bf[t % kSlots][j] = *reinterpret_cast<const half8_t *>(bsrc + j * 32 * kPitch + off);
                if (kk == 1) load_unit(load_set);
                half8_t af;
                __builtin_memcpy(&af, &cur_set[kk], 16);
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[kk % kSlots][j], af, acc[j], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < NJ; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 // 1 LDS read
                    if (kk == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);    // 1 global load
                }
            }
        };

        for (int sl = 0; sl < slices; ++sl) {
            const int g0 = sl * kSliceGroups;
            const int ng = min(kSliceGroups, G - g0);
            if (!(slices == 1 && pass > 0)) {
                if constexpr (PRE) {
                    __syncthreads();      // every wave is done reading the previous slice
                    copy_slice(g0, ng);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                } else {
                    if (!(pass == 0 && sl == 0)) fetch_slice(g0);
                    __syncthreads();      // every wave is done reading the previous slice (and the LUT is filled)
                    dequant_slice(ng);
                    __syncthreads();
                }
            }
            if (!live) continue;        // (once past its last block a wave stays past it: the ring no longer matters)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int a = 0; a < AHEAD; ++a)
                    bf[a][j] = *reinterpret_cast<const half8_t *>(slab_wave + j * 32 * kPitch + a * 16);
            // The ring is walked with fixed register names, three units at a time; every slice but the last has
            // six units, and a last slice that is not a multiple of three rotates the ring back into place.
            for (int gl = 0; gl < ng; gl += 3) {
                unit(r0, r2, gl);
                if (gl + 1 < ng) unit(r1, r0, gl + 1);
                if (gl + 2 < ng) unit(r2, r1, gl + 2);
            }

            const int rot = ng % 3;
            if (rot == 1) {             // r0 consumed (r2 refilled): next unit is in r1, the one after in r2
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4_t a0 = r1[t], a1 = r2[t];
                    r0[t] = a0;
                    r1[t] = a1;
                }
            } else if (rot == 2) {      // r0, r1 consumed (r2, r0 refilled): next unit is in r2, the one after in r0
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4_t a0 = r2[t], a1 = r0[t];
                    r0[t] = a0;
                    r1[t] = a1;
                }
            }
        }

        // ---- epilogue of this pass: the 32 x 128 block leaves in chunks of 128 bytes per row through the wave's
        // private staging tile (LDS operations of one wave execute in order: no wait is needed between them) ----
        constexpr int kChunkCols = 128 / static_cast<int>(sizeof(TOUT));     // 64 (fp16) / 32 (fp32)
        constexpr int kChunks = NJ * 32 / kChunkCols;
        constexpr int kBlocksPerChunk = kChunkCols / 32;
        constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));
        if (live) {
            // Whole 16-byte pieces everywhere in this slab (wave-uniform): the common case takes no per-piece branch.
            const bool whole = (N % kVec) == 0 && n_base + kSlabN <= N;
#pragma unroll
            for (int ch = 0; ch < kChunks; ++ch) {
                // Bias values first, a batch at a time (the whole chunk with eight waves; one 32-column block with
                // twelve, which have fewer registers): the compiler cannot tell the bias reads from the staging writes
                // (both LDS) and would otherwise wait for each read in turn.
                constexpr int kBiasBatch = WAVES == 8 ? kBlocksPerChunk : 1;
#pragma unroll
                for (int cb = 0; cb < kBlocksPerChunk; cb += kBiasBatch) {
                    float4 bv[kBiasBatch][4];
#pragma unroll
                    for (int jj = 0; jj < kBiasBatch; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            bv[jj][q] = *reinterpret_cast<const float4 *>(s_bias + (jb + ch * kBlocksPerChunk + cb + jj) * 32 + 8 * q + 4 * lh);
#pragma unroll
                    for (int jj = 0; jj < kBiasBatch; ++jj) {
                        const int j = ch * kBlocksPerChunk + cb + jj;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int cl = (cb + jj) * 32 + 8 * q + 4 * lh;            // column inside the chunk
                            const float o0 = acc[j][4 * q] + bv[jj][q].x, o1 = acc[j][4 * q + 1] + bv[jj][q].y;
                            const float o2 = acc[j][4 * q + 2] + bv[jj][q].z, o3 = acc[j][4 * q + 3] + bv[jj][q].w;
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
                constexpr int kStoreBatch = WAVES == 8 ? 4 : 2;       // staged pieces read back before they are stored
#pragma unroll
                for (int ib = 0; ib < 4; ib += kStoreBatch) {
                    u32x4_t v[kStoreBatch];
#pragma unroll
                    for (int i = 0; i < kStoreBatch; ++i)
                        v[i] = *reinterpret_cast<const u32x4_t *>(stage + ((ib + i) * 8 + (lane >> 3)) * kStageRow + (lane & 7) * 16);
                    if (residual || gelu) {          // wave-uniform
#pragma unroll
                        for (int i = 0; i < kStoreBatch; ++i)
                            if (row0 + (ib + i) * 8 < M && col < N)
                                post_ops16<TOUT>(v[i], residual ? residual + static_cast<int64_t>(row0 + (ib + i) * 8) * N + col : nullptr,
                                                 gelu != 0, (N % kVec) == 0 ? kVec : N - col);
                    }
                    if (whole) {
#pragma unroll
                        for (int i = 0; i < kStoreBatch; ++i)
                            if (row0 + (ib + i) * 8 < M)
                                store_streaming16(dst0 + static_cast<int64_t>(ib + i) * 8 * N, v[i][0], v[i][1], v[i][2], v[i][3]);
                    } else {
#pragma unroll
                        for (int i = 0; i < kStoreBatch; ++i) {
                            if (row0 + (ib + i) * 8 < M && col < N) {
                                TOUT *dst = dst0 + static_cast<int64_t>(ib + i) * 8 * N;
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
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    };

    for (int pass = 0; pass < passes; ++pass) {
        int pblk, jb, nj;
        assign(pass, pblk, jb, nj);
        const bool live = pblk < blk1;           // a wave without a block only keeps the barriers company
        if (!SPLIT || nj == kTJ) run_pass(std::integral_constant<int, kTJ>{}, pass, pblk, jb, live);
        else run_pass(std::integral_constant<int, kTJ / 2>{}, pass, pblk, jb, live);
    }
}

template <int BITS, typename TOUT, bool PRE, int WAVES, int AHEAD, int NQ = 0>
void launch_slab8_w(const GemmArgs &g, hipStream_t stream, const void *w_hat)
{
    constexpr int L = 1 << BITS;
    const size_t smem = kSlabBytes + WAVES * kStageTile + L * 64 * sizeof(float) + kSlabN * sizeof(float) +
                        (NQ ? next_quant_lds_bytes(NQ) : 0);
    auto kernel = gemm_slab8_kernel<BITS, TOUT, PRE, WAVES, AHEAD, NQ>;
    allow_dynamic_lds<gemm_slab8_kernel<BITS, TOUT, PRE, WAVES, AHEAD, NQ>>(static_cast<int>(smem));
    // One workgroup per CU where possible: split the 32-row blocks into as many ranges as CUs/slabs allow.
    const int n_slabs = (g.N + kSlabN - 1) / kSlabN;
    const int total_blocks = (g.M + 31) / 32;
    int ranges = device_cus() / n_slabs;
    if (ranges < 1) ranges = 1;
    if (ranges > total_blocks) ranges = total_blocks;
    const int blocks_per_range = (total_blocks + ranges - 1) / ranges;
    ranges = (total_blocks + blocks_per_range - 1) / blocks_per_range;
    const int tiles = n_slabs * ranges;
    hipLaunchKernelGGL(kernel, dim3(8 * ((tiles + 7) / 8)), dim3(64 * WAVES), smem, stream,
                       static_cast<const __half *>(g.x_hat), g.pw, g.cb, g.wc, g.ws, g.wcs, g.bias,
                       static_cast<TOUT *>(g.y), g.M, g.N, g.K, ranges, blocks_per_range,
                       static_cast<const __half *>(w_hat), static_cast<const TOUT *>(g.residual), g.gelu ? 1 : 0,
                       g.next_thr, g.next_cb);
}

// Waves per workgroup.  While one wave of a SIMD writes its block out (2-2.5 us per pass: the stores queue behind
// everybody else's) only the others multiply, so with two waves per SIMD much of the kernel runs one wave per SIMD,
// at the L2-stall-bound rate.  A third wave (12 per workgroup: the copying variant fits 168 VGPRs) keeps two
// multiplying: 5-15 % faster on the DeiT-B / ViT-L shapes (ViT-L fc1 562 -> 506 us, DeiT-B fc2 80.6 -> 68.0), but
// 5-10 % slower where a workgroup has little work to deal out (all four DeiT-S shapes: at most 19 blocks of at most
// 24 groups).  The variant that rebuilds weights in the kernel needs too many registers for three.
template <int BITS, typename TOUT, bool PRE>
void launch_slab8(const GemmArgs &g, hipStream_t stream, const void *w_hat)
{
    if constexpr (PRE) {
        const int n_slabs = (g.N + kSlabN - 1) / kSlabN;
        const int total_blocks = (g.M + 31) / 32;
        const int ranges = max(1, min(device_cus() / n_slabs, total_blocks));
        const int64_t units = static_cast<int64_t>((total_blocks + ranges - 1) / ranges) * (g.K / 64);
        if (units >= 256) {
            launch_slab8_w<BITS, TOUT, PRE, 12, 1>(g, stream, w_hat);
            return;
        }
    }
    launch_slab8_w<BITS, TOUT, PRE, 8, 2>(g, stream, w_hat);
}

}  // namespace

// g.x_hat is in the 32-row block layout; g.M must be positive and g.K a positive multiple of 64.  w_hat != nullptr:
// weights already reconstructed ([N,K] fp16), slab slices are copied from there.
void launch_gemm_slab8(const GemmArgs &g, const void *w_hat, hipStream_t stream)
{
    if (w_hat) {
        const char *e = tuning().pair;           // tuning aid: 0 / 1 pin the choice
        if (e ? e[0] != '0' : gemm_pair_pays(g)) {
            launch_gemm_pair(g, w_hat, stream);
            return;
        }
        if (g.next_thr) {      // quantize the output for the next layer: the eight-wave variant (fp16 output)
            if (g.bits == 4) launch_slab8_w<4, __half, true, 8, 2, 4>(g, stream, w_hat);
            else if (g.bits == 3) launch_slab8_w<4, __half, true, 8, 2, 3>(g, stream, w_hat);
            else launch_slab8_w<4, __half, true, 8, 2, 2>(g, stream, w_hat);
            return;
        }
        if (g.y_f16) launch_slab8<4, __half, true>(g, stream, w_hat);
        else launch_slab8<4, float, true>(g, stream, w_hat);
        return;
    }
    if (g.y_f16) {
        if (g.bits == 4) launch_slab8<4, __half, false>(g, stream, nullptr);
        else if (g.bits == 3) launch_slab8<3, __half, false>(g, stream, nullptr);
        else launch_slab8<2, __half, false>(g, stream, nullptr);
    } else {
        if (g.bits == 4) launch_slab8<4, float, false>(g, stream, nullptr);
        else if (g.bits == 3) launch_slab8<3, float, false>(g, stream, nullptr);
        else launch_slab8<2, float, false>(g, stream, nullptr);
    }
}

}  // namespace arcq
