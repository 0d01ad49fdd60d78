// Stage 1: activation group-residual quantizer (semantics:
// EXT/arcq_activation_kernel.cu:24-184; fused quantize+reconstruct as in
// FQ/arcq_packed_triton.py:123-178).
//
// Per group of gs input channels of one token:
//   mu = (x0 + x1 + ... ) / gs           serial, left to right
//   s  = sqrt((sum_j (x_j - mu)^2) / gs + eps)
//   t_j = (x_j - mu) / s                 correctly rounded
//   code_j = number of leading thresholds with t_j > thr[i]
//   S = sum_j cb[code_j]                 serial
//   x_hat_j = fma(s, cb[code_j] - S/gs, mu)
//
// gs == 64 kernel.  x is [rows, G*64], so the groups of the whole tensor are consecutive 64-element
// runs of one flat array.  A wave owns a tile of 64 consecutive groups and gives every lane ONE group,
// so the serial sums are plain register loops (64 independent chains per wave).  Data moves between
// the coalesced global layout (16-byte accesses) and the lane-per-group layout through a per-wave LDS
// tile whose row stride is odd in dwords (33 for fp16, 65 for fp32), which makes both the row-wise
// 16-byte phase and the per-lane column phase bank-conflict free.
//
// Two things keep the per-element VALU work low without changing a single result bit:
//  * t = d/s is evaluated as three fused corrections of d * RN(1/s) (q0 = d*y; e = fma(-s,q,d);
//    q = fma(e,y,q), twice).  With y the correctly rounded reciprocal and the second residual exact
//    this yields the correctly rounded quotient (Markstein); lanes whose s or mu fall outside the
//    range where no intermediate can under/overflow take the plain divide instead.
//  * the threshold search is one table lookup plus one compare: t is mapped by a monotone function
//    to one of up to 513 buckets over [-8, 8] (|t| <= 8 always, since s^2 >= d_j^2/64; the bucket width
//    adapts to the smallest gap between thresholds); a bucket stores how
//    many thresholds lie in lower buckets and the single threshold inside it.  Monotonicity makes
//    base + (t > thr_in_bucket) equal to the count of thresholds below t.  (Keeping the two candidate
//    codebook values in the bucket as well saves instructions but measured slower: the wider reads at
//    data-dependent addresses collide in LDS, while the per-lane codebook copy never does.)  If two
//    thresholds share a bucket, a threshold lies outside [-8, 8), or the thresholds are not sorted,
//    the kernel falls back to the compare chain.
// The arithmetic itself lives in arcq_act_quant_core.h (shared with the fused small-M layer kernel).
#include "arcq_act_quant_core.h"
#include "arcq_gemm.h"
#include "arcq_weight_dequant_core.h"

namespace arcq {

constexpr int kWaves = 4;          // waves (tiles in flight) per workgroup
constexpr int kTileGroups = 64;    // groups per tile = lanes per wave
template <typename T> struct Tile;
template <> struct Tile<float> { static constexpr int stride = 65; static constexpr int vec = 4; };
template <> struct Tile<__half> { static constexpr int stride = 33; static constexpr int vec = 8; };

// Coalesced 16-byte global loads of one tile (64 groups x 64 elements) into registers, and from there
// into the wave's LDS tile.  Two steps so that the first tile's loads can be in flight during the
// per-workgroup setup.
template <typename TIN> struct TileRegs { uint4 raw[kTileGroups * 64 / (64 * Tile<TIN>::vec)]; };

template <typename TIN>
__device__ __forceinline__ void fetch_tile(const TIN *__restrict__ x, int64_t elem0, int64_t elem_end,
                                           TileRegs<TIN> &r, int lane)
{
    constexpr int n = Tile<TIN>::vec;
    constexpr int iters = kTileGroups * 64 / (64 * n);
#pragma unroll
    for (int i = 0; i < iters; ++i) {
        const int e = (i * 64 + lane) * n;
        r.raw[i] = (elem0 + e < elem_end) ? *reinterpret_cast<const uint4 *>(x + elem0 + e) : make_uint4(0, 0, 0, 0);
    }
}

template <typename TIN>
__device__ __forceinline__ void commit_tile(const TileRegs<TIN> &r, uint32_t *__restrict__ tile, int lane)
{
    constexpr int n = Tile<TIN>::vec;
    constexpr int iters = kTileGroups * 64 / (64 * n);
#pragma unroll
    for (int i = 0; i < iters; ++i) {
        const int e = (i * 64 + lane) * n;
        uint32_t *dst = tile + (e >> 6) * Tile<TIN>::stride + (e & 63) * static_cast<int>(sizeof(TIN)) / 4;
        dst[0] = r.raw[i].x; dst[1] = r.raw[i].y; dst[2] = r.raw[i].z; dst[3] = r.raw[i].w;
    }
}

template <typename TOUT>
__device__ __forceinline__ void store_tile(TOUT *__restrict__ out, int64_t elem0, int64_t elem_end,
                                           const uint32_t *__restrict__ tile, int lane)
{
    constexpr int n = Tile<TOUT>::vec;
    constexpr int iters = kTileGroups * 64 / (64 * n);
#pragma unroll
    for (int i = 0; i < iters; ++i) {
        const int e = (i * 64 + lane) * n;
        if (elem0 + e >= elem_end) continue;
        const uint32_t *src = tile + (e >> 6) * Tile<TOUT>::stride + (e & 63) * static_cast<int>(sizeof(TOUT)) / 4;
        *reinterpret_cast<uint4 *>(out + elem0 + e) = make_uint4(src[0], src[1], src[2], src[3]);
    }
}

// The lane's own group (row `lane` of the tile) as 64 floats.
template <typename TIN>
__device__ __forceinline__ void read_row(const uint32_t *__restrict__ row, float (&v)[64])
{
    if constexpr (sizeof(TIN) == 4) {
#pragma unroll
        for (int j = 0; j < 64; ++j) v[j] = __uint_as_float(row[j]);
    } else {
#pragma unroll
        for (int p = 0; p < 32; ++p) {
            const uint32_t w = row[p];
            v[2 * p] = __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
            v[2 * p + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
        }
    }
}

template <typename TOUT>
__device__ __forceinline__ void write_row(uint32_t *__restrict__ row, const float (&v)[64])
{
    if constexpr (sizeof(TOUT) == 4) {
#pragma unroll
        for (int j = 0; j < 64; ++j) row[j] = __float_as_uint(v[j]);
    } else {
#pragma unroll
        for (int p = 0; p < 32; ++p) {
            const __half2 h = __floats2half2_rn(v[2 * p], v[2 * p + 1]);
            row[p] = *reinterpret_cast<const uint32_t *>(&h);
        }
    }
}

// Appends the 64 codes (one per array slot) to packed dwords, LSB first.
template <int BITS>
__device__ __forceinline__ void pack64(const uint32_t (&c)[64], uint32_t (&w)[2 * BITS])
{
    if constexpr (BITS == 4 || BITS == 2) {
        constexpr int per = 32 / BITS;
#pragma unroll
        for (int d = 0; d < 2 * BITS; ++d) {
            uint32_t v = 0;
#pragma unroll
            for (int q = 0; q < per; ++q) v |= c[d * per + q] << (BITS * q);
            w[d] = v;
        }
    } else {
        uint32_t ch[8];   // 8 codes -> one 24-bit chunk; 4 chunks -> 3 dwords
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint32_t v = 0;
#pragma unroll
            for (int q = 0; q < 8; ++q) v |= c[k * 8 + q] << (3 * q);
            ch[k] = v;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            w[3 * h + 0] = ch[4 * h + 0] | (ch[4 * h + 1] << 24);
            w[3 * h + 1] = (ch[4 * h + 1] >> 8) | (ch[4 * h + 2] << 16);
            w[3 * h + 2] = (ch[4 * h + 2] >> 16) | (ch[4 * h + 3] << 8);
        }
    }
}

// CODES = false drops everything only the code outputs need (the on-the-fly layer asks for x_hat alone).
// Weight reconstruction carried along by a block-layout stage-1 launch: the first `blocks` workgroups of the grid
// rebuild out[N,K] (fp16) from packed codes instead of quantizing activations.  Both are inputs of the same GEMM and
// independent of each other, so one launch does for two.  blocks == 0: nothing to carry.
struct WeightJob {
    const uint8_t *packed;
    const float *cb, *center, *scale, *code_sum;
    __half *out;
    int64_t N, K;
    unsigned blocks;
};

template <typename TIN, typename TOUT, int BITS, bool CODES>
__global__ void __launch_bounds__(64 * kWaves)
act_quant_g64_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                     uint8_t *__restrict__ packed, uint8_t *__restrict__ codes_u8,
                     float *__restrict__ center, float *__restrict__ scale, float *__restrict__ code_sum,
                     TOUT *__restrict__ x_hat, int64_t total_groups, float eps)
{
    constexpr int L = 1 << BITS;
    constexpr int kStride = (Tile<TIN>::stride > Tile<TOUT>::stride) ? Tile<TIN>::stride : Tile<TOUT>::stride;
    __shared__ uint32_t tiles[kWaves][kTileGroups * kStride];
    __shared__ float lut[L * 64];          // codebook replicated per lane: lut[c*64 + lane], conflict-free
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[kWaves];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    // The first tile of this wave is requested before anything else: its latency overlaps the setup below.
    const int64_t ntiles = (total_groups + kTileGroups - 1) / kTileGroups;
    const int64_t elem_end = total_groups * 64;
    TileRegs<TIN> regs;
    {
        const int64_t first = static_cast<int64_t>(blockIdx.x) * kWaves + wave;
        fetch_tile<TIN>(x, first * kTileGroups * 64, elem_end, regs, lane);      // zero-fills past the end
    }

    // Thresholds and codebook are requested now and first used after the first tile's statistics: the lookup
    // tables are built once per workgroup, between the two halves of the first tile, so that their load latency
    // and the tile's hide behind each other.
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    // The lookup tables are built once per workgroup, before the first tile's values are unpacked into registers.
    // (Built between the two halves of the first tile, or with both orders in the kernel and a flag to choose, the
    // variants that write codes run 20-40 % slower: registers.)
    build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid, 64 * kWaves);
    __syncthreads();
    bool table_ok = true;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) table_ok = table_ok && (slow_slots[w] == 0);

    uint32_t *tile = tiles[wave];

    // All four waves run the same number of iterations so that the barriers below are uniform.
    const int64_t tile_step = static_cast<int64_t>(gridDim.x) * kWaves;
    for (int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kWaves; tile0 < ntiles; tile0 += tile_step) {
        const int64_t group0 = (tile0 + wave) * kTileGroups;
        const int64_t elem0 = group0 * 64;
        commit_tile<TIN>(regs, tile, lane);
        __syncthreads();

        float xv[64];
        read_row<TIN>(tile + lane * Tile<TIN>::stride, xv);
        // The wave's next tile (zeros past the end) loads under this one's arithmetic.
        fetch_tile<TIN>(x, (group0 + tile_step * kTileGroups) * 64, elem_end, regs, lane);

        float mu, var, s, sum_codes;
        uint32_t code[CODES ? 64 : 1];
        group_stats64(xv, eps, mu, var, s);
        group_codes64<BITS, CODES>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes, code);

        const int64_t g = group0 + lane;
        if (g < total_groups) {
            if (center) center[g] = mu;
            if (scale) scale[g] = s;
            if (code_sum) code_sum[g] = sum_codes;
            if constexpr (CODES) {
                if (packed) {
                    uint32_t w[2 * BITS];
                    pack64<BITS>(code, w);
                    uint32_t *dst = reinterpret_cast<uint32_t *>(packed + g * (8 * BITS));
                    if constexpr (BITS == 4) {
                        reinterpret_cast<uint4 *>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
                        reinterpret_cast<uint4 *>(dst)[1] = make_uint4(w[4], w[5], w[6], w[7]);
                    } else if constexpr (BITS == 2) {
                        reinterpret_cast<uint4 *>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
                    } else {
#pragma unroll
                        for (int q = 0; q < 3; ++q)
                            reinterpret_cast<uint2 *>(dst)[q] = make_uint2(w[2 * q], w[2 * q + 1]);
                    }
                }
                if (codes_u8) {
                    uint4 *dst = reinterpret_cast<uint4 *>(codes_u8 + g * 64);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        uint32_t d[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int b = q * 16 + k * 4;
                            d[k] = code[b] | (code[b + 1] << 8) | (code[b + 2] << 16) | (code[b + 3] << 24);
                        }
                        dst[q] = make_uint4(d[0], d[1], d[2], d[3]);
                    }
                }
            }
        }

        if (x_hat) {
            const float code_mean = sum_codes * 0.015625f;
#pragma unroll
            for (int j = 0; j < 64; ++j) xv[j] = fma_f32(s, xv[j] - code_mean, mu);
            // Every lane has consumed its input row (program order within the wave), so rows may be
            // rewritten now, possibly with a different stride.
            write_row<TOUT>(tile + lane * Tile<TOUT>::stride, xv);
            __syncthreads();
            store_tile<TOUT>(x_hat, elem0, elem_end, tile, lane);
        }
        __syncthreads();   // the tile is reloaded in the next iteration
    }
}

// Small launches, x_hat only: two lanes per group, no LDS tile.  When the tensor is too small to fill the chip
// (a few hundred rows) the launch lasts as long as one lane's instruction chain, so the group is shared by two lanes
// (arcq_act_quant_core.h: half the per-element work per lane, the serial sums in two linked phases, same bits).  A
// lane's 32 inputs are contiguous and consecutive lanes hold consecutive halves, so plain 16-byte loads and stores
// are already coalesced.  Every lane reads all its inputs before it writes, so x_hat may alias x.
template <typename TIN, typename TOUT, int BITS>
__global__ void __launch_bounds__(64 * kWaves)
act_quant_small_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                       TOUT *__restrict__ x_hat, int64_t total_groups, float eps)
{
    constexpr int L = 1 << BITS;
    constexpr int kIn = 32 * sizeof(TIN) / 16, kOut = 32 * sizeof(TOUT) / 16;
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[kWaves];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int64_t f = (static_cast<int64_t>(blockIdx.x) * kWaves + (tid >> 6)) * 32 + (lane >> 1);   // this lane's group
    const bool valid = f < total_groups;
    const int64_t e0 = f * 64 + (lane & 1) * 32;                                                    // its first element

    uint4 raw[kIn];
#pragma unroll
    for (int i = 0; i < kIn; ++i)
        raw[i] = valid ? reinterpret_cast<const uint4 *>(x + e0)[i] : make_uint4(0, 0, 0, 0);
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    // The tables are built while the inputs are still on their way: their latency and the build's overlap (-0.2 us).
    build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid, 64 * kWaves);
    __syncthreads();

    float xv[32];
    if constexpr (sizeof(TIN) == 2) {
#pragma unroll
        for (int i = 0; i < kIn; ++i) {
            const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                xv[i * 8 + 2 * d] = __half2float(__ushort_as_half(static_cast<unsigned short>(w[d] & 0xffffu)));
                xv[i * 8 + 2 * d + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w[d] >> 16)));
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < kIn; ++i) {
            xv[4 * i] = __uint_as_float(raw[i].x); xv[4 * i + 1] = __uint_as_float(raw[i].y);
            xv[4 * i + 2] = __uint_as_float(raw[i].z); xv[4 * i + 3] = __uint_as_float(raw[i].w);
        }
    }
    float mu, var, s, sum_codes;
    group_stats32x2(xv, eps, mu, var, s);
    bool table_ok = true;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) table_ok = table_ok && (slow_slots[w] == 0);
    group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
    const float code_mean = sum_codes * 0.015625f;
#pragma unroll
    for (int j = 0; j < 32; ++j) xv[j] = fma_f32(s, xv[j] - code_mean, mu);
    if (!valid) return;
    uint4 *dst = reinterpret_cast<uint4 *>(x_hat + e0);
    if constexpr (sizeof(TOUT) == 2) {
#pragma unroll
        for (int i = 0; i < kOut; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const __half2 h = __floats2half2_rn(xv[i * 8 + 2 * d], xv[i * 8 + 2 * d + 1]);
                w[d] = *reinterpret_cast<const uint32_t *>(&h);
            }
            store_writethrough16(dst + i, w[0], w[1], w[2], w[3]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kOut; ++i)
            store_writethrough16(dst + i, __float_as_uint(xv[4 * i]), __float_as_uint(xv[4 * i + 1]),
                                 __float_as_uint(xv[4 * i + 2]), __float_as_uint(xv[4 * i + 3]));
    }
}

// Block-layout stage 1 with two lanes per group.  A wave tile is 32 rows x ONE group; lane l owns row l / 2 and the
// half l % 2 of the group (arcq_act_quant_core.h: two-phase serial sums, same bits as one lane per group).  Halving
// the tile doubles the number of work items, which is what the K = 384 layers of DeiT-S need: 1 182 whole tiles on
// 1 024 SIMDs leave 158 SIMDs with two tiles (2 x 1 470 instructions), 2 364 half tiles at most three (3 x 740).
// Data moves through a wave-private LDS tile (rows of the tile = rows of the tensor, odd dword pitch): coalesced
// 16-byte loads in, every piece column out as one 512-byte run of the block layout.
template <typename TIN, int BITS, bool BUILDER>
__global__ void __launch_bounds__(64 * (kWaves + (BUILDER ? 1 : 0)))
act_quant_blocked2_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                          __half *__restrict__ x_hat, float eps, int groups_per_row, int64_t rows, WeightJob wj)
{
    constexpr int L = 1 << BITS;
    constexpr int kInPitch = Tile<TIN>::stride, kOutPitch = Tile<__half>::stride;     // dwords per tile row
    constexpr int kPieces = 64 / Tile<TIN>::vec;           // 16-byte pieces per row of the tile (8 fp16 / 16 fp32)
    constexpr int kRowsPerInstr = 64 / kPieces;            // 8 / 4
    constexpr int kIters = 32 / kRowsPerInstr;             // 4 / 8
    __shared__ uint32_t tiles[kWaves][32 * kInPitch];
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[kWaves];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    if (blockIdx.x < wj.blocks) {          // workgroup-uniform: this workgroup rebuilds weights and is done
        if (!BUILDER || wave < kWaves)     // (256 threads per weight block; the fifth wave has nothing to do, and the
            weight_dequant8_block<__half, BITS, 64 * kWaves>(blockIdx.x, lut, wj.packed, wj.cb, wj.center, wj.scale,
                                                             wj.code_sum, wj.out, wj.N, wj.K, 64);
        else                               //  routine's barrier is counted per workgroup: it joins it)
            __syncthreads();
        return;
    }
    // BUILDER: the workgroup has a fifth wave that owns no tile; it builds the lookup tables while the four tile waves
    // load their first tile and take its statistics, meets them at the one barrier of the kernel, and is done.  That
    // takes the table construction (a third of a half tile's instruction chain) off every tile wave's path.  Without
    // it the four tile waves build the tables together between the two halves of their first tile.
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    if (BUILDER && wave == kWaves) {
        build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, lane, 64);
        __syncthreads();
        return;
    }
    const int64_t wg = blockIdx.x - wj.blocks;
    const int64_t act_blocks = gridDim.x - wj.blocks;
    const int64_t ntiles = ((rows + 31) / 32) * groups_per_row;
    const int64_t row_elems = static_cast<int64_t>(groups_per_row) * 64;
    uint32_t *tile = tiles[wave];

    uint4 raw[kIters];
    auto fetch = [&](int64_t t) {          // tile t = (row block t / G, group t % G); zero-fills past the end
        const int64_t rb = t / groups_per_row;
        const int g = static_cast<int>(t - rb * groups_per_row);
        const int64_t r0 = rb * 32 + lane / kPieces;
        const TIN *p = x + r0 * row_elems + g * 64 + (lane % kPieces) * Tile<TIN>::vec;
#pragma unroll
        for (int i = 0; i < kIters; ++i)         // rows past the tensor's end (a ragged last block) read as zeros
            raw[i] = (t < ntiles && r0 + i * kRowsPerInstr < rows) ? *reinterpret_cast<const uint4 *>(p + i * kRowsPerInstr * row_elems)
                                                                   : make_uint4(0, 0, 0, 0);
    };
    fetch(wg * kWaves + wave);
    bool table_ok = false, tables_built = false;
    const int row = lane >> 1, half = lane & 1;
    if constexpr (!BUILDER) {
        // Without a builder wave the four tile waves build the tables first, while their first tile is on its way:
        // nothing else is live in registers yet (building them between the halves of the first tile, with the tile's
        // 32 values held, took 169 VGPRs: two waves per SIMD instead of three).
        build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid, 64 * kWaves);
        __syncthreads();
        table_ok = true;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) table_ok = table_ok && (slow_slots[w] == 0);
        tables_built = true;
    }

    for (int64_t tile0 = wg * kWaves; tile0 < ntiles; tile0 += act_blocks * kWaves) {
        const int64_t t = tile0 + wave;
        {
            uint32_t *dst = tile + (lane / kPieces) * kInPitch + (lane % kPieces) * 4;
#pragma unroll
            for (int i = 0; i < kIters; ++i) {
                uint32_t *d = dst + i * kRowsPerInstr * kInPitch;
                d[0] = raw[i].x; d[1] = raw[i].y; d[2] = raw[i].z; d[3] = raw[i].w;
            }
        }
        __builtin_amdgcn_wave_barrier();      // the tile is private to the wave and LDS operations execute in order
        float xv[32];
        {
            const uint32_t *src = tile + row * kInPitch + half * (32 * static_cast<int>(sizeof(TIN)) / 4);
            if constexpr (sizeof(TIN) == 4) {
#pragma unroll
                for (int j = 0; j < 32; ++j) xv[j] = __uint_as_float(src[j]);
            } else {
#pragma unroll
                for (int p = 0; p < 16; ++p) {
                    const uint32_t w = src[p];
                    xv[2 * p] = __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
                    xv[2 * p + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
                }
            }
        }
        fetch(t + act_blocks * kWaves);       // the wave's next tile (nothing past the end) loads under this one's arithmetic
        float mu, var, s, sum_codes;
        group_stats32x2(xv, eps, mu, var, s);
        if (BUILDER && !tables_built) {       // once per workgroup: the builder wave's tables are ready
            __syncthreads();
            table_ok = (slow_slots[0] == 0);
            tables_built = true;
        }
        group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
        const float code_mean = sum_codes * 0.015625f;
        {
            // Every lane has read its inputs (program order within the wave), so rows may be rewritten, with the
            // output pitch.
            uint32_t *dst = tile + row * kOutPitch + half * 16;
#pragma unroll
            for (int p = 0; p < 16; ++p) {
                const __half2 h = __floats2half2_rn(fma_f32(s, xv[2 * p] - code_mean, mu), fma_f32(s, xv[2 * p + 1] - code_mean, mu));
                dst[p] = *reinterpret_cast<const uint32_t *>(&h);
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (t < ntiles) {
            const int64_t rb = t / groups_per_row;
            const int g = static_cast<int>(t - rb * groups_per_row);
            const int r = lane & 31;
            const int nrows = static_cast<int>(rows - rb * 32 < 32 ? rows - rb * 32 : 32);     // < 32 in a ragged last block,
            __half *base = x_hat + rb * (row_elems * 32) + (static_cast<int64_t>(g) * 8 * nrows + r) * 8;   // stored compactly
            if (r < nrows) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {  // instruction j: piece columns 2j and 2j + 1, nrows x 16 bytes each
                    const int kp = j * 2 + (lane >> 5);
                    const uint32_t *src = tile + r * kOutPitch + kp * 4;
                    store_writethrough16(base + kp * (nrows * 8), src[0], src[1], src[2], src[3]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();      // the tile is refilled in the next iteration
    }
}

// LayerNorm fused in front of the block-layout stage 1.  A workgroup owns one 32-row block and all G = K / 64 groups of
// it, one wave per group (wave tile = 32 rows x one group, two lanes per group, as act_quant_blocked2_kernel), so the
// row statistics LayerNorm needs are a sum over the workgroup: every lane folds its 32 values serially, the 2 G
// partial sums of a row meet in LDS and every lane of the row adds them up in the same fixed order.
//   mean = (sum of the partial sums, group by group, lower half first) / K
//   var  = (the same sum over (x - mean)^2) / K
//   y    = ((x - mean) * (1 / sqrt(var + ln_eps))) * gamma + beta        three roundings, no fma
// y is rounded to the input's type (what a stand-alone LayerNorm kernel would have stored) and then quantized and
// reconstructed exactly as act_quant_blocked2_kernel does.  MAXW = most waves (groups) per workgroup.
template <typename TIN, int BITS, int MAXW>
__global__ void __launch_bounds__(64 * MAXW)
act_quant_rows_ln_kernel(const TIN *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
                         float ln_eps, const float *__restrict__ thr, const float *__restrict__ cb,
                         __half *__restrict__ x_hat, float eps, int G, int64_t rows, WeightJob wj)
{
    constexpr int L = 1 << BITS;
    constexpr int kInPitch = Tile<TIN>::stride, kOutPitch = Tile<__half>::stride;     // dwords per tile row
    constexpr int kPieces = 64 / Tile<TIN>::vec;           // 16-byte pieces per row of the tile (8 fp16 / 16 fp32)
    constexpr int kRowsPerInstr = 64 / kPieces;            // 8 / 4
    constexpr int kIters = 32 / kRowsPerInstr;             // 4 / 8
    extern __shared__ __attribute__((aligned(16))) uint32_t rows_smem[];     // [G][32 * kInPitch] tiles, then [32][2 G + 1] partial sums
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[MAXW];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;          // = this wave's group
    if (blockIdx.x < wj.blocks) {       // workgroup-uniform: this workgroup rebuilds weights and is done
        weight_dequant8_block_n<__half, BITS>(blockIdx.x, 64 * G, lut, wj.packed, wj.cb, wj.center, wj.scale, wj.code_sum,
                                              wj.out, wj.N, wj.K, 64);
        return;
    }
    const int64_t rb = blockIdx.x - wj.blocks;
    const int64_t row_elems = static_cast<int64_t>(G) * 64;
    uint32_t *tile = rows_smem + wave * (32 * kInPitch);
    const int ppitch = 2 * G + 1;
    float *part = reinterpret_cast<float *>(rows_smem + G * (32 * kInPitch));

    uint4 raw[kIters];
    {
        const int64_t r0 = rb * 32 + lane / kPieces;
        const TIN *p = x + r0 * row_elems + wave * 64 + (lane % kPieces) * Tile<TIN>::vec;
#pragma unroll
        for (int i = 0; i < kIters; ++i)         // rows past the tensor's end (a ragged last block) read as zeros
            raw[i] = (r0 + i * kRowsPerInstr < rows) ? *reinterpret_cast<const uint4 *>(p + i * kRowsPerInstr * row_elems)
                                                     : make_uint4(0, 0, 0, 0);
    }
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid, 64 * G);      // while the tile is on its way

    const int row = lane >> 1, half = lane & 1;
    {
        uint32_t *dst = tile + (lane / kPieces) * kInPitch + (lane % kPieces) * 4;
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            uint32_t *d = dst + i * kRowsPerInstr * kInPitch;
            d[0] = raw[i].x; d[1] = raw[i].y; d[2] = raw[i].z; d[3] = raw[i].w;
        }
    }
    __builtin_amdgcn_wave_barrier();      // the tile is private to the wave and LDS operations execute in order
    float xv[32];
    {
        const uint32_t *src = tile + row * kInPitch + half * (32 * static_cast<int>(sizeof(TIN)) / 4);
        if constexpr (sizeof(TIN) == 4) {
#pragma unroll
            for (int j = 0; j < 32; ++j) xv[j] = __uint_as_float(src[j]);
        } else {
#pragma unroll
            for (int p = 0; p < 16; ++p) {
                const uint32_t w = src[p];
                xv[2 * p] = __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
                xv[2 * p + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
            }
        }
    }
    // ---- LayerNorm over the row ----
    const float fk = static_cast<float>(row_elems);
    auto row_total = [&](float mine) {          // sum over the row of every lane's `mine`, in the fixed order; two barriers
        part[row * ppitch + 2 * wave + half] = mine;
        __syncthreads();
        float acc = 0.0f;
        for (int i = 0; i < 2 * G; ++i) acc += part[row * ppitch + i];
        __syncthreads();                        // (the buffer is written again right away)
        return acc;
    };
    float a = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) a += xv[j];
    const float mean = row_total(a) / fk;
    float q = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        xv[j] -= mean;
        const float sq = xv[j] * xv[j];
        q += sq;
    }
    const float var_row = row_total(q) / fk;
    const float rstd = 1.0f / sqrtf(var_row + ln_eps);
    {
        const float4 *gp = reinterpret_cast<const float4 *>(gamma + wave * 64 + half * 32);
        const float4 *bp = reinterpret_cast<const float4 *>(beta + wave * 64 + half * 32);
#pragma unroll
        for (int j4 = 0; j4 < 8; ++j4) {
            const float4 gv = gp[j4], bv = bp[j4];
            const float g4[4] = {gv.x, gv.y, gv.z, gv.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float t = xv[4 * j4 + e] * rstd;
                const float u = t * g4[e];
                float yv = u + b4[e];
                if constexpr (sizeof(TIN) == 2) yv = __half2float(__float2half_rn(yv));     // what a LayerNorm kernel stores
                xv[4 * j4 + e] = yv;
            }
        }
    }
    // ---- stage 1 on the normalized row (the tables were finished before the first barrier above) ----
    bool table_ok = true;
    for (int w = 0; w < G; ++w) table_ok = table_ok && (slow_slots[w] == 0);
    float mu, var, s, sum_codes;
    group_stats32x2(xv, eps, mu, var, s);
    group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
    const float code_mean = sum_codes * 0.015625f;
    {
        uint32_t *dst = tile + row * kOutPitch + half * 16;
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const __half2 h = __floats2half2_rn(fma_f32(s, xv[2 * p] - code_mean, mu), fma_f32(s, xv[2 * p + 1] - code_mean, mu));
            dst[p] = *reinterpret_cast<const uint32_t *>(&h);
        }
    }
    __builtin_amdgcn_wave_barrier();
    {
        const int r = lane & 31;
        const int nrows = static_cast<int>(rows - rb * 32 < 32 ? rows - rb * 32 : 32);     // < 32 in a ragged last block,
        __half *base = x_hat + rb * (row_elems * 32) + (static_cast<int64_t>(wave) * 8 * nrows + r) * 8;   // stored compactly
        if (r < nrows) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {  // instruction j: piece columns 2j and 2j + 1, nrows x 16 bytes each
                const int kp = j * 2 + (lane >> 5);
                const uint32_t *src = tile + r * kOutPitch + kp * 4;
                store_writethrough16(base + kp * (nrows * 8), src[0], src[1], src[2], src[3]);
            }
        }
    }
}

// Any group size: one thread per group, straight from global memory.  Slow
// (strided reads) but has no layout assumptions; used when gs != 64 or the
// pointers are not 16-byte aligned.
template <typename TIN, typename TOUT>
__global__ void __launch_bounds__(128)
act_quant_generic_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                         uint8_t *__restrict__ packed, uint8_t *__restrict__ codes_u8,
                         float *__restrict__ center, float *__restrict__ scale, float *__restrict__ code_sum,
                         TOUT *__restrict__ x_hat, int64_t total_groups, int64_t groups_per_row,
                         int bits, int gs, float eps)
{
    const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (g >= total_groups) return;
    const int levels = 1 << bits;
    const int64_t row = g / groups_per_row;
    const int64_t gi = g - row * groups_per_row;
    const int64_t cols = groups_per_row * gs;
    const TIN *__restrict__ xg = x + g * gs;
    const float fgs = static_cast<float>(gs);

    float mu = 0.0f;
    for (int j = 0; j < gs; ++j) mu += to_float(xg[j]);
    mu /= fgs;
    float var = 0.0f;
    for (int j = 0; j < gs; ++j) {
        const float d = to_float(xg[j]) - mu;
        var += d * d;
    }
    const float s = sqrtf(var / fgs + eps);

    // Packed bytes of this group start at a byte boundary (checked on the host).
    uint8_t *pk = packed ? packed + row * packed_cols(cols, bits) + (gi * gs * bits) / 8 : nullptr;
    uint32_t acc = 0;
    int nacc = 0;
    float sum_codes = 0.0f;
    for (int j = 0; j < gs; ++j) {
        const float t = (to_float(xg[j]) - mu) / s;
        int c = 0;
        while (c < levels - 1 && t > thr[c]) ++c;
        sum_codes += cb[c];
        if (codes_u8) codes_u8[g * gs + j] = static_cast<uint8_t>(c);
        if (pk) {
            acc |= static_cast<uint32_t>(c) << nacc;
            nacc += bits;
            while (nacc >= 8) {
                *pk++ = static_cast<uint8_t>(acc & 0xffu);
                acc >>= 8;
                nacc -= 8;
            }
        }
    }
    if (center) center[g] = mu;
    if (scale) scale[g] = s;
    if (code_sum) code_sum[g] = sum_codes;
    if (x_hat) {
        // The codes are recomputed instead of stored: x_hat may alias x, so x is
        // re-read only at an index that has not been overwritten yet.
        const float code_mean = sum_codes / fgs;
        for (int j = 0; j < gs; ++j) {
            const float t = (to_float(xg[j]) - mu) / s;
            int c = 0;
            while (c < levels - 1 && t > thr[c]) ++c;
            x_hat[g * gs + j] = from_float<TOUT>(fma_f32(s, cb[c] - code_mean, mu));
        }
    }
}

template <typename TIN, typename TOUT>
static int launch(const void *x, const float *thr, const float *cb, uint8_t *packed, uint8_t *codes_u8,
                  float *center, float *scale, float *code_sum, void *x_hat,
                  int64_t rows, int64_t cols, int bits, int gs, float eps, hipStream_t stream)
{
    const int64_t groups_per_row = cols / gs;
    const int64_t total_groups = rows * groups_per_row;
    const TIN *xin = static_cast<const TIN *>(x);
    TOUT *xo = static_cast<TOUT *>(x_hat);
    const bool fast = gs == 64 && aligned(x, 16) && aligned(x_hat, 16) && aligned(packed, 16) && aligned(codes_u8, 16);
    // Fewer 64-group tiles than SIMDs and nothing but x_hat wanted: the two-lanes-per-group kernel.
    if (fast && x_hat && !packed && !codes_u8 && !center && !scale && !code_sum && total_groups <= 1024 * 64) {
        const unsigned blocks = static_cast<unsigned>((total_groups + 32 * kWaves - 1) / (32 * kWaves));
#define ARCQ_LAUNCH_SMALL(B) \
    hipLaunchKernelGGL((act_quant_small_kernel<TIN, TOUT, B>), dim3(blocks), dim3(64 * kWaves), 0, stream, xin, thr, cb, xo, \
                       total_groups, eps)
        if (bits == 4) ARCQ_LAUNCH_SMALL(4);
        else if (bits == 3) ARCQ_LAUNCH_SMALL(3);
        else ARCQ_LAUNCH_SMALL(2);
#undef ARCQ_LAUNCH_SMALL
    } else if (fast) {
        const int64_t ntiles = (total_groups + kTileGroups - 1) / kTileGroups;
        // Up to 3 workgroups fit a CU (LDS); more tiles than that are walked by the grid-stride loop.
        const int64_t want = (ntiles + kWaves - 1) / kWaves;
        // The kernel holds a whole group per lane (two waves per SIMD): 512 workgroups are what the chip runs at once,
        // and a launch with more tiles than that walks them (the next tile's loads in flight) instead of starting a
        // workgroup per four tiles.  With the tables built first: packed codes + metadata from fp32 19.3 -> 16.3 us
        // at 12 608 x 384, 47 -> 32 at K = 1 536, 113 -> 71 at 50 432 x 1 024; x_hat alone 10.2 -> 10.8, 24.5 -> 22.2,
        // 53 -> 51.5.
        const int64_t cap = 512;
        const unsigned blocks = static_cast<unsigned>(want < cap ? want : cap);
        const bool codes = packed || codes_u8;
#define ARCQ_LAUNCH_G64(B, C)                                                                                     \
    hipLaunchKernelGGL((act_quant_g64_kernel<TIN, TOUT, B, C>), dim3(blocks), dim3(64 * kWaves), 0, stream, xin, \
                       thr, cb, packed, codes_u8, center, scale, code_sum, xo, total_groups, eps)
        if (bits == 4) { if (codes) ARCQ_LAUNCH_G64(4, true); else ARCQ_LAUNCH_G64(4, false); }
        else if (bits == 3) { if (codes) ARCQ_LAUNCH_G64(3, true); else ARCQ_LAUNCH_G64(3, false); }
        else { if (codes) ARCQ_LAUNCH_G64(2, true); else ARCQ_LAUNCH_G64(2, false); }
#undef ARCQ_LAUNCH_G64
    } else {
        if (packed && (static_cast<int64_t>(gs) * bits) % 8 != 0)
            return fail(ARCQ_ERR_UNSUPPORTED,
                        "arcq_act_quant: packed output needs group_size*bits divisible by 8 (got %d*%d)", gs, bits);
        const unsigned blocks = static_cast<unsigned>((total_groups + 127) / 128);
        hipLaunchKernelGGL((act_quant_generic_kernel<TIN, TOUT>), dim3(blocks), dim3(128), 0, stream, xin, thr, cb,
                           packed, codes_u8, center, scale, code_sum, xo, total_groups, groups_per_row, bits, gs, eps);
    }
    return launch_status("arcq_act_quant");
}

template <typename TIN>
static int launch_blocked(const void *x, const float *thr, const float *cb, void *x_hat, int64_t rows, int64_t cols,
                          int bits, float eps, hipStream_t stream, const WeightJob &wj)
{
    const int groups_per_row = static_cast<int>(cols / 64);
    const int64_t ntiles = ((rows + 31) / 32) * groups_per_row;
    const int64_t want = (ntiles + kWaves - 1) / kWaves;
    // Up to 2 048 tiles (512 workgroups, two per CU) the launch is latency-bound: every wave takes one tile and a fifth
    // wave per workgroup builds the lookup tables meanwhile (M = 6 304, K = 384: 6.7 us against 7.6 without it).  Beyond
    // that the grid is what the chip holds at once (1 024 workgroups of four waves, four waves per SIMD), the tables are
    // built once per workgroup before its first tile, and each wave walks its tiles with the next one's loads in flight
    // (one workgroup per four tiles, tables rebuilt every time: K = 1 536 at M = 12 608 27-30 us instead of 18-19,
    // ViT-L's K = 4 096 input 230-258 instead of 171-178).
    const bool builder = ntiles <= 2048;
    const int64_t cap = 1024;
    const unsigned blocks = static_cast<unsigned>(want < cap ? want : cap) + wj.blocks;
#define ARCQ_LAUNCH_BLOCKED(B)                                                                                            \
    do {                                                                                                                  \
        if (builder)                                                                                                      \
            hipLaunchKernelGGL((act_quant_blocked2_kernel<TIN, B, true>), dim3(blocks), dim3(64 * (kWaves + 1)), 0, stream, \
                               static_cast<const TIN *>(x), thr, cb, static_cast<__half *>(x_hat), eps, groups_per_row, rows, wj); \
        else                                                                                                              \
            hipLaunchKernelGGL((act_quant_blocked2_kernel<TIN, B, false>), dim3(blocks), dim3(64 * kWaves), 0, stream,   \
                               static_cast<const TIN *>(x), thr, cb, static_cast<__half *>(x_hat), eps, groups_per_row, rows, wj); \
    } while (0)
    if (bits == 4) ARCQ_LAUNCH_BLOCKED(4);
    else if (bits == 3) ARCQ_LAUNCH_BLOCKED(3);
    else ARCQ_LAUNCH_BLOCKED(2);
#undef ARCQ_LAUNCH_BLOCKED
    return launch_status("arcq_act_quant_blocked");
}

}  // namespace arcq

using namespace arcq;

static int act_quant_blocked_checked(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                                     void *x_hat_blocked, int64_t rows, int64_t cols, int bits, float eps, void *stream,
                                     const WeightJob &wj)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant_blocked: bits must be 2, 3, or 4");
    if (rows < 0 || cols < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked: bad sizes");
    if (cols % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_act_quant_blocked: in_features must be divisible by 64");
    if (x_dtype != ARCQ_F32 && x_dtype != ARCQ_F16)
        return fail(ARCQ_ERR_DTYPE, "arcq_act_quant_blocked: x must be float32 or float16");
    if (rows * cols == 0 && wj.blocks == 0) return ARCQ_OK;
    if (!x || !thresholds || !codebook || !x_hat_blocked)
        return fail(ARCQ_ERR_NULL, "arcq_act_quant_blocked: x, thresholds, codebook and x_hat_blocked must not be NULL");
    if (x_hat_blocked == x) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_act_quant_blocked: x_hat_blocked must not alias x");
    if (rows * cols * 2 >= (int64_t(1) << 32)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked: tensor too large");
    if (!aligned(x, 16) || !aligned(x_hat_blocked, 16))
        return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_blocked: x and x_hat_blocked must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == ARCQ_F32)
        return launch_blocked<float>(x, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, st, wj);
    return launch_blocked<__half>(x, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, st, wj);
}

ARCQ_API int arcq_act_quant_blocked(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                                    void *x_hat_blocked, int64_t rows, int64_t cols, int bits, float eps, void *stream)
{
    return act_quant_blocked_checked(x, x_dtype, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, stream,
                                     WeightJob{});
}

// Stage 1 into the block layout and, in the same launch, w_hat[N, cols] (fp16, group size 64) from the layer's packed
// weights: the two inputs of the copying GEMM variant.
ARCQ_API int arcq_act_quant_blocked_with_weights(const void *x, int x_dtype, const float *thresholds,
                                                 const float *codebook, void *x_hat_blocked, int64_t rows, int64_t cols,
                                                 int bits, float eps, const uint8_t *packed_w, const float *w_codebook,
                                                 const float *w_center, const float *w_scale, const float *w_code_sum,
                                                 void *w_hat, int64_t N, void *stream)
{
    if (N < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked_with_weights: bad sizes");
    if (N == 0 || cols <= 0 || cols % 64 != 0)      // no weights to rebuild (or sizes the plain entry point reports)
        return arcq_act_quant_blocked(x, x_dtype, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, stream);
    if (!packed_w || !w_codebook || !w_center || !w_scale || !w_code_sum || !w_hat)
        return fail(ARCQ_ERR_NULL, "arcq_act_quant_blocked_with_weights: NULL weight tensor pointer");
    if (!aligned(w_hat, 16) || !aligned(packed_w, 4))
        return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_blocked_with_weights: w_hat must be 16-byte, packed_w 4-byte aligned");
    if (N * (cols / 8) >= (int64_t(1) << 38))
        return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked_with_weights: weight tensor too large");
    WeightJob wj{packed_w, w_codebook, w_center, w_scale, w_code_sum, static_cast<__half *>(w_hat), N, cols,
                 static_cast<unsigned>((N * (cols / 8) + 255) / 256)};
    return act_quant_blocked_checked(x, x_dtype, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, stream, wj);
}

template <typename TIN>
static int launch_rows_ln(const void *x, const float *gamma, const float *beta, float ln_eps, const float *thr, const float *cb,
                          void *x_hat, int64_t rows, int64_t cols, int bits, float eps, hipStream_t stream, WeightJob wj)
{
    const int G = static_cast<int>(cols / 64);
    const unsigned act_blocks = static_cast<unsigned>((rows + 31) / 32);
    if (wj.blocks) wj.blocks = static_cast<unsigned>((wj.N * (wj.K / 8) + 64 * G - 1) / (64 * G));      // 64 G threads per block here
    const size_t smem = (static_cast<size_t>(G) * 32 * Tile<TIN>::stride + 32 * (2 * G + 1)) * 4;
#define ARCQ_LAUNCH_ROWS(B, W)                                                                                   \
    do {                                                                                                         \
        allow_dynamic_lds<act_quant_rows_ln_kernel<TIN, B, W>>(160 * 1024 - 16 * 1024);                          \
        hipLaunchKernelGGL((act_quant_rows_ln_kernel<TIN, B, W>), dim3(act_blocks + wj.blocks), dim3(64 * G), smem, stream, \
                           static_cast<const TIN *>(x), gamma, beta, ln_eps, thr, cb, static_cast<__half *>(x_hat), eps, G, \
                           rows, wj);                                                                            \
    } while (0)
#define ARCQ_LAUNCH_ROWS_B(B) do { if (G <= 8) ARCQ_LAUNCH_ROWS(B, 8); else ARCQ_LAUNCH_ROWS(B, 16); } while (0)
    if (bits == 4) ARCQ_LAUNCH_ROWS_B(4);
    else if (bits == 3) ARCQ_LAUNCH_ROWS_B(3);
    else ARCQ_LAUNCH_ROWS_B(2);
#undef ARCQ_LAUNCH_ROWS_B
#undef ARCQ_LAUNCH_ROWS
    return launch_status("arcq_act_quant_blocked_ln");
}

// LayerNorm (weight ln_weight[cols], bias ln_bias[cols], fp32) followed by stage 1 into the block layout, in one
// launch; optionally (packed_w != NULL) the same launch reconstructs w_hat[N, cols] as
// arcq_act_quant_blocked_with_weights does.  cols / 64 must be between 1 and 16.
ARCQ_API int arcq_act_quant_blocked_ln(const void *x, int x_dtype, const float *ln_weight, const float *ln_bias, float ln_eps,
                                       const float *thresholds, const float *codebook, void *x_hat_blocked,
                                       int64_t rows, int64_t cols, int bits, float eps,
                                       const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                                       const float *w_scale, const float *w_code_sum, void *w_hat, int64_t N, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant_blocked_ln: bits must be 2, 3, or 4");
    if (rows < 0 || cols < 0 || N < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked_ln: bad sizes");
    if (cols % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_act_quant_blocked_ln: in_features must be divisible by 64");
    if (cols < 64 || cols > 1024)
        return fail(ARCQ_ERR_UNSUPPORTED, "arcq_act_quant_blocked_ln: in_features must be between 64 and 1024 (got %lld)",
                    static_cast<long long>(cols));
    if (x_dtype != ARCQ_F32 && x_dtype != ARCQ_F16)
        return fail(ARCQ_ERR_DTYPE, "arcq_act_quant_blocked_ln: x must be float32 or float16");
    WeightJob wj{};
    if (packed_w && N > 0) {
        if (!w_codebook || !w_center || !w_scale || !w_code_sum || !w_hat)
            return fail(ARCQ_ERR_NULL, "arcq_act_quant_blocked_ln: NULL weight tensor pointer");
        if (!aligned(w_hat, 16) || !aligned(packed_w, 4))
            return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_blocked_ln: w_hat must be 16-byte, packed_w 4-byte aligned");
        if (N * (cols / 8) >= (int64_t(1) << 38)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked_ln: weight tensor too large");
        wj = WeightJob{packed_w, w_codebook, w_center, w_scale, w_code_sum, static_cast<__half *>(w_hat), N, cols, 1};
    }
    if (rows == 0 && wj.blocks == 0) return ARCQ_OK;
    if (!x || !ln_weight || !ln_bias || !thresholds || !codebook || !x_hat_blocked)
        return fail(ARCQ_ERR_NULL, "arcq_act_quant_blocked_ln: x, ln_weight, ln_bias, thresholds, codebook and x_hat_blocked must not be NULL");
    if (x_hat_blocked == x) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_act_quant_blocked_ln: x_hat_blocked must not alias x");
    if (rows * cols * 2 >= (int64_t(1) << 32)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_blocked_ln: tensor too large");
    if (!aligned(x, 16) || !aligned(x_hat_blocked, 16) || !aligned(ln_weight, 16) || !aligned(ln_bias, 16))
        return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_blocked_ln: x, x_hat_blocked, ln_weight and ln_bias must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == ARCQ_F32)
        return launch_rows_ln<float>(x, ln_weight, ln_bias, ln_eps, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, st, wj);
    return launch_rows_ln<__half>(x, ln_weight, ln_bias, ln_eps, thresholds, codebook, x_hat_blocked, rows, cols, bits, eps, st, wj);
}

ARCQ_API int arcq_act_quant(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                            uint8_t *packed, uint8_t *codes_u8, float *center, float *scale, float *code_sum,
                            void *x_hat, int x_hat_dtype,
                            int64_t rows, int64_t cols, int bits, int group_size, float eps, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant: bits must be 2, 3, or 4");
    if (rows < 0 || cols < 0 || group_size <= 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant: bad sizes");
    if (cols % group_size != 0)
        return fail(ARCQ_ERR_GROUP, "arcq_act_quant: in_features must be divisible by group_size");
    if (x_dtype != ARCQ_F32 && x_dtype != ARCQ_F16) return fail(ARCQ_ERR_DTYPE, "arcq_act_quant: x must be float32 or float16");
    if (x_hat && x_hat_dtype != ARCQ_F32 && x_hat_dtype != ARCQ_F16)
        return fail(ARCQ_ERR_DTYPE, "arcq_act_quant: x_hat must be float32 or float16");
    if (x_hat && x_hat == x && x_hat_dtype != x_dtype)
        return fail(ARCQ_ERR_DTYPE, "arcq_act_quant: x_hat may alias x only when the dtypes match");
    if (rows * cols == 0) return ARCQ_OK;
    if (!x || !thresholds || !codebook) return fail(ARCQ_ERR_NULL, "arcq_act_quant: x, thresholds and codebook must not be NULL");
    if (rows * (cols / group_size) >= (int64_t(1) << 36)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int od = x_hat ? x_hat_dtype : x_dtype;
#define ARCQ_GO(TI, TO) \
    return launch<TI, TO>(x, thresholds, codebook, packed, codes_u8, center, scale, code_sum, x_hat, rows, cols, bits, group_size, eps, st)
    if (x_dtype == ARCQ_F32 && od == ARCQ_F32) ARCQ_GO(float, float);
    if (x_dtype == ARCQ_F32 && od == ARCQ_F16) ARCQ_GO(float, __half);
    if (x_dtype == ARCQ_F16 && od == ARCQ_F32) ARCQ_GO(__half, float);
    ARCQ_GO(__half, __half);
#undef ARCQ_GO
}
