// Stages 2+3 fused, weight-stationary kernel: y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias.
//
// A workgroup (4 waves) owns a slab of 128 output columns and a contiguous range of 32-row blocks.
// For every K slice of up to 6 quantization groups (384 values) it
//   1. rebuilds the slab's slice of w_hat from the packed codes ONCE, into LDS as fp16
//      (exact stage-2 arithmetic, FQ/arcq_packed_triton.py:59-74), all 256 threads cooperating;
//   2. runs a barrier-free MFMA loop: every wave multiplies its own row blocks, two at a time
//      (2 x 4 accumulator blocks of 32x32), with the resident slab.  The rows of a wave are private to
//      it, so its x_hat stream needs no workgroup barrier: a "unit" (64 rows x one group, 8 KiB) is
//      fetched with fully coalesced 16-byte loads (8 rows x 128 B per instruction) two units ahead,
//      parked in registers, written to a wave-private LDS tile and read back as MFMA fragments;
//      LDS operations of one wave execute in order, which is all the synchronization this needs.
// The dequantization cost is paid once per (workgroup, slice) instead of once per 256 rows, and when K
// fits one slice the slab stays resident while the wave walks all its row blocks.
//
// k order inside a group: lane half h covers k = 32h + 8*step ... + 7 in k-step `step`, for both
// operands (the MFMA sums over k, so any order shared by the operands is valid).
// Operand roles are swapped (w_hat is the MFMA "A" operand): accumulator element v of lane l is
// y[m = 32i + l%32][n = 32j + 8*(v/4) + 4*(l/32) + v%4], four consecutive columns per lane.
#include "arcq_common.h"
#include "arcq_gemm.h"

#include <type_traits>

namespace arcq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kSlabN = 128;                 // columns per slab
constexpr int kSliceGroups = 6;             // groups per K slice
constexpr int kPitch = kSliceGroups * 128 + 16;   // bytes per slab row: 384 halves + 16 B pad (conflict-free 16-B reads)
constexpr int kStageRow = 272;              // bytes per staged output row: 256 + 16 pad
constexpr int kSlabBytes = kSlabN * kPitch;                 // 100352
constexpr int kTJ = kSlabN / 32;            // 4 column blocks
constexpr int kTI = 2;                      // row blocks per wave and pass
constexpr int kAPitch = 144;                // bytes per x_hat row in the wave's tile: one group (128 B) + 16 B pad
constexpr int kATile = kTI * 32 * kAPitch;  // 9216 B per wave; doubles as the epilogue staging tile (32 x 272 B)
constexpr int kStageBytes = 4 * kATile;
static_assert(32 * kStageRow <= kATile, "epilogue staging must fit the wave's x_hat tile");

template <int BITS>
__device__ __forceinline__ void slab_load_codes(const uint8_t *__restrict__ p, uint32_t (&w)[BITS])
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
__device__ __forceinline__ uint32_t slab_code_at(const uint32_t (&w)[BITS], int q)
{
    const int bit = q * BITS;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + BITS > 32) v |= w[d + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}

// Ordering point between LDS accesses of different lanes of one wave.  LDS operations of a wave execute in issue
// order, so no wait is needed; this only keeps the compiler from moving code across.  (A release/acquire fence here
// would also wait for the wave's outstanding global stores and serialize the epilogue on their latency.)
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_wave_barrier();
}

// PRE = true: the weights were reconstructed beforehand (arcq_weight_dequant into a caller-provided fp16 [N,K]
// buffer); the slab slices are then copied, global -> LDS directly, instead of rebuilt, which is what pays when many
// workgroups would otherwise repeat the rebuild (long K, few columns, many passes).  (Copying the next slice under the
// running slice's MFMA loop measured 2-4x slower: vector memory operations complete in issue order, so the x_hat
// loads issued behind a copy wait for it.)
template <int BITS, typename TOUT, bool PRE>
__global__ void __launch_bounds__(256)
gemm_slab_kernel(const __half *__restrict__ a, const uint8_t *__restrict__ pw, const float *__restrict__ cb,
                 const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                 const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K,
                 int row_ranges, int blocks_per_range, const __half *__restrict__ w_hat)
{
    constexpr int L = 1 << BITS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *slab = smem;
    unsigned char *stage_all = smem + kSlabBytes;
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
    const int n_base = (tile % n_slabs) * kSlabN;
    const int total_blocks = (M + 31) / 32;
    const int blk0 = (tile / n_slabs) * blocks_per_range;
    const int blk1 = min(total_blocks, blk0 + blocks_per_range);
    // Row blocks of this wave: a contiguous quarter of the workgroup's range.
    const int per_wave = (blk1 - blk0 + 3) / 4;
    const int wblk0 = min(blk1, blk0 + wave * per_wave);
    const int wblk1 = min(blk1, wblk0 + per_wave);
    const int passes = (per_wave + kTI - 1) / kTI;          // same for all four waves: barriers stay uniform
    const int slices = (G + kSliceGroups - 1) / kSliceGroups;


    // Dequantization roles: a slab slice is 128 rows x 12 half groups (32 codes = 4*BITS bytes each, the 12 of a row
    // contiguous in memory); half group number p = round * 256 + tid, so that consecutive lanes read consecutive
    // pieces of a row and a wave's load touches about six rows instead of thirty-two.
    constexpr int kHalves = 2 * kSliceGroups;

    const unsigned char *slab_lane = slab + lr * kPitch + lh * 64;
    unsigned char *a_tile = stage_all + wave * kATile;
    unsigned char *stage = a_tile;
    // x_hat unit loads: instruction t of a unit covers rows 8t..8t+7, lane -> (row 8t + lane/8, 16-byte piece lane%8).
    const int ld_row = lane >> 3, ld_c = lane & 7;
    unsigned char *a_wr = a_tile + ld_row * kAPitch + ld_c * 16;
    const unsigned char *a_rd = a_tile + lr * kAPitch + lh * 64;

    // Codes and metadata of one slice: fetched into registers first (for the first slice at the very top of the
    // kernel, so that this latency, the codebook's and the first x_hat units' all overlap), converted afterwards.
    uint32_t codes[kSliceGroups][BITS];
    float c[kSliceGroups], s[kSliceGroups], m[kSliceGroups];
    auto fetch_slice = [&](int g0) {
#pragma unroll
        for (int r = 0; r < kSliceGroups; ++r) {
            const int p = r * 256 + tid;
            const int row = p / kHalves, q = p % kHalves;
            const int n = min(n_base + row, N - 1);
            const int g = min(g0 + (q >> 1), G - 1);
            slab_load_codes<BITS>(pw + static_cast<int64_t>(n) * pcols + g * (8 * BITS) + (q & 1) * (4 * BITS), codes[r]);
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
    // PRE: one direct global -> LDS load per slab row and wave (lanes 0..47 carry the row's 48 16-byte pieces, the
    // hardware writes lane l's piece at the wave-uniform LDS base + 16 l); the caller waits for vmcnt and the barrier.
    auto copy_slice = [&](int g0, int ng) {
        const bool active = lane < 8 * ng;
        for (int rr = 0; rr < kSlabN / 4; ++rr) {
            const int row = wave * (kSlabN / 4) + rr;
            const int n = min(n_base + row, N - 1);
            if (active)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(w_hat + static_cast<int64_t>(n) * K + g0 * 64 + lane * 8),
                    (__attribute__((address_space(3))) void *)(slab + row * kPitch), 16, 0, 0);
        }
    };
    auto dequant_slice = [&](int ng) {
#pragma unroll
        for (int r = 0; r < kSliceGroups; ++r) {
            const int p = r * 256 + tid;
            const int row = p / kHalves, q = p % kHalves;
            if ((q >> 1) < ng) {
                // All 32 table lookups of this half group are issued before the first is used.
                const float mg = m[r] * 0.015625f;          // S/64, exact
                float v[32];
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    const uint32_t code = slab_code_at<BITS>(codes[r], e);
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

    // Load cursor: the next unit (pass, group) to fetch from global memory; it runs ahead of the MFMA loop.
    int ld_pass = 0, ld_g = 0;
    uint32_t voff[8];
    auto set_offsets = [&](int pass) {
        const int row0 = (wblk0 + pass * kTI) * 32 + ld_row;
#pragma unroll
        for (int t = 0; t < 8; ++t)
            voff[t] = static_cast<uint32_t>(min(row0 + t * 8, M - 1)) * static_cast<uint32_t>(K * 2) + ld_c * 16;
    };
    auto load_unit = [&](u32x4_t (&r)[8]) {
        const char *base = reinterpret_cast<const char *>(a) + ld_g * 128;
#pragma unroll
        for (int t = 0; t < 8; ++t) r[t] = *reinterpret_cast<const u32x4_t *>(base + voff[t]);
        if (++ld_g == G) {
            ld_g = 0;
            if (ld_pass + 1 < passes) set_offsets(++ld_pass);      // past the end: keep re-reading the last pass
        }
    };
    auto park_unit = [&](const u32x4_t (&r)[8]) {
#pragma unroll
        for (int t = 0; t < 8; ++t) *reinterpret_cast<u32x4_t *>(a_wr + t * 8 * kAPitch) = r[t];
    };

    u32x4_t r0[8], r1[8];          // units in flight (two ahead of the MFMA loop)
    u32x4_t frag[kTI][4];          // x_hat fragments of the current unit
    set_offsets(0);
    load_unit(r0);
    load_unit(r1);
    park_unit(r0);
#pragma unroll
    for (int i = 0; i < kTI; ++i)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            frag[i][kk] = *reinterpret_cast<const u32x4_t *>(a_rd + i * 32 * kAPitch + kk * 16);
    load_unit(r0);
    // From here on, at the start of every unit: `frag` holds the unit, `rw` (alternating r1, r0) the next one, the
    // other buffer the one after.

    for (int pass = 0; pass < passes; ++pass) {
        const int pblk0 = wblk0 + pass * kTI;
        const int nf = max(0, min(kTI, wblk1 - pblk0));        // row blocks of this wave in this pass
        float16_t acc[kTI][kTJ];
#pragma unroll
        for (int i = 0; i < kTI; ++i)
#pragma unroll
            for (int j = 0; j < kTJ; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

        // One unit = one group for this wave's two row blocks = four k-steps of 8 MFMAs.  Every k-step also issues the
        // LDS reads of the next k-step's w_hat fragments and refills the x_hat fragments it has consumed with the next
        // unit's; k-step 0 parks the next unit in the LDS tile, k-step 1 fetches the unit after the one in flight.
        // `bf[0]` holds the fragments of (gl, k-step 0) on entry and of (gl + 1, k-step 0) on exit.
        half8_t bf[2][kTJ];
        auto unit = [&](u32x4_t (&rw)[8], int gl, auto nfc) {
            constexpr int NFU = decltype(nfc)::value;      // row blocks really multiplied (1 on a wave's last, odd pass)
            const unsigned char *bsrc = slab_lane + gl * 128;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int cur = kk & 1, nxt = cur ^ 1;
#pragma unroll
                for (int j = 0; j < kTJ; ++j)       // kk == 3 reads the next group (past the slice on its last unit: unused)
                    bf[nxt][j] = *reinterpret_cast<const half8_t *>(bsrc + j * 32 * kPitch + (kk + 1) * 16 + (kk == 3 ? 64 : 0));
                if (kk == 0) park_unit(rw);
                if (kk == 1) load_unit(rw);
#pragma unroll
                for (int i = 0; i < NFU; ++i) {
                    half8_t af;
                    __builtin_memcpy(&af, &frag[i][kk], 16);
#pragma unroll
                    for (int j = 0; j < kTJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af, acc[i][j], 0, 0, 0);
                    frag[i][kk] = *reinterpret_cast<const u32x4_t *>(a_rd + i * 32 * kAPitch + kk * 16);
                }
#pragma unroll
                for (int q = 0; q < 4 * NFU; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 // 1 LDS read
                    if (kk == 0) __builtin_amdgcn_sched_group_barrier(0x200, 2 / NFU, 0);    // LDS writes
                    if (kk == 1) __builtin_amdgcn_sched_group_barrier(0x020, 2 / NFU, 0);    // global loads
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
#pragma unroll
            for (int j = 0; j < kTJ; ++j) bf[0][j] = *reinterpret_cast<const half8_t *>(slab_lane + j * 32 * kPitch);
            // A pass with a single row block (the tail of an odd count; later passes are then empty) skips the
            // second block's MFMAs and fragment reads instead of multiplying a duplicate.
            if (nf == 1) {
                for (int gl = 0; gl < ng; gl += 2) {
                    unit(r1, gl, std::integral_constant<int, 1>{});
                    if (gl + 1 < ng) unit(r0, gl + 1, std::integral_constant<int, 1>{});
                }
            } else {
                for (int gl = 0; gl < ng; gl += 2) {
                    unit(r1, gl, std::integral_constant<int, 2>{});
                    if (gl + 1 < ng) unit(r0, gl + 1, std::integral_constant<int, 2>{});
                }
            }
            if (ng & 1) {               // odd unit count: restore the alternation for the next slice
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const u32x4_t tmp = r0[t];
                    r0[t] = r1[t];
                    r1[t] = tmp;
                }
            }
        }

        // ---- epilogue of this pass: one 32-row block at a time through the wave's private staging tile ----
        constexpr int kChunks = (sizeof(TOUT) == 2) ? 1 : 2;        // staged columns per chunk: 128 (fp16) / 64 (fp32)
        constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));
#pragma unroll
        for (int i = 0; i < kTI; ++i) {
            if (i < nf) {
#pragma unroll
                for (int ch = 0; ch < kChunks; ++ch) {
#pragma unroll
                    for (int jj = 0; jj < kTJ / kChunks; ++jj) {
                        const int j = ch * (kTJ / kChunks) + jj;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int cl = jj * 32 + 8 * q + 4 * lh;            // column inside the chunk
                            const float4 bv = *reinterpret_cast<const float4 *>(s_bias + j * 32 + 8 * q + 4 * lh);
                            const float o0 = acc[i][j][4 * q] + bv.x, o1 = acc[i][j][4 * q + 1] + bv.y;
                            const float o2 = acc[i][j][4 * q + 2] + bv.z, o3 = acc[i][j][4 * q + 3] + bv.w;
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
                    wave_sync();
                    const int col0 = n_base + ch * (kSlabN / kChunks);
#pragma unroll
                    for (int it = 0; it < 8; ++it) {
                        const int r = it * 4 + (lane >> 4);
                        const int cseg = lane & 15;
                        const int row = (pblk0 + i) * 32 + r;
                        const int col = col0 + cseg * kVec;
                        if (row < M && col < N) {
                            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(stage + r * kStageRow + cseg * 16);
                            TOUT *dst = y + static_cast<int64_t>(row) * N + col;
                            if ((N % kVec) == 0 && col + kVec <= N) {
                                store_streaming16(dst, v[0], v[1], v[2], v[3]);
                            } else {
                                const TOUT *e = reinterpret_cast<const TOUT *>(&v);
#pragma unroll
                                for (int k = 0; k < kVec; ++k)
                                    if (col + k < N) dst[k] = e[k];
                            }
                        }
                    }
                    wave_sync();
                }
            }
        }
    }
}

template <int BITS, typename TOUT, bool PRE>
static void launch_slab(const GemmArgs &g, hipStream_t stream, const void *w_hat)
{
    constexpr int L = 1 << BITS;
    const size_t smem = kSlabBytes + kStageBytes + L * 64 * sizeof(float) + kSlabN * sizeof(float);
    auto kernel = gemm_slab_kernel<BITS, TOUT, PRE>;
    allow_dynamic_lds<gemm_slab_kernel<BITS, TOUT, PRE>>(static_cast<int>(smem));
    // One workgroup per CU where possible: split the 32-row blocks into as many ranges as CUs/slabs allow.
    const int n_slabs = (g.N + kSlabN - 1) / kSlabN;
    const int total_blocks = (g.M + 31) / 32;
    int ranges = 256 / n_slabs;
    if (ranges < 1) ranges = 1;
    if (ranges > total_blocks) ranges = total_blocks;
    const int blocks_per_range = (total_blocks + ranges - 1) / ranges;
    ranges = (total_blocks + blocks_per_range - 1) / blocks_per_range;
    const int tiles = n_slabs * ranges;
    hipLaunchKernelGGL(kernel, dim3(8 * ((tiles + 7) / 8)), dim3(256), smem, stream,
                       static_cast<const __half *>(g.x_hat), g.pw, g.cb, g.wc, g.ws, g.wcs, g.bias,
                       static_cast<TOUT *>(g.y), g.M, g.N, g.K, ranges, blocks_per_range,
                       static_cast<const __half *>(w_hat));
}

void launch_gemm_slab(const GemmArgs &g, hipStream_t stream)
{
    if (g.y_f16) {
        if (g.bits == 4) launch_slab<4, __half, false>(g, stream, nullptr);
        else if (g.bits == 3) launch_slab<3, __half, false>(g, stream, nullptr);
        else launch_slab<2, __half, false>(g, stream, nullptr);
    } else {
        if (g.bits == 4) launch_slab<4, float, false>(g, stream, nullptr);
        else if (g.bits == 3) launch_slab<3, float, false>(g, stream, nullptr);
        else launch_slab<2, float, false>(g, stream, nullptr);
    }
}

// Same product with the weights already reconstructed into w_hat ([N,K] fp16).
void launch_gemm_slab_prebuilt(const GemmArgs &g, const void *w_hat, hipStream_t stream)
{
    if (g.y_f16) launch_slab<4, __half, true>(g, stream, w_hat);
    else launch_slab<4, float, true>(g, stream, w_hat);
}

}  // namespace arcq
