// Stages 2+3 fused, large-M kernel: y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias.
//
// Workgroup = 4*WM waves laid out WM (rows) x 4 (columns), tile = (32*TI*WM) rows x 256 columns; a
// wave owns 32*TI rows x 64 columns, i.e. TI x 2 MFMA 32x32x16 accumulator blocks.  The shipped
// configuration is WM = 1, TI = 8 (four waves, one per SIMD, 256 accumulator registers each): every
// dequantized weight fragment then feeds 8 MFMAs.  WM = 2, TI = 4 (two waves per SIMD) is kept
// instantiable; it measured slower because the dequantization work per MFMA doubles.  The K loop
// advances one quantization group (64) at a time.
//
//  * x_hat (fp16) goes global -> registers -> LDS (double buffered, row stride 144 B so that the
//    16-byte fragment reads are bank-conflict free) and is read by all four waves.
//  * packed weight codes never touch LDS: a lane needs, per group and per 32-column block, exactly
//    the 32 codes k in [32h, 32h+32) of ONE weight row (h = lane/32), which are 4*BITS contiguous
//    bytes, one 16-byte load for 4-bit codes.  The MFMA sums over k, so the k order inside a group is
//    free as long as both operands agree; here the four k-steps of lane half h cover
//    k = 32h + 8*step ... + 7, for x_hat and w_hat alike.
//  * codes are turned into values two at a time: a byte (two 4-bit codes; 6 bits for 3-bit codes)
//    indexes an LDS table of float pairs (cb[lo], cb[hi]).  The table holds 32 copies, copy c in
//    banks 2c, 2c+1, and lane l uses copy l%32, so the 8-byte reads never conflict.  Then
//    w_hat = fp16(fma(cb - S/64, s, mu)), exactly the stand-alone stage-2 arithmetic
//    (FQ/arcq_packed_triton.py:59-74).
#include "arcq_common.h"
#include "arcq_gemm.h"

#include <type_traits>

namespace arcq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // native vectors keep staging arrays in registers
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;
constexpr int kAStride = 72;       // halves per LDS row of x_hat: 64 + 8 pad = 144 bytes
constexpr int kBN = 256;           // columns per workgroup

// 32 codes of one weight row and one lane half: the little-endian bit string in w[].
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

// Pair index (2*BITS bits) number `p` (0..15) of the 32-code string.
template <int BITS>
__device__ __forceinline__ uint32_t pair_at(const uint32_t (&w)[BITS], int p)
{
    constexpr int PB = 2 * BITS;
    const int bit = p * PB;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + PB > 32) v |= w[d + 1] << (32 - sh);
    return v & ((1u << PB) - 1u);
}

template <int BITS, typename TOUT, int TI, int WM>
__global__ void __launch_bounds__(256 * WM)
gemm_stream_kernel(const __half *__restrict__ a, const uint8_t *__restrict__ pw, const float *__restrict__ cb,
                   const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                   const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K)
{
    constexpr int THREADS = 256 * WM;
    constexpr int BM = 32 * TI * WM;
    constexpr int L = 1 << BITS;
    constexpr int PAIRS = 1 << (2 * BITS);
    constexpr int ROWS_PER_PASS = THREADS / 8;   // 8 threads x 16 B cover one row of 64 halves
    constexpr int A_PASSES = BM / ROWS_PER_PASS;

    // LDS map: [2 x_hat buffers: BM rows x 144 B][pair LUT: PAIRS entries x 32 copies x 8 B][bias: 256 floats]
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    _Float16 *sa = reinterpret_cast<_Float16 *>(smem);
    float2 *pair_lut = reinterpret_cast<float2 *>(smem + 2 * BM * kAStride * 2);
    float *s_bias = reinterpret_cast<float *>(smem + 2 * BM * kAStride * 2 + PAIRS * 256);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave & 3;          // column block of 64
    const int wm = wave >> 2;         // row block of 32*TI
    const int lr = lane & 31;         // row inside a 32-row / 32-column block
    const int lh = lane >> 5;         // k half
    // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Tiles are numbered with
    // the column tile fastest and XCD x takes the contiguous range [x*per, (x+1)*per), so the column
    // tiles that share a row tile of x_hat (and neighbouring row tiles, which share the weights) run on
    // one XCD at about the same time and re-read their operands from that L2 instead of from HBM.
    const int n_tiles = (N + kBN - 1) / kBN;
    const int tiles = n_tiles * ((M + BM - 1) / BM);
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    const int tile_n = tile % n_tiles;
    const int m0 = (tile / n_tiles) * BM;
    const int n0 = tile_n * kBN + wn * 64;
    const int G = K / kBK;
    const int64_t pcols = static_cast<int64_t>(K) * BITS / 8;

    // ---- global -> register staging of the next group -------------------------------------------
    const int a_row = tid >> 3, a_col = (tid & 7) * 8;
    const __half *a_src[A_PASSES];
#pragma unroll
    for (int p = 0; p < A_PASSES; ++p)
        a_src[p] = a + static_cast<int64_t>(min(m0 + p * ROWS_PER_PASS + a_row, M - 1)) * K + a_col;

    const uint8_t *w_src[2];
    const float *wc_src[2], *ws_src[2], *wcs_src[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = min(n0 + j * 32 + lr, N - 1);
        w_src[j] = pw + static_cast<int64_t>(n) * pcols + lh * (4 * BITS);
        wc_src[j] = wc + static_cast<int64_t>(n) * G;
        ws_src[j] = ws + static_cast<int64_t>(n) * G;
        wcs_src[j] = wcs + static_cast<int64_t>(n) * G;
    }

    u32x4_t a_reg[A_PASSES];
    uint32_t w_reg[2][BITS], w_cur[2][BITS];
    float c_reg[2], s_reg[2], m_reg[2], c_cur[2], s_cur[2], m_cur[2];

    auto fetch = [&](int g) {
#pragma unroll
        for (int p = 0; p < A_PASSES; ++p) a_reg[p] = *reinterpret_cast<const u32x4_t *>(a_src[p] + g * kBK);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            load_codes<BITS>(w_src[j] + g * (8 * BITS), w_reg[j]);
            c_reg[j] = wc_src[j][g];
            s_reg[j] = ws_src[j][g];
            m_reg[j] = wcs_src[j][g];
        }
    };
    auto commit_a = [&](int buf) {
        _Float16 *dst = sa + buf * (BM * kAStride);
#pragma unroll
        for (int p = 0; p < A_PASSES; ++p)
            *reinterpret_cast<u32x4_t *>(dst + (p * ROWS_PER_PASS + a_row) * kAStride + a_col) = a_reg[p];
    };
    auto take_b = [&]() {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < BITS; ++q) w_cur[j][q] = w_reg[j][q];
            c_cur[j] = c_reg[j];
            s_cur[j] = s_reg[j];
            m_cur[j] = m_reg[j] * 0.015625f;     // S/64, exact
        }
    };

    float16_t acc[TI][2];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const char *lut_lane = reinterpret_cast<const char *>(pair_lut) + lr * 8;
    const int lane_off = (wm * TI * 32 + lr) * kAStride + lh * 32;   // this lane's row / k-half inside an A buffer

    // Fragments are double buffered in registers: while the MFMAs of k-step s run on buffer s%2, the
    // x_hat fragments of step s+1 are read from LDS and the w_hat fragments of step s+1 are rebuilt.
    half8_t af[2][TI], bf[2][2];

    auto load_a = [&](int buf, const _Float16 *abase, int kk) {
#pragma unroll
        for (int i = 0; i < TI; ++i)
            af[buf][i] = *reinterpret_cast<const half8_t *>(abase + i * 32 * kAStride + kk * 8);
    };
    auto make_b = [&](int buf, int kk) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t e = pair_at<BITS>(w_cur[j], kk * 4 + p);
                const float2 v = *reinterpret_cast<const float2 *>(lut_lane + (e << 8));
                bf[buf][j][2 * p] = static_cast<_Float16>(fma_f32(v.x - m_cur[j], s_cur[j], c_cur[j]));
                bf[buf][j][2 * p + 1] = static_cast<_Float16>(fma_f32(v.y - m_cur[j], s_cur[j], c_cur[j]));
            }
        }
    };
    // Operand roles are swapped (w_hat is the MFMA "A" operand): accumulator element v of lane l is
    // y[m = 32i + l%32][n = 32j + 8*(v/4) + 4*(l/32) + v%4], four consecutive columns per lane.
    auto mma = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[buf][j], af[buf][i], acc[i][j], 0, 0, 0);
    };
    // Asks the scheduler to spread one k-step's LDS reads and dequantization VALU work between its MFMAs.
    auto interleave = [&]() {
#pragma unroll
        for (int q = 0; q < 2 * TI; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 LDS read
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);   // 4 VALU
        }
    };

    if (G > 0) fetch(0);
    // While the first group's loads are in flight: codebook pairs and bias into LDS.
    if (tid < 256) {
        const int col = tile_n * kBN + tid;
        s_bias[tid] = (bias && col < N) ? bias[col] : 0.0f;
    }
    for (int idx = tid; idx < PAIRS * 16; idx += THREADS) {   // 16 x 16-byte writes cover the 32 copies of an entry
        const int e = idx >> 4;
        const float lo = cb[e & (L - 1)], hi = cb[e >> BITS];
        reinterpret_cast<float4 *>(pair_lut)[idx] = make_float4(lo, hi, lo, hi);
    }
    if (G > 0) {
        commit_a(0);
        take_b();
    }
    __syncthreads();
    if (G > 0) {
        load_a(0, sa + lane_off, 0);
        make_b(0, 0);
    }

    // One barrier per group, placed before the last k-step: buffer `nxt` is written after every wave has
    // passed the previous group's barrier (hence finished reading it) and is read only after this one.
    auto group_step = [&](int g, auto last) {
        constexpr bool kLast = decltype(last)::value;
        const _Float16 *cur = sa + (g & 1) * (BM * kAStride) + lane_off;
        const _Float16 *nxt = sa + ((g + 1) & 1) * (BM * kAStride) + lane_off;
        if constexpr (!kLast) fetch(g + 1);
        load_a(1, cur, 1); make_b(1, 1); mma(0); interleave();
        load_a(0, cur, 2); make_b(0, 2); mma(1); interleave();
        load_a(1, cur, 3); make_b(1, 3); mma(0); interleave();
        if constexpr (!kLast) commit_a((g + 1) & 1);
        __syncthreads();
        if constexpr (!kLast) {
            take_b();
            load_a(0, nxt, 0);
            make_b(0, 0);
        }
        mma(1);
        if constexpr (!kLast) interleave();
    };
    for (int g = 0; g + 1 < G; ++g) group_step(g, std::false_type{});
    if (G > 0) group_step(G - 1, std::true_type{});

    // ---- epilogue ----------------------------------------------------------------------------------
    // Each wave stages 32*CH rows x 64 columns of its tile (bias added, rounded to TOUT) in its own LDS
    // region, row-major with a 16-byte pad, and writes it out as 16-byte row-contiguous stores.
    constexpr int CH = 4 / WM;                                       // 32-row blocks per pass
    constexpr int kOutStride = 64 * static_cast<int>(sizeof(TOUT)) + 16;   // bytes per staged row
    constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));        // elements per 16-byte store
    constexpr int kLanesPerRow = 64 / kVec;
    constexpr int kRowsPerIter = 64 / kLanesPerRow;
    const bool vec_ok = (N % kVec) == 0;

    float bv[2][4][4];   // bias of this lane's 32 columns, read before the staging writes reuse the block
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) bv[j][q][r] = s_bias[wn * 64 + j * 32 + 8 * q + 4 * lh + r];
    __syncthreads();     // every wave is done with the x_hat buffers, the LUT and the bias
    unsigned char *stage = smem + wave * (CH * 32 * kOutStride);

#pragma unroll
    for (int pass = 0; pass < TI / CH; ++pass) {
#pragma unroll
        for (int ii = 0; ii < CH; ++ii) {
            const int i = pass * CH + ii;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    unsigned char *dst = stage + (ii * 32 + lr) * kOutStride +
                                         (j * 32 + 8 * q + 4 * lh) * static_cast<int>(sizeof(TOUT));
                    float o[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] = acc[i][j][4 * q + r] + bv[j][q][r];
                    if constexpr (sizeof(TOUT) == 2) {
                        const __half2 lo = __floats2half2_rn(o[0], o[1]), hi = __floats2half2_rn(o[2], o[3]);
                        u32x2_t pk;
                        pk[0] = *reinterpret_cast<const uint32_t *>(&lo);
                        pk[1] = *reinterpret_cast<const uint32_t *>(&hi);
                        *reinterpret_cast<u32x2_t *>(dst) = pk;
                    } else {
                        u32x4_t pk;
#pragma unroll
                        for (int r = 0; r < 4; ++r) pk[r] = __float_as_uint(o[r]);
                        *reinterpret_cast<u32x4_t *>(dst) = pk;
                    }
                }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < CH * 32 / kRowsPerIter; ++t) {
            const int r = t * kRowsPerIter + lane / kLanesPerRow;     // staged row
            const int cseg = lane % kLanesPerRow;
            const int row = m0 + (wm * TI + pass * CH) * 32 + r;
            const int col = n0 + cseg * kVec;
            if (row < M && col < N) {
                const u32x4_t v = *reinterpret_cast<const u32x4_t *>(stage + r * kOutStride + cseg * 16);
                TOUT *dst = y + static_cast<int64_t>(row) * N + col;
                if (vec_ok && col + kVec <= N) {
                    store_streaming16(dst, v[0], v[1], v[2], v[3]);
                } else {
                    const TOUT *e = reinterpret_cast<const TOUT *>(&v);
#pragma unroll
                    for (int k = 0; k < kVec; ++k)
                        if (col + k < N) dst[k] = e[k];
                }
            }
        }
        if (pass + 1 < TI / CH) __syncthreads();
    }
}

template <int BITS, typename TOUT, int TI, int WM>
static void launch_ti(const GemmArgs &g, hipStream_t stream)
{
    constexpr int BM = 32 * TI * WM;
    const size_t main_bytes = 2 * BM * kAStride * 2 + (size_t(1) << (2 * BITS)) * 256 + 1024;   // x_hat buffers + pair LUT + bias
    const size_t stage_bytes = size_t(4 * WM) * (4 / WM) * 32 * (64 * sizeof(TOUT) + 16);       // epilogue staging
    const size_t smem = main_bytes > stage_bytes ? main_bytes : stage_bytes;
    auto kernel = gemm_stream_kernel<BITS, TOUT, TI, WM>;
    allow_dynamic_lds<gemm_stream_kernel<BITS, TOUT, TI, WM>>(static_cast<int>(smem));
    const int tiles = ((g.N + kBN - 1) / kBN) * ((g.M + BM - 1) / BM);
    dim3 grid(8 * ((tiles + 7) / 8));
    hipLaunchKernelGGL(kernel, grid, dim3(256 * WM), smem, stream, static_cast<const __half *>(g.x_hat), g.pw, g.cb,
                       g.wc, g.ws, g.wcs, g.bias, static_cast<TOUT *>(g.y), g.M, g.N, g.K);
}

template <int BITS, typename TOUT>
static void launch_bits(const GemmArgs &g, hipStream_t stream)
{
    // One wave per SIMD with 256-row x 64-column wave tiles measured faster than two waves per SIMD
    // with 128-row tiles (the dequantization work per MFMA doubles with the smaller tile).
    launch_ti<BITS, TOUT, 8, 1>(g, stream);
}

void launch_gemm_stream(const GemmArgs &g, hipStream_t stream)
{
    if (g.y_f16) {
        if (g.bits == 4) launch_bits<4, __half>(g, stream);
        else if (g.bits == 3) launch_bits<3, __half>(g, stream);
        else launch_bits<2, __half>(g, stream);
    } else {
        if (g.bits == 4) launch_bits<4, float>(g, stream);
        else if (g.bits == 3) launch_bits<3, float>(g, stream);
        else launch_bits<2, float>(g, stream);
    }
}

}  // namespace arcq
