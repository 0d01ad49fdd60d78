// Low-precision formulation of the layer (the direction EXT/arcq_linear_kernel.cu:22-202 points at: the product on
// matrix units at less than fp16): stage 1 and stage 2 as everywhere else -- same codes, same mu / s, same
// reconstruction in fp32 -- but the reconstructed operands are rounded to FP8 (OCP E4M3: 3 mantissa bits, largest
// finite value 448) instead of fp16, so that stage 3 can run as an FP8 matrix product with fp32 accumulation (twice
// the fp16 MFMA rate).  The per-group scales are inside the operands, as in the fp16 path; putting them behind the
// product instead (codebook values as operands, scales in an epilogue per output and group) costs more vector-ALU
// time than the matrix units save.
//
//   x8[m,k] = fp8( clamp( s (cb[code] - code_sum/64) + mu ) )                 row-major [M,K]
//   w8[n,k] = fp8( clamp( w_mult ((cb_w[code] - code_sum/64) scale + center) ) )   row-major [N,K]
//   y = (x8 * w8^T) / w_mult + bias            (the product itself is a plain library GEMM, outside this file)
//
// w_mult is a power of two chosen by the caller so that the weights (|w| ~ 0.01 .. 1) land in FP8's normal range;
// it changes no bit of the significands.  This path does NOT reproduce the reference's numbers: each operand carries
// a relative rounding error of up to 2^-4 where fp16 has 2^-11.
#include "arcq_common.h"
#include "arcq_act_quant_core.h"

namespace arcq {
namespace {

constexpr float kFp8Max = 448.0f;
constexpr int kFp8Waves = 4;

// Eight floats -> eight FP8 (E4M3, round to nearest even, finite values saturating at +-448, NaN kept) in two dwords.
__device__ __forceinline__ void to_fp8x8(const float (&v)[8], uint32_t &lo, uint32_t &hi)
{
    float c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = v[i] != v[i] ? v[i] : fminf(fmaxf(v[i], -kFp8Max), kFp8Max);      // (NaN stays NaN)
    int a = 0, b = 0;
    a = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], a, false);
    a = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], a, true);
    b = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], b, false);
    b = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], b, true);
    lo = static_cast<uint32_t>(a);
    hi = static_cast<uint32_t>(b);
}

// Stage 2 with FP8 output: one thread per eight weights (one piece of codes), value = w_mult * w_hat.  Rows of w8 are
// `ldw` bytes apart (ldw >= K, a multiple of 8); the bytes from K to ldw are written as zeros (FP8 0.0).  Thread t of
// nt walks the pieces t, t + nt, ...; s_cb = the codebook in LDS.
template <int BITS>
__device__ __forceinline__ void weight_dequant_fp8_share(const uint8_t *__restrict__ packed, const float *s_cb,
                                                         const float *__restrict__ center, const float *__restrict__ scale,
                                                         const float *__restrict__ code_sum, uint8_t *__restrict__ w8,
                                                         int64_t N, int K, int ldw, float w_mult, int64_t t, int64_t nt)
{
    constexpr int L = 1 << BITS;
    const int pieces_per_row = ldw / 8, live_pieces = K / 8;
    const int64_t pieces = N * pieces_per_row;
    const int pcols = K * BITS / 8;
    const int G = K / 64;
    for (int64_t idx = t; idx < pieces; idx += nt) {
        const int64_t n = idx / pieces_per_row;
        const int pp = static_cast<int>(idx - n * pieces_per_row);
        uint32_t lo = 0, hi = 0;
        if (pp < live_pieces) {
            const uint32_t w = load_codes8<BITS>(packed + n * pcols + pp * BITS);
            const int64_t mi = n * G + (pp >> 3);
            const float c = center[mi], s = scale[mi], m = code_sum[mi] * 0.015625f;
            float v[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = fma_f32(s_cb[(w >> (BITS * q)) & (L - 1)] - m, s, c) * w_mult;
            to_fp8x8(v, lo, hi);
        }
        *reinterpret_cast<uint2 *>(w8 + idx * 8) = make_uint2(lo, hi);
    }
}

template <int BITS>
__global__ void __launch_bounds__(256)
weight_dequant_fp8_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ cb,
                          const float *__restrict__ center, const float *__restrict__ scale,
                          const float *__restrict__ code_sum, uint8_t *__restrict__ w8, int64_t N, int K, int ldw, float w_mult)
{
    constexpr int L = 1 << BITS;
    __shared__ float s_cb[L];
    if (threadIdx.x < L) s_cb[threadIdx.x] = cb[threadIdx.x];
    __syncthreads();
    weight_dequant_fp8_share<BITS>(packed, s_cb, center, scale, code_sum, w8, N, K, ldw, w_mult,
                                   static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x,
                                   static_cast<int64_t>(gridDim.x) * blockDim.x);
}

// What the block-layout stage-1 launch carries along: the layer's weights reconstructed to FP8 by `blocks` extra
// workgroups in front of the grid (activations and weights are independent inputs of the same product).
struct Fp8Carry {
    const uint8_t *packed;
    const float *cb, *center, *scale, *code_sum;
    uint8_t *w8;
    int64_t N;
    int ldw;
    float w_mult;
    int blocks;
};

// Stage 1 with FP8 output.  Wave tile = 32 rows x one group, two lanes per group (arcq_act_quant_core.h); the inputs
// come straight from global memory (each lane 32 consecutive values), the outputs go straight back (each lane 32
// consecutive bytes).  The four waves of a workgroup build the lookup tables together, then walk the tiles.
// BLK: x8 in the block layout of the FP8 GEMM, 16-byte pieces [rows/32][Kp/16][32 rows][16 values] with
// Kp = K rounded up to 128 (the pieces from K to Kp written as zeros; a last block of r < 32 rows as [Kp/16][r][16]).
template <typename TIN, int BITS, bool BLK>
__global__ void __launch_bounds__(64 * kFp8Waves)
act_quant_fp8_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                     uint8_t *__restrict__ x8, float eps, int groups_per_row, int64_t rows, const Fp8Carry carry)
{
    constexpr int L = 1 << BITS;
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[kFp8Waves];
    if constexpr (BLK) {
        if (static_cast<int>(blockIdx.x) < carry.blocks) {      // a weight workgroup (workgroup-uniform)
            float *s_cb = lut;
            if (threadIdx.x < L) s_cb[threadIdx.x] = carry.cb[threadIdx.x];
            __syncthreads();
            weight_dequant_fp8_share<BITS>(carry.packed, s_cb, carry.center, carry.scale, carry.code_sum, carry.w8, carry.N,
                                           groups_per_row * 64, carry.ldw, carry.w_mult,
                                           static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x,
                                           static_cast<int64_t>(carry.blocks) * blockDim.x);
            return;
        }
    }
    const int wg = BLK ? static_cast<int>(blockIdx.x) - carry.blocks : static_cast<int>(blockIdx.x);
    const int n_wg = BLK ? static_cast<int>(gridDim.x) - carry.blocks : static_cast<int>(gridDim.x);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid, 64 * kFp8Waves);
    __syncthreads();
    bool table_ok = true;
#pragma unroll
    for (int w = 0; w < kFp8Waves; ++w) table_ok = table_ok && (slow_slots[w] == 0);

    const int row = lane >> 1, half = lane & 1;
    const int64_t K = static_cast<int64_t>(groups_per_row) * 64;
    const int64_t ntiles = ((rows + 31) / 32) * groups_per_row;
    for (int64_t t = static_cast<int64_t>(wg) * kFp8Waves + wave; t < ntiles;
         t += static_cast<int64_t>(n_wg) * kFp8Waves) {
        const int64_t rb = t / groups_per_row;
        const int g = static_cast<int>(t - rb * groups_per_row);
        const int64_t r = rb * 32 + row;
        const bool live = r < rows;                  // (a ragged last block: the lanes past the end quantize zeros)
        const int64_t at = r * K + g * 64 + half * 32;
        float xv[32];
        if constexpr (sizeof(TIN) == 2) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 q = live ? *reinterpret_cast<const uint4 *>(x + at + i * 8) : make_uint4(0, 0, 0, 0);
                const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    xv[8 * i + 2 * e] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] & 0xffffu)));
                    xv[8 * i + 2 * e + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] >> 16)));
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint4 q = live ? *reinterpret_cast<const uint4 *>(x + at + i * 4) : make_uint4(0, 0, 0, 0);
                xv[4 * i] = __uint_as_float(q.x); xv[4 * i + 1] = __uint_as_float(q.y);
                xv[4 * i + 2] = __uint_as_float(q.z); xv[4 * i + 3] = __uint_as_float(q.w);
            }
        }
        float mu, var, s, sum_codes;
        group_stats32x2(xv, eps, mu, var, s);
        group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
        const float code_mean = sum_codes * 0.015625f;
        uint32_t out[8];
#pragma unroll
        for (int q8 = 0; q8 < 4; ++q8) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = fma_f32(s, xv[8 * q8 + e] - code_mean, mu);
            to_fp8x8(v, out[2 * q8], out[2 * q8 + 1]);
        }
        if constexpr (BLK) {
            if (live) {
                const int Kp = (groups_per_row * 64 + 127) / 128 * 128;
                const int64_t R = rows - rb * 32 < 32 ? rows - rb * 32 : 32;      // rows of this block
                uint8_t *blk = x8 + rb * 32 * Kp;
                const int p0 = g * 4 + half * 2;                                  // this lane's two pieces
                *reinterpret_cast<uint4 *>(blk + (p0 * R + row) * 16) = make_uint4(out[0], out[1], out[2], out[3]);
                *reinterpret_cast<uint4 *>(blk + ((p0 + 1) * R + row) * 16) = make_uint4(out[4], out[5], out[6], out[7]);
                if (g == groups_per_row - 1 && Kp > groups_per_row * 64) {         // the row's padding: 64 zero bytes
                    const int z0 = groups_per_row * 4 + half * 2;
                    *reinterpret_cast<uint4 *>(blk + (z0 * R + row) * 16) = make_uint4(0, 0, 0, 0);
                    *reinterpret_cast<uint4 *>(blk + ((z0 + 1) * R + row) * 16) = make_uint4(0, 0, 0, 0);
                }
            }
        } else if (live) {
            uint4 *dst = reinterpret_cast<uint4 *>(x8 + at);
            dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
            dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
        }
    }
}

template <typename TIN, bool BLK>
void launch_act_fp8(const void *x, const float *thr, const float *cb, uint8_t *x8, int64_t rows, int64_t cols, int bits,
                    float eps, Fp8Carry carry, hipStream_t stream)
{
    const int groups = static_cast<int>(cols / 64);
    const int64_t ntiles = ((rows + 31) / 32) * groups;
    int64_t blocks = (ntiles + kFp8Waves - 1) / kFp8Waves;
    if (blocks > 2048) blocks = 2048;
    if (carry.packed) {          // one weight workgroup per 2048 pieces of eight values, at most 256
        const int64_t pieces = carry.N * (carry.ldw / 8);
        int64_t wb = (pieces + 2047) / 2048;
        carry.blocks = static_cast<int>(wb < 1 ? 1 : (wb > 256 ? 256 : wb));
    } else {
        carry.blocks = 0;
    }
    const dim3 grid(static_cast<unsigned>(blocks + carry.blocks));
    const TIN *xin = static_cast<const TIN *>(x);
    if (bits == 4)
        hipLaunchKernelGGL((act_quant_fp8_kernel<TIN, 4, BLK>), grid, dim3(64 * kFp8Waves), 0, stream, xin, thr, cb, x8, eps, groups, rows, carry);
    else if (bits == 3)
        hipLaunchKernelGGL((act_quant_fp8_kernel<TIN, 3, BLK>), grid, dim3(64 * kFp8Waves), 0, stream, xin, thr, cb, x8, eps, groups, rows, carry);
    else
        hipLaunchKernelGGL((act_quant_fp8_kernel<TIN, 2, BLK>), grid, dim3(64 * kFp8Waves), 0, stream, xin, thr, cb, x8, eps, groups, rows, carry);
}

}  // namespace
}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_act_quant_fp8(const void *x, int x_dtype, const float *thresholds, const float *codebook, void *x8,
                                int64_t rows, int64_t cols, int bits, float eps, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant_fp8: bits must be 2, 3, or 4");
    if (rows < 0 || cols < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_fp8: negative size");
    if (cols % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_act_quant_fp8: the row length must be a multiple of the group size 64");
    if (x_dtype != ARCQ_F16 && x_dtype != ARCQ_F32) return fail(ARCQ_ERR_DTYPE, "arcq_act_quant_fp8: x must be float16 or float32");
    if (rows * cols == 0) return ARCQ_OK;
    if (!x || !thresholds || !codebook || !x8) return fail(ARCQ_ERR_NULL, "arcq_act_quant_fp8: NULL tensor pointer");
    if (!aligned(x, 16) || !aligned(x8, 16)) return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_fp8: x and x8 must be 16-byte aligned");
    if (rows * cols >= (int64_t(1) << 40)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_fp8: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == ARCQ_F16) launch_act_fp8<__half, false>(x, thresholds, codebook, static_cast<uint8_t *>(x8), rows, cols, bits, eps, Fp8Carry{}, st);
    else launch_act_fp8<float, false>(x, thresholds, codebook, static_cast<uint8_t *>(x8), rows, cols, bits, eps, Fp8Carry{}, st);
    return launch_status("arcq_act_quant_fp8");
}

// Stage 1 into the FP8 GEMM's block layout; with packed_w != NULL the same launch reconstructs the layer's weights to
// FP8 as well (w8 [N, Kp], Kp = cols rounded up to 128, the padding zero).
ARCQ_API int arcq_act_quant_fp8_blocked(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                                        void *x8_blocked, int64_t rows, int64_t cols, int bits, float eps,
                                        const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                                        const float *w_scale, const float *w_code_sum, void *w8, int64_t N, float w_mult,
                                        void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant_fp8_blocked: bits must be 2, 3, or 4");
    if (rows < 0 || cols < 0 || N < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_fp8_blocked: negative size");
    if (cols % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_act_quant_fp8_blocked: the row length must be a multiple of the group size 64");
    if (x_dtype != ARCQ_F16 && x_dtype != ARCQ_F32) return fail(ARCQ_ERR_DTYPE, "arcq_act_quant_fp8_blocked: x must be float16 or float32");
    if (rows * cols == 0) return ARCQ_OK;
    if (!x || !thresholds || !codebook || !x8_blocked) return fail(ARCQ_ERR_NULL, "arcq_act_quant_fp8_blocked: NULL tensor pointer");
    if (!aligned(x, 16) || !aligned(x8_blocked, 16)) return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_fp8_blocked: x and x8_blocked must be 16-byte aligned");
    const int64_t Kp = (cols + 127) / 128 * 128;
    if (rows * Kp >= (int64_t(1) << 32) || cols > (1 << 24)) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_fp8_blocked: tensor too large");
    Fp8Carry carry{};
    if (packed_w && N > 0) {
        if (!w_codebook || !w_center || !w_scale || !w_code_sum || !w8)
            return fail(ARCQ_ERR_NULL, "arcq_act_quant_fp8_blocked: NULL weight tensor pointer");
        if (!(w_mult > 0.0f)) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_act_quant_fp8_blocked: w_mult must be positive");
        if (!aligned(w8, 16) || !aligned(packed_w, 4))
            return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_fp8_blocked: w8 must be 16-byte, packed_w 4-byte aligned");
        carry = Fp8Carry{packed_w, w_codebook, w_center, w_scale, w_code_sum, static_cast<uint8_t *>(w8), N, static_cast<int>(Kp), w_mult, 0};
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == ARCQ_F16) launch_act_fp8<__half, true>(x, thresholds, codebook, static_cast<uint8_t *>(x8_blocked), rows, cols, bits, eps, carry, st);
    else launch_act_fp8<float, true>(x, thresholds, codebook, static_cast<uint8_t *>(x8_blocked), rows, cols, bits, eps, carry, st);
    return launch_status("arcq_act_quant_fp8_blocked");
}

// The whole layer with FP8 operands in two launches: stage 1 into the block layout with the FP8 weights carried along,
// then the FP8 MFMA GEMM.  x8_ws: M * Kp bytes, w8_ws: N * Kp bytes (Kp = K rounded up to 128), both 16-byte aligned.
ARCQ_API int arcq_linear_otf_fp8(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                                 const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                                 const float *w_scale, const float *w_code_sum, const float *bias, float w_mult,
                                 void *x8_ws, void *w8_ws, void *y, int y_dtype, int64_t M, int64_t N, int64_t K, int bits,
                                 void *stream)
{
    if (M < 0 || N < 0 || K < 0) return fail(ARCQ_ERR_SHAPE, "arcq_linear_otf_fp8: negative size");
    if (M == 0 || N == 0) return ARCQ_OK;
    if (K == 0 || K % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_linear_otf_fp8: in_features must be a positive multiple of the group size 64");
    if (!packed_w || !w8_ws) return fail(ARCQ_ERR_NULL, "arcq_linear_otf_fp8: NULL tensor pointer");
    const int rc = arcq_act_quant_fp8_blocked(x, x_dtype, a_thresholds, a_codebook, x8_ws, M, K, bits, 1.0e-6f, packed_w, w_codebook,
                                              w_center, w_scale, w_code_sum, w8_ws, N, w_mult, stream);
    if (rc != ARCQ_OK) return rc;
    return arcq_linear_fp8_blocked(x8_ws, w8_ws, bias, w_mult, y, y_dtype, M, N, (K + 127) / 128 * 128, stream);
}

ARCQ_API int arcq_weight_dequant_fp8(const uint8_t *packed, const float *codebook, const float *center, const float *scale,
                                     const float *code_sum, void *w8, int64_t N, int64_t K, int bits, int group_size,
                                     float w_mult, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_weight_dequant_fp8: bits must be 2, 3, or 4");
    if (N < 0 || K < 0) return fail(ARCQ_ERR_SHAPE, "arcq_weight_dequant_fp8: negative size");
    if (group_size != 64 || K % 64 != 0)
        return fail(ARCQ_ERR_GROUP, "arcq_weight_dequant_fp8: group_size must be 64 and divide in_features");
    if (!(w_mult > 0.0f)) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_weight_dequant_fp8: w_mult must be positive");
    if (N * K == 0) return ARCQ_OK;
    if (!packed || !codebook || !center || !scale || !code_sum || !w8)
        return fail(ARCQ_ERR_NULL, "arcq_weight_dequant_fp8: NULL tensor pointer");
    if (!aligned(w8, 8) || !aligned(packed, 4)) return fail(ARCQ_ERR_ALIGN, "arcq_weight_dequant_fp8: w8 must be 8-byte, packed 4-byte aligned");
    if (N * K >= (int64_t(1) << 40) || K > (1 << 24)) return fail(ARCQ_ERR_SHAPE, "arcq_weight_dequant_fp8: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t pieces = N * (K / 8);
    int64_t blocks = (pieces + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    uint8_t *out = static_cast<uint8_t *>(w8);
    const int k = static_cast<int>(K);
    if (bits == 4)
        hipLaunchKernelGGL((weight_dequant_fp8_kernel<4>), dim3(blocks), dim3(256), 0, st, packed, codebook, center, scale, code_sum, out, N, k, k, w_mult);
    else if (bits == 3)
        hipLaunchKernelGGL((weight_dequant_fp8_kernel<3>), dim3(blocks), dim3(256), 0, st, packed, codebook, center, scale, code_sum, out, N, k, k, w_mult);
    else
        hipLaunchKernelGGL((weight_dequant_fp8_kernel<2>), dim3(blocks), dim3(256), 0, st, packed, codebook, center, scale, code_sum, out, N, k, k, w_mult);
    return launch_status("arcq_weight_dequant_fp8");
}
