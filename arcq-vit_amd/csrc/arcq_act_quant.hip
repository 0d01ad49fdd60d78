// Stage 1: activation group-residual quantizer (semantics:
// EXT/arcq_activation_kernel.cu:24-184; fused quantize+reconstruct as in
// FQ/arcq_packed_triton.py:123-178).
//
// Per group of gs input channels of one token:
//   mu = (x0 + x1 + ... ) / gs           serial, left to right
//   s  = sqrt((sum_j (x_j - mu)^2) / gs + eps)
//   t_j = (x_j - mu) / s                 IEEE divide
//   code_j = number of leading thresholds with t_j > thr[i]
//   S = sum_j cb[code_j]                 serial
//   x_hat_j = fma(s, cb[code_j] - S/gs, mu)
//
// Data layout.  x is [rows, cols] with cols = G*gs, so the groups of the whole
// tensor are consecutive 64-element runs of one flat array and "group index"
// is simply flat_offset/64.  The gs == 64 kernel gives every lane ONE group (so
// the serial sums are plain register loops, 64 independent chains per wave) and
// moves data between the coalesced global layout and that lane-per-group layout
// through an LDS tile of 64 groups x 64 elements, padded to a row stride of 65
// floats so that the per-lane column reads hit 64 different banks.
#include "arcq_common.h"

namespace arcq {

constexpr int kTileGroups = 64;   // groups per wave-sized workgroup
constexpr int kTileStride = 65;   // floats per group row in LDS (64 + 1 pad)

template <typename T> struct Vec16B;  // 16-byte global access unit
template <> struct Vec16B<float> { static constexpr int n = 4; };
template <> struct Vec16B<__half> { static constexpr int n = 8; };

// Coalesced 16-byte loads of one tile (4096 elements) into the padded LDS tile.
template <typename TIN>
__device__ __forceinline__ void load_tile(const TIN *__restrict__ x, int64_t elem0, int64_t elem_end,
                                          float *__restrict__ tile, int lane)
{
    constexpr int n = Vec16B<TIN>::n;
    constexpr int iters = kTileGroups * 64 / (64 * n);
#pragma unroll
    for (int i = 0; i < iters; ++i) {
        const int e = (i * 64 + lane) * n;  // element offset inside the tile
        float v[n];
        if (elem0 + e < elem_end) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(x + elem0 + e);
            if constexpr (n == 4) {
                v[0] = __uint_as_float(raw.x); v[1] = __uint_as_float(raw.y);
                v[2] = __uint_as_float(raw.z); v[3] = __uint_as_float(raw.w);
            } else {
                const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float2 f = __half22float2(h[q]);
                    v[2 * q] = f.x; v[2 * q + 1] = f.y;
                }
            }
        } else {
#pragma unroll
            for (int q = 0; q < n; ++q) v[q] = 0.0f;
        }
        float *dst = tile + (e >> 6) * kTileStride + (e & 63);
#pragma unroll
        for (int q = 0; q < n; ++q) dst[q] = v[q];
    }
}

template <typename TOUT>
__device__ __forceinline__ void store_tile(TOUT *__restrict__ out, int64_t elem0, int64_t elem_end,
                                           const float *__restrict__ tile, int lane)
{
    constexpr int n = Vec16B<TOUT>::n;
    constexpr int iters = kTileGroups * 64 / (64 * n);
#pragma unroll
    for (int i = 0; i < iters; ++i) {
        const int e = (i * 64 + lane) * n;
        if (elem0 + e >= elem_end) continue;
        const float *src = tile + (e >> 6) * kTileStride + (e & 63);
        uint4 raw;
        if constexpr (n == 4) {
            raw.x = __float_as_uint(src[0]); raw.y = __float_as_uint(src[1]);
            raw.z = __float_as_uint(src[2]); raw.w = __float_as_uint(src[3]);
        } else {
            __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
            for (int q = 0; q < 4; ++q) h[q] = __floats2half2_rn(src[2 * q], src[2 * q + 1]);
        }
        *reinterpret_cast<uint4 *>(out + elem0 + e) = raw;
    }
}

// Packs the lane's 64 codes (one byte each in `c`) into 2*BITS dwords, LSB first.
template <int BITS>
__device__ __forceinline__ void pack64(const uint8_t (&c)[64], uint32_t (&w)[2 * BITS])
{
    if constexpr (BITS == 4) {
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            uint32_t v = 0;
#pragma unroll
            for (int q = 0; q < 8; ++q) v |= static_cast<uint32_t>(c[d * 8 + q]) << (4 * q);
            w[d] = v;
        }
    } else if constexpr (BITS == 2) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t v = 0;
#pragma unroll
            for (int q = 0; q < 16; ++q) v |= static_cast<uint32_t>(c[d * 16 + q]) << (2 * q);
            w[d] = v;
        }
    } else {
        // 8 codes -> one 24-bit chunk; 4 chunks -> 3 dwords.
        uint32_t ch[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint32_t v = 0;
#pragma unroll
            for (int q = 0; q < 8; ++q) v |= static_cast<uint32_t>(c[k * 8 + q]) << (3 * q);
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

template <typename TIN, typename TOUT, int BITS>
__global__ void __launch_bounds__(64)
act_quant_g64_kernel(const TIN *__restrict__ x, const float *__restrict__ thr, const float *__restrict__ cb,
                     uint8_t *__restrict__ packed, uint8_t *__restrict__ codes_u8,
                     float *__restrict__ center, float *__restrict__ scale, float *__restrict__ code_sum,
                     TOUT *__restrict__ x_hat, int64_t total_groups, float eps)
{
    constexpr int L = 1 << BITS;
    __shared__ float tile[kTileGroups * kTileStride];
    __shared__ float lut[L * 64];  // codebook replicated per lane: lut[c*64 + lane], conflict-free

    const int lane = threadIdx.x;
    const int64_t group0 = static_cast<int64_t>(blockIdx.x) * kTileGroups;
    const int64_t elem0 = group0 * 64;
    const int64_t elem_end = total_groups * 64;

    float th[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) th[i] = thr[i];
#pragma unroll
    for (int c = 0; c < L; ++c) lut[c * 64 + lane] = cb[c];

    load_tile<TIN>(x, elem0, elem_end, tile, lane);
    __syncthreads();

    const int64_t g = group0 + lane;
    const bool live = g < total_groups;
    float *col = tile + lane * kTileStride;

    float xv[64];
#pragma unroll
    for (int j = 0; j < 64; ++j) xv[j] = col[j];

    float mu = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; ++j) mu += xv[j];
    mu /= 64.0f;

    float var = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
        const float d = xv[j] - mu;
        var += d * d;
    }
    const float s = sqrtf(var / 64.0f + eps);

    uint8_t code[64];
    float sum_codes = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
        const float t = (xv[j] - mu) / s;
        int c = 0;
        bool alive = true;
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            alive = alive && (t > th[i]);
            c += alive ? 1 : 0;
        }
        code[j] = static_cast<uint8_t>(c);
        const float v = lut[c * 64 + lane];
        xv[j] = v;  // the input value is not needed any more
        sum_codes += v;
    }

    if (live) {
        if (center) center[g] = mu;
        if (scale) scale[g] = s;
        if (code_sum) code_sum[g] = sum_codes;
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
                for (int q = 0; q < 3; ++q) reinterpret_cast<uint2 *>(dst)[q] = make_uint2(w[2 * q], w[2 * q + 1]);
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
                    d[k] = static_cast<uint32_t>(code[b]) | (static_cast<uint32_t>(code[b + 1]) << 8) |
                           (static_cast<uint32_t>(code[b + 2]) << 16) | (static_cast<uint32_t>(code[b + 3]) << 24);
                }
                dst[q] = make_uint4(d[0], d[1], d[2], d[3]);
            }
        }
    }

    if (x_hat) {
        const float code_mean = sum_codes / 64.0f;
#pragma unroll
        for (int j = 0; j < 64; ++j) col[j] = fma_f32(s, xv[j] - code_mean, mu);
        __syncthreads();
        store_tile<TOUT>(x_hat, elem0, elem_end, tile, lane);
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
    if (fast) {
        const unsigned blocks = static_cast<unsigned>((total_groups + kTileGroups - 1) / kTileGroups);
#define ARCQ_LAUNCH_G64(B)                                                                                   \
    hipLaunchKernelGGL((act_quant_g64_kernel<TIN, TOUT, B>), dim3(blocks), dim3(64), 0, stream, xin, thr, cb, \
                       packed, codes_u8, center, scale, code_sum, xo, total_groups, eps)
        if (bits == 4) ARCQ_LAUNCH_G64(4);
        else if (bits == 3) ARCQ_LAUNCH_G64(3);
        else ARCQ_LAUNCH_G64(2);
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

}  // namespace arcq

using namespace arcq;

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
