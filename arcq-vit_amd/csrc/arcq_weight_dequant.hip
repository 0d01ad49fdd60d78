// Stage 2 stand-alone: packed weight codes -> dense reconstructed weight
// (FQ/arcq_packed_triton.py:11-74):  w[n,k] = fma(cb[code] - S[n,g]/gs, s[n,g], mu[n,g]).
//
// Eight consecutive codes starting at a multiple of eight occupy exactly `bits`
// whole bytes, so a thread that owns eight outputs never sees a code straddle
// its slice.  The codebook sits in LDS replicated per lane (lut[c*64 + lane])
// so that the per-element lookup is bank-conflict free.
#include "arcq_common.h"

namespace arcq {

template <typename TOUT, int BITS>
__global__ void __launch_bounds__(256)
weight_dequant8_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ cb,
                       const float *__restrict__ center, const float *__restrict__ scale,
                       const float *__restrict__ code_sum, TOUT *__restrict__ out,
                       int64_t N, int64_t K, int gs)
{
    constexpr int L = 1 << BITS;
    __shared__ float lut[L * 64];
    const int lane = threadIdx.x & 63;
    if (threadIdx.x < 64) {
#pragma unroll
        for (int c = 0; c < L; ++c) lut[c * 64 + lane] = cb[c];
    }
    __syncthreads();

    const int64_t chunks_per_row = K / 8;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= N * chunks_per_row) return;
    const int64_t n = idx / chunks_per_row;
    const int64_t k0 = (idx - n * chunks_per_row) * 8;
    const int64_t pcols = K * BITS / 8;
    const uint32_t w = load_codes8<BITS>(packed + n * pcols + k0 * BITS / 8);

    const float fgs = static_cast<float>(gs);
    const int64_t groups = K / gs;
    float v[8];
    // A run of eight outputs may cross a group boundary when gs is not a multiple of 8.
    int64_t g_prev = -1;
    float c = 0.f, s = 0.f, m = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int64_t g = (k0 + q) / gs;
        if (g != g_prev) {
            c = center[n * groups + g];
            s = scale[n * groups + g];
            m = code_sum[n * groups + g] / fgs;
            g_prev = g;
        }
        const int code = (w >> (BITS * q)) & (L - 1);
        v[q] = fma_f32(lut[code * 64 + lane] - m, s, c);
    }
    TOUT *dst = out + n * K + k0;
    if constexpr (sizeof(TOUT) == 2) {
        uint4 raw;
        __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
        for (int q = 0; q < 4; ++q) h[q] = __floats2half2_rn(v[2 * q], v[2 * q + 1]);
        *reinterpret_cast<uint4 *>(dst) = raw;
    } else {
        reinterpret_cast<float4 *>(dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4 *>(dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// Any K: one thread per element.
template <typename TOUT>
__global__ void __launch_bounds__(256)
weight_dequant_generic_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ cb,
                              const float *__restrict__ center, const float *__restrict__ scale,
                              const float *__restrict__ code_sum, TOUT *__restrict__ out,
                              int64_t N, int64_t K, int bits, int gs)
{
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= N * K) return;
    const int64_t n = idx / K;
    const int64_t k = idx - n * K;
    const int64_t groups = K / gs;
    const int64_t g = k / gs;
    const int code = get_code(packed + n * packed_cols(K, bits), k, bits);
    const float m = code_sum[n * groups + g] / static_cast<float>(gs);
    out[idx] = from_float<TOUT>(fma_f32(cb[code] - m, scale[n * groups + g], center[n * groups + g]));
}

template <typename TOUT>
static int launch(const uint8_t *packed, const float *cb, const float *center, const float *scale,
                  const float *code_sum, void *out, int64_t N, int64_t K, int bits, int gs, hipStream_t stream)
{
    TOUT *o = static_cast<TOUT *>(out);
    const bool fast = (K % 8 == 0) && aligned(out, 16) && aligned(packed, 4);
    if (fast) {
        const int64_t total = N * (K / 8);
        const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
#define ARCQ_LAUNCH_W8(B)                                                                                       \
    hipLaunchKernelGGL((weight_dequant8_kernel<TOUT, B>), dim3(blocks), dim3(256), 0, stream, packed, cb, center, \
                       scale, code_sum, o, N, K, gs)
        if (bits == 4) ARCQ_LAUNCH_W8(4);
        else if (bits == 3) ARCQ_LAUNCH_W8(3);
        else ARCQ_LAUNCH_W8(2);
#undef ARCQ_LAUNCH_W8
    } else {
        const int64_t total = N * K;
        const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
        hipLaunchKernelGGL((weight_dequant_generic_kernel<TOUT>), dim3(blocks), dim3(256), 0, stream, packed, cb,
                           center, scale, code_sum, o, N, K, bits, gs);
    }
    return launch_status("arcq_weight_dequant");
}

}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_weight_dequant(const uint8_t *packed, const float *codebook,
                                 const float *center, const float *scale, const float *code_sum,
                                 void *out, int out_dtype,
                                 int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_weight_dequant: bits must be 2, 3, or 4");
    if (N < 0 || K < 0 || group_size <= 0) return fail(ARCQ_ERR_SHAPE, "arcq_weight_dequant: bad sizes");
    if (K % group_size != 0)
        return fail(ARCQ_ERR_GROUP, "arcq_weight_dequant: in_features must be divisible by group_size");
    if (out_dtype != ARCQ_F16 && out_dtype != ARCQ_F32)
        return fail(ARCQ_ERR_DTYPE, "arcq_weight_dequant: out must be float16 or float32");
    if (N * K == 0) return ARCQ_OK;
    if (!packed || !codebook || !center || !scale || !code_sum || !out)
        return fail(ARCQ_ERR_NULL, "arcq_weight_dequant: NULL tensor pointer");
    if (N * K >= (int64_t(1) << 40)) return fail(ARCQ_ERR_SHAPE, "arcq_weight_dequant: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (out_dtype == ARCQ_F16)
        return launch<__half>(packed, codebook, center, scale, code_sum, out, N, K, bits, group_size, st);
    return launch<float>(packed, codebook, center, scale, code_sum, out, N, K, bits, group_size, st);
}
