// Stage 2 stand-alone: packed weight codes -> dense reconstructed weight
// (FQ/arcq_packed_triton.py:11-74):  w[n,k] = fma(cb[code] - S[n,g]/gs, s[n,g], mu[n,g]).
//
// Eight consecutive codes starting at a multiple of eight occupy exactly `bits`
// whole bytes, so a thread that owns eight outputs never sees a code straddle
// its slice.  The codebook sits in LDS replicated per lane (lut[c*64 + lane])
// so that the per-element lookup is bank-conflict free.
#include "arcq_common.h"
#include "arcq_weight_dequant_core.h"

namespace arcq {

template <typename TOUT, int BITS>
__global__ void __launch_bounds__(256)
weight_dequant8_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ cb,
                       const float *__restrict__ center, const float *__restrict__ scale,
                       const float *__restrict__ code_sum, TOUT *__restrict__ out,
                       int64_t N, int64_t K, int gs)
{
    __shared__ float lut[(1 << BITS) * 64];
    weight_dequant8_block<TOUT, BITS>(blockIdx.x, lut, packed, cb, center, scale, code_sum, out, N, K, gs);
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
