// Stage 1 of a quantized patch-embedding convolution (QuantConv2dPCARCQ with kernel == stride, FQ/quant_backends.py:
// 329-384): every pixel's three channels are one quantization group (its act_group_size is min(64, in_channels) = 3),
// and the reconstructed values are written straight as the rows of the patch matrix the convolution multiplies,
// row = patch (b, py, px), column k = c * 256 + i * 16 + j -- row-major [M, 768] fp16, or in the 32-row block layout
// [M/32][96][32][8] that arcq_linear_fused_blocked reads (a last block of r < 32 rows as [96][r][8]).
//
// The arithmetic per group is that of the any-group-size kernel of arcq_act_quant (which restates
// EXT/arcq_activation_kernel.cu:24-77 for a group of three): serial sums from zero, mean and variance divided by the
// group size with IEEE divisions, t = d / s, compare chain, x_hat = fma(s, cb[code] - code_sum / 3, mu) -- so the values
// equal, bit for bit, what that kernel writes for the NHWC pixels; what is new is the order of the work: one wave = 32
// patches x one pixel row of theirs, a lane = eight neighbouring pixels, loads and stores of 16 contiguous bytes, no
// NHWC copy of the image and no gather of the patch rows afterwards.
#include "arcq_common.h"

namespace arcq {
namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kP = 16, kC = 3, kKP = kC * kP * kP;      // patch side, channels, 768 values per patch row

template <typename TIN, int BITS>
__global__ void __launch_bounds__(256)
act_quant_patches_kernel(const TIN *__restrict__ img, const float *__restrict__ thr, const float *__restrict__ cb,
                         __half *__restrict__ x_hat, int B, int H, int W, float eps, int blocked)
{
    constexpr int L = 1 << BITS;
    const int tid = threadIdx.x, lane = tid & 63;
    const int lr = lane & 31, lh = lane >> 5;
    const int pw = W / kP, np = (H / kP) * pw;
    const int M = B * np;
    const int64_t wv = static_cast<int64_t>(blockIdx.x) * 4 + (tid >> 6);      // wave = (block of 32 patches, pixel row i)
    const int blk = static_cast<int>(wv >> 4), i = static_cast<int>(wv & 15);
    const int m = blk * 32 + lr;
    if (blk * 32 >= M) return;
    float th[L - 1], cbv[L];
#pragma unroll
    for (int q = 0; q < L - 1; ++q) th[q] = thr[q];
#pragma unroll
    for (int q = 0; q < L; ++q) cbv[q] = cb[q];
    const int mc = min(m, M - 1);
    const int b = mc / np, p = mc - b * np, py = p / pw, px = p - py * pw;
    const TIN *src = img + (static_cast<int64_t>(b) * kC * H + py * kP + i) * W + px * kP + 8 * lh;
    const int64_t plane = static_cast<int64_t>(H) * W;
    float x[kC][8];
#pragma unroll
    for (int c = 0; c < kC; ++c) {
        if constexpr (sizeof(TIN) == 2) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(src + c * plane);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[c][2 * e] = __half2float(__ushort_as_half(static_cast<unsigned short>(v[e] & 0xffffu)));
                x[c][2 * e + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(v[e] >> 16)));
            }
        } else {
            const float4 v0 = *reinterpret_cast<const float4 *>(src + c * plane);
            const float4 v1 = *reinterpret_cast<const float4 *>(src + c * plane + 4);
            x[c][0] = v0.x, x[c][1] = v0.y, x[c][2] = v0.z, x[c][3] = v0.w;
            x[c][4] = v1.x, x[c][5] = v1.y, x[c][6] = v1.z, x[c][7] = v1.w;
        }
    }
    const float fgs = static_cast<float>(kC);
    __half out[kC][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float mu = 0.0f;
#pragma unroll
        for (int c = 0; c < kC; ++c) mu += x[c][e];
        mu /= fgs;
        float var = 0.0f;
#pragma unroll
        for (int c = 0; c < kC; ++c) {
            const float d = x[c][e] - mu;
            var += d * d;
        }
        const float s = sqrtf(var / fgs + eps);
        float cv[kC], sum_codes = 0.0f;
#pragma unroll
        for (int c = 0; c < kC; ++c) {
            const float t = (x[c][e] - mu) / s;
            // while (code < L - 1 && t > thr[code]) ++code, with the codebook value picked along the way
            float v = cbv[0];
            bool alive = true;
#pragma unroll
            for (int q = 0; q < L - 1; ++q) {
                alive = alive && (t > th[q]);
                v = alive ? cbv[q + 1] : v;
            }
            cv[c] = v;
            sum_codes += v;
        }
        const float code_mean = sum_codes / fgs;
#pragma unroll
        for (int c = 0; c < kC; ++c) out[c][e] = __float2half_rn(fma_f32(s, cv[c] - code_mean, mu));
    }
    if (m >= M) return;
    // piece column of (c, i, half): k / 8 = c * 32 + 2 i + lh
    const int rows = min(32, M - blk * 32);
#pragma unroll
    for (int c = 0; c < kC; ++c) {
        const int kp = c * 32 + 2 * i + lh;
        __half *dst = blocked ? x_hat + static_cast<int64_t>(blk) * 32 * kKP + (static_cast<int64_t>(kp) * rows + lr) * 8
                              : x_hat + static_cast<int64_t>(m) * kKP + kp * 8;
        *reinterpret_cast<u32x4_t *>(dst) = *reinterpret_cast<const u32x4_t *>(out[c]);
    }
}

template <typename TIN, int BITS>
void launch_patches(const void *img, const float *thr, const float *cb, void *x_hat, int B, int H, int W, float eps, int blocked,
                    hipStream_t stream)
{
    const int64_t M = static_cast<int64_t>(B) * (H / kP) * (W / kP);
    const int64_t waves = (M + 31) / 32 * 16;
    hipLaunchKernelGGL((act_quant_patches_kernel<TIN, BITS>), dim3(static_cast<unsigned>((waves + 3) / 4)), dim3(256), 0, stream,
                       static_cast<const TIN *>(img), thr, cb, static_cast<__half *>(x_hat), B, H, W, eps, blocked);
}

}  // namespace
}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_act_quant_patches(const void *img, int img_dtype, const float *thresholds, const float *codebook, void *x_hat,
                                    int64_t B, int64_t C, int64_t H, int64_t W, int64_t patch, int bits, float eps, int blocked,
                                    void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_act_quant_patches: bits must be 2, 3, or 4");
    if (B < 0 || H < 0 || W < 0) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_patches: negative size");
    if (C != kC || patch != kP)
        return fail(ARCQ_ERR_UNSUPPORTED, "arcq_act_quant_patches: three channels and 16 x 16 patches only (got C=%lld, patch=%lld)",
                    static_cast<long long>(C), static_cast<long long>(patch));
    if (H % kP || W % kP) return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_patches: image sides must be multiples of 16");
    if (img_dtype != ARCQ_F32 && img_dtype != ARCQ_F16) return fail(ARCQ_ERR_DTYPE, "arcq_act_quant_patches: img must be float32 or float16");
    if (B * H * W == 0) return ARCQ_OK;
    if (!img || !thresholds || !codebook || !x_hat) return fail(ARCQ_ERR_NULL, "arcq_act_quant_patches: NULL pointer");
    if (!aligned(img, 16) || !aligned(x_hat, 16)) return fail(ARCQ_ERR_ALIGN, "arcq_act_quant_patches: img and x_hat must be 16-byte aligned");
    if (B > (1 << 20) || H > (1 << 14) || W > (1 << 14) || B * (H / kP) * (W / kP) >= (int64_t(1) << 26))
        return fail(ARCQ_ERR_SHAPE, "arcq_act_quant_patches: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int b = static_cast<int>(B), h = static_cast<int>(H), w = static_cast<int>(W);
#define ARCQ_GO(T) \
    do { \
        if (bits == 4) launch_patches<T, 4>(img, thresholds, codebook, x_hat, b, h, w, eps, blocked, st); \
        else if (bits == 3) launch_patches<T, 3>(img, thresholds, codebook, x_hat, b, h, w, eps, blocked, st); \
        else launch_patches<T, 2>(img, thresholds, codebook, x_hat, b, h, w, eps, blocked, st); \
    } while (0)
    if (img_dtype == ARCQ_F16) ARCQ_GO(__half);
    else ARCQ_GO(float);
#undef ARCQ_GO
    return launch_status("arcq_act_quant_patches");
}
