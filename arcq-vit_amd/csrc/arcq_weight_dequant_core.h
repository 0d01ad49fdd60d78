// Stage-2 arithmetic for eight consecutive weights per thread (FQ/arcq_packed_triton.py:11-74), shared by the
// stand-alone weight kernel and by the stage-1 kernel that carries weight-reconstruction workgroups along.
#pragma once

#include "arcq_common.h"

namespace arcq {

// Work of workgroup number `block` (THREADS participating threads, numbered by threadIdx.x) of a launch that
// reconstructs out[N,K] from packed codes: thread idx = block * THREADS + threadIdx.x owns outputs [8 idx, 8 idx + 8)
// of the flattened tensor.  `lut` is an LDS array of
// (1 << BITS) * 64 floats that this call fills with the codebook replicated per lane (conflict-free lookups); every
// thread of the workgroup must call it (it contains a barrier).
// `threads` = number of participating threads per workgroup (a template constant in the overload below).
template <typename TOUT, int BITS>
__device__ __forceinline__ void weight_dequant8_block_n(int64_t block, int threads, float *lut, const uint8_t *__restrict__ packed,
                                                        const float *__restrict__ cb, const float *__restrict__ center,
                                                        const float *__restrict__ scale, const float *__restrict__ code_sum,
                                                        TOUT *__restrict__ out, int64_t N, int64_t K, int gs)
{
    constexpr int L = 1 << BITS;
    const int lane = threadIdx.x & 63;
    if (threadIdx.x < 64) {
#pragma unroll
        for (int c = 0; c < L; ++c) lut[c * 64 + lane] = cb[c];
    }
    __syncthreads();

    const int64_t chunks_per_row = K / 8;
    const int64_t idx = block * threads + threadIdx.x;
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

template <typename TOUT, int BITS, int THREADS = 256>
__device__ __forceinline__ void weight_dequant8_block(int64_t block, float *lut, const uint8_t *__restrict__ packed,
                                                      const float *__restrict__ cb, const float *__restrict__ center,
                                                      const float *__restrict__ scale, const float *__restrict__ code_sum,
                                                      TOUT *__restrict__ out, int64_t N, int64_t K, int gs)
{
    weight_dequant8_block_n<TOUT, BITS>(block, THREADS, lut, packed, cb, center, scale, code_sum, out, N, K, gs);
}

}  // namespace arcq
