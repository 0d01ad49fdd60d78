// Internal interface between the fused-GEMM entry point and its kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace arcq {

struct GemmArgs {
    const void *x_hat;       // [M,K] fp16
    const uint8_t *pw;       // [N, K*bits/8]
    const float *cb;         // [2^bits]
    const float *wc, *ws, *wcs;   // [N, K/64]
    const float *bias;       // [N] or nullptr
    void *y;                 // [M,N]
    bool y_f16;
    int M, N, K, bits;
};

// Large-M kernel (256-column x up-to-256-row workgroup tiles); requires K >= 64.
void launch_gemm_stream(const GemmArgs &g, hipStream_t stream);

// Large-M weight-stationary kernel (128-column slabs dequantized once per workgroup into LDS); requires K >= 64.
void launch_gemm_slab(const GemmArgs &g, hipStream_t stream);

// Small-M kernel (64 x 64 tiles, K split across the waves of a workgroup); requires K >= 64.
void launch_gemm_splitk(const GemmArgs &g, hipStream_t stream);

}  // namespace arcq
