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
    // Post-operations on the rounded outputs (arcq_common.h, post_ops16 / post_op1); only the block-layout kernels
    // (launch_gemm_slab8, launch_gemm_pair) and the small-M kernel (launch_gemm_splitk) apply them, the entry points
    // keep them away from the others.
    const void *residual = nullptr;   // [M,N] of y's type, or nullptr
    bool gelu = false;
    // Quantize-the-output mode of the block-layout kernels fed from reconstructed weights: y (fp16, N a multiple of 64)
    // receives stage 1 of the layer that consumes this one's output (its thresholds / codebook, `bits` levels) in
    // that layer's 32-row block layout.  No residual in this mode.
    const float *next_thr = nullptr, *next_cb = nullptr;
};

// Large-M kernel (256-column x up-to-256-row workgroup tiles); requires K >= 64.
void launch_gemm_stream(const GemmArgs &g, hipStream_t stream);

// Large-M weight-stationary kernel (128-column slabs dequantized once per workgroup into LDS); requires K >= 64.
void launch_gemm_slab(const GemmArgs &g, hipStream_t stream);
// The same kernel fed from weights reconstructed beforehand into w_hat ([N,K] fp16, 16-byte aligned).
void launch_gemm_slab_prebuilt(const GemmArgs &g, const void *w_hat, hipStream_t stream);
// Eight-wave weight-stationary kernel; g.x_hat is in the 32-row block layout ([M/32][K/8][32][8] fp16, a last
// block of fewer rows stored compactly), g.M positive, g.K a positive multiple of 64.  w_hat != nullptr: weights already reconstructed ([N,K] fp16).
void launch_gemm_slab8(const GemmArgs &g, const void *w_hat, hipStream_t stream);
// The same with two row blocks per wave and pass (wave tile 64 x 128); weights must be reconstructed already.
void launch_gemm_pair(const GemmArgs &g, const void *w_hat, hipStream_t stream);
// Whether launch_gemm_pair is the kernel of choice for this shape.
bool gemm_pair_pays(const GemmArgs &g);
// Whether the whole-layer entry point with scratch-only workspaces runs stage 1 into the block layout and the
// eight-wave kernel for this shape.
bool otf_blocked_pays(int64_t M, int64_t N, int64_t K);
// Whether the eight-wave kernel, given a weight workspace, copies weights reconstructed beforehand for this shape.
bool blocked_uses_workspace(int64_t N, int64_t K);
// arcq_linear_fused_blocked with the state of the workspace made explicit: w_hat_ready means w_hat_ws already holds
// the reconstructed weights (and is to be used); otherwise they are rebuilt first where that pays.
int linear_fused_blocked(const void *x_hat_blocked, const uint8_t *packed_w, const float *w_codebook,
                         const float *w_center, const float *w_scale, const float *w_code_sum, const float *bias,
                         void *w_hat_ws, bool w_hat_ready, void *y, int y_dtype, int64_t M, int64_t N, int64_t K, int bits,
                         int group_size, void *stream, const void *residual = nullptr, bool gelu = false,
                         const float *next_thr = nullptr, const float *next_cb = nullptr);


// Compute units of the current device (256 when there is none to ask: the host-side predicates also run without a
// GPU); what the weight-stationary kernels size their row ranges by (one workgroup per compute unit).
int device_cus();

// Small-M kernel (64 x 64 tiles, K split across the waves of a workgroup); requires K >= 64.
void launch_gemm_splitk(const GemmArgs &g, hipStream_t stream);
// arcq_linear_fused with GELU / a residual ([M,N] of y's type) on the rounded outputs; with either set it needs the
// small-M kernel's shapes (fewer than 512 rows, K >= 64) and reports ARCQ_ERR_UNSUPPORTED otherwise.
int linear_fused_post(const void *x_hat, const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                      const float *w_scale, const float *w_code_sum, const float *bias, void *y, int y_dtype,
                      int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream,
                      const void *residual, bool gelu);

// Whole on-the-fly layer in one launch (activation quantizer + split-K product) for M < 512.
struct OtfSmallArgs {
    const void *x;           // [M,K] fp16 or fp32
    bool x_f16;
    const float *a_thr, *a_cb;
    const uint8_t *pw;
    const float *w_cb, *wc, *ws, *wcs, *bias;
    void *x_hat_ws;          // [M,K] fp16, must not alias x; may be nullptr
    void *y;
    bool y_f16;
    int M, N, K, bits;
    float eps;
    // Optional work fused around the layer: a LayerNorm over the rows of x in front of stage 1 (fp32 weight / bias
    // [K], 16-byte aligned; nullptr: none) and GELU / a residual ([M,N] of y's type) on the rounded outputs.
    const float *ln_weight = nullptr, *ln_bias = nullptr;
    float ln_eps = 0.0f;
    const void *residual = nullptr;
    bool gelu = false;
    // Quantize-the-output mode: y (fp16, N a multiple of 64) receives not the layer's output but stage 1 of the layer
    // that consumes it (that layer's activation thresholds / codebook, same bits), row-major.
    const float *next_thr = nullptr, *next_cb = nullptr;
};
bool otf_small_supported(int64_t M, int64_t N, int64_t K, bool any_supported);
void launch_otf_small(const OtfSmallArgs &a, hipStream_t stream);

// Whole layer in one launch for short rows: stage 1 (optionally LayerNorm first) into LDS, product with weights that
// the same launch reconstructs into the weight workspace in its 32-column block layout ([N/32][K/8][32][8] fp16).
struct OtfRowsArgs {
    const void *x;           // [M,K] fp16
    const float *a_thr, *a_cb;
    const float *ln_weight, *ln_bias;    // fp32 [K], or nullptr: no LayerNorm
    float ln_eps;
    const uint8_t *pw;
    const float *w_cb, *wc, *ws, *wcs, *bias;
    void *w_hat_ws;          // at least N*K fp16, 16-byte aligned
    void *y;
    bool y_f16;
    const void *residual;    // [M,N] of y's type, or nullptr
    bool gelu;
    int M, N, K, bits;
    float eps;
};
// Shapes the kernels can run: M >= 512 and few enough rows that one workgroup per 64 of them is resident at once
// (M <= 64 x compute units, twice that for K = 192), N a multiple of 32 and either K = 192 / 256 / 384 / 768 with
// everything within LDS (otf_rows_kernel; K = 768: fp16 outputs only, which launch_otf_rows checks) or K = 768 / 1536
// with N <= 384 or K = 3072 with N <= 768, no LayerNorm in front (otf_rows_phased_kernel).
bool otf_rows_supported(int64_t M, int64_t N, int64_t K, bool layernorm = false);
bool otf_rows_is_phased(int64_t N, int64_t K);      // which of the two one-launch kernels serves the shape
// Whether the whole-layer entry points take it for this shape (fp16 input, both workspaces given).
bool otf_rows_pays(int64_t M, int64_t N, int64_t K, bool layernorm = false);
// Returns kNotLaunched (having launched nothing and recorded no error) when the stream cannot be given a counter or
// the device would not hold all the launch's workgroups at once: the caller takes the two-launch path.
constexpr int kNotLaunched = -1000;
// Slot of `key` in a table of `slots` keys (nullptr = free): its own if it has one, else the first free one on its
// probe sequence, which it then owns; -1 when the table is full.  (The per-workspace counters of launch_otf_rows.)
int rows_counter_slot(const void **table, int slots, const void *key);
int launch_otf_rows(const OtfRowsArgs &a, hipStream_t stream);

}  // namespace arcq
