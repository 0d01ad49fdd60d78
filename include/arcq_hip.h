/*
 * arcq_hip.h -- C ABI of libarcq_hip.so: ARCQ packed quantized-linear kernels
 * for AMD MI355X (gfx950 / CDNA4).
 *
 * Every entry point is a plain-C replacement for one binding of the
 * reference's pybind11 extension `arcq_infer_cuda_ext`
 * (methods/fair_qat_framework/fair_qat/arcq_infer_cuda/arcq_infer_bind.cpp:57-66)
 * or for one of its Triton launchers
 * (methods/fair_qat_framework/fair_qat/arcq_packed_triton.py).  Abbreviations
 * in the citations below: FQ = methods/fair_qat_framework/fair_qat,
 * EXT = FQ/arcq_infer_cuda.
 *
 * Conventions
 *   - All pointers are DEVICE pointers on the current HIP device unless said
 *     otherwise.  Tensors are dense row-major.  The library never allocates,
 *     frees or synchronises; the caller owns every buffer.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Every
 *     call only enqueues kernels on that stream and returns.
 *   - Return value: 0 = ok; < 0 = argument error (ARCQ_ERR_*), nothing was
 *     enqueued; > 0 = the hipError_t of a failed launch.  arcq_last_error()
 *     returns a message for the calling thread's most recent non-zero return.
 *   - bits is 2, 3 or 4; a codebook has L = 2^bits fp32 entries and L-1
 *     non-decreasing fp32 thresholds.  Code j of a row lives at bits
 *     [j*bits, (j+1)*bits) of the row's little-endian byte stream
 *     (EXT/arcq_pack_kernel.cu:8-36); a row of n codes takes
 *     ceil(n*bits/8) bytes.
 *   - Floating-point contract: fp32 IEEE arithmetic with round-to-nearest,
 *     correctly rounded divide and sqrt, group sums taken serially left to
 *     right (the loop order of EXT/arcq_activation_kernel.cu:49-60); fused
 *     multiply-add only in the two reconstructions x_hat = fma(s, v, mu) and
 *     w_hat = fma(v, s, mu).
 */
#ifndef ARCQ_HIP_H
#define ARCQ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARCQ_VERSION 100 /* major*10000 + minor*100 + patch */

/* element types for the void* tensor arguments */
#define ARCQ_F32 0
#define ARCQ_F16 1

/* argument errors (negative return values) */
#define ARCQ_OK 0
#define ARCQ_ERR_BITS (-1)        /* "bits must be 2, 3, or 4" */
#define ARCQ_ERR_GROUP (-2)       /* "in_features must be divisible by group_size" */
#define ARCQ_ERR_NULL (-3)        /* a required pointer is NULL */
#define ARCQ_ERR_SHAPE (-4)       /* negative or inconsistent sizes */
#define ARCQ_ERR_DTYPE (-5)       /* dtype code not supported by this entry point */
#define ARCQ_ERR_UNSUPPORTED (-6) /* valid for the reference, not built here (message says what) */
#define ARCQ_ERR_ALIGN (-7)       /* pointer not aligned as the kernel requires */

int arcq_version(void);
const char *arcq_last_error(void);
/* The library reads its tuning variables (ARCQ_GEMM_KERNEL, ARCQ_OTF_FUSED, ARCQ_PAIR: they pin kernel choices for
 * experiments; results are the same bits either way) once per process; this reads them again.  A hook for tests
 * and tuning scripts with no counterpart in the reference; do not call it while other threads are inside the library. */
void arcq_reload_tuning(void);

/* ---- bit packing --------------------------------------------------------
 * Replaces pack_codes_cuda / unpack_codes_cuda / unpack_codes_u8_cuda,
 * EXT/arcq_pack_kernel.cu:94-114, :116-136, :138-158.
 * codes [rows, length]; packed [rows, ceil(length*bits/8)].  `packed` need not
 * be zeroed beforehand (the reference pre-zeroes and ORs).  Codes are masked
 * to their low `bits` bits, as set_packed_code_u8 does. */
int arcq_pack_codes(const int64_t *codes, uint8_t *packed, int64_t rows, int64_t length, int bits, void *stream);
int arcq_unpack_codes(const uint8_t *packed, int64_t *codes, int64_t rows, int64_t length, int bits, void *stream);
int arcq_unpack_codes_u8(const uint8_t *packed, uint8_t *codes, int64_t rows, int64_t length, int bits, void *stream);

/* ---- stage 1: activation group-residual quantizer -------------------------
 * One kernel replaces quantize_activation_cuda, quantize_activation_u8_cuda and
 * quantize_activation_dequant_cuda (EXT/arcq_activation_kernel.cu:188-237,
 * :239-285, :287-326) and dequant_activation_triton
 * (FQ/arcq_packed_triton.py:181-215); which outputs are produced is chosen by
 * which output pointers are non-NULL:
 *   packed   [rows, ceil(cols*bits/8)] u8   bit-packed codes
 *   codes_u8 [rows, cols] u8                one byte per code
 *   center, scale, code_sum [rows, cols/group_size] f32
 *   x_hat    [rows, cols] of x_hat_dtype    mu + s*(cb[code] - code_sum/gs)
 * x is [rows, cols] of x_dtype (ARCQ_F32 or ARCQ_F16; fp16 is widened to fp32
 * before any arithmetic).  x_hat may alias x when the two dtypes are equal
 * (the in-place use at FQ/arcq_packed_on_the_fly.py:143-145).
 * eps is added to the variance inside the square root; the reference kernels
 * hard-code 1e-6f.  thresholds [L-1], codebook [L], both fp32. */
int arcq_act_quant(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                   uint8_t *packed, uint8_t *codes_u8, float *center, float *scale, float *code_sum,
                   void *x_hat, int x_hat_dtype,
                   int64_t rows, int64_t cols, int bits, int group_size, float eps, void *stream);

/* ---- stage 2: packed weight -> dense weight -------------------------------
 * Replaces unpack_weight_triton (FQ/arcq_packed_triton.py:77-120):
 * out[n,k] = (cb[code] - code_sum[n,g]/gs) * scale[n,g] + center[n,g], g = k/gs,
 * rounded once to out_dtype (ARCQ_F16 as the reference, or ARCQ_F32).
 * packed [N, ceil(K*bits/8)]; center/scale/code_sum [N, K/group_size]. */
int arcq_weight_dequant(const uint8_t *packed, const float *codebook,
                        const float *center, const float *scale, const float *code_sum,
                        void *out, int out_dtype,
                        int64_t N, int64_t K, int bits, int group_size, void *stream);

/* ---- stages 2+3 fused: y = x_hat * w_hat^T + bias --------------------------
 * Replaces the pair unpack_weight_triton + F.linear at
 * FQ/arcq_packed_on_the_fly.py:148-160 (and F.linear on weight_dequant at
 * FQ/arcq_packed_linear.py:175-176) without materialising w_hat in HBM: packed
 * codes are streamed, reconstructed exactly as arcq_weight_dequant does,
 * rounded to fp16, and fed to fp16 MFMA with fp32 accumulation.
 * x_hat [M,K] fp16; y [M,N] of y_dtype (ARCQ_F16 or ARCQ_F32); bias [N] fp32 or
 * NULL, added in fp32 before the output rounding.  Requires group_size == 64;
 * x_hat and y must be 16-byte aligned, packed_w 4-byte aligned. */
int arcq_linear_fused(const void *x_hat,
                      const uint8_t *packed_w, const float *w_codebook,
                      const float *w_center, const float *w_scale, const float *w_code_sum,
                      const float *bias, void *y, int y_dtype,
                      int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);

/* Name of the kernel arcq_linear_fused launches for an [M,K] x [N,K] problem ("gemm_splitk_kernel",
 * "gemm_slab_kernel", "gemm_stream_kernel" or "gemm_fused_kernel"), as it appears in a kernel trace.  A profiling
 * aid with no counterpart in the reference; the returned string is static. */
const char *arcq_linear_fused_kernel(int64_t M, int64_t N, int64_t K);

/* ---- whole packed on-the-fly layer: stage 1 then stages 2+3 ----------------
 * Replaces ARCQPackedLinearOnTheFly.forward's device work
 * (FQ/arcq_packed_on_the_fly.py:137-161).  x [M,K] of x_dtype; x_hat_ws is a
 * caller-owned fp16 [M,K] workspace that receives the reconstructed activation
 * (it may alias x when x_dtype == ARCQ_F16, as the reference overwrites its
 * fp16 copy of x). */
int arcq_linear_otf(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                    const uint8_t *packed_w, const float *w_codebook,
                    const float *w_center, const float *w_scale, const float *w_code_sum,
                    const float *bias, void *x_hat_ws, void *y, int y_dtype,
                    int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);

/* The two entry points above with one more caller-owned scratch buffer, w_hat_ws: fp16 [N,K], 16-byte aligned, the
 * counterpart of the reference module's optional _weight_buffer (FQ/arcq_packed_on_the_fly.py:148-158, the `out=` of
 * unpack_weight_triton).  For shapes where many workgroups would each repeat the weight reconstruction (long K with few
 * output columns, large models) the weights are rebuilt once into w_hat_ws (arcq_weight_dequant) and the GEMM copies
 * them; for all other shapes, or with w_hat_ws == NULL, these behave exactly like arcq_linear_fused / arcq_linear_otf.
 * arcq_linear_otf_ws with a workspace and 512 rows or more always takes the workspace route: the fp16 weights are
 * reconstructed into w_hat_ws inside the layer's first (or only) launch and the GEMM reads them from there, i.e. the
 * dense weight does pass through memory (L2-resident: at most a few MB) -- the reference's unpack-then-GEMM order,
 * without a launch of its own.  Without a workspace the weights are reconstructed inside the GEMM kernel.
 * y is bit-identical in every case; the contents of w_hat_ws after the call are unspecified.  arcq_linear_otf_ws treats
 * x_hat_ws as scratch too (unspecified contents afterwards: it may hold x_hat in the block layout described below, or
 * be left untouched); call arcq_linear_otf to get x_hat row-major in x_hat_ws.
 * With fp16 x, N a multiple of 32, w_hat_ws given (128-byte aligned) and 512 <= M <= 64 x the device's compute units
 * (twice that for K = 192), arcq_linear_otf_ws runs the whole layer as ONE launch for K = 192 / 256 / 384 and, with
 * fp16 outputs, K = 768 with more than 384 outputs (from M >= 8800 - 1.15e9 / (N K) rows on: below that the two
 * launches are faster), and for K = 768 / 1536 with N <= 384 or K = 3072 with N <= 768 from 86 / 128 / 128 blocks of
 * 64 rows on (x_hat stays on chip; w_hat_ws is filled
 * cooperatively, in 32-column blocks [N/32][K/8][32][8]).  The upper limit on M keeps every workgroup of the launch
 * resident at once: each waits, for at most 0.5 ms, until all the others have written their share of w_hat; if the
 * device is shared with other kernels at that moment the wait can run out, after which a workgroup rebuilds all of
 * w_hat itself (same result, late; arcq_rows_wait_timeouts counts these).  That launch counts in a word of the
 * library's static device memory chosen by the address of w_hat_ws: calls that may overlap in time (different
 * streams, graphs replayed side by side) must use different weight workspaces -- which they must anyway, since each
 * call overwrites its workspace -- and then never share a word; the first 4096 workspace addresses a process uses on a
 * device get a word each, calls with further ones take the two-launch path.  ARCQ_ROWS=0 in the environment keeps
 * the two-launch path everywhere. */
int arcq_linear_fused_ws(const void *x_hat,
                         const uint8_t *packed_w, const float *w_codebook,
                         const float *w_center, const float *w_scale, const float *w_code_sum,
                         const float *bias, void *w_hat_ws, void *y, int y_dtype,
                         int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);
int arcq_linear_otf_ws(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                       const uint8_t *packed_w, const float *w_codebook,
                       const float *w_center, const float *w_scale, const float *w_code_sum,
                       const float *bias, void *x_hat_ws, void *w_hat_ws, void *y, int y_dtype,
                       int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);

/* As arcq_linear_fused_kernel, for arcq_linear_fused_ws: "weight_dequant8_kernel+gemm_slab_kernel" when a call with
 * these sizes and a workspace (have_workspace != 0) rebuilds the weights first, else arcq_linear_fused_kernel's
 * answer.  A profiling aid with no counterpart in the reference. */
const char *arcq_linear_fused_ws_kernel(int64_t M, int64_t N, int64_t K, int have_workspace);

/* ---- 32-row block layout for x_hat ------------------------------------------
 * No counterpart in the reference (its x_hat goes to cuBLAS row-major, FQ/arcq_packed_on_the_fly.py:141-160): these
 * are the two halves arcq_linear_otf_ws is made of when its workspaces are scratch only, exposed so that each can be
 * called, timed and tested on its own.  The layout stores 16-byte pieces of 8 values as
 *     x_hat_blocked[((row / 32) * (K / 8) + k / 8) * 32 + row % 32][k % 8]        (K a multiple of 64),
 * and a last block of r = rows % 32 rows compactly as [(k / 8) * r + row % 32][k % 8] behind the whole blocks, so the
 * tensor takes exactly rows * K values.  An MFMA operand fragment (32 rows x 8 values) is one contiguous 512-byte run.  Values are the ones
 * arcq_act_quant writes row-major, bit for bit; arcq_linear_fused_blocked's result equals arcq_linear_fused's on the
 * row-major tensor, bit for bit.  group_size is 64; M * K must stay below 2^31. */
int arcq_act_quant_blocked(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                           void *x_hat_blocked, int64_t rows, int64_t cols, int bits, float eps, void *stream);
/* The same launch also reconstructs w_hat[N, cols] (fp16, what arcq_weight_dequant writes) from the layer's packed
 * weights, in extra workgroups: the two inputs of arcq_linear_fused_blocked(..., w_hat_ready = 1) for one launch. */
int arcq_act_quant_blocked_with_weights(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                                        void *x_hat_blocked, int64_t rows, int64_t cols, int bits, float eps,
                                        const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                                        const float *w_scale, const float *w_code_sum, void *w_hat, int64_t N,
                                        void *stream);
/* w_hat_ws: NULL, or a fp16 [N,K] buffer.  w_hat_ready != 0: it already holds the reconstructed weights (from
 * arcq_weight_dequant, arcq_act_quant_blocked_with_weights or an earlier call with the same weights) and the kernel
 * copies from it; w_hat_ready == 0: scratch, filled first for the shapes where that pays. */
int arcq_linear_fused_blocked(const void *x_hat_blocked,
                              const uint8_t *packed_w, const float *w_codebook,
                              const float *w_center, const float *w_scale, const float *w_code_sum,
                              const float *bias, void *w_hat_ws, int w_hat_ready, void *y, int y_dtype,
                              int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);

/* ---- the layer with the elementwise work around it fused in ------------------------------------------------
 * The transformer block the reference's models are built from (timm's Block via FQ/timm_quant_models.py:63-121) is
 *     x = x + proj(attention(qkv(LayerNorm1(x))));   x = x + fc2(GELU(fc1(LayerNorm2(x))))
 * with qkv / proj / fc1 / fc2 the packed linears.  This entry point runs one packed on-the-fly layer together with
 * the work that sits directly in front of and behind it, so that the tensors in between never make a round trip
 * through HBM in a launch of their own:
 *     y = residual + activation(linear(stage1(producer(x))))
 *   producer   ARCQ_PRODUCER_LAYERNORM: LayerNorm over the last dimension (ln_weight, ln_bias [K] fp32, ln_eps), its
 *              result rounded to x's type, inside the stage-1 launch (arcq_act_quant_blocked_ln; K <= 1024)
 *   activation ARCQ_ACT_GELU: the exact (erf) GELU of the rounded linear output, rounded again, in the GEMM's epilogue
 *   residual   [M,N] of y's type, added to the rounded value, rounded again, in the GEMM's epilogue
 * Every step rounds where a separate kernel would have stored its result, so y equals the unfused sequence bit for
 * bit given the same LayerNorm output.  With no option set it is arcq_linear_otf_ws.  With an option set it needs
 * group_size 64 and M >= 512 (the block-layout path or the one-launch kernel described at arcq_linear_otf_ws, which
 * then also runs the LayerNorm, GELU and residual) and returns ARCQ_ERR_UNSUPPORTED otherwise: compose the
 * layer from the separate operations then.  Workspaces as arcq_linear_otf_ws (w_hat_ws may be NULL).
 * struct_size = sizeof(arcq_linear_ex_args). */
#define ARCQ_PRODUCER_NONE 0
#define ARCQ_PRODUCER_LAYERNORM 1
#define ARCQ_PRODUCER_XHAT 2
#define ARCQ_ACT_NONE 0
#define ARCQ_ACT_GELU 1
typedef struct arcq_linear_ex_args {
    uint32_t struct_size;
    int32_t x_dtype, y_dtype, producer, activation, bits, group_size;
    float ln_eps;
    int64_t M, N, K;
    const void *x;
    const float *ln_weight, *ln_bias;
    const float *a_thresholds, *a_codebook;
    const uint8_t *packed_w;
    const float *w_codebook, *w_center, *w_scale, *w_code_sum, *bias;
    const void *residual;
    void *x_hat_ws, *w_hat_ws, *y;
    /* fields added after the first version of this struct (a caller that passes the shorter struct_size gets NULL) */
    const float *next_a_thresholds, *next_a_codebook;
} arcq_linear_ex_args;
int arcq_linear_otf_ex(const arcq_linear_ex_args *args, void *stream);

/* Two layers chained through their quantizer (fc1 -> GELU -> fc2 of the block: the GELU output is only ever consumed
 * quantized, FQ/arcq_packed_on_the_fly.py:139-145 is the stage-1 call that disappears).
 *   next_a_thresholds / next_a_codebook set (the activation quantizer of the layer that consumes y; same bits, group
 *   size 64, N a multiple of 64, y_dtype ARCQ_F16): y receives, instead of the layer's output, that output's
 *   reconstruction x_hat = stage1(post-processed, fp16-rounded output), fp16, in the layout arcq_xhat_layout(M) --
 *   exactly what the consuming layer's stage 1 would have produced from the stored output, bit for bit.
 *   producer == ARCQ_PRODUCER_XHAT on the consuming layer's call: x [M,K] fp16 already is that x_hat in
 *   arcq_xhat_layout(M); stage 1 is skipped (a_thresholds / a_codebook are not read) and the call runs stages 2+3 with
 *   the optional GELU / residual.
 * arcq_xhat_layout: 0 = row-major [M,K] (fewer than 512 rows), 1 = the 32-row block layout described above.
 * Both return ARCQ_ERR_UNSUPPORTED for shapes the kernels that hold a whole group per output row do not serve; the
 * caller then runs the two layers the ordinary way. */
int arcq_xhat_layout(int64_t M);

/* LayerNorm + stage 1 into the block layout in one launch (the first half of arcq_linear_otf_ex with
 * ARCQ_PRODUCER_LAYERNORM), exposed so that it can be called and tested on its own; no counterpart in the
 * reference.  LayerNorm arithmetic, fp32: every lane's 32 values (half a group) are summed serially, a row's partial
 * sums are added group by group, lower half first; mean = sum / cols; var = the same sum over (x - mean)^2, / cols;
 * y = ((x - mean) * (1 / sqrt(var + ln_eps))) * ln_weight + ln_bias with one rounding per operation, then rounded to
 * x's type.  64 <= cols <= 1024.  packed_w != NULL: the launch also reconstructs w_hat[N, cols] (fp16), as
 * arcq_act_quant_blocked_with_weights does. */
int arcq_act_quant_blocked_ln(const void *x, int x_dtype, const float *ln_weight, const float *ln_bias, float ln_eps,
                              const float *thresholds, const float *codebook, void *x_hat_blocked,
                              int64_t rows, int64_t cols, int bits, float eps,
                              const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                              const float *w_scale, const float *w_code_sum, void *w_hat, int64_t N, void *stream);

/* arcq_linear_otf_ws for callers that cannot allocate device memory or lend workspaces (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The two
 * scratch buffers come from a static device array of ARCQ_STATIC_SCRATCH_BYTES inside the library, of which every GPU
 * the library runs on holds its own copy until the process ends; the call itself allocates and frees nothing.  It
 * needs 2*N*K (rounded up to 256) + 2*M*K bytes of it and returns ARCQ_ERR_SHAPE beyond that (the limit covers every
 * DeiT-Small layer at batch 64).  y equals arcq_linear_otf_ws's bit for bit.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU (different streams, or threads) race; calls on one stream are ordered.  The
 * first call on a device looks up the array's address; make it outside a graph capture. */
#define ARCQ_STATIC_SCRATCH_BYTES (40 * 1024 * 1024)
int arcq_linear_otf_static(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                           const uint8_t *packed_w, const float *w_codebook,
                           const float *w_center, const float *w_scale, const float *w_code_sum,
                           const float *bias, void *y, int y_dtype,
                           int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream);

/* The two operands of the layer rounded to FP8 (OCP E4M3, round to nearest even; finite values beyond +-448 saturate --
 * activations carry no multiplier, so |x_hat| > 448 is clipped and |x_hat| < 2^-6 loses precision -- NaN stays NaN) instead of fp16, for
 * a product on FP8 matrix units: the low-precision formulation that EXT/arcq_linear_kernel.cu:22-202 points at.  They
 * have no counterpart in the reference and do NOT reproduce its numbers (3 mantissa bits per operand where fp16 has
 * 10); codes, mu, s and the fp32 reconstruction are those of arcq_act_quant / arcq_weight_dequant.
 *   arcq_act_quant_fp8:      x8[rows, cols]  = fp8(x_hat), row-major, cols a multiple of 64 (group size 64 only)
 *   arcq_weight_dequant_fp8: w8[N, K]        = fp8(w_mult * w_hat), row-major; w_mult > 0, a power of two chosen by the
 *                                              caller so that the weights fall into FP8's normal range (2^-6 .. 448)
 * The product y = (x8 w8^T) / w_mult + bias on these row-major operands is a plain FP8 GEMM with fp32 accumulation that
 * any GEMM library can run; arcq_linear_otf_fp8 below is the layer on this library's own FP8 kernel. */
int arcq_act_quant_fp8(const void *x, int x_dtype, const float *thresholds, const float *codebook, void *x8,
                       int64_t rows, int64_t cols, int bits, float eps, void *stream);
int arcq_weight_dequant_fp8(const uint8_t *packed, const float *codebook, const float *center, const float *scale,
                            const float *code_sum, void *w8, int64_t N, int64_t K, int bits, int group_size,
                            float w_mult, void *stream);

/* The FP8-operand layer end to end on hand-written kernels (no counterpart in the reference; same caveat: FP8 operands
 * do not reproduce its numbers).  Kp below is K rounded up to a multiple of 128.
 *   arcq_act_quant_fp8_blocked: stage 1 with x8 in the FP8 GEMM's block layout, 16-byte pieces
 *       x8_blocked[((row / 32) * (Kp / 16) + k / 16) * 32 + row % 32][k % 16]
 *     (a last block of r = rows % 32 rows compactly as [(k / 16) * r + row % 32][k % 16]); the pieces from K to Kp are
 *     written as zeros; rows * Kp bytes in all.  packed_w != NULL: extra workgroups of the same launch also write
 *     w8[N, Kp] = fp8(w_mult * w_hat), rows Kp bytes apart, zero from K to Kp (what arcq_weight_dequant_fp8 computes).
 *   arcq_linear_fp8_blocked: y[M,N] = (x8 w8^T) / w_mult + bias on v_mfma_f32_32x32x64_f8f6f4 (fp32 accumulation in
 *     ascending k; bias fp32 or NULL, added in fp32 before the one output rounding; y ARCQ_F16 or ARCQ_F32).  K here is
 *     the padded length Kp (a multiple of 128); x8_blocked and w8 as written by arcq_act_quant_fp8_blocked.
 *   arcq_linear_otf_fp8: the two of them, i.e. the whole layer in two launches.  x8_ws: M * Kp bytes, w8_ws: N * Kp
 *     bytes, both 16-byte aligned scratch. */
int arcq_act_quant_fp8_blocked(const void *x, int x_dtype, const float *thresholds, const float *codebook,
                               void *x8_blocked, int64_t rows, int64_t cols, int bits, float eps,
                               const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                               const float *w_scale, const float *w_code_sum, void *w8, int64_t N, float w_mult,
                               void *stream);
int arcq_linear_fp8_blocked(const void *x8_blocked, const void *w8, const float *bias, float w_mult, void *y, int y_dtype,
                            int64_t M, int64_t N, int64_t K, void *stream);
int arcq_linear_otf_fp8(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                        const uint8_t *packed_w, const float *w_codebook, const float *w_center, const float *w_scale,
                        const float *w_code_sum, const float *bias, float w_mult, void *x8_ws, void *w8_ws, void *y,
                        int y_dtype, int64_t M, int64_t N, int64_t K, int bits, void *stream);

/* ---- softmax attention between the packed qkv and proj layers ---------------
 * No counterpart in the reference's packed path: its models leave attention to timm / torch
 * (scripts/benchmark_arcq_on_the_fly.py:202-243 times the model with it).  Here so that a ViT block is the four packed
 * layers plus one more launch, with no reshaping copies: it reads the qkv layer's output as it lies and writes the
 * proj layer's input as it lies.
 *   qkv [B, n, 3, H, 64] fp16 (= [B*n, 3*H*64] row-major), out [B, n, H*64] fp16:
 *   out[b, i, h*64 + j] = sum_k softmax_k(scale * q_i . k_k) v_k[j], fp32 scores / softmax / accumulation, the
 *   probabilities rounded to fp16 before the second product.
 * head_dim must be 64, n <= 256 and scale > 0 (ARCQ_ERR_UNSUPPORTED otherwise); qkv 16-byte, out 8-byte aligned. */
int arcq_attention_fwd(const void *qkv, void *out, int64_t B, int64_t n, int64_t H, int64_t head_dim, float scale,
                       void *stream);

/* ---- stage 1 of a quantized patch-embedding convolution ---------------------
 * QuantConv2dPCARCQ (FQ/quant_backends.py:329-384; the activation quantizer groups min(64, in_channels) = 3 channels
 * of one pixel, :351) for kernel == stride == 16 on three channels: the pixels' groups are quantized with the
 * arithmetic of arcq_act_quant (group_size 3) and the reconstructions written as the rows of the patch matrix,
 * row = (b, py, px), column = c * 256 + i * 16 + j, fp16 -- the values arcq_act_quant gives for the NHWC pixels, bit for
 * bit, without the NHWC copy and the gather of the rows.
 *   img [B, 3, H, W] ARCQ_F16 or ARCQ_F32; x_hat: blocked == 0: [B * (H/16) * (W/16), 768] row-major (the input of
 *   arcq_linear_fused), blocked != 0: the 32-row block layout of arcq_linear_fused_blocked.  img and x_hat 16-byte
 *   aligned.  Other channel counts or patch sizes: ARCQ_ERR_UNSUPPORTED (compose arcq_act_quant on NHWC pixels). */
int arcq_act_quant_patches(const void *img, int img_dtype, const float *thresholds, const float *codebook, void *x_hat,
                           int64_t B, int64_t C, int64_t H, int64_t W, int64_t patch, int bits, float eps, int blocked,
                           void *stream);

/* ---- fp16 patch embedding of a ViT in one launch ----------------------------
 * No counterpart in the reference's packed path: the fp16 patch embedding of its models is a torch convolution
 * followed by the class-token concatenation and the position-embedding addition (timm's VisionTransformer, which
 * scripts/benchmark_arcq_on_the_fly.py:202-243 times as part of the model).  The quantized patch convolution
 * (QuantConv2dPCARCQ, FQ/timm_quant_models.py) does not go through this entry point.
 *   img [B, 3, H, W] fp16; w [N, 768] fp16 (the Conv2d weight [N, 3, 16, 16] as it lies); bias [N] fp16 or NULL;
 *   cls [N], pos [1 + (H/16)(W/16), N], out [B, 1 + (H/16)(W/16), N] fp16:
 *   out[b, 0] = cls + pos[0];  out[b, 1 + p] = fp16(fp16(patch(b, p) . w^T + bias) + pos[1 + p]), fp32 accumulation.
 * patch must be 16, H and W multiples of 16, N a multiple of 32; img and w 16-byte, the others 8-byte aligned. */
int arcq_patch_embed_fwd(const void *img, const void *w, const void *bias, const void *cls, const void *pos, void *out,
                         int64_t B, int64_t H, int64_t W, int64_t patch, int64_t N, void *stream);

/* Diagnostics of the one-launch layer kernels; no counterpart in the reference.
 * arcq_rows_wait_timeouts: number of workgroups that, on the current device since the library was loaded, gave up
 * their bounded wait for the other workgroups' weight shares and rebuilt all of w_hat themselves (results stay
 * correct; such a launch is many times slower -- the sign of a device shared with other work, or of a launch larger
 * than the device holds).  Blocks until the device has finished (a synchronous copy); -1 if it cannot be read.
 * arcq_rows_counter_slot: the host-side logic that assigns a weight workspace its counter word (`table`: `slots`
 * pointers, NULL = free; returns the slot of `key`, claiming a free one on its probe sequence, or -1 when full). */
long long arcq_rows_wait_timeouts(void);
int arcq_rows_counter_slot(const void **table, int slots, const void *key);

/* Kernels arcq_linear_otf_ws runs after stage 1 for these sizes: "gemm_slab8_kernel", or, with the weights rebuilt
 * in the stage-1 launch and copied by the GEMM, "gemm_slab8_kernel<copy>" or "gemm_pair_kernel" (two row blocks per
 * wave), when it takes the block layout, else arcq_linear_fused_ws_kernel's answer.  A profiling aid with no
 * counterpart in the reference. */
const char *arcq_linear_otf_ws_kernel(int64_t M, int64_t N, int64_t K, int have_workspace);

/* ---- index-space linears (no reconstruction, product-table gather) ---------
 * Replace arcq_linear_forward_cuda (EXT/arcq_linear_kernel.cu:206-278; fp64
 * accumulation, kernel :22-78) and arcq_linear_forward_u8_cuda (:280-353; fp32,
 * 32-lane strided partial sums folded by a shuffle-down tree, kernel :136-202).
 * Both reproduce the reference's summation order, so results are bit-identical
 * to a serial CPU evaluation in that order.  product_table [levels, levels]
 * fp32 = cb_a (x) cb_w; bias [out_features] fp32 or NULL; y [rows, out_features]
 * fp32. */
int arcq_linear_forward_packed(const uint8_t *packed_x, const float *x_center, const float *x_scale,
                               const float *x_code_sum,
                               const uint8_t *packed_w, const float *w_center, const float *w_scale,
                               const float *w_code_sum,
                               const float *product_table, const float *bias, float *y,
                               int64_t rows, int64_t out_features, int64_t in_features,
                               int bits, int group_size, int levels, void *stream);
int arcq_linear_forward_u8(const uint8_t *x_codes, const float *x_center, const float *x_scale,
                           const float *x_code_sum,
                           const uint8_t *w_codes, const float *w_center, const float *w_scale,
                           const float *w_code_sum,
                           const float *product_table, const float *bias, float *y,
                           int64_t rows, int64_t out_features, int64_t in_features,
                           int group_size, int levels, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ARCQ_HIP_H */
