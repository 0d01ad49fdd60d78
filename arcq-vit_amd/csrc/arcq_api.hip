// Library-level pieces of libarcq_hip.so: version, per-thread error text and
// the whole-layer entry point that chains stage 1 into the fused stages 2+3.
#include <stdarg.h>
#include <stddef.h>
#include <string.h>

#include <stdlib.h>

#include <mutex>

#include "arcq_common.h"
#include "arcq_gemm.h"

namespace arcq {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int launch_status(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return ARCQ_OK;
    return fail(static_cast<int>(e), "%s: launch failed: %s", what, hipGetErrorString(e));
}

namespace {
struct TuningStore {
    char gemm_kernel[32], otf_fused[8], pair[8], rows[8];
    Tuning view;
};
TuningStore g_tuning;
std::once_flag g_tuning_once;
std::mutex g_tuning_mutex;

void read_tuning()
{
    auto grab = [](const char *name, char *buf, size_t n) -> const char * {
        const char *e = getenv(name);
        if (!e) return nullptr;
        strncpy(buf, e, n - 1);
        buf[n - 1] = 0;
        return buf;
    };
    std::lock_guard<std::mutex> lock(g_tuning_mutex);
    g_tuning.view.gemm_kernel = grab("ARCQ_GEMM_KERNEL", g_tuning.gemm_kernel, sizeof(g_tuning.gemm_kernel));
    g_tuning.view.otf_fused = grab("ARCQ_OTF_FUSED", g_tuning.otf_fused, sizeof(g_tuning.otf_fused));
    g_tuning.view.pair = grab("ARCQ_PAIR", g_tuning.pair, sizeof(g_tuning.pair));
    g_tuning.view.rows = grab("ARCQ_ROWS", g_tuning.rows, sizeof(g_tuning.rows));
    // (ARCQ_ROWS_WAIT_TICKS=0 makes every workgroup of the one-launch kernels give up waiting at once and rebuild the
    // weights itself: how the tests reach that path)
    const char *ticks = getenv("ARCQ_ROWS_WAIT_TICKS");
    g_tuning.view.rows_wait_ticks = ticks ? strtoll(ticks, nullptr, 10) : kRowsWaitTicks;
    if (g_tuning.view.rows_wait_ticks < 0) g_tuning.view.rows_wait_ticks = kRowsWaitTicks;
}
}  // namespace

const Tuning &tuning()
{
    std::call_once(g_tuning_once, read_tuning);
    return g_tuning.view;
}

}  // namespace arcq

// Reads the ARCQ_* tuning variables again (they are otherwise read once per process).  Not safe against calls
// running in other threads at the same moment; a hook for tests and tuning scripts.
ARCQ_API void arcq_reload_tuning(void)
{
    (void)arcq::tuning();
    arcq::read_tuning();
}

ARCQ_API int arcq_version(void) { return ARCQ_VERSION; }

ARCQ_API const char *arcq_last_error(void) { return arcq::g_last_error; }

// FQ/arcq_packed_on_the_fly.py:137-161: quantize+reconstruct the activation
// into an fp16 buffer, then run the fused unpack+GEMM on it.
static int linear_otf_impl(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                             const uint8_t *packed_w, const float *w_codebook,
                             const float *w_center, const float *w_scale, const float *w_code_sum,
                             const float *bias, void *x_hat_ws, void *w_hat_ws, bool scratch_only, void *y, int y_dtype,
                             int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    if (!x_hat_ws) return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf: x_hat_ws must not be NULL");
    if (x_hat_ws == x && x_dtype != ARCQ_F16)
        return arcq::fail(ARCQ_ERR_DTYPE, "arcq_linear_otf: x_hat_ws may alias x only when x is fp16");
    // A few hundred rows: one launch for the whole layer (same results bit for bit).  Taken only when every argument
    // is plainly valid; anything else goes through the two entry points below, which report what is wrong.
    // ARCQ_OTF_FUSED=0 switches the single-launch path off, =2 takes it for every shape the kernel can run (tuning aids).
    {
        const char *e = arcq::tuning().otf_fused;
        const bool enabled = !(e && e[0] == '0');
        if (enabled && group_size == 64 && arcq::bits_ok(bits) && M > 0 && N > 0 && N < (int64_t(1) << 30) &&
            arcq::otf_small_supported(M, N, K, e && e[0] == '2') && x && x != x_hat_ws && a_thresholds && a_codebook && packed_w &&
            w_codebook && w_center && w_scale && w_code_sum && y && (x_dtype == ARCQ_F16 || x_dtype == ARCQ_F32) &&
            (y_dtype == ARCQ_F16 || y_dtype == ARCQ_F32) && arcq::aligned(x, 16) && arcq::aligned(x_hat_ws, 16) &&
            arcq::aligned(y, 16) && arcq::aligned(packed_w, 16)) {
            // (with scratch-only workspaces nobody reads x_hat afterwards: the kernel then keeps it in LDS only)
            arcq::OtfSmallArgs a{x, x_dtype == ARCQ_F16, a_thresholds, a_codebook, packed_w, w_codebook, w_center, w_scale,
                                 w_code_sum, bias, scratch_only ? nullptr : x_hat_ws, y, y_dtype == ARCQ_F16, static_cast<int>(M),
                                 static_cast<int>(N), static_cast<int>(K), bits, 1.0e-6f};
            arcq::launch_otf_small(a, static_cast<hipStream_t>(stream));
            return arcq::launch_status("arcq_linear_otf");
        }
    }
    // Short rows, many of them, fp16 input, both workspaces scratch: the whole layer in one launch (x_hat stays in
    // LDS, the weight workspace takes w_hat in the 32-column block layout); same results bit for bit.
    if (scratch_only && w_hat_ws && x_dtype == ARCQ_F16 && group_size == 64 && arcq::bits_ok(bits) &&
        arcq::otf_rows_pays(M, N, K) && x && a_thresholds && a_codebook && packed_w && w_codebook && w_center && w_scale &&
        w_code_sum && y && (y_dtype == ARCQ_F16 || y_dtype == ARCQ_F32) && arcq::aligned(x, 16) && arcq::aligned(y, 16) &&
        arcq::aligned(w_hat_ws, 128) && arcq::aligned(packed_w, 4)) {
        arcq::OtfRowsArgs a{x, a_thresholds, a_codebook, nullptr, nullptr, 0.0f, packed_w, w_codebook, w_center, w_scale,
                            w_code_sum, bias, w_hat_ws, y, y_dtype == ARCQ_F16, nullptr, false, static_cast<int>(M),
                            static_cast<int>(N), static_cast<int>(K), bits, 1.0e-6f};
        const int rc = arcq::launch_otf_rows(a, static_cast<hipStream_t>(stream));
        if (rc != arcq::kNotLaunched) return rc;
    }
    // Scratch-only workspaces and 512 rows or more: x_hat in the block layout, eight-wave weight-stationary GEMM
    // (bit-identical results; invalid arguments fall through to the entry points below, which report them).
    if (scratch_only && group_size == 64 && arcq::bits_ok(bits) && arcq::otf_blocked_pays(M, N, K) && x != x_hat_ws) {
        // With a weight workspace that pays, its reconstruction rides along in the stage-1 launch.
        const bool carry = w_hat_ws && arcq::blocked_uses_workspace(N, K) && packed_w && w_codebook && w_center &&
                           w_scale && w_code_sum && arcq::aligned(w_hat_ws, 16) && arcq::aligned(packed_w, 16);
        const int rc = carry ? arcq_act_quant_blocked_with_weights(x, x_dtype, a_thresholds, a_codebook, x_hat_ws, M, K, bits,
                                                                    1.0e-6f, packed_w, w_codebook, w_center, w_scale,
                                                                    w_code_sum, w_hat_ws, N, stream)
                             : arcq_act_quant_blocked(x, x_dtype, a_thresholds, a_codebook, x_hat_ws, M, K, bits, 1.0e-6f, stream);
        if (rc != ARCQ_OK) return rc;
        return arcq::linear_fused_blocked(x_hat_ws, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, w_hat_ws, carry,
                                          y, y_dtype, M, N, K, bits, group_size, stream);
    }
    int rc = arcq_act_quant(x, x_dtype, a_thresholds, a_codebook, nullptr, nullptr, nullptr, nullptr, nullptr,
                            x_hat_ws, ARCQ_F16, M, K, bits, group_size, 1.0e-6f, stream);
    if (rc != ARCQ_OK) return rc;
    return arcq_linear_fused_ws(x_hat_ws, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, w_hat_ws, y, y_dtype,
                                M, N, K, bits, group_size, stream);
}

ARCQ_API int arcq_linear_otf(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                             const uint8_t *packed_w, const float *w_codebook,
                             const float *w_center, const float *w_scale, const float *w_code_sum,
                             const float *bias, void *x_hat_ws, void *y, int y_dtype,
                             int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    return linear_otf_impl(x, x_dtype, a_thresholds, a_codebook, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias,
                           x_hat_ws, nullptr, false, y, y_dtype, M, N, K, bits, group_size, stream);
}

// The same layer with a second scratch buffer, for the reconstructed weights ([N,K] fp16; the counterpart of the
// reference module's _weight_buffer, FQ/arcq_packed_on_the_fly.py:148-158).  NULL behaves like arcq_linear_otf.
ARCQ_API int arcq_linear_otf_ws(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                                const uint8_t *packed_w, const float *w_codebook,
                                const float *w_center, const float *w_scale, const float *w_code_sum,
                                const float *bias, void *x_hat_ws, void *w_hat_ws, void *y, int y_dtype,
                                int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    return linear_otf_impl(x, x_dtype, a_thresholds, a_codebook, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias,
                           x_hat_ws, w_hat_ws, true, y, y_dtype, M, N, K, bits, group_size, stream);
}

// The layer with LayerNorm in front and GELU / a residual behind fused in (see arcq_hip.h).
ARCQ_API int arcq_linear_otf_ex(const arcq_linear_ex_args *a, void *stream)
{
    if (!a) return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf_ex: args must not be NULL");
    constexpr size_t kFirstVersion = offsetof(arcq_linear_ex_args, next_a_thresholds);
    if (a->struct_size < kFirstVersion)
        return arcq::fail(ARCQ_ERR_SHAPE, "arcq_linear_otf_ex: struct_size %u is smaller than this library's %zu",
                          a->struct_size, kFirstVersion);
    const bool has_next = a->struct_size >= sizeof(arcq_linear_ex_args);
    const float *next_thr = has_next ? a->next_a_thresholds : nullptr;
    const float *next_cb = has_next ? a->next_a_codebook : nullptr;
    if ((next_thr == nullptr) != (next_cb == nullptr))
        return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf_ex: next_a_thresholds and next_a_codebook go together");
    if (a->producer != ARCQ_PRODUCER_NONE && a->producer != ARCQ_PRODUCER_LAYERNORM && a->producer != ARCQ_PRODUCER_XHAT)
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: unknown producer %d", a->producer);
    if (a->activation != ARCQ_ACT_NONE && a->activation != ARCQ_ACT_GELU)
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: unknown activation %d", a->activation);
    const bool options = a->producer != ARCQ_PRODUCER_NONE || a->activation != ARCQ_ACT_NONE || a->residual || next_thr;
    if (!options)
        return linear_otf_impl(a->x, a->x_dtype, a->a_thresholds, a->a_codebook, a->packed_w, a->w_codebook, a->w_center,
                               a->w_scale, a->w_code_sum, a->bias, a->x_hat_ws, a->w_hat_ws, true, a->y, a->y_dtype, a->M,
                               a->N, a->K, a->bits, a->group_size, stream);
    if (a->group_size != 64 || !arcq::bits_ok(a->bits))
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: the fused options need group_size 64 and bits 2/3/4 "
                          "(got group_size=%d bits=%d)", a->group_size, a->bits);
    const bool from_xhat = a->producer == ARCQ_PRODUCER_XHAT;
    if (from_xhat && a->x_dtype != ARCQ_F16)
        return arcq::fail(ARCQ_ERR_DTYPE, "arcq_linear_otf_ex: ARCQ_PRODUCER_XHAT needs x as float16 (it is x_hat)");
    if (next_thr && (a->y_dtype != ARCQ_F16 || a->N % 64 != 0))
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: quantizing the output for the next layer needs a float16 y "
                          "and out_features a multiple of 64");
    if (!from_xhat) {
        if (!a->x_hat_ws) return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf_ex: x_hat_ws must not be NULL");
        if (a->x_hat_ws == a->x) return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: x_hat_ws must not alias x");
    }
    if (a->residual && !arcq::aligned(a->residual, 16))
        return arcq::fail(ARCQ_ERR_ALIGN, "arcq_linear_otf_ex: residual must be 16-byte aligned");
    const bool want_ln = a->producer == ARCQ_PRODUCER_LAYERNORM;
    if (want_ln && (!a->ln_weight || !a->ln_bias || !arcq::aligned(a->ln_weight, 16) || !arcq::aligned(a->ln_bias, 16)))
        return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf_ex: ln_weight and ln_bias must be 16-byte aligned fp32 [K] tensors");
    // A few hundred rows (batch 1): the whole layer, LayerNorm and post-operations included, in the one launch of the
    // small-M kernel wherever that kernel can run (always with a LayerNorm: it is the only small-M kernel that has
    // one); else stage 1 row-major + the split-K kernel with the post-operations in its epilogue.
    if (a->M > 0 && a->M < 512 && a->N > 0 && a->N < (int64_t(1) << 30) && a->K >= 64 && a->K % 64 == 0) {
        if (!a->x || (!from_xhat && (!a->a_thresholds || !a->a_codebook)) || !a->packed_w || !a->w_codebook || !a->w_center ||
            !a->w_scale || !a->w_code_sum || !a->y)
            return arcq::fail(ARCQ_ERR_NULL, "arcq_linear_otf_ex: NULL tensor pointer");
        if ((a->x_dtype != ARCQ_F16 && a->x_dtype != ARCQ_F32) || (a->y_dtype != ARCQ_F16 && a->y_dtype != ARCQ_F32))
            return arcq::fail(ARCQ_ERR_DTYPE, "arcq_linear_otf_ex: x and y must be float16 or float32");
        if (!arcq::aligned(a->x, 16) || (!from_xhat && !arcq::aligned(a->x_hat_ws, 16)) || !arcq::aligned(a->y, 16) ||
            !arcq::aligned(a->packed_w, 16))
            return arcq::fail(ARCQ_ERR_ALIGN, "arcq_linear_otf_ex: x, x_hat_ws, y and packed_w must be 16-byte aligned");
        if (from_xhat) {          // x is this layer's x_hat, row-major: stages 2+3 only
            if (next_thr)
                return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: below 512 rows a layer that starts from x_hat cannot "
                                  "quantize its output for the next one");
            return arcq::linear_fused_post(a->x, a->packed_w, a->w_codebook, a->w_center, a->w_scale, a->w_code_sum, a->bias,
                                           a->y, a->y_dtype, a->M, a->N, a->K, a->bits, 64, stream, a->residual,
                                           a->activation == ARCQ_ACT_GELU);
        }
        if (next_thr && !arcq::otf_small_supported(a->M, a->N, a->K, true))
            return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: below 512 rows quantizing the output for the next layer "
                              "needs in_features <= 1536");
        const char *e = arcq::tuning().otf_fused;
        const bool one_launch = next_thr ? true : want_ln ? arcq::otf_small_supported(a->M, a->N, a->K, true)
                                        : (!(e && e[0] == '0') && arcq::otf_small_supported(a->M, a->N, a->K, e && e[0] == '2'));
        if (one_launch) {
            arcq::OtfSmallArgs s{a->x, a->x_dtype == ARCQ_F16, a->a_thresholds, a->a_codebook, a->packed_w, a->w_codebook,
                                 a->w_center, a->w_scale, a->w_code_sum, a->bias, nullptr, a->y, a->y_dtype == ARCQ_F16,
                                 static_cast<int>(a->M), static_cast<int>(a->N), static_cast<int>(a->K), a->bits, 1.0e-6f};
            if (want_ln) s.ln_weight = a->ln_weight, s.ln_bias = a->ln_bias, s.ln_eps = a->ln_eps;
            s.residual = a->residual;
            s.gelu = a->activation == ARCQ_ACT_GELU;
            s.next_thr = next_thr, s.next_cb = next_cb;
            arcq::launch_otf_small(s, static_cast<hipStream_t>(stream));
            return arcq::launch_status("arcq_linear_otf_ex");
        }
        if (want_ln)
            return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: below 512 rows the fused LayerNorm needs in_features <= 1536");
        const int rc = arcq_act_quant(a->x, a->x_dtype, a->a_thresholds, a->a_codebook, nullptr, nullptr, nullptr, nullptr,
                                      nullptr, a->x_hat_ws, ARCQ_F16, a->M, a->K, a->bits, 64, 1.0e-6f, stream);
        if (rc != ARCQ_OK) return rc;
        return arcq::linear_fused_post(a->x_hat_ws, a->packed_w, a->w_codebook, a->w_center, a->w_scale, a->w_code_sum, a->bias,
                                       a->y, a->y_dtype, a->M, a->N, a->K, a->bits, 64, stream, a->residual,
                                       a->activation == ARCQ_ACT_GELU);
    }
    if (!arcq::otf_blocked_pays(a->M, a->N, a->K))
        return arcq::fail(ARCQ_ERR_UNSUPPORTED,
                          "arcq_linear_otf_ex: the fused options need in_features a positive multiple of 64 and a shape the "
                          "block-layout kernels run (got M=%lld K=%lld)", static_cast<long long>(a->M),
                          static_cast<long long>(a->K));
    // From 512 rows on two chained layers hand x_hat over in the 32-row block layout.  The consumer runs stages 2+3 on
    // it (the weights rebuilt into the workspace first where that pays); the producer is the block-layout GEMM on
    // copied weights with the consumer's stage 1 in its epilogue (which needs the weight workspace).
    if (from_xhat) {
        if (next_thr)
            return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: a layer that starts from x_hat cannot quantize its output "
                              "for the next one");
        return arcq::linear_fused_blocked(a->x, a->packed_w, a->w_codebook, a->w_center, a->w_scale, a->w_code_sum, a->bias,
                                          a->w_hat_ws, false, a->y, a->y_dtype, a->M, a->N, a->K, a->bits, a->group_size, stream,
                                          a->residual, a->activation == ARCQ_ACT_GELU);
    }
    if (next_thr && (!a->w_hat_ws || a->residual))
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: from 512 rows on quantizing the output for the next layer needs "
                          "w_hat_ws and no residual");
    if (!next_thr && a->w_hat_ws && a->x_dtype == ARCQ_F16 &&
        arcq::otf_rows_pays(a->M, a->N, a->K, a->producer == ARCQ_PRODUCER_LAYERNORM) && a->x && a->a_thresholds &&
        a->a_codebook && a->packed_w && a->w_codebook && a->w_center && a->w_scale && a->w_code_sum && a->y &&
        (a->y_dtype == ARCQ_F16 || a->y_dtype == ARCQ_F32) && arcq::aligned(a->x, 16) && arcq::aligned(a->y, 16) &&
        arcq::aligned(a->w_hat_ws, 128) && arcq::aligned(a->packed_w, 4) &&
        (a->producer != ARCQ_PRODUCER_LAYERNORM || (a->ln_weight && a->ln_bias && arcq::aligned(a->ln_weight, 16) &&
                                                    arcq::aligned(a->ln_bias, 16)))) {
        const bool ln = a->producer == ARCQ_PRODUCER_LAYERNORM;
        arcq::OtfRowsArgs r{a->x, a->a_thresholds, a->a_codebook, ln ? a->ln_weight : nullptr, ln ? a->ln_bias : nullptr,
                            a->ln_eps, a->packed_w, a->w_codebook, a->w_center, a->w_scale, a->w_code_sum, a->bias,
                            a->w_hat_ws, a->y, a->y_dtype == ARCQ_F16, a->residual, a->activation == ARCQ_ACT_GELU,
                            static_cast<int>(a->M), static_cast<int>(a->N), static_cast<int>(a->K), a->bits, 1.0e-6f};
        const int rc = arcq::launch_otf_rows(r, static_cast<hipStream_t>(stream));
        if (rc != arcq::kNotLaunched) return rc;
    }
    const bool carry = a->w_hat_ws && (next_thr || arcq::blocked_uses_workspace(a->N, a->K)) && a->packed_w && a->w_codebook &&
                       a->w_center && a->w_scale && a->w_code_sum && arcq::aligned(a->w_hat_ws, 16) && arcq::aligned(a->packed_w, 16);
    if (next_thr && !carry)
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: quantizing the output for the next layer needs a 16-byte aligned "
                          "weight workspace and packed weights");
    int rc;
    if (a->producer == ARCQ_PRODUCER_LAYERNORM) {
        if (a->K > 1024)
            return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_ex: the fused LayerNorm needs in_features <= 1024");
        rc = arcq_act_quant_blocked_ln(a->x, a->x_dtype, a->ln_weight, a->ln_bias, a->ln_eps, a->a_thresholds, a->a_codebook,
                                       a->x_hat_ws, a->M, a->K, a->bits, 1.0e-6f, carry ? a->packed_w : nullptr, a->w_codebook,
                                       a->w_center, a->w_scale, a->w_code_sum, a->w_hat_ws, carry ? a->N : 0, stream);
    } else if (carry) {
        rc = arcq_act_quant_blocked_with_weights(a->x, a->x_dtype, a->a_thresholds, a->a_codebook, a->x_hat_ws, a->M, a->K,
                                                 a->bits, 1.0e-6f, a->packed_w, a->w_codebook, a->w_center, a->w_scale,
                                                 a->w_code_sum, a->w_hat_ws, a->N, stream);
    } else {
        rc = arcq_act_quant_blocked(a->x, a->x_dtype, a->a_thresholds, a->a_codebook, a->x_hat_ws, a->M, a->K, a->bits, 1.0e-6f,
                                    stream);
    }
    if (rc != ARCQ_OK) return rc;
    return arcq::linear_fused_blocked(a->x_hat_ws, a->packed_w, a->w_codebook, a->w_center, a->w_scale, a->w_code_sum, a->bias,
                                      a->w_hat_ws, carry, a->y, a->y_dtype, a->M, a->N, a->K, a->bits, a->group_size, stream,
                                      a->residual, a->activation == ARCQ_ACT_GELU, next_thr, next_cb);
}

ARCQ_API int arcq_xhat_layout(int64_t M) { return M < 512 ? 0 : 1; }

// ---- the same layer for callers that cannot allocate --------------------------------------------------------
// Both scratch buffers of arcq_linear_otf_ws live in a file-scope device array instead of caller memory.  Every GPU
// the library runs on holds its own copy of the array (at its own address) until the process ends.
static __device__ __align__(256) unsigned char scratch[ARCQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[kMaxDevices];        // device address of `scratch` on each device, once resolved
}

ARCQ_API int arcq_linear_otf_static(const void *x, int x_dtype, const float *a_thresholds, const float *a_codebook,
                                    const uint8_t *packed_w, const float *w_codebook,
                                    const float *w_center, const float *w_scale, const float *w_code_sum,
                                    const float *bias, void *y, int y_dtype,
                                    int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    if (M < 0 || N < 0 || K < 0) return arcq::fail(ARCQ_ERR_SHAPE, "arcq_linear_otf_static: negative size");
    // Layout of the array: [w_hat: N*K fp16, rounded up to 256 bytes][x_hat: M*K fp16].
    const int64_t limit = ARCQ_STATIC_SCRATCH_BYTES;
    if (K > limit || N > limit || M > limit)
        return arcq::fail(ARCQ_ERR_SHAPE, "arcq_linear_otf_static: sizes exceed the static scratch of %lld bytes",
                          static_cast<long long>(limit));
    const int64_t w_bytes = (N * K * 2 + 255) / 256 * 256;
    const int64_t x_bytes = M * K * 2;
    if (w_bytes + x_bytes > limit)
        return arcq::fail(ARCQ_ERR_SHAPE,
                          "arcq_linear_otf_static: 2*N*K + 2*M*K = %lld bytes of scratch needed, the static scratch holds "
                          "%lld; use arcq_linear_otf_ws with caller-owned workspaces",
                          static_cast<long long>(w_bytes + x_bytes), static_cast<long long>(limit));
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return arcq::fail(static_cast<int>(e), "arcq_linear_otf_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return arcq::fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_otf_static: device index %d not supported", dev);
    unsigned char *base;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[dev]) {
            // In host code the array's name is only a handle: its device address has to be asked for, once per
            // device, with that device current.
            void *p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p)
                return arcq::fail(e != hipSuccess ? static_cast<int>(e) : ARCQ_ERR_NULL,
                                  "arcq_linear_otf_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
        }
        base = g_scratch_ptr[dev];
    }
    // Nothing in the array has to start at zero: stage 1 writes every x_hat value and the weight reconstruction every
    // w_hat value before the GEMM reads them.
    return linear_otf_impl(x, x_dtype, a_thresholds, a_codebook, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias,
                           base + w_bytes, base, true, y, y_dtype, M, N, K, bits, group_size, stream);
}
