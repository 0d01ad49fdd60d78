/*
 * CPU oracle for the ARCQ packed quantized-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the arithmetic of the reference
 * implementation (WangHY0325/ARCQ-ViT).  It is the checker the GPU kernels are
 * compared with; nothing in the shipped product path may call it.  Every
 * function names the reference lines it follows (paths relative to the
 * reference root; FQ = methods/fair_qat_framework/fair_qat,
 * EXT = FQ/arcq_infer_cuda).
 *
 * Arithmetic contract of this oracle (what "bit-exact" is measured against):
 *   - IEEE-754 binary32 for every float op, round-to-nearest-even, no
 *     contraction except where fmaf() is written explicitly, no fast-math.
 *     (The reference's CUDA build uses --use_fast_math, EXT/setup.py:23, whose
 *     approximate divide/sqrt no CPU can restate; IEEE divide/sqrt is what the
 *     reference's torch paths do.)
 *   - group sums run serially, left to right, exactly like the loops at
 *     EXT/arcq_activation_kernel.cu:49-60.
 *
 * Pinning status of each function is listed in oracle/README.md; all of them
 * are pinned by tests/test_oracle_*.py without importing the reference.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fno-fast-math).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__GNUC__)
#define ORACLE_API __attribute__((visibility("default")))
#else
#define ORACLE_API
#endif

/* ------------------------------------------------------------------------- */
/* a1: LSB-first bitstream layout.                                           */
/* Follows EXT/arcq_pack_kernel.cu:8-20 (get) and :22-36 (set): code j of a  */
/* row occupies bits [j*bits, (j+1)*bits) of the row's little-endian byte    */
/* stream and may straddle two bytes.                                        */
/* ------------------------------------------------------------------------- */
static inline int get_code(const uint8_t *row, int64_t idx, int bits)
{
    const int64_t bit_offset = idx * bits;
    const int64_t byte_idx = bit_offset >> 3;
    const int shift = (int)(bit_offset & 7);
    unsigned value = (unsigned)row[byte_idx] >> shift;
    if (shift + bits > 8)
        value |= (unsigned)row[byte_idx + 1] << (8 - shift);
    return (int)(value & ((1u << bits) - 1u));
}

static inline void set_code(uint8_t *row, int64_t idx, int bits, int code)
{
    const int64_t bit_offset = idx * bits;
    const int64_t byte_idx = bit_offset >> 3;
    const int shift = (int)(bit_offset & 7);
    const unsigned mask = (1u << bits) - 1u;
    const unsigned value = ((unsigned)code & mask) << shift;
    row[byte_idx] |= (uint8_t)(value & 0xffu);
    if (shift + bits > 8)
        row[byte_idx + 1] |= (uint8_t)((value >> 8) & 0xffu);
}

ORACLE_API int64_t oracle_packed_cols(int64_t length, int bits)
{
    /* EXT/arcq_pack_kernel.cu:101 */
    return (length * bits + 7) / 8;
}

/* a3 pack: EXT/arcq_pack_kernel.cu:38-54 (+ zero-init at :102);
 * same bytes as FQ/arcq_packed_py.py:8-47. */
ORACLE_API void oracle_pack_codes(const int64_t *codes, uint8_t *packed,
                                  int64_t rows, int64_t length, int bits)
{
    const int64_t pc = oracle_packed_cols(length, bits);
    memset(packed, 0, (size_t)(rows * pc));
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < length; ++j)
            set_code(packed + r * pc, j, bits, (int)codes[r * length + j]);
}

/* a3 unpack to int64: EXT/arcq_pack_kernel.cu:56-72; FQ/arcq_packed_py.py:50-78 */
ORACLE_API void oracle_unpack_codes(const uint8_t *packed, int64_t *codes,
                                    int64_t rows, int64_t length, int bits)
{
    const int64_t pc = oracle_packed_cols(length, bits);
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < length; ++j)
            codes[r * length + j] = get_code(packed + r * pc, j, bits);
}

/* a3 unpack to uint8: EXT/arcq_pack_kernel.cu:74-90 */
ORACLE_API void oracle_unpack_codes_u8(const uint8_t *packed, uint8_t *codes,
                                       int64_t rows, int64_t length, int bits)
{
    const int64_t pc = oracle_packed_cols(length, bits);
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < length; ++j)
            codes[r * length + j] = (uint8_t)get_code(packed + r * pc, j, bits);
}

/* ------------------------------------------------------------------------- */
/* a6: stage 1, activation group-residual quantizer.                         */
/* Follows EXT/arcq_activation_kernel.cu:24-77 (packed), :79-130 (u8) and    */
/* :132-184 (dequant), one group at a time:                                  */
/*   mu  = (x0 + x1 + ... serial) / gs                         (:49-53)      */
/*   var = sum_j (x_j - mu)^2 serial;  s = sqrtf(var/gs + eps) (:55-60)      */
/*   t_j = (x_j - mu) / s                                      (:64)         */
/*   code_j: while (code < L-1 && t > thr[code]) ++code        (:65-68)      */
/*   code_sum = sum_j cb[code_j] serial                        (:70)         */
/*   x_hat_j = mu + s * (cb[code_j] - code_sum/gs)             (:175-182)    */
/* The reference hard-codes eps = 1e-6f; it is a parameter here because the  */
/* offline weight encoder passes the quantizer's eps                          */
/* (FQ/arcq_packed_linear.py:48).  `fma` selects how x_hat is rounded:       */
/*   1: fmaf(s, d, mu)  -- what a contracting GPU compiler emits for the     */
/*      expression at :182 and FQ/arcq_packed_triton.py:175                  */
/*   0: mu + (s * d)    -- two roundings, what torch does                    */
/*      (FQ/arcq_packed_on_the_fly.py:87-89)                                 */
/* Any output pointer may be NULL.                                           */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_act_quant(const float *x, const float *thr, const float *cb,
                                 int64_t rows, int64_t cols, int bits, int gs,
                                 float eps, int fma,
                                 uint8_t *packed, uint8_t *codes_u8,
                                 float *center, float *scale, float *code_sum,
                                 float *x_hat)
{
    const int levels = 1 << bits;
    const int64_t groups = cols / gs;
    const int64_t pc = oracle_packed_cols(cols, bits);
    uint8_t *tmp = (uint8_t *)malloc((size_t)gs);
    if (packed)
        memset(packed, 0, (size_t)(rows * pc));
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t g = 0; g < groups; ++g) {
            const float *xg = x + r * cols + g * gs;
            float mu = 0.0f;
            for (int j = 0; j < gs; ++j)
                mu += xg[j];
            mu /= (float)gs;
            float var = 0.0f;
            for (int j = 0; j < gs; ++j) {
                const float d = xg[j] - mu;
                var += d * d;
            }
            const float s = sqrtf(var / (float)gs + eps);
            float sum_codes = 0.0f;
            for (int j = 0; j < gs; ++j) {
                const float t = (xg[j] - mu) / s;
                int code = 0;
                while (code < levels - 1 && t > thr[code])
                    ++code;
                tmp[j] = (uint8_t)code;
                sum_codes += cb[code];
            }
            const float code_mean = sum_codes / (float)gs;
            for (int j = 0; j < gs; ++j) {
                const int64_t col = g * gs + j;
                if (packed)
                    set_code(packed + r * pc, col, bits, tmp[j]);
                if (codes_u8)
                    codes_u8[r * cols + col] = tmp[j];
                if (x_hat) {
                    const float d = cb[tmp[j]] - code_mean;
                    x_hat[r * cols + col] = fma ? fmaf(s, d, mu) : (mu + s * d);
                }
            }
            if (center)
                center[r * groups + g] = mu;
            if (scale)
                scale[r * groups + g] = s;
            if (code_sum)
                code_sum[r * groups + g] = sum_codes;
        }
    }
    free(tmp);
}

/* ------------------------------------------------------------------------- */
/* a9: stage 2, packed weight -> reconstructed weight (fp32 before the fp16  */
/* rounding, which the Python side applies with numpy's round-to-nearest).   */
/* Follows FQ/arcq_packed_triton.py:33-74:                                   */
/*   code -> cb[code]; result = (cb - cs / gs) * s + c                       */
/* fma = 1: fmaf(cb - cs/gs, s, c) (Triton contracts the mul+add at :71);    */
/* fma = 0: c + s * (cb - cs/gs) with two roundings                          */
/*          (FQ/arcq_packed_on_the_fly.py:54-61).                            */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_weight_dequant(const uint8_t *packed, const float *cb,
                                      const float *center, const float *scale,
                                      const float *code_sum,
                                      int64_t N, int64_t K, int bits, int gs,
                                      int fma, float *out)
{
    const int64_t groups = K / gs;
    const int64_t pc = oracle_packed_cols(K, bits);
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t k = 0; k < K; ++k) {
            const int64_t g = k / gs;
            const int code = get_code(packed + n * pc, k, bits);
            const float c = center[n * groups + g];
            const float s = scale[n * groups + g];
            const float cs = code_sum[n * groups + g];
            const float d = cb[code] - cs / (float)gs;
            out[n * K + k] = fma ? fmaf(d, s, c) : (c + s * d);
        }
    }
}

/* ------------------------------------------------------------------------- */
/* a11: stage 3, y = a * w^T + bias with a, w already rounded to fp16 and    */
/* passed here widened to fp32.  Products of two fp16 values are exact in    */
/* fp32/fp64; the sum is taken in fp64, so this is the correctly rounded     */
/* value every fp32-accumulating GEMM (cuBLAS at                             */
/* FQ/arcq_packed_on_the_fly.py:160, MFMA here) approximates.  Also returns  */
/* sum |a*w| per output, the scale of the fp32 accumulation error bound.     */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_linear_f64(const float *a, const float *w, const float *bias,
                                  int64_t M, int64_t N, int64_t K,
                                  double *y, double *abs_sum)
{
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0, aacc = 0.0;
            const float *ar = a + m * K;
            const float *wr = w + n * K;
            for (int64_t k = 0; k < K; ++k) {
                const double p = (double)ar[k] * (double)wr[k];
                acc += p;
                aacc += fabs(p);
            }
            if (bias)
                acc += (double)bias[n];
            y[m * N + n] = acc;
            if (abs_sum)
                abs_sum[m * N + n] = aacc + (bias ? fabs((double)bias[n]) : 0.0);
        }
    }
}

/* ------------------------------------------------------------------------- */
/* a12: index-space linear, packed codes, fp64 accumulate.                   */
/* Follows EXT/arcq_linear_kernel.cu:22-78 statement by statement (no        */
/* contraction): per group                                                   */
/*   cross = sum_j (double)P[xc_j*L + wc_j]  serial                          */
/*   mu_term = gs * xc * wc                                                  */
/*   residual_term = xs * ws * (cross - (xcs * wcs) / gs)                    */
/*   acc += mu_term + residual_term;   y = (float)acc, acc starts at bias    */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_linear_forward_packed(
    const uint8_t *packed_x, const float *x_center, const float *x_scale, const float *x_code_sum,
    const uint8_t *packed_w, const float *w_center, const float *w_scale, const float *w_code_sum,
    const float *product_table, const float *bias,
    int64_t rows, int64_t out_features, int64_t in_features,
    int bits, int gs, int levels, float *y)
{
    const int64_t groups = in_features / gs;
    const int64_t pc = oracle_packed_cols(in_features, bits);
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t o = 0; o < out_features; ++o) {
            const uint8_t *xr = packed_x + r * pc;
            const uint8_t *wr = packed_w + o * pc;
            double acc = bias ? (double)bias[o] : 0.0;
            for (int64_t g = 0; g < groups; ++g) {
                double cross = 0.0;
                const int64_t base = g * gs;
                for (int j = 0; j < gs; ++j) {
                    const int xc = get_code(xr, base + j, bits);
                    const int wc = get_code(wr, base + j, bits);
                    cross += (double)product_table[xc * levels + wc];
                }
                const int64_t xm = r * groups + g, wm = o * groups + g;
                const double mu_term = (double)gs * (double)x_center[xm] * (double)w_center[wm];
                const double residual_term = (double)x_scale[xm] * (double)w_scale[wm] *
                    (cross - ((double)x_code_sum[xm] * (double)w_code_sum[wm]) / (double)gs);
                acc += mu_term + residual_term;
            }
            y[r * out_features + o] = (float)acc;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* a12: index-space linear, one byte per code, fp32, 32-lane order.          */
/* Follows EXT/arcq_linear_kernel.cu:136-202: lane l of 32 sums              */
/* P[...] for j = l, l+32, ... serially (:176-180), the 32 partials are      */
/* folded by a shuffle-down tree with offsets 16,8,4,2,1 (:182-185) and lane */
/* 0 applies the per-group closed form in fp32 (:187-197).                   */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_linear_forward_u8(
    const uint8_t *x_codes, const float *x_center, const float *x_scale, const float *x_code_sum,
    const uint8_t *w_codes, const float *w_center, const float *w_scale, const float *w_code_sum,
    const float *product_table, const float *bias,
    int64_t rows, int64_t out_features, int64_t in_features,
    int gs, int levels, float *y)
{
    const int64_t groups = in_features / gs;
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t o = 0; o < out_features; ++o) {
            const uint8_t *xr = x_codes + r * in_features;
            const uint8_t *wr = w_codes + o * in_features;
            float acc = bias ? bias[o] : 0.0f;
            for (int64_t g = 0; g < groups; ++g) {
                float lane[32];
                const int64_t base = g * gs;
                for (int l = 0; l < 32; ++l) {
                    float cross = 0.0f;
                    for (int j = l; j < gs; j += 32)
                        cross += product_table[(int)xr[base + j] * levels + (int)wr[base + j]];
                    lane[l] = cross;
                }
                /* __shfl_down_sync: lane l reads lane l+offset when that lane
                 * exists, else keeps its own value; only lane 0 is consumed. */
                for (int offset = 16; offset > 0; offset >>= 1) {
                    float next[32];
                    for (int l = 0; l < 32; ++l)
                        next[l] = lane[l] + ((l + offset < 32) ? lane[l + offset] : lane[l]);
                    memcpy(lane, next, sizeof(lane));
                }
                const float cross = lane[0];
                const int64_t xm = r * groups + g, wm = o * groups + g;
                const float mu_term = (float)gs * x_center[xm] * w_center[wm];
                const float residual_term = x_scale[xm] * w_scale[wm] *
                    (cross - (x_code_sum[xm] * w_code_sum[wm]) / (float)gs);
                acc += mu_term + residual_term;
            }
            y[r * out_features + o] = acc;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Checker for the GPU stage-1 kernel's divide: t = d/s evaluated as          */
/*   y = 1/s;  q = d*y;  e = fma(-s,q,d);  q = fma(e,y,q);  (twice)           */
/* must equal the IEEE quotient d/s for every input its guard admits          */
/* (2^-60 <= s <= 2^60, |d| <= 8s, and d == 0 or |d| >= 2^-90).  Draws n      */
/* pseudo-random (d, s) pairs in that range, mantissa extremes included, and  */
/* returns how many disagree (0 expected).  Not part of the reference; it     */
/* exists so that the equivalence is tested on the CPU as well as on the GPU. */
/* ------------------------------------------------------------------------- */
static inline float u32_as_float(uint32_t b)
{
    float f;
    memcpy(&f, &b, 4);
    return f;
}

ORACLE_API float oracle_div_sequence(float d, float s)
{
    const float y = 1.0f / s;
    float q = d * y;
    float e = fmaf(-s, q, d);
    q = fmaf(e, y, q);
    e = fmaf(-s, q, d);
    return fmaf(e, y, q);
}

ORACLE_API int64_t oracle_check_div_sequence(int64_t n, uint64_t seed)
{
    uint64_t rng = seed ? seed : 88172645463325252ull;
    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) {
        rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
        const uint64_t a = rng;
        rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
        const uint64_t b = rng;
        const int es = (int)(a % 121) - 60;
        uint32_t ms = (uint32_t)(a >> 20) & 0x7fffffu;
        if ((i & 15) == 0) ms = (i & 16) ? 0x7fffffu : 0u;
        float s = u32_as_float(((uint32_t)(es + 127) << 23) | ms);
        if (s > 0x1p60f) s = 0x1p60f;
        int er = es + 3 - (int)((b >> 8) % 44);
        if (er < -90) er = -90;
        uint32_t mr = (uint32_t)(b >> 24) & 0x7fffffu;
        if ((i & 31) == 1) mr = 0u;
        float d = u32_as_float(((uint32_t)(b & 1u) << 31) | ((uint32_t)(er + 127) << 23) | mr);
        if (fabsf(d) > 8.0f * s) d = ((b & 1u) ? -7.9f : 7.9f) * s;
        const float want = d / s, got = oracle_div_sequence(d, s);
        if (memcmp(&want, &got, 4) != 0) ++bad;
    }
    return bad;
}
