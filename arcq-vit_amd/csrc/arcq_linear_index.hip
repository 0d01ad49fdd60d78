// Index-space linears: y = sum over groups of
//   gs*mu_x*mu_w + s_x*s_w*(sum_j P[xcode_j][wcode_j] - Sx*Sw/gs)
// with P = cb_a (x) cb_w, i.e. no reconstruction of either operand
// (EXT/arcq_linear_kernel.cu:22-78 for packed codes / fp64, :136-202 for byte
// codes / fp32).  These are the reference's "packed" and "u8" runtime formats.
// Both kernels keep the reference's summation order so that the result equals a
// serial CPU evaluation bit for bit; contraction is switched off for that reason.
#include "arcq_common.h"

namespace arcq {

constexpr int kIdxTile = 16;  // 16 x 16 outputs per 256-thread workgroup

// fp64 accumulation, codes extracted from the packed rows on the fly.
__global__ void __launch_bounds__(256)
linear_index_packed_kernel(const uint8_t *__restrict__ px, const float *__restrict__ xc, const float *__restrict__ xs,
                           const float *__restrict__ xcs, const uint8_t *__restrict__ pw,
                           const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                           const float *__restrict__ table, const float *__restrict__ bias, float *__restrict__ y,
                           int64_t rows, int64_t out_f, int64_t in_f, int bits, int gs, int levels)
{
#pragma clang fp contract(off)
    extern __shared__ float s_table[];
    for (int i = threadIdx.x; i < levels * levels; i += blockDim.x) s_table[i] = table[i];
    __syncthreads();
    const int64_t r = static_cast<int64_t>(blockIdx.y) * kIdxTile + (threadIdx.x >> 4);
    const int64_t o = static_cast<int64_t>(blockIdx.x) * kIdxTile + (threadIdx.x & 15);
    if (r >= rows || o >= out_f) return;
    const int64_t groups = in_f / gs;
    const int64_t pcols = packed_cols(in_f, bits);
    const uint8_t *__restrict__ xr = px + r * pcols;
    const uint8_t *__restrict__ wr = pw + o * pcols;
    double acc = bias ? static_cast<double>(bias[o]) : 0.0;
    for (int64_t g = 0; g < groups; ++g) {
        double cross = 0.0;
        const int64_t base = g * gs;
        for (int j = 0; j < gs; ++j) {
            const int a = get_code(xr, base + j, bits);
            const int b = get_code(wr, base + j, bits);
            cross += static_cast<double>(s_table[a * levels + b]);
        }
        const int64_t xm = r * groups + g, wm = o * groups + g;
        const double mu_term = static_cast<double>(gs) * static_cast<double>(xc[xm]) * static_cast<double>(wc[wm]);
        const double residual_term = static_cast<double>(xs[xm]) * static_cast<double>(ws[wm]) *
            (cross - (static_cast<double>(xcs[xm]) * static_cast<double>(wcs[wm])) / static_cast<double>(gs));
        acc += mu_term + residual_term;
    }
    y[r * out_f + o] = static_cast<float>(acc);
}

// fp32, byte codes.  The reference gives each output a 32-lane warp: lane l sums
// the table entries of j = l, l+32, ... and the 32 partials are folded by a
// shuffle-down tree (16, 8, 4, 2, 1).  Here one thread owns the output and
// evaluates the same 32 partials and the same tree in registers.
__global__ void __launch_bounds__(256)
linear_index_u8_kernel(const uint8_t *__restrict__ xcodes, const float *__restrict__ xc, const float *__restrict__ xs,
                       const float *__restrict__ xcs, const uint8_t *__restrict__ wcodes,
                       const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                       const float *__restrict__ table, const float *__restrict__ bias, float *__restrict__ y,
                       int64_t rows, int64_t out_f, int64_t in_f, int gs, int levels)
{
#pragma clang fp contract(off)
    extern __shared__ float s_table[];
    for (int i = threadIdx.x; i < levels * levels; i += blockDim.x) s_table[i] = table[i];
    __syncthreads();
    const int64_t r = static_cast<int64_t>(blockIdx.y) * kIdxTile + (threadIdx.x >> 4);
    const int64_t o = static_cast<int64_t>(blockIdx.x) * kIdxTile + (threadIdx.x & 15);
    if (r >= rows || o >= out_f) return;
    const int64_t groups = in_f / gs;
    const uint8_t *__restrict__ xr = xcodes + r * in_f;
    const uint8_t *__restrict__ wr = wcodes + o * in_f;
    float acc = bias ? bias[o] : 0.0f;
    for (int64_t g = 0; g < groups; ++g) {
        const int64_t base = g * gs;
        float p[32];
#pragma unroll
        for (int l = 0; l < 32; ++l) {
            float cross = 0.0f;
            for (int j = l; j < gs; j += 32)
                cross += s_table[static_cast<int>(xr[base + j]) * levels + static_cast<int>(wr[base + j])];
            p[l] = cross;
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
#pragma unroll
            for (int l = 0; l < off; ++l) p[l] = p[l] + p[l + off];
        }
        const float cross = p[0];
        const int64_t xm = r * groups + g, wm = o * groups + g;
        const float mu_term = static_cast<float>(gs) * xc[xm] * wc[wm];
        const float residual_term = xs[xm] * ws[wm] * (cross - (xcs[xm] * wcs[wm]) / static_cast<float>(gs));
        acc += mu_term + residual_term;
    }
    y[r * out_f + o] = acc;
}

static int check_common(const char *fn, int64_t rows, int64_t out_f, int64_t in_f, int gs, int levels)
{
    if (rows < 0 || out_f < 0 || in_f < 0 || gs <= 0) return fail(ARCQ_ERR_SHAPE, "%s: bad sizes", fn);
    if (in_f % gs != 0) return fail(ARCQ_ERR_GROUP, "%s: in_features must be divisible by group_size", fn);
    if (levels < 1 || levels > 256) return fail(ARCQ_ERR_SHAPE, "%s: product_table must be [levels, levels] with 1 <= levels <= 256", fn);
    if ((out_f + kIdxTile - 1) / kIdxTile > 0x7fffffff || (rows + kIdxTile - 1) / kIdxTile > 65535)
        return fail(ARCQ_ERR_SHAPE, "%s: too many rows or outputs", fn);
    return ARCQ_OK;
}

}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_linear_forward_packed(const uint8_t *packed_x, const float *x_center, const float *x_scale,
                                        const float *x_code_sum,
                                        const uint8_t *packed_w, const float *w_center, const float *w_scale,
                                        const float *w_code_sum,
                                        const float *product_table, const float *bias, float *y,
                                        int64_t rows, int64_t out_features, int64_t in_features,
                                        int bits, int group_size, int levels, void *stream)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_linear_forward_packed: bits must be 2, 3, or 4");
    int rc = check_common("arcq_linear_forward_packed", rows, out_features, in_features, group_size, levels);
    if (rc != ARCQ_OK) return rc;
    if (levels < (1 << bits))
        return fail(ARCQ_ERR_SHAPE, "arcq_linear_forward_packed: product_table has %d levels, %d-bit codes need %d",
                    levels, bits, 1 << bits);
    if (rows * out_features == 0) return ARCQ_OK;
    if (!y || !product_table) return fail(ARCQ_ERR_NULL, "arcq_linear_forward_packed: NULL tensor pointer");
    if (in_features > 0 && (!packed_x || !x_center || !x_scale || !x_code_sum || !packed_w || !w_center || !w_scale || !w_code_sum))
        return fail(ARCQ_ERR_NULL, "arcq_linear_forward_packed: NULL tensor pointer");
    dim3 grid(static_cast<unsigned>((out_features + kIdxTile - 1) / kIdxTile),
              static_cast<unsigned>((rows + kIdxTile - 1) / kIdxTile));
    hipLaunchKernelGGL(linear_index_packed_kernel, grid, dim3(256), levels * levels * sizeof(float),
                       static_cast<hipStream_t>(stream), packed_x, x_center, x_scale, x_code_sum, packed_w, w_center,
                       w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, bits, group_size,
                       levels);
    return launch_status("arcq_linear_forward_packed");
}

ARCQ_API int arcq_linear_forward_u8(const uint8_t *x_codes, const float *x_center, const float *x_scale,
                                    const float *x_code_sum,
                                    const uint8_t *w_codes, const float *w_center, const float *w_scale,
                                    const float *w_code_sum,
                                    const float *product_table, const float *bias, float *y,
                                    int64_t rows, int64_t out_features, int64_t in_features,
                                    int group_size, int levels, void *stream)
{
    int rc = check_common("arcq_linear_forward_u8", rows, out_features, in_features, group_size, levels);
    if (rc != ARCQ_OK) return rc;
    if (rows * out_features == 0) return ARCQ_OK;
    if (!y || !product_table) return fail(ARCQ_ERR_NULL, "arcq_linear_forward_u8: NULL tensor pointer");
    if (in_features > 0 && (!x_codes || !x_center || !x_scale || !x_code_sum || !w_codes || !w_center || !w_scale || !w_code_sum))
        return fail(ARCQ_ERR_NULL, "arcq_linear_forward_u8: NULL tensor pointer");
    dim3 grid(static_cast<unsigned>((out_features + kIdxTile - 1) / kIdxTile),
              static_cast<unsigned>((rows + kIdxTile - 1) / kIdxTile));
    hipLaunchKernelGGL(linear_index_u8_kernel, grid, dim3(256), levels * levels * sizeof(float),
                       static_cast<hipStream_t>(stream), x_codes, x_center, x_scale, x_code_sum, w_codes, w_center,
                       w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, group_size, levels);
    return launch_status("arcq_linear_forward_u8");
}
