// Index-space linears: y = sum over groups of
//   gs*mu_x*mu_w + s_x*s_w*(sum_j P[xcode_j][wcode_j] - Sx*Sw/gs)
// with P = cb_a (x) cb_w, i.e. no reconstruction of either operand
// (EXT/arcq_linear_kernel.cu:22-78 for packed codes / fp64, :136-202 for byte
// codes / fp32).  These are the reference's "packed" and "u8" runtime formats.
// All kernels keep the reference's summation order per output, so that the result equals a
// serial CPU evaluation bit for bit; contraction is switched off for that reason.  Group size 64
// runs the tiled kernels further down; the two kernels right below take any group size.
#include "arcq_common.h"

#include <type_traits>

namespace arcq {

constexpr int kIdxTile = 16;  // 16 x 16 outputs per 256-thread workgroup (the any-group-size kernels)

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

// ---- group size 64: tiled kernels -------------------------------------------------------------------------------
// A workgroup owns 16 rows x 64 outputs; a thread one row and four consecutive outputs.  Per group the tile's codes
// are fetched once (packed rows: `bits` bytes = eight codes per load, consecutive threads reading consecutive bytes),
// unpacked once into LDS as bytes -- x as [row][j], w transposed as [j][output], so that a thread's four weight codes
// of one j are a single dword read -- and every product-table lookup is one LDS read.  What fixes the result's bits is
// the order in which one output's terms are added; that is the reference's, per output: serial over j in fp64 for
// the packed format; for the byte format the 32 strided partial sums folded by the shuffle-down tree, which is
// evaluated here depth first (the same additions, associated the same way) so that only five values per output are live.
constexpr int kTileRows = 16, kTileOuts = 64;

// BITS = 2 / 3 / 4: packed codes, fp64 accumulation.  BITS = 0: byte codes, fp32, tree order.
// OPT = outputs per thread: four (256 threads per workgroup) for launches that fill the chip; one (1024 threads) for
// small ones, whose duration is the length of one thread's chain of additions (197 x 768 x 192: 156 tiles).
template <int BITS, int OPT>
__global__ void __launch_bounds__(1024 / OPT)
linear_index_tile_kernel(const uint8_t *__restrict__ xq, const float *__restrict__ xc, const float *__restrict__ xs,
                         const float *__restrict__ xcs, const uint8_t *__restrict__ wq,
                         const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                         const float *__restrict__ table, const float *__restrict__ bias, float *__restrict__ y,
                         int64_t rows, int64_t out_f, int64_t in_f, int levels)
{
#pragma clang fp contract(off)
    extern __shared__ float s_table[];
    __shared__ __attribute__((aligned(16))) uint8_t s_x[kTileRows][64];
    __shared__ __attribute__((aligned(16))) uint8_t s_w[64][kTileOuts];          // [j][output]
    constexpr int kOutsPerThread = OPT;
    constexpr int kThreads = 1024 / OPT;
    constexpr int kThreadsPerRow = kTileOuts / OPT;
    const int tid = threadIdx.x;
    for (int i = tid; i < levels * levels; i += kThreads) s_table[i] = table[i];
    const int tr = tid / kThreadsPerRow;                       // row of the tile
    const int to = (tid % kThreadsPerRow) * kOutsPerThread;    // first of this thread's outputs in the tile
    const int64_t r = static_cast<int64_t>(blockIdx.y) * kTileRows + tr;
    const int64_t o0 = static_cast<int64_t>(blockIdx.x) * kTileOuts + to;
    const int64_t groups = in_f / 64;
    const int64_t rc = r < rows ? r : rows - 1;    // rows / outputs past the end repeat the last one and are not stored
    constexpr int kRowBytes = BITS ? 8 * BITS : 64;      // bytes of one group in a row of codes
    const int64_t pcols = groups * kRowBytes;

    using acc_t = typename std::conditional<BITS != 0, double, float>::type;
    acc_t acc[kOutsPerThread];
    int64_t oc[kOutsPerThread];
#pragma unroll
    for (int i = 0; i < kOutsPerThread; ++i) {
        oc[i] = o0 + i < out_f ? o0 + i : out_f - 1;
        acc[i] = bias ? static_cast<acc_t>(bias[oc[i]]) : static_cast<acc_t>(0);
    }

    for (int64_t g = 0; g < groups; ++g) {
        __syncthreads();          // the previous group's codes have been used (first round: the table is complete)
        // ---- this group's codes into LDS, unpacked ----
        if constexpr (BITS != 0) {
            if (tid < kTileRows * 8) {                               // x: 16 rows x 8 chunks of eight codes
                const int row = tid >> 3, ch = tid & 7;
                const int64_t rr = static_cast<int64_t>(blockIdx.y) * kTileRows + row;
                const uint32_t w8 = load_codes8<BITS>(xq + (rr < rows ? rr : rows - 1) * pcols + g * kRowBytes + ch * BITS);
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    lo |= ((w8 >> (BITS * q)) & ((1u << BITS) - 1u)) << (8 * q);
                    hi |= ((w8 >> (BITS * (q + 4))) & ((1u << BITS) - 1u)) << (8 * q);
                }
                *reinterpret_cast<uint2 *>(&s_x[row][ch * 8]) = make_uint2(lo, hi);
            }
            for (int job = tid; job < kTileOuts * 8; job += kThreads) {      // w: 64 outputs x 8 chunks of eight codes
                const int out = job >> 3, ch = job & 7;
                const int64_t oo = static_cast<int64_t>(blockIdx.x) * kTileOuts + out;
                const uint32_t w8 = load_codes8<BITS>(wq + (oo < out_f ? oo : out_f - 1) * pcols + g * kRowBytes + ch * BITS);
#pragma unroll
                for (int q = 0; q < 8; ++q) s_w[ch * 8 + q][out] = static_cast<uint8_t>((w8 >> (BITS * q)) & ((1u << BITS) - 1u));
            }
        } else {
            if (tid < 256) {                                         // x: 16 rows x 64 bytes, one dword per thread
                const int row = tid >> 4, c4 = (tid & 15) * 4;
                const int64_t rr = static_cast<int64_t>(blockIdx.y) * kTileRows + row;
                *reinterpret_cast<uint32_t *>(&s_x[row][c4]) =
                    *reinterpret_cast<const uint32_t *>(xq + (rr < rows ? rr : rows - 1) * pcols + g * 64 + c4);
            }
            if (tid < 256) {                                         // w: 64 outputs x 64 bytes, sixteen bytes per thread
                const int out = tid >> 2, c16 = (tid & 3) * 16;
                const int64_t oo = static_cast<int64_t>(blockIdx.x) * kTileOuts + out;
                const uint4 v = *reinterpret_cast<const uint4 *>(wq + (oo < out_f ? oo : out_f - 1) * pcols + g * 64 + c16);
                const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 16; ++q) s_w[c16 + q][out] = static_cast<uint8_t>(d[q >> 2] >> (8 * (q & 3)));
            }
        }
        __syncthreads();
        // one j for this thread's row and its four outputs: the table entries P[x code][w code]
        auto entries = [&](int j, float (&e)[kOutsPerThread]) __attribute__((always_inline)) {
            const int a = static_cast<int>(s_x[tr][j]) * levels;
            if constexpr (OPT == 4) {
                const uint32_t wb = *reinterpret_cast<const uint32_t *>(&s_w[j][to]);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) e[i] = s_table[a + static_cast<int>((wb >> (8 * i)) & 255u)];
            } else {
                e[0] = s_table[a + static_cast<int>(s_w[j][to])];
            }
        };
        acc_t cross[kOutsPerThread];
        if constexpr (BITS != 0) {
#pragma unroll
            for (int i = 0; i < kOutsPerThread; ++i) cross[i] = 0.0;
#pragma unroll 8
            for (int j = 0; j < 64; ++j) {
                float e[kOutsPerThread];
                entries(j, e);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) cross[i] += static_cast<double>(e[i]);
            }
        } else {
            // leaf l = the partial sum of lane l: j = l, then j = l + 32; node(level, l) = what lane l holds after the
            // fold with offset 32 >> level (lane l adds lane l + offset): node(5, 0) is the group's sum.
            auto leaf = [&](int l, float (&p)[kOutsPerThread]) __attribute__((always_inline)) {
                float e0[kOutsPerThread], e1[kOutsPerThread];
                entries(l, e0);
                entries(l + 32, e1);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) {
                    float c = 0.0f;
                    c += e0[i];
                    c += e1[i];
                    p[i] = c;
                }
            };
            auto node1 = [&](int l, float (&v)[kOutsPerThread]) __attribute__((always_inline)) {      // offset 16
                float b[kOutsPerThread];
                leaf(l, v);
                leaf(l + 16, b);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) v[i] = v[i] + b[i];
            };
            auto node2 = [&](int l, float (&v)[kOutsPerThread]) __attribute__((always_inline)) {      // offset 8
                float b[kOutsPerThread];
                node1(l, v);
                node1(l + 8, b);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) v[i] = v[i] + b[i];
            };
            auto node3 = [&](int l, float (&v)[kOutsPerThread]) __attribute__((always_inline)) {      // offset 4
                float b[kOutsPerThread];
                node2(l, v);
                node2(l + 4, b);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) v[i] = v[i] + b[i];
            };
            auto node4 = [&](int l, float (&v)[kOutsPerThread]) __attribute__((always_inline)) {      // offset 2
                float b[kOutsPerThread];
                node3(l, v);
                node3(l + 2, b);
#pragma unroll
                for (int i = 0; i < kOutsPerThread; ++i) v[i] = v[i] + b[i];
            };
            float b[kOutsPerThread];
            node4(0, cross);                                                                             // offset 1
            node4(1, b);
#pragma unroll
            for (int i = 0; i < kOutsPerThread; ++i) cross[i] = cross[i] + b[i];
        }
        // ---- the group's closed form (EXT/arcq_linear_kernel.cu:65-74 / :187-197) ----
        const int64_t xm = rc * groups + g;
        const float xcv = xc[xm], xsv = xs[xm], xcsv = xcs[xm];
#pragma unroll
        for (int i = 0; i < kOutsPerThread; ++i) {
            const int64_t wm = oc[i] * groups + g;
            if constexpr (BITS != 0) {
                const double mu_term = 64.0 * static_cast<double>(xcv) * static_cast<double>(wc[wm]);
                const double residual_term = static_cast<double>(xsv) * static_cast<double>(ws[wm]) *
                    (cross[i] - (static_cast<double>(xcsv) * static_cast<double>(wcs[wm])) / 64.0);
                acc[i] += mu_term + residual_term;
            } else {
                const float mu_term = 64.0f * xcv * wc[wm];
                const float residual_term = xsv * ws[wm] * (cross[i] - (xcsv * wcs[wm]) / 64.0f);
                acc[i] += mu_term + residual_term;
            }
        }
    }
    if (groups == 0) __syncthreads();
    if (r < rows) {
#pragma unroll
        for (int i = 0; i < kOutsPerThread; ++i)
            if (o0 + i < out_f) y[r * out_f + o0 + i] = static_cast<float>(acc[i]);
    }
}

// Launches of at most this many 16 x 64 tiles give every thread one output instead of four.
constexpr int kSmallTiles = 512;
static size_t tile_table_bytes(int levels) { return static_cast<size_t>(levels) * levels * sizeof(float); }

static int check_common(const char *fn, int64_t rows, int64_t out_f, int64_t in_f, int gs, int levels)
{
    if (rows < 0 || out_f < 0 || in_f < 0 || gs <= 0) return fail(ARCQ_ERR_SHAPE, "%s: bad sizes", fn);
    if (in_f % gs != 0) return fail(ARCQ_ERR_GROUP, "%s: in_features must be divisible by group_size", fn);
    // (the table is held in LDS: 128 x 128 floats are 64 KB)
    if (levels < 1 || levels > 128) return fail(ARCQ_ERR_SHAPE, "%s: product_table must be [levels, levels] with 1 <= levels <= 128 (got %d)", fn, levels);
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
    if (group_size == 64 && in_features > 0 && (rows + kTileRows - 1) / kTileRows <= 65535 && aligned(packed_x, 4) &&
        aligned(packed_w, 4)) {
        dim3 tgrid(static_cast<unsigned>((out_features + kTileOuts - 1) / kTileOuts),
                   static_cast<unsigned>((rows + kTileRows - 1) / kTileRows));
        const bool small = static_cast<int64_t>(tgrid.x) * tgrid.y <= kSmallTiles;
#define ARCQ_LAUNCH_TILE(B, O)                                                                                           \
    do {                                                                                                                  \
        allow_dynamic_lds<linear_index_tile_kernel<B, O>>(64 * 1024);                                                     \
        hipLaunchKernelGGL((linear_index_tile_kernel<B, O>), tgrid, dim3(1024 / O), tile_table_bytes(levels),              \
                           static_cast<hipStream_t>(stream), packed_x, x_center, x_scale, x_code_sum, packed_w, w_center, \
                           w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, levels);         \
    } while (0)
        if (bits == 4) { if (small) ARCQ_LAUNCH_TILE(4, 1); else ARCQ_LAUNCH_TILE(4, 4); }
        else if (bits == 3) { if (small) ARCQ_LAUNCH_TILE(3, 1); else ARCQ_LAUNCH_TILE(3, 4); }
        else { if (small) ARCQ_LAUNCH_TILE(2, 1); else ARCQ_LAUNCH_TILE(2, 4); }
#undef ARCQ_LAUNCH_TILE
        return launch_status("arcq_linear_forward_packed");
    }
    // Any other group size: one thread per output, codes extracted from global memory (slow, no layout assumptions).
    dim3 grid(static_cast<unsigned>((out_features + kIdxTile - 1) / kIdxTile),
              static_cast<unsigned>((rows + kIdxTile - 1) / kIdxTile));
    allow_dynamic_lds<linear_index_packed_kernel>(64 * 1024);
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
    if (group_size == 64 && in_features > 0 && (rows + kTileRows - 1) / kTileRows <= 65535 && aligned(x_codes, 4) &&
        aligned(w_codes, 16)) {
        dim3 tgrid(static_cast<unsigned>((out_features + kTileOuts - 1) / kTileOuts),
                   static_cast<unsigned>((rows + kTileRows - 1) / kTileRows));
        if (static_cast<int64_t>(tgrid.x) * tgrid.y <= kSmallTiles) {
            allow_dynamic_lds<linear_index_tile_kernel<0, 1>>(64 * 1024);
            hipLaunchKernelGGL((linear_index_tile_kernel<0, 1>), tgrid, dim3(1024), tile_table_bytes(levels),
                               static_cast<hipStream_t>(stream), x_codes, x_center, x_scale, x_code_sum, w_codes, w_center,
                               w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, levels);
        } else {
            allow_dynamic_lds<linear_index_tile_kernel<0, 4>>(64 * 1024);
            hipLaunchKernelGGL((linear_index_tile_kernel<0, 4>), tgrid, dim3(256), tile_table_bytes(levels),
                               static_cast<hipStream_t>(stream), x_codes, x_center, x_scale, x_code_sum, w_codes, w_center,
                               w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, levels);
        }
        return launch_status("arcq_linear_forward_u8");
    }
    dim3 grid(static_cast<unsigned>((out_features + kIdxTile - 1) / kIdxTile),
              static_cast<unsigned>((rows + kIdxTile - 1) / kIdxTile));
    allow_dynamic_lds<linear_index_u8_kernel>(64 * 1024);
    hipLaunchKernelGGL(linear_index_u8_kernel, grid, dim3(256), levels * levels * sizeof(float),
                       static_cast<hipStream_t>(stream), x_codes, x_center, x_scale, x_code_sum, w_codes, w_center,
                       w_scale, w_code_sum, product_table, bias, y, rows, out_features, in_features, group_size, levels);
    return launch_status("arcq_linear_forward_u8");
}
