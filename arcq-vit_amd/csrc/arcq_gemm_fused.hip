// Stages 2+3 fused: y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias, with w_hat
// reconstructed on the fly from packed codes (never written to HBM).
//
// Reference semantics: unpack_weight_triton (FQ/arcq_packed_triton.py:11-74)
// followed by F.linear in fp16 (FQ/arcq_packed_on_the_fly.py:159-160):
// w_hat = fp16(fma(cb[code] - S/gs, s, mu)); products of fp16 operands are
// accumulated in fp32; bias is added in fp32; the result is rounded once.
//
// Kernel shape (gs == 64): the K step of the main loop is one quantization group,
// so each weight row needs exactly one (mu, s, S) triple per step.  Both
// operands are K-contiguous, which is the layout v_mfma_f32_32x32x16_f16 wants:
// lane l supplies 8 consecutive k for row (l % 32), k offset 8*(l / 32).
#include "arcq_common.h"
#include "arcq_gemm.h"
#include <stdlib.h>
#include <string.h>

namespace arcq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // native vectors keep staging arrays in registers
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int BK = 64;            // one quantization group per main-loop step
constexpr int LDS_STRIDE = 72;    // halves per tile row: 64 + 8 pad (144 B) -> conflict-free b128 reads

// Reads the 32 codes [32*h, 32*h+32) of group g of one packed weight row.
template <int BITS>
__device__ __forceinline__ void load_codes32(const uint8_t *__restrict__ row_g, int h, uint32_t (&w)[BITS])
{
    const uint32_t *p = reinterpret_cast<const uint32_t *>(row_g + h * (4 * BITS));
    if constexpr (BITS == 4) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(p);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
    } else if constexpr (BITS == 2) {
        const u32x2_t v = *reinterpret_cast<const u32x2_t *>(p);
        w[0] = v[0]; w[1] = v[1];
    } else {
        w[0] = p[0]; w[1] = p[1]; w[2] = p[2];
    }
}

// Code q (0..31) out of the little-endian bit string held in w[].
template <int BITS>
__device__ __forceinline__ int code_at(const uint32_t (&w)[BITS], int q)
{
    const int bit = q * BITS;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + BITS > 32) v |= w[d + 1] << (32 - sh);   // only for BITS == 3
    return static_cast<int>(v & ((1u << BITS) - 1u));
}

template <int BITS, typename TOUT, int BM, int BN>
__global__ void __launch_bounds__(256)
gemm_fused_kernel(const __half *__restrict__ a, const uint8_t *__restrict__ pw, const float *__restrict__ cb,
                  const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                  const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K)
{
    static_assert(BM % 64 == 0 && BN == 128, "tile shape");
    constexpr int L = 1 << BITS;
    constexpr int WM = BM / 2;          // wave tile rows (2x2 waves)
    constexpr int WN = BN / 2;          // wave tile cols
    constexpr int TI = WM / 32, TJ = WN / 32;
    constexpr int A_PASSES = BM / 32;   // 256 threads x 16 B cover 32 rows of 64 halves

    __shared__ __attribute__((aligned(16))) _Float16 sa[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 sb[BN * LDS_STRIDE];
    __shared__ float lut[L * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;
    const int G = K / BK;
    const int64_t pcols = static_cast<int64_t>(K) * BITS / 8;

    if (tid < 64) {
#pragma unroll
        for (int c = 0; c < L; ++c) lut[c * 64 + lane] = cb[c];
    }

    // global -> register staging
    const int a_row = tid >> 3, a_col = (tid & 7) * 8;
    const int b_row = tid >> 1, b_h = tid & 1;
    const int bn = min(n0 + b_row, N - 1);
    const uint8_t *pw_row = pw + static_cast<int64_t>(bn) * pcols;
    const float *wc_row = wc + static_cast<int64_t>(bn) * G;
    const float *ws_row = ws + static_cast<int64_t>(bn) * G;
    const float *wcs_row = wcs + static_cast<int64_t>(bn) * G;

    u32x4_t a_reg[A_PASSES];
    uint32_t b_reg[BITS];
    float b_c, b_s, b_m;

    auto fetch = [&](int g) {
#pragma unroll
        for (int p = 0; p < A_PASSES; ++p) {
            const int r = min(m0 + p * 32 + a_row, M - 1);
            a_reg[p] = *reinterpret_cast<const u32x4_t *>(a + static_cast<int64_t>(r) * K + g * BK + a_col);
        }
        load_codes32<BITS>(pw_row + g * (8 * BITS), b_h, b_reg);
        b_c = wc_row[g];
        b_s = ws_row[g];
        b_m = wcs_row[g] / 64.0f;
    };

    auto stage = [&]() {
#pragma unroll
        for (int p = 0; p < A_PASSES; ++p)
            *reinterpret_cast<u32x4_t *>(&sa[(p * 32 + a_row) * LDS_STRIDE + a_col]) = a_reg[p];
        _Float16 *dst = &sb[b_row * LDS_STRIDE + b_h * 32];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            half8_t hv;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int code = code_at<BITS>(b_reg, q4 * 8 + q);
                hv[q] = static_cast<_Float16>(fma_f32(lut[code * 64 + lane] - b_m, b_s, b_c));
            }
            *reinterpret_cast<half8_t *>(dst + q4 * 8) = hv;
        }
    };

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    if (G > 0) fetch(0);
    __syncthreads();  // lut visible
    for (int g = 0; g < G; ++g) {
        stage();
        __syncthreads();
        if (g + 1 < G) fetch(g + 1);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8_t af[TI], bf[TJ];
            const int kof = kk * 16 + 8 * (lane >> 5);
#pragma unroll
            for (int i = 0; i < TI; ++i)
                af[i] = *reinterpret_cast<const half8_t *>(&sa[(wm * WM + i * 32 + (lane & 31)) * LDS_STRIDE + kof]);
#pragma unroll
            for (int j = 0; j < TJ; ++j)
                bf[j] = *reinterpret_cast<const half8_t *>(&sb[(wn * WN + j * 32 + (lane & 31)) * LDS_STRIDE + kof]);
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // Epilogue.  Accumulator element v of lane l is C[8*(v/4) + 4*(l/32) + v%4][l%32].
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int col = n0 + wn * WN + j * 32 + (lane & 31);
        if (col >= N) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < M) y[static_cast<int64_t>(row) * N + col] = from_float<TOUT>(acc[i][j][v] + bv);
            }
        }
    }
}

template <int BITS, typename TOUT>
static void launch_bits(const void *x_hat, const uint8_t *pw, const float *cb, const float *wc, const float *ws,
                        const float *wcs, const float *bias, void *y, int M, int N, int K, hipStream_t stream)
{
    const __half *a = static_cast<const __half *>(x_hat);
    TOUT *out = static_cast<TOUT *>(y);
    // Small M (batch 1: 197 tokens) gets the 64-row tile so more workgroups exist.
    const int64_t wg128 = static_cast<int64_t>((M + 127) / 128) * ((N + 127) / 128);
    if (wg128 >= 256) {
        dim3 grid((N + 127) / 128, (M + 127) / 128);
        hipLaunchKernelGGL((gemm_fused_kernel<BITS, TOUT, 128, 128>), grid, dim3(256), 0, stream, a, pw, cb, wc, ws,
                           wcs, bias, out, M, N, K);
    } else {
        dim3 grid((N + 127) / 128, (M + 63) / 64);
        hipLaunchKernelGGL((gemm_fused_kernel<BITS, TOUT, 64, 128>), grid, dim3(256), 0, stream, a, pw, cb, wc, ws,
                           wcs, bias, out, M, N, K);
    }
}

template <typename TOUT>
static void launch_out(const void *x_hat, const uint8_t *pw, const float *cb, const float *wc, const float *ws,
                       const float *wcs, const float *bias, void *y, int M, int N, int K, int bits, hipStream_t stream)
{
    if (bits == 4) launch_bits<4, TOUT>(x_hat, pw, cb, wc, ws, wcs, bias, y, M, N, K, stream);
    else if (bits == 3) launch_bits<3, TOUT>(x_hat, pw, cb, wc, ws, wcs, bias, y, M, N, K, stream);
    else launch_bits<2, TOUT>(x_hat, pw, cb, wc, ws, wcs, bias, y, M, N, K, stream);
}

}  // namespace arcq

using namespace arcq;

// Tuning aid: ARCQ_GEMM_KERNEL=stream|slab|small|splitk pins the kernel choice (read once per process).
static int forced_kernel()
{
    const char *e = tuning().gemm_kernel;
    if (!e) return 0;
    if (!strcmp(e, "stream")) return 1;
    if (!strcmp(e, "slab")) return 2;
    if (!strcmp(e, "small")) return 3;
    if (!strcmp(e, "splitk")) return 4;
    return 0;
}

// Cost model of the large-M kernels, fitted to measured launch durations (microseconds, output write-out excluded
// since all pay it alike):
//   streaming kernel: waves of 256 workgroup tiles (256 x 256), each 5 + 2.0 per quantization group;
//   weight-stationary kernel: 5.5 + 0.85 per (64-row x group) unit of a wave + 3.5 per slab slice rebuilt
//   (4.2 when K spans several slices, which adds two barriers per slice);
// The weight-stationary kernel wins when K fits one slice or N is small (few slabs, many row ranges); the
// streaming kernel wins for wide N and long K.
struct GemmCosts { double stream, slab; };

static GemmCosts gemm_costs(int64_t M, int64_t N, int64_t K)
{
    const int64_t G = K / 64;
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    GemmCosts c;
    c.stream = static_cast<double>((tiles + 255) / 256) * (5.0 + 2.0 * static_cast<double>(G));
    const int64_t n_slabs = (N + 127) / 128, blocks = (M + 31) / 32;
    int64_t ranges = 256 / n_slabs;
    if (ranges < 1) ranges = 1;
    if (ranges > blocks) ranges = blocks;
    const int64_t per_range = (blocks + ranges - 1) / ranges;
    ranges = (blocks + per_range - 1) / per_range;
    const int64_t rounds = (n_slabs * ranges + 255) / 256;
    const int64_t passes = ((per_range + 3) / 4 + 1) / 2;
    const int64_t slices = (G + 5) / 6;
    const double fills = slices == 1 ? 1.0 : static_cast<double>(passes * slices);
    const double units = 0.85 * static_cast<double>(passes * G);
    c.slab = static_cast<double>(rounds) * (5.5 + (slices == 1 ? 3.5 : 4.2) * fills + units);
    if (M * K * 2 >= (int64_t(1) << 32)) c.slab = 1.0e30;      // 32-bit byte offsets into x_hat
    return c;
}

static bool prefer_slab(int64_t M, int64_t N, int64_t K)
{
    const GemmCosts c = gemm_costs(M, N, K);
    return c.slab < c.stream;
}

enum GemmKernel { kTiled = 0, kStream = 1, kSlab = 2, kSplitK = 4 };

// Kernel that arcq_linear_fused runs for this shape: K below one group goes to the tiled kernel (it handles K = 0),
// fewer than 512 rows to the split-K kernel, larger M to whichever of the two large-M kernels the cost model favours.
static GemmKernel pick_kernel(int64_t M, int64_t N, int64_t K)
{
    const int forced = forced_kernel();
    if (K < 64 || forced == 3) return kTiled;
    const bool slab_ok = M * K * 2 < (int64_t(1) << 32);
    if (forced == 4) return kSplitK;
    if (forced == 2) return slab_ok ? kSlab : kStream;
    if (forced == 1) return kStream;
    if (M < 512) return kSplitK;
    return prefer_slab(M, N, K) ? kSlab : kStream;
}

ARCQ_API const char *arcq_linear_fused_kernel(int64_t M, int64_t N, int64_t K)
{
    switch (pick_kernel(M, N, K)) {
    case kSplitK: return "gemm_splitk_kernel";
    case kSlab: return "gemm_slab_kernel";
    case kStream: return "gemm_stream_kernel";
    default: return "gemm_fused_kernel";
    }
}

// arcq_linear_fused, optionally with GELU / a residual on the rounded outputs; those are built into the small-M
// kernel only (the large-M row-major kernels do not have them: callers with 512 rows or more use the block layout).
int arcq::linear_fused_post(const void *x_hat, const uint8_t *packed_w, const float *w_codebook, const float *w_center,
                            const float *w_scale, const float *w_code_sum, const float *bias, void *y, int y_dtype,
                            int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream,
                            const void *residual, bool gelu)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_linear_fused: bits must be 2, 3, or 4");
    if (M < 0 || N < 0 || K < 0 || group_size <= 0) return fail(ARCQ_ERR_SHAPE, "arcq_linear_fused: bad sizes");
    if (K % group_size != 0)
        return fail(ARCQ_ERR_GROUP, "arcq_linear_fused: in_features must be divisible by group_size");
    if (group_size != 64)
        return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fused: only group_size 64 is built (got %d)", group_size);
    if (y_dtype != ARCQ_F16 && y_dtype != ARCQ_F32)
        return fail(ARCQ_ERR_DTYPE, "arcq_linear_fused: y must be float16 or float32");
    if (M * N == 0) return ARCQ_OK;
    if (!y) return fail(ARCQ_ERR_NULL, "arcq_linear_fused: y must not be NULL");
    if (K > 0 && (!x_hat || !packed_w || !w_codebook || !w_center || !w_scale || !w_code_sum))
        return fail(ARCQ_ERR_NULL, "arcq_linear_fused: NULL tensor pointer");
    if (M >= (int64_t(1) << 31) - 256 || N >= (int64_t(1) << 31) - 256 || K >= (int64_t(1) << 31) - 256 ||
        (N + 127) / 128 > 0x7fffffff || (M + 63) / 64 > 65535)
        return fail(ARCQ_ERR_SHAPE, "arcq_linear_fused: M, N or K too large");
    if (!aligned(x_hat, 16) || !aligned(y, 16) || !aligned(packed_w, 16))
        return fail(ARCQ_ERR_ALIGN, "arcq_linear_fused: x_hat, y and packed_w must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
    GemmArgs g{x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, y_dtype == ARCQ_F16, m, n, k, bits};
    if (residual || gelu) {
        if (pick_kernel(M, N, K) != kSplitK)
            return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fused: GELU / residual on row-major x_hat need fewer than 512 rows "
                        "and in_features >= 64");
        if (residual && !aligned(residual, 16))
            return fail(ARCQ_ERR_ALIGN, "arcq_linear_fused: residual must be 16-byte aligned");
        g.residual = residual;
        g.gelu = gelu;
    }
    switch (pick_kernel(M, N, K)) {
    case kSplitK: launch_gemm_splitk(g, st); break;
    case kSlab: launch_gemm_slab(g, st); break;
    case kStream: launch_gemm_stream(g, st); break;
    default:
        if (y_dtype == ARCQ_F16)
            launch_out<__half>(x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, m, n, k, bits, st);
        else
            launch_out<float>(x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, m, n, k, bits, st);
    }
    return launch_status("arcq_linear_fused");
}

ARCQ_API int arcq_linear_fused(const void *x_hat,
                               const uint8_t *packed_w, const float *w_codebook,
                               const float *w_center, const float *w_scale, const float *w_code_sum,
                               const float *bias, void *y, int y_dtype,
                               int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    return linear_fused_post(x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, y_dtype, M, N, K, bits,
                             group_size, stream, nullptr, false);
}

// Whether arcq_linear_fused_ws, given a workspace, rebuilds the weights into it and runs the copying slab kernel.
static bool workspace_pays(int64_t M, int64_t N, int64_t K)
{
    if (M < 512 || K < 64 || K % 64 != 0 || M * K * 2 >= (int64_t(1) << 32)) return false;
    const char *e = tuning().gemm_kernel;
    if (e) return !strcmp(e, "prebuilt");
    // Measured: copying beats both fused kernels when few slabs (N <= 1024) meet a K of three or more slab slices,
    // i.e. when up to 256 / slabs workgroups per slab would each rebuild the same long weight rows (fc2 of DeiT-S:
    // 36.9 us against 42.2; 50432 x 1024 x 4096: 533 us against 667 and 693).
    return (N + 127) / 128 <= 8 && (K / 64 + 5) / 6 >= 3;
}

// The same question for the eight-wave kernel.  Measured: copying wins whenever K spans three or more slab slices
// (DeiT-S fc2 31.1 us against 33.9, DeiT-B fc2 87.5 against 108, ViT-L proj 136 against 160, fc1 450 against 468,
// fc2 461 against 588), with two slices only while the slabs are few (DeiT-B proj 31.4 against 33.0, but qkv 76.6
// against 72.1), and never when the slab stays resident (one slice).  "prebuilt" forces the copy.
static bool workspace_pays_blocked(int64_t N, int64_t K)
{
    if (K < 64 || K % 64 != 0) return false;
    const char *e = tuning().gemm_kernel;
    if (e && !strcmp(e, "prebuilt")) return true;
    const int64_t slabs = (N + 127) / 128, slices = (K / 64 + 5) / 6;
    return slices >= 3 || (slices == 2 && slabs <= 8);
}

ARCQ_API const char *arcq_linear_fused_ws_kernel(int64_t M, int64_t N, int64_t K, int have_workspace)
{
    if (have_workspace && N > 0 && workspace_pays(M, N, K)) return "weight_dequant8_kernel+gemm_slab_kernel";
    return arcq_linear_fused_kernel(M, N, K);
}

// Shapes for which arcq_linear_otf_ws quantizes into the 32-row block layout and multiplies with the eight-wave
// weight-stationary kernel: from 512 rows on.  Measured against the row-major kernels on the
// twelve DeiT-S / DeiT-B / ViT-L layer shapes it is the fastest on ten and within 3 % (DeiT-B proj, ViT-L fc1) on
// two.  ARCQ_GEMM_KERNEL pins a row-major kernel, or this one with "slab8" / "prebuilt".
bool arcq::otf_blocked_pays(int64_t M, int64_t N, int64_t K)
{
    if (M < 512 || N <= 0 || K < 64 || K % 64 != 0 || M * K * 2 >= (int64_t(1) << 32)) return false;
    if (M >= (int64_t(1) << 31) - 256 || N >= (int64_t(1) << 31) - 256) return false;
    const char *e = tuning().gemm_kernel;
    if (e) return !strcmp(e, "slab8") || !strcmp(e, "prebuilt");
    return true;
}

ARCQ_API const char *arcq_linear_otf_ws_kernel(int64_t M, int64_t N, int64_t K, int have_workspace)
{
    if (have_workspace && otf_rows_pays(M, N, K)) return otf_rows_is_phased(N, K) ? "otf_rows_phased_kernel" : "otf_rows_kernel";      // (for fp16 input)
    if (otf_blocked_pays(M, N, K)) {
        if (!(have_workspace && blocked_uses_workspace(N, K))) return "gemm_slab8_kernel";
        GemmArgs g{};
        g.M = static_cast<int>(M), g.N = static_cast<int>(N), g.K = static_cast<int>(K);
        const char *e = tuning().pair;
        return (e ? e[0] != '0' : gemm_pair_pays(g)) ? "gemm_pair_kernel" : "gemm_slab8_kernel<copy>";
    }
    return arcq_linear_fused_ws_kernel(M, N, K, have_workspace);
}

// The fused GEMM on x_hat in the 32-row block layout (what arcq_act_quant_blocked writes): always the eight-wave
// weight-stationary kernel; with a weight workspace, and a shape where that pays, on weights reconstructed once.
// In the whole-layer entry point the reconstruction costs no launch of its own (it rides in the stage-1 launch), and
// copying is then never slower than rebuilding inside the GEMM: for shapes whose K spans several slab slices it is
// the large win measured above, for the others what the GEMM gains (a 1 us copy instead of a 3.6 us rebuild) the
// stage-1 launch pays (whole steps of DeiT-S / DeiT-B / ViT-L: 0.5 % / 0.3 % / 0.0 % faster than copying by the
// stand-alone rule).  "slab8" pins the in-kernel rebuild, "prebuilt" the copy.
bool arcq::blocked_uses_workspace(int64_t N, int64_t K)
{
    if (N <= 0 || K < 64 || K % 64 != 0) return false;
    const char *e = tuning().gemm_kernel;
    if (e) return !strcmp(e, "prebuilt");
    return true;
}

ARCQ_API int arcq_linear_fused_blocked(const void *x_hat_blocked,
                                       const uint8_t *packed_w, const float *w_codebook,
                                       const float *w_center, const float *w_scale, const float *w_code_sum,
                                       const float *bias, void *w_hat_ws, int w_hat_ready, void *y, int y_dtype,
                                       int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    if (w_hat_ready && !w_hat_ws)
        return fail(ARCQ_ERR_NULL, "arcq_linear_fused_blocked: w_hat_ready needs w_hat_ws");
    return linear_fused_blocked(x_hat_blocked, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, w_hat_ws,
                                w_hat_ready != 0, y, y_dtype, M, N, K, bits, group_size, stream);
}

int arcq::linear_fused_blocked(const void *x_hat_blocked, const uint8_t *packed_w, const float *w_codebook,
                               const float *w_center, const float *w_scale, const float *w_code_sum, const float *bias,
                               void *w_hat_ws, bool w_hat_ready, void *y, int y_dtype, int64_t M, int64_t N, int64_t K,
                               int bits, int group_size, void *stream, const void *residual, bool gelu,
                               const float *next_thr, const float *next_cb)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "arcq_linear_fused_blocked: bits must be 2, 3, or 4");
    if (group_size != 64) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fused_blocked: group_size must be 64 (got %d)", group_size);
    if (M < 0 || N < 0 || K < 0) return fail(ARCQ_ERR_SHAPE, "arcq_linear_fused_blocked: negative size");
    if (K % 64 != 0) return fail(ARCQ_ERR_GROUP, "arcq_linear_fused_blocked: in_features must be divisible by group_size");
    if (y_dtype != ARCQ_F16 && y_dtype != ARCQ_F32)
        return fail(ARCQ_ERR_DTYPE, "arcq_linear_fused_blocked: y must be float16 or float32");
    if (M == 0 || N == 0) return ARCQ_OK;
    if (K == 0) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fused_blocked: in_features must not be 0");
    if (!y || !x_hat_blocked || !packed_w || !w_codebook || !w_center || !w_scale || !w_code_sum)
        return fail(ARCQ_ERR_NULL, "arcq_linear_fused_blocked: NULL tensor pointer");
    if (M >= (int64_t(1) << 31) - 256 || N >= (int64_t(1) << 31) - 256 || M * K * 2 >= (int64_t(1) << 32))
        return fail(ARCQ_ERR_SHAPE, "arcq_linear_fused_blocked: M, N or K too large");
    if (!aligned(x_hat_blocked, 16) || !aligned(y, 16) || !aligned(packed_w, 16) || !aligned(w_hat_ws, 16))
        return fail(ARCQ_ERR_ALIGN, "arcq_linear_fused_blocked: x_hat_blocked, y, packed_w and w_hat_ws must be 16-byte aligned");
    if (next_thr) {          // y receives the consuming layer's x_hat: built into the kernels that copy reconstructed weights
        if (!next_cb || !w_hat_ws || y_dtype != ARCQ_F16 || N % 64 != 0 || residual)
            return fail(ARCQ_ERR_UNSUPPORTED, "arcq_linear_fused_blocked: quantizing the output for the next layer needs a weight "
                        "workspace, a float16 output, out_features a multiple of 64 and no residual");
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool prebuilt = w_hat_ws && (w_hat_ready || next_thr || workspace_pays_blocked(N, K));
    if (prebuilt && !w_hat_ready) {
        const int rc = arcq_weight_dequant(packed_w, w_codebook, w_center, w_scale, w_code_sum, w_hat_ws, ARCQ_F16, N, K,
                                           bits, group_size, stream);
        if (rc != ARCQ_OK) return rc;
    }
    GemmArgs g{x_hat_blocked, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, y_dtype == ARCQ_F16,
               static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), bits};
    g.residual = residual;
    g.gelu = gelu;
    g.next_thr = next_thr;
    g.next_cb = next_cb;
    launch_gemm_slab8(g, prebuilt ? w_hat_ws : nullptr, st);
    return launch_status("arcq_linear_fused_blocked");
}

// arcq_linear_fused with a scratch buffer for the reconstructed weights.  When the cost model says that rebuilding
// the weights once (arcq_weight_dequant into w_hat_ws) and copying slab slices beats both fused kernels, that is
// what runs; otherwise, or without a workspace, this is arcq_linear_fused.  Results are bit-identical either way.
ARCQ_API int arcq_linear_fused_ws(const void *x_hat,
                                  const uint8_t *packed_w, const float *w_codebook,
                                  const float *w_center, const float *w_scale, const float *w_code_sum,
                                  const float *bias, void *w_hat_ws, void *y, int y_dtype,
                                  int64_t M, int64_t N, int64_t K, int bits, int group_size, void *stream)
{
    const bool prebuilt = w_hat_ws && group_size == 64 && bits_ok(bits) && N > 0 &&
        M < (int64_t(1) << 31) - 256 && N < (int64_t(1) << 31) - 256 && K < (int64_t(1) << 31) - 256 &&
        (y_dtype == ARCQ_F16 || y_dtype == ARCQ_F32) && x_hat && y && packed_w && w_codebook && w_center && w_scale &&
        w_code_sum && aligned(x_hat, 16) && aligned(y, 16) && aligned(packed_w, 16) && aligned(w_hat_ws, 16) &&
        workspace_pays(M, N, K);
    if (!prebuilt)
        return arcq_linear_fused(x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, y_dtype, M, N, K,
                                 bits, group_size, stream);
    const int rc = arcq_weight_dequant(packed_w, w_codebook, w_center, w_scale, w_code_sum, w_hat_ws, ARCQ_F16, N, K, bits,
                                       group_size, stream);
    if (rc != ARCQ_OK) return rc;
    GemmArgs g{x_hat, packed_w, w_codebook, w_center, w_scale, w_code_sum, bias, y, y_dtype == ARCQ_F16,
               static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), bits};
    launch_gemm_slab_prebuilt(g, w_hat_ws, static_cast<hipStream_t>(stream));
    return launch_status("arcq_linear_fused_ws");
}
