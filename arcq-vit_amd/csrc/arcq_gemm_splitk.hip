// Stages 2+3 fused, small-M kernel: y[M,N] = x_hat[M,K] * w_hat[N,K]^T + bias for a few hundred rows.
//
// With so few rows a launch cannot fill the chip and its duration is the length of one workgroup's dependent
// chain: (global load -> dequantize -> MFMA) once per quantization group.  This kernel shortens that chain by
// splitting K across the waves of a workgroup: a workgroup owns a 32 x 32, 32 x 64 or 64 x 64 output tile (the
// smallest that still leaves the grid within the chip), wave w of NW handles the
// groups g = w, w + NW, w + 2 NW, ... entirely on its own (operands straight from global memory into registers, no
// barrier inside the loop), and the NW partial tiles are added in LDS in the fixed order w = 0, 1, ..., NW-1, so
// results do not depend on timing.  Weight reconstruction is the stand-alone stage-2 arithmetic
// (FQ/arcq_packed_triton.py:59-74): w_hat = fp16(fma(cb[code] - S/64, s, mu)).
//
// k order inside a group: lane half h covers k = 32h + 8*step ... + 7 in k-step `step`, for both operands.
// Operand roles are swapped (w_hat is the MFMA "A" operand): accumulator element v of lane l is
// y[m = 32i + l%32][n = 32j + 8*(v/4) + 4*(l/32) + v%4].
#include "arcq_common.h"
#include "arcq_gemm.h"

#include <type_traits>

namespace arcq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// A workgroup's tile is 32 * RB rows x 32 * CB columns; a row of a partial tile in LDS takes 32 * CB * 4 + 16 bytes.

template <int BITS>
__device__ __forceinline__ void sk_load_codes(const uint8_t *__restrict__ p, uint32_t (&w)[BITS])
{
    if constexpr (BITS == 4) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(p);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
    } else if constexpr (BITS == 2) {
        const u32x2_t v = *reinterpret_cast<const u32x2_t *>(p);
        w[0] = v[0]; w[1] = v[1];
    } else {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
        w[0] = q[0]; w[1] = q[1]; w[2] = q[2];
    }
}

template <int BITS>
__device__ __forceinline__ uint32_t sk_code_at(const uint32_t (&w)[BITS], int q)
{
    const int bit = q * BITS;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + BITS > 32) v |= w[d + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}

template <int BITS, int RB, int CB>
struct SkOperands {                 // everything one wave needs for one group
    u32x4_t a[RB][4];               // x_hat: RB row blocks x 4 k-steps, 8 halves each
    uint32_t codes[CB][BITS];       // 32 codes of this lane's weight row, per column block
    float c[CB], s[CB], m[CB];
};

template <int BITS, typename TOUT, int NW, int RB, int CB>
__global__ void __launch_bounds__(NW * 64)
gemm_splitk_kernel(const __half *__restrict__ a, const uint8_t *__restrict__ pw, const float *__restrict__ cb,
                   const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                   const float *__restrict__ bias, TOUT *__restrict__ y, int M, int N, int K,
                   const TOUT *residual, int gelu)
{
    constexpr int L = 1 << BITS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *lut = reinterpret_cast<float *>(smem);                              // [L][64], one copy per lane
    unsigned char *partial = smem + L * 64 * sizeof(float);                    // [NW][RT rows][kSkPitch]
    constexpr int RT = 32 * RB;
    constexpr int kSkTile = 32 * CB;
    constexpr int kSkPitch = kSkTile * 4 + 16;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int lh = lane >> 5;
    const int m0 = blockIdx.y * RT, n0 = blockIdx.x * kSkTile;
    const int G = K / 64;
    const int64_t pcols = static_cast<int64_t>(K) * BITS / 8;

    const __half *a_src[RB];
    const uint8_t *w_src[CB];
    const float *wc_src[CB], *ws_src[CB], *wcs_src[CB];
#pragma unroll
    for (int i = 0; i < RB; ++i) a_src[i] = a + static_cast<int64_t>(min(m0 + i * 32 + lr, M - 1)) * K + lh * 32;
#pragma unroll
    for (int i = 0; i < CB; ++i) {
        const int n = min(n0 + i * 32 + lr, N - 1);
        w_src[i] = pw + static_cast<int64_t>(n) * pcols + lh * (4 * BITS);
        wc_src[i] = wc + static_cast<int64_t>(n) * G;
        ws_src[i] = ws + static_cast<int64_t>(n) * G;
        wcs_src[i] = wcs + static_cast<int64_t>(n) * G;
    }
    auto fetch = [&](int g, SkOperands<BITS, RB, CB> &o) {
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) o.a[i][kk] = *reinterpret_cast<const u32x4_t *>(a_src[i] + g * 64 + kk * 8);
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            sk_load_codes<BITS>(w_src[i] + g * (8 * BITS), o.codes[i]);
            o.c[i] = wc_src[i][g];
            o.s[i] = ws_src[i][g];
            o.m[i] = wcs_src[i][g];
        }
    };

    SkOperands<BITS, RB, CB> o0, o1;
    if (wave < G) fetch(wave, o0);             // in flight while the codebook is staged
    if (tid < 64) {
#pragma unroll
        for (int c = 0; c < L; ++c) lut[c * 64 + lane] = cb[c];
    }
    __syncthreads();

    float16_t acc[RB][CB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const char *lut_lane = reinterpret_cast<const char *>(lut) + lane * 4;
    auto compute = [&](const SkOperands<BITS, RB, CB> &o) {
        float mg[CB];
#pragma unroll
        for (int j = 0; j < CB; ++j) mg[j] = o.m[j] * 0.015625f;       // S/64, exact
        float wv[CB][32];         // all table lookups are issued before the first is used
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int q = 0; q < 32; ++q)
                wv[j][q] = *reinterpret_cast<const float *>(lut_lane + (sk_code_at<BITS>(o.codes[j], q) << 8));
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            half8_t bf[CB];
#pragma unroll
            for (int j = 0; j < CB; ++j)
#pragma unroll
                for (int q = 0; q < 8; ++q)
                    bf[j][q] = static_cast<_Float16>(fma_f32(wv[j][kk * 8 + q] - mg[j], o.s[j], o.c[j]));
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                half8_t af;
                __builtin_memcpy(&af, &o.a[i][kk], 16);
#pragma unroll
                for (int j = 0; j < CB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af, acc[i][j], 0, 0, 0);
            }
        }
    };
    // The thread's outputs in the epilogue (E consecutive ones of a row) are known now: their bias and residual values
    // are requested here, so that the loads travel under the product instead of after it.
    constexpr int E = RT * kSkTile / (NW * 64);            // outputs per thread, consecutive in a row (8, 4 or 2)
    constexpr int TPR = kSkTile / E;                       // threads per row
    constexpr int BYTES = E * static_cast<int>(sizeof(TOUT));
    const int row = tid / TPR, col = (tid % TPR) * E;
    const int gr = m0 + row, gc = n0 + col;
    const bool vec_out = gr < M && gc + E <= N && (N % E) == 0 && BYTES % 4 == 0;
    float bv[E];
    TOUT rv[E];
#pragma unroll
    for (int e = 0; e < E; ++e) bv[e] = 0.0f, rv[e] = from_float<TOUT>(0.0f);
    if (vec_out) {
        if (bias) {
#pragma unroll
            for (int e = 0; e < E; ++e) bv[e] = bias[gc + e];
        }
        if (residual) {    // (N % E == 0 and a 16-byte aligned tensor: the E values are aligned 4-, 8- or 16-byte loads)
            const TOUT *rp = residual + static_cast<int64_t>(gr) * N + gc;
            if constexpr (BYTES % 16 == 0) {
#pragma unroll
                for (int b = 0; b < BYTES / 16; ++b) {
                    const u32x4_t v = reinterpret_cast<const u32x4_t *>(rp)[b];
                    __builtin_memcpy(reinterpret_cast<char *>(rv) + 16 * b, &v, 16);
                }
            } else if constexpr (BYTES == 8) {
                const u32x2_t v = *reinterpret_cast<const u32x2_t *>(rp);
                __builtin_memcpy(rv, &v, 8);
            } else {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(rp);
                __builtin_memcpy(rv, &v, 4);
            }
        }
    }
    // Groups of this wave, two per trip so that the operand sets alternate statically: the next group's loads are
    // issued before the current group is multiplied.  (A third set in flight measured slower: the loop is bound by
    // the address processing of its row-strided loads, not by their latency, and the extra registers cost more.)
    for (int g = wave; g < G; g += 2 * NW) {
        if (g + NW < G) fetch(g + NW, o1);
        compute(o0);
        if (g + NW < G) {
            if (g + 2 * NW < G) fetch(g + 2 * NW, o0);
            compute(o1);
        }
    }

    // ---- reduction over the waves, bias, output ----------------------------------------------------------
    unsigned char *mine = partial + wave * (RT * kSkPitch);
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4_t v;
                v[0] = acc[i][j][4 * q]; v[1] = acc[i][j][4 * q + 1]; v[2] = acc[i][j][4 * q + 2]; v[3] = acc[i][j][4 * q + 3];
                *reinterpret_cast<f32x4_t *>(mine + (i * 32 + lr) * kSkPitch + (j * 32 + 8 * q + 4 * lh) * 4) = v;
            }
    __syncthreads();
    float sum[E];
#pragma unroll
    for (int e = 0; e < E; ++e) sum[e] = 0.0f;
    const int waves_used = min(NW, G);                     // the others hold zeros; skipping them changes nothing
    for (int w = 0; w < waves_used; ++w) {
        const unsigned char *src = partial + w * (RT * kSkPitch) + row * kSkPitch + col * 4;
        if constexpr (E % 4 == 0) {
#pragma unroll
            for (int e = 0; e < E; e += 4) {
                const f32x4_t v = *reinterpret_cast<const f32x4_t *>(src + e * 4);
                sum[e] += v[0]; sum[e + 1] += v[1]; sum[e + 2] += v[2]; sum[e + 3] += v[3];
            }
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) sum[e] += *reinterpret_cast<const float *>(src + e * 4);
        }
    }
    if (gr < M && gc < N) {
        TOUT *dst = y + static_cast<int64_t>(gr) * N + gc;
        // Optional GELU / residual on the rounded output (post_op1): what separate elementwise kernels would store.
        const bool post = residual || gelu;
        if (vec_out) {
            TOUT out[E];
#pragma unroll
            for (int e = 0; e < E; ++e) out[e] = from_float<TOUT>(sum[e] + bv[e]);
            if (post) {
#pragma unroll
                for (int e = 0; e < E; ++e) out[e] = post_op1<TOUT>(out[e], residual != nullptr, rv[e], gelu != 0);
            }
            if constexpr (BYTES % 16 == 0) {
#pragma unroll
                for (int b = 0; b < BYTES; b += 16)
                    *reinterpret_cast<u32x4_t *>(reinterpret_cast<char *>(dst) + b) =
                        *reinterpret_cast<const u32x4_t *>(reinterpret_cast<const char *>(out) + b);
            } else if constexpr (BYTES == 8) {
                *reinterpret_cast<u32x2_t *>(dst) = *reinterpret_cast<const u32x2_t *>(out);
            } else {
                static_assert(BYTES == 4, "outputs per thread");
                *reinterpret_cast<uint32_t *>(dst) = *reinterpret_cast<const uint32_t *>(out);
            }
        } else {
            const TOUT *res = residual ? residual + static_cast<int64_t>(gr) * N + gc : nullptr;
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (gc + e < N) {
                    TOUT o = from_float<TOUT>(sum[e] + (bias ? bias[gc + e] : 0.0f));
                    if (post) o = post_op1<TOUT>(o, res != nullptr, res ? res[e] : o, gelu != 0);
                    dst[e] = o;
                }
        }
    }
}

template <int BITS, typename TOUT, int RB, int CB>
static void launch_splitk_rb(const GemmArgs &g, hipStream_t stream)
{
    constexpr int NW = 8;
    constexpr int L = 1 << BITS;
    constexpr int RT = 32 * RB;
    constexpr int kSkTile = 32 * CB;
    constexpr int kSkPitch = kSkTile * 4 + 16;
    const size_t smem = L * 64 * sizeof(float) + static_cast<size_t>(NW) * RT * kSkPitch;
    auto kernel = gemm_splitk_kernel<BITS, TOUT, NW, RB, CB>;
    allow_dynamic_lds<gemm_splitk_kernel<BITS, TOUT, NW, RB, CB>>(static_cast<int>(smem));
    const dim3 grid((g.N + kSkTile - 1) / kSkTile, (g.M + RT - 1) / RT);
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), smem, stream, static_cast<const __half *>(g.x_hat), g.pw, g.cb, g.wc,
                       g.ws, g.wcs, g.bias, static_cast<TOUT *>(g.y), g.M, g.N, g.K, static_cast<const TOUT *>(g.residual),
                       g.gelu ? 1 : 0);
}

template <int BITS, typename TOUT>
static void launch_splitk_t(const GemmArgs &g, hipStream_t stream)
{
    // 32-row tiles while the grid still fits the chip: more workgroups in flight and half the row-strided x_hat
    // loads per wave; 64-row tiles otherwise (the weights are then rebuilt half as often).
    // 32 x 32 tiles while the grid stays within about one and a half workgroups per CU: a wave then rebuilds 32 weight
    // rows per group instead of 64 and the chain a launch this small waits for is a third shorter (M = 197:
    // 384 x 1536 11.9 -> 8.0 us, 384 x 384 5.0 -> 3.8, 1024 x 1024 10.0 -> 6.9; 1536 x 384, 336 tiles, 5.2 -> 4.8;
    // equal at 504 tiles, slower beyond).  Same k order per output: bit-identical.
    const int64_t tiles32 = static_cast<int64_t>((g.N + 63) / 64) * ((g.M + 31) / 32);
    const int64_t tiles32x32 = static_cast<int64_t>((g.N + 31) / 32) * ((g.M + 31) / 32);
    if (tiles32x32 <= 400) launch_splitk_rb<BITS, TOUT, 1, 1>(g, stream);
    else if (tiles32 <= 256) launch_splitk_rb<BITS, TOUT, 1, 2>(g, stream);
    else launch_splitk_rb<BITS, TOUT, 2, 2>(g, stream);
}

void launch_gemm_splitk(const GemmArgs &g, hipStream_t stream)
{
    if (g.y_f16) {
        if (g.bits == 4) launch_splitk_t<4, __half>(g, stream);
        else if (g.bits == 3) launch_splitk_t<3, __half>(g, stream);
        else launch_splitk_t<2, __half>(g, stream);
    } else {
        if (g.bits == 4) launch_splitk_t<4, float>(g, stream);
        else if (g.bits == 3) launch_splitk_t<3, float>(g, stream);
        else launch_splitk_t<2, float>(g, stream);
    }
}

}  // namespace arcq
