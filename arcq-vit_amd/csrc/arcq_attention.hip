// Softmax attention of a ViT block, placed between the packed qkv and proj layers so that neither needs a reshaping
// kernel around it: it reads the qkv layer's output as it is and writes the proj layer's input as it is.
//
//   qkv [B, n, 3, H, 64] fp16  (= the qkv layer's y, [B*n, 3*H*64] row-major: q, k, v of head h at columns
//                               (0|1|2)*H*64 + h*64 ...)
//   out [B, n, H*64]     fp16  (= the proj layer's x):  out[b, i, h*64 + j] = sum_k softmax_k(q_i . k_k * scale) v_k[j]
//
// No counterpart in the reference's packed path (its models run timm's attention through torch); part of the
// whole-block fusion around the packed linears: at batch 1 the library attention plus the two copies that reshape
// its operands take as long as two packed layers.
//
// One workgroup per (batch, head); wave w owns the 32 queries 32 w ... (n <= 256 tokens: at most eight waves).  K of
// the head sits in LDS row-major, V transposed, both zero-padded to whole 32-key blocks.  Scores: S^T = K Q^T on
// v_mfma_f32_32x32x16_f16 with K as the first operand, so that a lane (query q = lane % 32, half h = lane / 32) ends
// up holding, of every 32-key block, the 16 keys 8 t + 4 h + c (t, c = 0..3) of its own query: the row maximum and sum
// are in-lane reductions plus one exchange with lane ^ 32, and -- since the contraction index of the second product
// may be enumerated in any order as long as both operands use the same one -- eight consecutive accumulator registers,
// rounded to fp16, ARE the second operand of O^T = V^T P^T for the keys {16 s + 4 h + c, 16 s + 8 + 4 h + c}; the
// matching eight values of V^T are two 8-byte LDS reads.  fp32 scores, softmax and accumulation; P rounded to fp16;
// normalisation by the row sum at the end.  Beyond 128 keys the keys go in two chunks with a running maximum and sum.
#include "arcq_common.h"

namespace arcq {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kHeadDim = 64;
constexpr int kKPitch = kHeadDim * 2 + 16;          // bytes per key row of K in LDS

template <int NKB>      // 32-key blocks (= 32-query tiles = waves): ceil(n / 32)
__global__ void __launch_bounds__(64 * NKB) __attribute__((amdgpu_waves_per_eu(4)))     // two workgroups of up to 8 waves on a CU
attention_kernel(const __half *__restrict__ qkv, __half *__restrict__ out, int n, int H, float scale)
{
    constexpr int kKeys = 32 * NKB;
    // bytes per dim row of V^T in LDS: the row stride in dwords is 2 mod 4, which spreads both the transposing writes
    // (rows 8 apart, 4-byte) and the product's reads (32 consecutive rows, 8-byte) over the banks
    constexpr int kVPitch = kKeys * 2 + 8;
    constexpr int CH = NKB <= 4 ? 4 : NKB == 6 ? 2 : 3;   // key blocks whose scores are live at a time (no spills at 128 registers)
    constexpr int NCH = (NKB + CH - 1) / CH;
    __shared__ __attribute__((aligned(16))) unsigned char ks[kKeys * kKPitch];
    __shared__ __attribute__((aligned(16))) unsigned char vt[kHeadDim * kVPitch];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int h = blockIdx.x, b = blockIdx.y;
    const int C = H * kHeadDim;
    const int64_t row0 = static_cast<int64_t>(b) * n;           // first token row of this image
    const __half *base = qkv + h * kHeadDim;                    // + (row * 3 + which) * C

    // ---- K row-major and V transposed into LDS (keys past n as zeros).  16 NKB key pairs x 8 pieces of 8 dims =
    //      exactly two items per thread; all eight loads are in flight before the first LDS write ----
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    u32x4_t kreg[2][2], vreg[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int p = tid + i * 64 * NKB, kp = p >> 3, piece = p & 7;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int key = 2 * kp + j;
            const __half *src = base + ((row0 + min(key, n - 1)) * 3 + 1) * C + piece * 8;
            kreg[i][j] = key < n ? *reinterpret_cast<const u32x4_t *>(src) : zero4;
            vreg[i][j] = key < n ? *reinterpret_cast<const u32x4_t *>(src + C) : zero4;
        }
    }
    // ---- this wave's queries: lane (q, half) holds Q[q][16 kk + 8 half ... + 7] for kk = 0..3 ----
    const int q = wave * 32 + lr;
    u32x4_t qf[4];
    {
        const __half *src = base + (row0 + min(q, n - 1)) * 3 * C + 8 * lh;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) qf[kk] = q < n ? *reinterpret_cast<const u32x4_t *>(src + 16 * kk) : zero4;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int p = tid + i * 64 * NKB, kp = p >> 3, piece = p & 7;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            *reinterpret_cast<u32x4_t *>(ks + (2 * kp + j) * kKPitch + piece * 16) = kreg[i][j];
#pragma unroll
        for (int e = 0; e < 8; ++e) {       // dim piece*8 + e of the two keys as one dword
            const uint32_t a = vreg[i][0][e >> 1], c = vreg[i][1][e >> 1];
            const uint32_t pair = (e & 1) ? ((a >> 16) | (c & 0xffff0000u)) : ((a & 0xffffu) | (c << 16));
            *reinterpret_cast<uint32_t *>(vt + (piece * 8 + e) * kVPitch + kp * 4) = pair;
        }
    }
    __syncthreads();

    // Keys in chunks of CH blocks with a running maximum and sum (the scores of one chunk are live at a time, which
    // keeps the wave at half the registers and two workgroups on a CU); one chunk is the plain two-pass softmax.
    const float ninf = -__builtin_inff();
    const float c2 = scale * 1.44269504088896341f;      // exp(scale x) = exp2(c2 x)
    float m = ninf, l = 0.0f;
    float16_t oacc[2];      // oacc[jb][v]: dim jb*32 + 8 (v / 4) + 4 lh + v % 4 of this lane's query
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[jb][v] = 0.0f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
        constexpr int kLast = NKB - CH * (NCH - 1);
        const int nb = ch == NCH - 1 ? kLast : CH;          // constant after unrolling
        if (ch > 0) __builtin_amdgcn_sched_barrier(0);      // keep the next chunk's scores out of this one's live range
        // ---- scores: acc[i][v] = q . k for key (ch*CH + i)*32 + 8 (v / 4) + 4 lh + v % 4 ----
        float16_t acc[CH];
        float cm = ninf;
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if (i >= nb) continue;
            const int kb = ch * CH + i;
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const half8_t kf = *reinterpret_cast<const half8_t *>(ks + (kb * 32 + lr) * kKPitch + (16 * kk + 8 * lh) * 2);
                half8_t qv;
                __builtin_memcpy(&qv, &qf[kk], 16);
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qv, acc[i], 0, 0, 0);
            }
            // (raw scores: the scale is positive, so it commutes with the maximum and is applied inside the exponential;
            // only the last key block can hold keys past n)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                if (kb == NKB - 1) {
                    const int key = kb * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                    acc[i][v] = key < n ? acc[i][v] : ninf;
                }
                cm = fmaxf(cm, acc[i][v]);
            }
        }
        cm = fmaxf(cm, __shfl_xor(cm, 32));
        const float m_new = fmaxf(m, cm);       // finite: every chunk holds at least one key < n
        if (ch > 0) {                           // rescale what the earlier chunks left (exp(-inf) never occurs here)
            const float alpha = __builtin_amdgcn_exp2f((m - m_new) * c2);
            l *= alpha;
#pragma unroll
            for (int jb = 0; jb < 2; ++jb)
#pragma unroll
                for (int v = 0; v < 16; ++v) oacc[jb][v] *= alpha;
        }
        m = m_new;
        const float mc = -m * c2;
        // ---- probabilities (this lane's share of the row sum; the two halves are added at the end) and O^T += V^T P^T ----
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if (i >= nb) continue;
            const int kb = ch * CH + i;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[i][v], c2, mc));      // exp(scale (s - m))
                acc[i][v] = p;
                l += p;
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                half8_t pf;
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = static_cast<_Float16>(acc[i][8 * s + e]);
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    const unsigned char *vrow = vt + (jb * 32 + lr) * kVPitch + (kb * 32 + 16 * s + 4 * lh) * 2;
                    const u32x2_t lo = *reinterpret_cast<const u32x2_t *>(vrow);
                    const u32x2_t hi = *reinterpret_cast<const u32x2_t *>(vrow + 16);
                    half8_t vf;
                    __builtin_memcpy(&vf, &lo, 8);
                    __builtin_memcpy(reinterpret_cast<char *>(&vf) + 8, &hi, 8);
                    oacc[jb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, oacc[jb], 0, 0, 0);
                }
            }
        }
    }
    l += __shfl_xor(l, 32);
    // ---- normalise, round, store: each lane 4 runs of 4 consecutive dims per 32-dim block ----
    if (q < n) {
        const float inv = 1.0f / l;
        __half *dst = out + (row0 + q) * C + h * kHeadDim;
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const __half2 a = __floats2half2_rn(oacc[jb][4 * t] * inv, oacc[jb][4 * t + 1] * inv);
                const __half2 c = __floats2half2_rn(oacc[jb][4 * t + 2] * inv, oacc[jb][4 * t + 3] * inv);
                u32x2_t pk;
                pk[0] = *reinterpret_cast<const uint32_t *>(&a);
                pk[1] = *reinterpret_cast<const uint32_t *>(&c);
                *reinterpret_cast<u32x2_t *>(dst + jb * 32 + 8 * t + 4 * lh) = pk;
            }
    }
}

template <int NKB>
void launch_attention(const void *qkv, void *out, int B, int n, int H, float scale, hipStream_t stream)
{
    hipLaunchKernelGGL((attention_kernel<NKB>), dim3(H, B), dim3(64 * NKB), 0, stream, static_cast<const __half *>(qkv),
                       static_cast<__half *>(out), n, H, scale);
}

}  // namespace
}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_attention_fwd(const void *qkv, void *out, int64_t B, int64_t n, int64_t H, int64_t head_dim, float scale,
                                void *stream)
{
    if (B < 0 || n < 0 || H < 0) return fail(ARCQ_ERR_SHAPE, "arcq_attention_fwd: negative size");
    if (!(scale > 0.0f)) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_attention_fwd: scale must be positive");
    if (head_dim != kHeadDim) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_attention_fwd: head_dim must be 64 (got %lld)", static_cast<long long>(head_dim));
    if (n > 256) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_attention_fwd: at most 256 tokens (got %lld)", static_cast<long long>(n));
    if (B * n * H == 0) return ARCQ_OK;
    if (!qkv || !out) return fail(ARCQ_ERR_NULL, "arcq_attention_fwd: NULL tensor pointer");
    if (!aligned(qkv, 16) || !aligned(out, 8)) return fail(ARCQ_ERR_ALIGN, "arcq_attention_fwd: qkv must be 16-byte, out 8-byte aligned");
    if (B > 65535 || H > (1 << 20) || B * n * 3 * H * head_dim >= (int64_t(1) << 40))
        return fail(ARCQ_ERR_SHAPE, "arcq_attention_fwd: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int b = static_cast<int>(B), nn = static_cast<int>(n), hh = static_cast<int>(H);
    switch ((nn + 31) / 32) {
    case 1: launch_attention<1>(qkv, out, b, nn, hh, scale, st); break;
    case 2: launch_attention<2>(qkv, out, b, nn, hh, scale, st); break;
    case 3: launch_attention<3>(qkv, out, b, nn, hh, scale, st); break;
    case 4: launch_attention<4>(qkv, out, b, nn, hh, scale, st); break;
    case 5: launch_attention<5>(qkv, out, b, nn, hh, scale, st); break;
    case 6: launch_attention<6>(qkv, out, b, nn, hh, scale, st); break;
    case 7: launch_attention<7>(qkv, out, b, nn, hh, scale, st); break;
    default: launch_attention<8>(qkv, out, b, nn, hh, scale, st); break;
    }
    return launch_status("arcq_attention_fwd");
}
