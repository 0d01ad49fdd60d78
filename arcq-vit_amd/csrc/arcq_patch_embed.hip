// Front end of a ViT in one launch: the 16 x 16 stride-16 patch convolution as an MFMA product straight from the NCHW
// image (no im2col tensor), its bias, the class token in front and the position embedding added:
//
//   out[b, 0, :]     = cls + pos[0]
//   out[b, 1 + p, :] = fp16( fp16( patch(b, p) . w^T + bias ) + pos[1 + p] ),   p = py * (W / 16) + px
//
// img [B, 3, H, W] fp16, w [N, 3 * 16 * 16] fp16 (a Conv2d weight as it lies: k = c * 256 + i * 16 + j), bias / cls [N],
// pos [1 + (H/16)(W/16), N], out [B, 1 + (H/16)(W/16), N], all fp16.  fp32 accumulation; the two roundings are those of
// the separate convolution and addition it replaces.
//
// No counterpart in the reference's packed path (the fp16 patch embedding of its models is a torch convolution); here
// because with the blocks down to five launches each, torch's im2col + GEMM + concatenation + addition are the largest
// single item of a batch-1 forward.  The quantized patch convolution (ARCQPackedPatchConv) does not go through this.
//
// A k-step of 16 covers half of one 16-pixel image row of a patch: the eight values a lane needs of it are 16
// contiguous bytes of the image, so the fragments are plain 16-byte loads from the image (and from w, whose row is the
// patch in the same order).  Two kernels: patch_embed_kernel (workgroup = 256 patches x 32 channels, weight rows in LDS)
// and, up to 256 tiles of 32 x 32, patch_embed_small_kernel (a workgroup per tile, the k-steps split over its waves).
#include "arcq_common.h"

namespace arcq {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kPatch = 16, kChannels = 3, kK = kChannels * kPatch * kPatch, kSteps = kK / 16;      // 768, 48

// Workgroup = 256 patches (four waves of 64) x 32 channels.  The 32 weight rows (48 KB) are copied into LDS once, with
// coalesced loads, and every wave reads its weight fragments from there: straight from global memory a weight
// fragment touches 32 different cache lines per instruction (one row each), which costs the vector memory path a clock
// per line and bounded the launch; an image fragment is 1 KB in two or three contiguous runs and stays a global load.
constexpr int kTM = 2;                                  // 32-patch blocks per wave
constexpr int kWPitch = kK * 2 + 16;                    // bytes per weight row in LDS (odd number of 16-byte pieces)

__global__ void __launch_bounds__(256)
patch_embed_kernel(const __half *__restrict__ img, const __half *__restrict__ w, const __half *__restrict__ bias,
                   const __half *__restrict__ cls, const __half *__restrict__ pos, __half *__restrict__ out, int B, int H,
                   int W, int N, int row_groups, int col_tiles)
{
    __shared__ __attribute__((aligned(16))) unsigned char ws[32 * kWPitch];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int pw = W / kPatch, np = (H / kPatch) * pw;
    const int M = B * np;
    const int tiles = row_groups * col_tiles;
    if (static_cast<int>(blockIdx.x) >= tiles) {        // the class-token rows: element e = b * N + n
        const int64_t e0 = (static_cast<int64_t>(blockIdx.x - tiles) * 256 + tid) * 8;
        if (e0 < static_cast<int64_t>(B) * N) {
            const int b = static_cast<int>(e0 / N), n = static_cast<int>(e0 - static_cast<int64_t>(b) * N);
            __half *dst = out + static_cast<int64_t>(b) * (np + 1) * N + n;
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[i] = __float2half_rn(__half2float(cls[n + i]) + __half2float(pos[n + i]));
        }
        return;
    }
    const int rg = blockIdx.x / col_tiles, ct = blockIdx.x - rg * col_tiles;      // neighbours share the patches
    const int n0 = ct * 32;
    // ---- the weight rows n0 .. n0 + 31 into LDS: 3072 pieces of 16 bytes, twelve per thread, all in flight ----
    {
        constexpr int kPiecesPerRow = kK / 8;           // 96
        u32x4_t t[12];
#pragma unroll
        for (int j = 0; j < 12; ++j) {
            const int p = tid + 256 * j, row = p / kPiecesPerRow, col = p - row * kPiecesPerRow;
            t[j] = *reinterpret_cast<const u32x4_t *>(w + static_cast<int64_t>(n0 + row) * kK + col * 8);
        }
#pragma unroll
        for (int j = 0; j < 12; ++j) {
            const int p = tid + 256 * j, row = p / kPiecesPerRow, col = p - row * kPiecesPerRow;
            *reinterpret_cast<u32x4_t *>(ws + row * kWPitch + col * 16) = t[j];
        }
    }
    // per row block: this lane's patch, its first image row (channel 0, i = 0) at column 8 lh, its output row
    const __half *a_base[kTM];
    int64_t out_row[kTM];
    int pos_row[kTM];
    bool valid[kTM];
#pragma unroll
    for (int tm = 0; tm < kTM; ++tm) {
        const int m = ((rg * 4 + wave) * kTM + tm) * 32 + lr;
        const int mc = min(m, M - 1);
        const int b = mc / np, p = mc - b * np, py = p / pw, px = p - py * pw;
        a_base[tm] = img + (static_cast<int64_t>(b) * kChannels * H + py * kPatch) * W + px * kPatch + 8 * lh;
        out_row[tm] = static_cast<int64_t>(b) * (np + 1) + 1 + p;
        pos_row[tm] = 1 + p;
        valid[tm] = m < M;
    }
    const int64_t plane = static_cast<int64_t>(H) * W;
    auto load_step = [&](int s, u32x4_t (&af)[kTM]) {
        const int c = s >> 4, i = s & 15;
        const int64_t a_off = c * plane + static_cast<int64_t>(i) * W;
#pragma unroll
        for (int tm = 0; tm < kTM; ++tm) af[tm] = *reinterpret_cast<const u32x4_t *>(a_base[tm] + a_off);
    };
    float16_t acc[kTM];
#pragma unroll
    for (int tm = 0; tm < kTM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tm][v] = 0.0f;
    constexpr int kAhead = 8;                  // k-steps of image fragments in flight
    u32x4_t af[kAhead][kTM];
#pragma unroll
    for (int s = 0; s < kAhead - 1; ++s) load_step(s, af[s]);
    __syncthreads();                           // the weight rows are in LDS
    const unsigned char *w_lane = ws + lr * kWPitch + lh * 16;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        if (s + kAhead - 1 < kSteps) load_step(s + kAhead - 1, af[(s + kAhead - 1) % kAhead]);
        const half8_t wb = *reinterpret_cast<const half8_t *>(w_lane + s * 32);
        __builtin_amdgcn_sched_barrier(0);     // (left alone, the compiler sinks the loads towards their use)
#pragma unroll
        for (int tm = 0; tm < kTM; ++tm) {
            half8_t xa;
            __builtin_memcpy(&xa, &af[s % kAhead][tm], 16);
            acc[tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wb, xa, acc[tm], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    // acc[tm][v]: patch lr of row block tm, channel n0 + 8 (v / 4) + 4 lh + v % 4
#pragma unroll
    for (int tm = 0; tm < kTM; ++tm) {
        if (!valid[tm]) continue;
        __half *dst = out + out_row[tm] * N;
        const __half *ps = pos + static_cast<int64_t>(pos_row[tm]) * N;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = n0 + 8 * q + 4 * lh;
            const u32x2_t pv = *reinterpret_cast<const u32x2_t *>(ps + n);
            u32x2_t bv = {0u, 0u};
            if (bias) bv = *reinterpret_cast<const u32x2_t *>(bias + n);
            const __half *ph = reinterpret_cast<const __half *>(&pv), *bh = reinterpret_cast<const __half *>(&bv);
            __half o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const __half y = __float2half_rn(acc[tm][4 * q + e] + __half2float(bh[e]));
                o[e] = __float2half_rn(__half2float(y) + __half2float(ph[e]));
            }
            *reinterpret_cast<u32x2_t *>(dst + n) = *reinterpret_cast<const u32x2_t *>(o);
        }
    }
}

// The same for few patches (batch 1-2): one 32 x 32 tile per workgroup, its 48 k-steps dealt to the four waves (twelve
// each, all 24 fragment loads of a wave in flight at once: the launch is one memory latency, twelve MFMAs and a
// reduction of the four partial tiles through LDS, in wave order).
__global__ void __launch_bounds__(256)
patch_embed_small_kernel(const __half *__restrict__ img, const __half *__restrict__ w, const __half *__restrict__ bias,
                         const __half *__restrict__ cls, const __half *__restrict__ pos, __half *__restrict__ out, int B,
                         int H, int W, int N, int row_tiles, int col_tiles)
{
    __shared__ float part[3][16][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int pw = W / kPatch, np = (H / kPatch) * pw;
    const int M = B * np;
    const int tile = blockIdx.x, tiles = row_tiles * col_tiles;
    if (tile >= tiles) {        // the class-token rows: element e = b * N + n
        const int64_t e0 = (static_cast<int64_t>(tile - tiles) * 256 + tid) * 8;
        if (e0 < static_cast<int64_t>(B) * N) {
            const int b = static_cast<int>(e0 / N), n = static_cast<int>(e0 - static_cast<int64_t>(b) * N);
            __half *dst = out + static_cast<int64_t>(b) * (np + 1) * N + n;
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[i] = __float2half_rn(__half2float(cls[n + i]) + __half2float(pos[n + i]));
        }
        return;
    }
    const int rt = tile / col_tiles, ct = tile - rt * col_tiles;
    const int m = rt * 32 + lr, mc = min(m, M - 1);
    const int b = mc / np, p = mc - b * np, py = p / pw, px = p - py * pw;
    const __half *a_base = img + (static_cast<int64_t>(b) * kChannels * H + py * kPatch) * W + px * kPatch + 8 * lh;
    const __half *w_base = w + static_cast<int64_t>(min(ct * 32 + lr, N - 1)) * kK + 8 * lh;
    const int64_t plane = static_cast<int64_t>(H) * W;
    constexpr int kMine = kSteps / 4;          // 12 k-steps per wave
    u32x4_t af[kMine], bf[kMine];
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
        const int s = wave * kMine + j, c = s >> 4, i = s & 15;
        af[j] = *reinterpret_cast<const u32x4_t *>(a_base + c * plane + static_cast<int64_t>(i) * W);
        bf[j] = *reinterpret_cast<const u32x4_t *>(w_base + s * 16);
    }
    __builtin_amdgcn_sched_barrier(0);         // every load is issued before the first wait
    float16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
        half8_t xa, wb;
        __builtin_memcpy(&xa, &af[j], 16);
        __builtin_memcpy(&wb, &bf[j], 16);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(wb, xa, acc, 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) part[wave - 1][v][lane] = acc[v];
    }
    __syncthreads();
    if (wave > 0 || m >= M) return;
#pragma unroll
    for (int q = 0; q < 3; ++q)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] += part[q][v][lane];
    __half *dst = out + (static_cast<int64_t>(b) * (np + 1) + 1 + p) * N;
    const __half *ps = pos + static_cast<int64_t>(1 + p) * N;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int n = ct * 32 + 8 * q + 4 * lh;
        const u32x2_t pv = *reinterpret_cast<const u32x2_t *>(ps + n);
        u32x2_t bv = {0u, 0u};
        if (bias) bv = *reinterpret_cast<const u32x2_t *>(bias + n);
        const __half *ph = reinterpret_cast<const __half *>(&pv), *bh = reinterpret_cast<const __half *>(&bv);
        __half o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const __half y = __float2half_rn(acc[4 * q + e] + __half2float(bh[e]));
            o[e] = __float2half_rn(__half2float(y) + __half2float(ph[e]));
        }
        *reinterpret_cast<u32x2_t *>(dst + n) = *reinterpret_cast<const u32x2_t *>(o);
    }
}

}  // namespace
}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_patch_embed_fwd(const void *img, const void *w, const void *bias, const void *cls, const void *pos, void *out,
                                  int64_t B, int64_t H, int64_t W, int64_t patch, int64_t N, void *stream)
{
    if (B < 0 || H < 0 || W < 0 || N < 0) return fail(ARCQ_ERR_SHAPE, "arcq_patch_embed_fwd: negative size");
    if (patch != kPatch) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_patch_embed_fwd: patch size must be 16 (got %lld)", static_cast<long long>(patch));
    if (H % kPatch || W % kPatch) return fail(ARCQ_ERR_SHAPE, "arcq_patch_embed_fwd: image sides must be multiples of 16");
    if (N % 32) return fail(ARCQ_ERR_UNSUPPORTED, "arcq_patch_embed_fwd: embedding width must be a multiple of 32 (got %lld)", static_cast<long long>(N));
    if (B == 0 || N == 0) return ARCQ_OK;
    if (H == 0 || W == 0) return fail(ARCQ_ERR_SHAPE, "arcq_patch_embed_fwd: empty image");
    if (!img || !w || !cls || !pos || !out) return fail(ARCQ_ERR_NULL, "arcq_patch_embed_fwd: NULL tensor pointer");
    if (!aligned(img, 16) || !aligned(w, 16) || !aligned(out, 8) || !aligned(pos, 8) || (bias && !aligned(bias, 8)))
        return fail(ARCQ_ERR_ALIGN, "arcq_patch_embed_fwd: img and w must be 16-byte, bias / pos / out 8-byte aligned");
    const int64_t M = B * (H / kPatch) * (W / kPatch);
    if (B > (1 << 20) || H > (1 << 14) || W > (1 << 14) || N > (1 << 16) || M >= (int64_t(1) << 30) || (M + B) * N >= (int64_t(1) << 40))
        return fail(ARCQ_ERR_SHAPE, "arcq_patch_embed_fwd: tensor too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int b = static_cast<int>(B), h = static_cast<int>(H), wd = static_cast<int>(W), n = static_cast<int>(N);
    const auto *pi = static_cast<const __half *>(img), *pwt = static_cast<const __half *>(w), *pb = static_cast<const __half *>(bias);
    const auto *pc = static_cast<const __half *>(cls), *pp = static_cast<const __half *>(pos);
    auto *po = static_cast<__half *>(out);
    const int cls_wgs = static_cast<int>((B * N / 8 + 255) / 256);
    const int col_tiles = n / 32;
    if (((M + 31) / 32) * col_tiles <= 256) {
        const int row_tiles = static_cast<int>((M + 31) / 32);
        hipLaunchKernelGGL(patch_embed_small_kernel, dim3(row_tiles * col_tiles + cls_wgs), dim3(256), 0, st, pi, pwt, pb, pc, pp, po,
                           b, h, wd, n, row_tiles, col_tiles);
    } else {
        const int row_groups = static_cast<int>((M + 128 * kTM - 1) / (128 * kTM));      // four waves of 32 kTM patches
        hipLaunchKernelGGL(patch_embed_kernel, dim3(row_groups * col_tiles + cls_wgs), dim3(256), 0, st, pi, pwt, pb, pc, pp, po, b, h, wd,
                           n, row_groups, col_tiles);
    }
    return launch_status("arcq_patch_embed_fwd");
}
