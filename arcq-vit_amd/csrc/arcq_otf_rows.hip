// Whole on-the-fly layer in ONE launch for many rows of moderate length: a workgroup owns 64 rows of x, quantizes
// them into LDS (stage 1, optionally with the LayerNorm in front of it) and multiplies them with every column of
// w_hat, which streams through the registers from a 32-column block layout in the weight workspace.  Two kernels:
// otf_rows_kernel (K = 192 / 256 / 384: the whole row at once; also K = 768 with fp16 outputs, twelve waves that
// quantize two tiles each and a 97 KB x_hat tile) and otf_rows_phased_kernel (K = 768 / 1536 with at most 384 output
// columns, K = 3072 with at most 768: the row in slices of 384 or 256 values, stage 1 of a slice under the MFMAs of the
// one before).
//
//   y[M,N] = post( stage1( [LayerNorm] x )[M,K] * w_hat[N,K]^T + bias )
//
// Why a second design beside the weight-stationary kernels: with K = 384 a launch of those does 4-20 us of work per
// CU, and the fixed costs of two launches (launch ramp, first loads, the x_hat round trip through L2, the drain)
// are a third of the layer.  Here x_hat never leaves the CU (64 rows x K fp16 = 48 KB of LDS at K = 384), stage 1
// runs on all twelve waves at once (wave = 32 rows x one group, two lanes per group), and the product starts the
// moment the workgroup's own rows are done.  The price is that every workgroup reads all of w_hat from L2
// (N*K*2 bytes, 0.9 MB for DeiT-S qkv) -- affordable only while N*K is small -- and that the launch must not have
// more workgroups than the device holds at once (see resident_workgroups below).
//
// Weights: w_hat is rebuilt from the packed codes inside the same launch, cooperatively: every workgroup
// reconstructs 1/gridDim of it into the workspace (16-byte pieces, written through to memory), adds to a counter,
// does its stage 1, and then waits for the counter to show that all shares have been written.  While the row tiles
// leave compute units free, otf_rows_kernel's launch carries extra workgroups that do nothing but this
// reconstruction, and the row workgroups only count (a quarter off the layer at 1 024 rows, nothing at 12 608).
// The wait is bounded:
// a workgroup that has not seen the others finish within half a millisecond (they may not be resident) rebuilds
// the whole matrix itself -- same values, so a share written twice is harmless -- and goes on.  No workgroup ever
// waits before it has contributed its share, so the counter always completes.
//
// Layout of the weight workspace: [N/32][K/8][32 columns][8 values] fp16 -- the MFMA fragment of a 32-column block
// and k-step (lane = column, 8 consecutive k) is one 16-byte load per lane, 512 contiguous bytes per half wave.
// Accumulation order per output (groups ascending, four k-steps of 16 per group, fp32) is that of the
// weight-stationary kernels, so y is bit-identical to theirs.
#include "arcq_common.h"
#include "arcq_gemm.h"
#include "arcq_act_quant_core.h"

#include <mutex>
#include <vector>

namespace arcq {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWaveLds = 4608;               // bytes of LDS per wave: the output staging tile (32 rows of 128 + 16 bytes)
// otf_rows_kernel's staging tile: kWaveLds, or, where a wave quantizes two tiles (K = 768: LDS is short), just the
// 32 rows of 32 outputs + 16 bytes that the epilogue uses.
constexpr int rows_stage_bytes(int rounds, size_t out_size) { return rounds == 1 ? kWaveLds : 32 * (32 * static_cast<int>(out_size) + 16); }
constexpr unsigned long long kEpoch = 1ull << 20;     // what one launch adds to its counter, whatever its grid

constexpr int gcd_of(int a, int b) { return b == 0 ? a : gcd_of(b, a % b); }

struct RowsParams {
    const __half *x;                 // [M,K] fp16
    const float *thr, *cb_a;         // activation thresholds / codebook
    float eps;
    const float *gamma, *beta;       // LayerNorm weight / bias (fp32), gamma == nullptr: no LayerNorm
    float ln_eps;
    const uint8_t *pw;               // packed weight codes [N, K*bits/8]
    const float *cb_w, *wc, *ws, *wcs;
    __half *w_blk;                   // weight workspace, block layout
    unsigned long long *counter;     // nullptr: w_blk is complete already
    long long wait_ticks;            // bound of the wait for the other workgroups' shares, ticks of the 100 MHz clock
    unsigned long long *timeouts;    // counts the workgroups whose wait ran out (a diagnostic: arcq_rows_wait_timeouts)
    const float *bias;               // [N] or nullptr
    void *y;
    const void *residual;
    int gelu;
    int M, N, G;
};

// Piece idx of the block-layout w_hat, idx = ((n / 32) * (K / 8) + k / 8) * 32 + n % 32, holds w_hat[n][k .. k + 8):
// value (cb[code] - code_sum/64) * scale + center with one fma (FQ/arcq_packed_triton.py:59-74), stored at
// out + 8 idx, written through to memory.  In two steps so that the loads of the first can travel under other work.
struct Piece {
    uint32_t w;
    float c, s, m;
};
template <int BITS, int G>
__device__ __forceinline__ void fetch_piece(const RowsParams &p, int64_t idx, Piece &pc)
{
    constexpr int K = 64 * G, P = K / 8, pcols = K * BITS / 8;     // compile-time: the divisions below are multiplications
    const uint32_t i = static_cast<uint32_t>(idx);                 // N * K / 8 < 2^31 (N <= 16384, K <= 384)
    const uint32_t r = i & 31u;
    const uint32_t t = i >> 5;
    const uint32_t nb = t / P;
    const uint32_t pp = t - nb * P;
    const uint32_t n = nb * 32u + r;
    pc.w = load_codes8<BITS>(p.pw + n * pcols + pp * BITS);
    const uint32_t mi = n * G + (pp >> 3);
    pc.c = p.wc[mi];
    pc.s = p.ws[mi];
    pc.m = p.wcs[mi] * 0.015625f;      // code_sum / 64, exact
}
template <int BITS>
__device__ __forceinline__ void finish_piece(const RowsParams &p, int64_t idx, const Piece &pc)
{
    constexpr int L = 1 << BITS;
    float cbv[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) cbv[q] = p.cb_w[(pc.w >> (BITS * q)) & (L - 1)];      // 64 bytes, cached
    uint32_t out[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const __half2 h = __floats2half2_rn(fma_f32(cbv[2 * q] - pc.m, pc.s, pc.c), fma_f32(cbv[2 * q + 1] - pc.m, pc.s, pc.c));
        out[q] = *reinterpret_cast<const uint32_t *>(&h);
    }
    store_writethrough16(p.w_blk + idx * 8, out[0], out[1], out[2], out[3]);
}

// G = K / 64 groups per row (the workgroup has 2 G waves); RING = groups of w_hat fragments a wave holds (the one
// being multiplied and RING - 1 on their way from L2); AHEAD = k-steps by which the LDS reads of the x_hat fragments
// run ahead of the MFMAs that use them.
// WV = waves per workgroup: 2 G (every wave one stage-1 tile) or, for K = 768, G (two tiles per wave, one after the
// other: sixteen waves are the most a workgroup can have).
template <int BITS, typename TOUT, int G, int RING, int AHEAD, int WV = 2 * G>
__global__ void __launch_bounds__(64 * WV)
otf_rows_kernel(const RowsParams p)
{
    constexpr int L = 1 << BITS;
    constexpr int MAXW = WV;
    constexpr int ROUNDS = 2 * G / WV;                              // stage-1 tiles per wave
    static_assert(ROUNDS * WV == 2 * G, "waves must divide the 2 G stage-1 tiles");
    constexpr int kStage = rows_stage_bytes(ROUNDS, sizeof(TOUT));  // bytes of a wave's output staging tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[MAXW];
    __shared__ int s_flag;

    constexpr int K = 64 * G, W = WV;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int nthreads = 64 * W;
    constexpr int pitch = K * 2 + 16;                               // bytes per x_hat row in LDS (conflict-free 16-byte reads)
    unsigned char *xs = smem;                                   // [64][pitch]
    unsigned char *wave_lds = smem + 64 * pitch + wave * kStage;
    float *part = reinterpret_cast<float *>(smem + 64 * pitch + W * kStage);        // [64][2 G + 1]
    float *s_bias = part + 64 * (2 * G + 1);                    // [N]
    const int64_t row_base = static_cast<int64_t>(blockIdx.x) * 64;
    const int64_t pieces = static_cast<int64_t>(p.N) * (K / 8);

    // The wave's stage-1 inputs (wave = (row block rb2, group g): 32 rows x 64 values; a lane pair holds one row's 64,
    // each lane 64 contiguous bytes) are requested first, so that they travel while the weights are rebuilt.
    // (tile t = wave + round * W: row block t / G, group t % G)
    uint4 raws[ROUNDS][4];
#pragma unroll
    for (int rnd = 0; rnd < ROUNDS; ++rnd) {
        // Rows past the tensor's end re-read its last row (their outputs are never stored).  Unconditional loads on
        // purpose: with a per-lane condition around them the compiler waits for the first load before it issues the next.
        const int t = wave + rnd * W, rb2 = t / G, g = t - rb2 * G;
        const int64_t r0 = min(row_base + rb2 * 32 + (lane >> 1), static_cast<int64_t>(p.M) - 1);
        const __half *src = p.x + r0 * K + g * 64 + (lane & 1) * 32;
#pragma unroll
        for (int i = 0; i < 4; ++i) raws[rnd][i] = *reinterpret_cast<const uint4 *>(src + i * 8);
    }

    // ---- this workgroup's share of w_hat: the inputs of this thread's first piece are requested here, the piece is
    // finished under stage 1's set-up ----
    // Division of the extra work over the waves (stage 1 is instruction-bound and waves w, w + 4, w + 8 share a SIMD):
    // waves 1-3 build the activation lookup tables, the others reconstruct the weight pieces -- wave 0 and waves 4..
    // are piece threads 0..63, 64.. -- so that no SIMD carries more than one builder and one piece wave beside
    // its plain ones (two piece waves on SIMD 0).
    constexpr int kBuilders = W < 4 ? 1 : 3;
    constexpr int kBuilder0 = W < 4 ? 0 : 1;
    constexpr int kPieceThreads = W < 4 ? 64 * W : 64 * (W - 3);
    const int ptid = W < 4 ? tid : (wave == 0 ? lane : (wave >= 4 ? (wave - 3) * 64 + lane : -1));
    int64_t share_lo = 0, share_hi = 0;
    Piece pc{};
    unsigned long long target = 0;
    // Workgroups beyond the row tiles are helpers (the launcher adds them while compute units are free): they
    // reconstruct all of w_hat between them, count, and are done; the row workgroups then only count.
    const int row_wgs = (p.M + 63) / 64;
    const int helpers = static_cast<int>(gridDim.x) - row_wgs;
    if (static_cast<int>(blockIdx.x) >= row_wgs) {
        int64_t per = (pieces + helpers - 1) / helpers;
        per = (per + 7) & ~int64_t(7);
        const int64_t lo = (static_cast<int>(blockIdx.x) - row_wgs) * per;
        const int64_t hi = lo + per < pieces ? lo + per : pieces;
        for (int64_t idx = lo + tid; idx < hi; idx += nthreads) {
            fetch_piece<BITS, G>(p, idx, pc);
            finish_piece<BITS>(p, idx, pc);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) __hip_atomic_fetch_add(p.counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    const bool own_share = p.counter && helpers == 0;
    if (own_share) {
        int64_t per = (pieces + gridDim.x - 1) / gridDim.x;
        per = (per + 7) & ~int64_t(7);                          // whole 128-byte lines per workgroup
        share_lo = blockIdx.x * per;
        share_hi = share_lo + per < pieces ? share_lo + per : pieces;
        if (ptid >= 0 && share_lo + ptid < share_hi) fetch_piece<BITS, G>(p, share_lo + ptid, pc);
    }

    // ---- stage 1: wave = (row block rb2, group g), two lanes per (row, group) ----
    for (int i = tid; i < p.N; i += nthreads) s_bias[i] = p.bias ? p.bias[i] : 0.0f;
    {
        float th[L - 1], cbv[L];
        load_quant_params<BITS>(p.thr, p.cb_a, th, cbv);
        const BucketScale bq = pick_bucket_scale<BITS>(th);
        // The lookup tables are built by three waves while the tiles are on their way (every participating thread
        // pays ~250 instructions of set-up whether or not it owns a table entry: all 2 G waves building cost 17 % of
        // the phase).
        if (wave >= kBuilder0 && wave < kBuilder0 + kBuilders)
            build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid - 64 * kBuilder0, 64 * kBuilders);
        if (own_share) {
            if (ptid >= 0 && share_lo + ptid < share_hi) finish_piece<BITS>(p, share_lo + ptid, pc);
            for (int64_t idx = share_lo + kPieceThreads + ptid; ptid >= 0 && idx < share_hi; idx += kPieceThreads) {     // (large N*K only)
                fetch_piece<BITS, G>(p, idx, pc);
                finish_piece<BITS>(p, idx, pc);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the written-through pieces have reached memory
        }
        const int row = lane >> 1, half = lane & 1;
        __syncthreads();                          // the tables are complete, and so is the workgroup's share of w_hat
        if (p.counter && tid == 0) {
            const unsigned long long inc = blockIdx.x == 0 ? kEpoch - (gridDim.x - 1) : 1ull;
            const unsigned long long old = __hip_atomic_fetch_add(p.counter, inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            target = (old & ~(kEpoch - 1)) + kEpoch;            // every launch adds kEpoch in total
        }
#pragma unroll
      for (int rnd = 0; rnd < ROUNDS; ++rnd) {
        const int tile = wave + rnd * W, rb2 = tile / G, g = tile - rb2 * G;
        const uint4 (&raw)[4] = raws[rnd];
        float xv[32];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w4[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                xv[8 * i + 2 * e] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] & 0xffffu)));
                xv[8 * i + 2 * e + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] >> 16)));
            }
        }
        if (p.gamma) {
            // LayerNorm over the row, arithmetic and summation order of act_quant_rows_ln_kernel: every lane folds its
            // 32 values serially, the 2 G partial sums of a row meet in LDS and are added group by group, lower half
            // first; y = ((x - mean) * rstd) * gamma + beta, rounded to fp16 as a LayerNorm kernel would store it.
            const float fk = static_cast<float>(K);
            const int ppitch = 2 * G + 1;
            float *prow = part + (rb2 * 32 + row) * ppitch;
            auto row_total = [&](float mine) {
                prow[2 * g + half] = mine;
                __syncthreads();
                float acc = 0.0f;
                for (int i = 0; i < 2 * G; ++i) acc += prow[i];
                __syncthreads();
                return acc;
            };
            float a = 0.0f;
#pragma unroll
            for (int j = 0; j < 32; ++j) a += xv[j];
            const float mean = row_total(a) / fk;
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                xv[j] -= mean;
                const float sq = xv[j] * xv[j];
                q += sq;
            }
            const float var_row = row_total(q) / fk;
            const float rstd = 1.0f / sqrtf(var_row + p.ln_eps);
            const float4 *gp = reinterpret_cast<const float4 *>(p.gamma + g * 64 + half * 32);
            const float4 *bp = reinterpret_cast<const float4 *>(p.beta + g * 64 + half * 32);
#pragma unroll
            for (int j4 = 0; j4 < 8; ++j4) {
                const float4 gv = gp[j4], bv = bp[j4];
                const float g4[4] = {gv.x, gv.y, gv.z, gv.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = xv[4 * j4 + e] * rstd;
                    const float u = t * g4[e];
                    xv[4 * j4 + e] = __half2float(__float2half_rn(u + b4[e]));
                }
            }
        }
        bool table_ok = true;
        for (int w = 0; w < kBuilders; ++w) table_ok = table_ok && (slow_slots[w] == 0);
        float mu, var, s, sum_codes;
        group_stats32x2(xv, p.eps, mu, var, s);
        group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
        const float code_mean = sum_codes * 0.015625f;
        unsigned char *dst = xs + (rb2 * 32 + row) * pitch + g * 128 + half * 64;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            u32x4_t o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = 8 * q4 + 2 * e;
                const __half2 h = __floats2half2_rn(fma_f32(s, xv[j] - code_mean, mu), fma_f32(s, xv[j + 1] - code_mean, mu));
                o[e] = *reinterpret_cast<const uint32_t *>(&h);
            }
            *reinterpret_cast<u32x4_t *>(dst + q4 * 16) = o;
        }
      }
    }

    // ---- every share of w_hat written? ----
    if (p.counter && tid == 0) {
        int ok = p.wait_ticks > 0;      // (a bound of zero: give up without looking -- how the tests reach the rebuild)
        const long long t0 = wall_clock64();
        while (ok && __hip_atomic_load(p.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            if (wall_clock64() - t0 > p.wait_ticks) {
                ok = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
        if (!ok) __hip_atomic_fetch_add(p.timeouts, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_flag = ok;
    }
    // One wave drops whatever this CU's L1 and this XCD's L2 may hold of the workspace (nothing, unless a line was
    // fetched before its writer was done), before anyone reads it.
    if (p.counter && wave == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    __syncthreads();                              // x_hat is complete in LDS; s_flag is set
    if (p.counter) {
        if (!s_flag) {                            // workgroup-uniform
            for (int64_t idx = tid; idx < pieces; idx += nthreads) {
                fetch_piece<BITS, G>(p, idx, pc);
                finish_piece<BITS>(p, idx, pc);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }

    // ---- the product: wave tile = 64 rows x one 32-column block; every wave a run of N / 32 / W blocks ----
    const int lr = lane & 31, lh = lane >> 5;
    const int ncb = p.N / 32;
    const unsigned char *xs_lane = xs + lr * pitch + lh * 64;
    const char *w_lane = reinterpret_cast<const char *>(p.w_blk) + lh * 2048 + lr * 16;
    const int64_t cb_bytes = static_cast<int64_t>(K) * 64;     // bytes per 32-column block
    // The wave's blocks are a run of adjacent ones: a row's 64-byte segments of two neighbouring blocks share a
    // 128-byte line, and written by one wave shortly after each other they are more often merged on their way to
    // memory than when twelve waves write them at unrelated times (qkv: 38.5 -> 35.7 MB written per launch).
    const int bpw = (ncb + W - 1) / W;
    const int cb_first = wave * bpw, cb_last = cb_first + bpw < ncb ? cb_first + bpw : ncb;
    int ld_cb = cb_first, ld_g = 0;
    auto load_unit = [&](u32x4_t (&r)[4]) {      // the four fragments of one group; past the wave's last block it re-reads a valid one
        const int c = ld_cb < cb_last ? ld_cb : ncb - 1;
        const char *q = w_lane + c * cb_bytes + ld_g * 4096;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) r[kk] = *reinterpret_cast<const u32x4_t *>(q + kk * 512);
        if (++ld_g == G) {
            ld_g = 0;
            ++ld_cb;
        }
    };
    // Ring of RING groups, walked with compile-time slot numbers: group number s (counted over the wave's column
    // blocks) sits in slot s % RING and, once multiplied, its slot takes group s + RING - 1.  kUnroll column blocks
    // bring the ring back to where it started.
    constexpr int kUnroll = RING / gcd_of(G, RING);
    static_assert((kUnroll * G) % RING == 0, "ring does not close");
    u32x4_t ring[RING][4];
#pragma unroll
    for (int i = 0; i < RING - 1; ++i) load_unit(ring[i]);

    constexpr int kSlots = 2 * AHEAD;
    constexpr int kStageRow = 32 * static_cast<int>(sizeof(TOUT)) + 16;      // bytes per staged output row
    // fp16 outputs with the full-size staging tile: two column blocks per write-out, rows of 128 + 16 bytes
    constexpr bool kPairOut = sizeof(TOUT) == 2 && kStage >= 32 * 144 && G > 3;      // (K = 192 needs its registers for two workgroups per CU)
    constexpr int kOutRow = kPairOut ? 144 : kStageRow;
    float16_t held[2];
    bool have_held = false;
    constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));
    constexpr int kPiecesPerRow = 32 / kVec;                                  // 4 (fp16) / 8 (fp32)
    constexpr int kRowsPerInstr = 64 / kPiecesPerRow;                         // 16 / 8
    TOUT *y = static_cast<TOUT *>(p.y);
    const TOUT *residual = static_cast<const TOUT *>(p.residual);

    for (int cb0 = cb_first; cb0 < cb_last; cb0 += kUnroll) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int cbk = cb0 + u;
        if (cbk >= cb_last) break;
        float16_t acc[2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;
        half8_t xf[kSlots][2];
#pragma unroll
        for (int a = 0; a < AHEAD; ++a)
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
                xf[a][rb] = *reinterpret_cast<const half8_t *>(xs_lane + rb * 32 * pitch + a * 16);
#pragma unroll
        for (int gl = 0; gl < G; ++gl) {
            const u32x4_t (&cur_set)[4] = ring[(u * G + gl) % RING];
            u32x4_t (&load_set)[4] = ring[(u * G + gl + RING - 1) % RING];
            const unsigned char *xsrc = xs_lane + gl * 128;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int t = kk + AHEAD;           // the k-step whose x_hat fragments are read now; t >= 4: of the next group
                const int off = t < 4 ? t * 16 : 128 + (t - 4) * 16;      // (past the row on the last group: unused)
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    xf[t % kSlots][rb] = *reinterpret_cast<const half8_t *>(xsrc + rb * 32 * pitch + off);
                if (kk == 1) load_unit(load_set);
                half8_t wf;
                __builtin_memcpy(&wf, &cur_set[kk], 16);
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, xf[kk % kSlots][rb], acc[rb], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 // 1 LDS read
                    if (kk == 1) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);    // 2 global loads
                }
            }
        }

        // ---- epilogue: bias, rounding, optional GELU / residual, through the wave's staging tile so that every lane
        // stores 16 contiguous bytes.  fp16 outputs leave two column blocks at a time where the wave has two in a row
        // (the first one's accumulators wait in `held`): a row's segment is then a whole 128-byte line instead of two
        // halves written at different times, which do not always meet again before they reach memory. ----
        if constexpr (kPairOut) {
            if (!have_held && cbk + 1 < cb_last) {
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) held[rb] = acc[rb];
                have_held = true;
                continue;
            }
        }
        const int nblk = have_held ? 2 : 1;          // column blocks in this write-out
        const int cb_out = have_held ? cbk - 1 : cbk;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int hb = 0; hb < (kPairOut ? 2 : 1); ++hb) {
                if (hb >= nblk) continue;
                const float16_t &src = (kPairOut && nblk == 2 && hb == 0) ? held[rb] : acc[rb];
                float4 bv[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) bv[q] = *reinterpret_cast<const float4 *>(s_bias + (cb_out + hb) * 32 + 8 * q + 4 * lh);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cl = hb * 32 + 8 * q + 4 * lh;
                    const float o0 = src[4 * q] + bv[q].x, o1 = src[4 * q + 1] + bv[q].y;
                    const float o2 = src[4 * q + 2] + bv[q].z, o3 = src[4 * q + 3] + bv[q].w;
                    unsigned char *dst = wave_lds + lr * kOutRow + cl * static_cast<int>(sizeof(TOUT));
                    if constexpr (sizeof(TOUT) == 2) {
                        const __half2 lo = __floats2half2_rn(o0, o1), hi = __floats2half2_rn(o2, o3);
                        u32x2_t pk;
                        pk[0] = *reinterpret_cast<const uint32_t *>(&lo);
                        pk[1] = *reinterpret_cast<const uint32_t *>(&hi);
                        *reinterpret_cast<u32x2_t *>(dst) = pk;
                    } else {
                        u32x4_t pk;
                        pk[0] = __float_as_uint(o0); pk[1] = __float_as_uint(o1);
                        pk[2] = __float_as_uint(o2); pk[3] = __float_as_uint(o3);
                        *reinterpret_cast<u32x4_t *>(dst) = pk;
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
            if (kPairOut && nblk == 2) {              // 8 lanes per row of 128 bytes, 8 rows per instruction
                const int col = cb_out * 32 + (lane & 7) * kVec;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = i * 8 + (lane >> 3);
                    u32x4_store_t v = *reinterpret_cast<const u32x4_store_t *>(wave_lds + r * kOutRow + (lane & 7) * 16);
                    const int64_t grow = row_base + rb * 32 + r;
                    if (grow < p.M) {
                        if (residual || p.gelu)
                            post_ops16<TOUT>(v, residual ? residual + grow * p.N + col : nullptr, p.gelu != 0, kVec);
                        store_streaming16(y + grow * p.N + col, v[0], v[1], v[2], v[3]);
                    }
                }
            } else {
                const int col = cb_out * 32 + (lane % kPiecesPerRow) * kVec;
#pragma unroll
                for (int i = 0; i < 32 / kRowsPerInstr; ++i) {
                    const int r = i * kRowsPerInstr + lane / kPiecesPerRow;
                    u32x4_store_t v = *reinterpret_cast<const u32x4_store_t *>(wave_lds + r * kOutRow + (lane % kPiecesPerRow) * 16);
                    const int64_t grow = row_base + rb * 32 + r;
                    if (grow < p.M) {
                        if (residual || p.gelu)
                            post_ops16<TOUT>(v, residual ? residual + grow * p.N + col : nullptr, p.gelu != 0, kVec);
                        store_streaming16(y + grow * p.N + col, v[0], v[1], v[2], v[3]);
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        have_held = false;
      }
    }
}

// The same layer for rows of PHASES * 64 G values (K = 768, 1536: fc2 of the small models) and at most 32 * 2 G
// output columns: the row is taken in PHASES slices of G groups.  Two x_hat slice buffers alternate in LDS; while the
// MFMAs of slice p run from one, stage 1 of slice p + 1 fills the other (stage 1 is bound by vector-ALU issue, the
// product by the stream of w_hat through L1 -- different units, so waves of one SIMD that are in different halves
// of the phase overlap: every second wave quad multiplies first and quantizes second).  Every wave owns one
// 32-column block for the whole launch, so the accumulators stay in registers across the slices; k order per output
// is ascending as everywhere else.  A lane pair reads its 64 inputs of the next slice straight from global memory
// (two whole 64-byte halves of a 128-byte line) as soon as the registers of the current one are converted.
// NB = column blocks per wave (block nb of wave w is w + nb * 2 G): with eight waves (G = 4) and three blocks each the
// kernel serves K = 3072 with up to 768 outputs (fc2 of DeiT-B) inside the 256 registers two waves per SIMD have.
template <int BITS, typename TOUT, int G, int PHASES, int NB = 1>
__global__ void __launch_bounds__(128 * G)
otf_rows_phased_kernel(const RowsParams p)
{
    constexpr int L = 1 << BITS;
    constexpr int W = 2 * G, GT = G * PHASES, K = 64 * GT, KS = 64 * G;
    static_assert(G % 2 == 0, "the two-slot fragment ring must close on a slice boundary");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ float lut[L * 64];
    __shared__ Bucket table[kMaxBuckets + 1];
    __shared__ int slow_slots[W];
    __shared__ int s_flag;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int nthreads = 64 * W;
    constexpr int pitch = KS * 2 + 16;                           // bytes per x_hat row of a slice
    constexpr int kBuf = 64 * pitch;
    unsigned char *xs = smem;                                    // [2][64][pitch]
    float *s_bias = reinterpret_cast<float *>(smem + 2 * kBuf);  // [32 W NB]
    unsigned char *wave_lds = smem + wave * kWaveLds;            // output staging: reuses the slice buffers at the end
    static_assert(W * kWaveLds <= 2 * kBuf, "output staging must fit into the slice buffers");
    const int64_t pieces = static_cast<int64_t>(p.N) * (K / 8);
    const int64_t row_base = static_cast<int64_t>(blockIdx.x) * 64;

    // stage-1 role: wave = (row block rb2, group g of the slice); lane pair = one row
    const int rb2 = wave / G, g = wave - rb2 * G;
    const int row = lane >> 1, half = lane & 1;
    uint4 raw[4];
    auto load_slice = [&](int ph) {                              // rows past the tensor's end read as zeros
        const int64_t my_row = row_base + rb2 * 32 + row;
        const __half *src = p.x + my_row * K + ph * KS + g * 64 + half * 32;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            raw[i] = my_row < p.M ? *reinterpret_cast<const uint4 *>(src + i * 8) : make_uint4(0, 0, 0, 0);
    };
    load_slice(0);

    // ---- this workgroup's share of w_hat and the lookup tables, as in otf_rows_kernel ----
    constexpr int kBuilders = 3, kBuilder0 = 1;
    constexpr int kPieceThreads = 64 * (W - 3);
    const int ptid = wave == 0 ? lane : (wave >= 4 ? (wave - 3) * 64 + lane : -1);
    int64_t share_lo = 0, share_hi = 0;
    Piece pc{};
    unsigned long long target = 0;
    if (p.counter) {
        int64_t per = (pieces + gridDim.x - 1) / gridDim.x;
        per = (per + 7) & ~int64_t(7);
        share_lo = blockIdx.x * per;
        share_hi = share_lo + per < pieces ? share_lo + per : pieces;
        if (ptid >= 0 && share_lo + ptid < share_hi) fetch_piece<BITS, GT>(p, share_lo + ptid, pc);
    }
    for (int i = tid; i < 32 * W * NB; i += nthreads) s_bias[i] = (p.bias && i < p.N) ? p.bias[i] : 0.0f;
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(p.thr, p.cb_a, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    if (wave >= kBuilder0 && wave < kBuilder0 + kBuilders)
        build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slow_slots, tid - 64 * kBuilder0, 64 * kBuilders);
    if (p.counter) {
        if (ptid >= 0 && share_lo + ptid < share_hi) finish_piece<BITS>(p, share_lo + ptid, pc);
        for (int64_t idx = share_lo + kPieceThreads + ptid; ptid >= 0 && idx < share_hi; idx += kPieceThreads) {
            fetch_piece<BITS, GT>(p, idx, pc);
            finish_piece<BITS>(p, idx, pc);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // the written-through pieces have reached memory
    }
    __syncthreads();                                             // tables complete, and the workgroup's share of w_hat
    if (p.counter && tid == 0) {
        const unsigned long long inc = blockIdx.x == 0 ? kEpoch - (gridDim.x - 1) : 1ull;
        const unsigned long long old = __hip_atomic_fetch_add(p.counter, inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        target = (old & ~(kEpoch - 1)) + kEpoch;
    }
    bool table_ok = true;
    for (int w = 0; w < kBuilders; ++w) table_ok = table_ok && (slow_slots[w] == 0);

    // ---- product role: wave = the 32-column blocks wave, wave + W, ... (idle in the product if it has none) ----
    const int lr = lane & 31, lh = lane >> 5;
    const int ncb = p.N / 32;
    const int nv = wave < ncb ? min(NB, (ncb - wave + W - 1) / W) : 0;      // this wave's blocks: nb < nv
    const bool has_block = nv > 0;
    const char *w_col = reinterpret_cast<const char *>(p.w_blk) + lh * 2048 + lr * 16 +
                        static_cast<int64_t>(has_block ? wave : 0) * (static_cast<int64_t>(K) * 64);
    constexpr int64_t kBlockStride = static_cast<int64_t>(W) * K * 64;      // bytes from a wave's block to its next one
    // The fragment groups are consumed slice by slice, within a slice block by block, within a block group by group;
    // load_unit walks the same order (ld_s = G * (slice * nv + block) + group) and re-reads the last group past the end.
    int ld_ph = 0, ld_nb = 0, ld_g = 0;
    auto load_unit = [&](u32x4_t (&r)[4]) {
        const char *q = w_col + ld_nb * kBlockStride + (ld_ph * G + ld_g) * 4096;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) r[kk] = *reinterpret_cast<const u32x4_t *>(q + kk * 512);
        const bool last = ld_ph == PHASES - 1 && ld_nb == nv - 1 && ld_g == G - 1;      // (the last group: stay)
        const bool wrap_g = ld_g == G - 1, wrap_nb = wrap_g && ld_nb >= nv - 1;
        ld_g = last ? ld_g : (wrap_g ? 0 : ld_g + 1);
        ld_nb = last ? ld_nb : (wrap_nb ? 0 : (wrap_g ? ld_nb + 1 : ld_nb));
        ld_ph = last ? ld_ph : (wrap_nb ? ld_ph + 1 : ld_ph);
    };
    u32x4_t ring[2][4];
    float16_t acc[NB][2];

    auto stage1 = [&](int ph) {                  // slice ph: registers -> xs[ph & 1]; then requests slice ph + 1
        float xv[32];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w4[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                xv[8 * i + 2 * e] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] & 0xffffu)));
                xv[8 * i + 2 * e + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w4[e] >> 16)));
            }
        }
        if (ph + 1 < PHASES) load_slice(ph + 1);
        float mu, var, s, sum_codes;
        group_stats32x2(xv, p.eps, mu, var, s);
        group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, lut, table_ok, lane, sum_codes);
        const float code_mean = sum_codes * 0.015625f;
        unsigned char *dst = xs + (ph & 1) * kBuf + (rb2 * 32 + row) * pitch + g * 128 + half * 64;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            u32x4_t o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = 8 * q4 + 2 * e;
                const __half2 h = __floats2half2_rn(fma_f32(s, xv[j] - code_mean, mu), fma_f32(s, xv[j + 1] - code_mean, mu));
                o[e] = *reinterpret_cast<const uint32_t *>(&h);
            }
            *reinterpret_cast<u32x4_t *>(dst + q4 * 16) = o;
        }
    };

    auto product = [&](int ph) {                 // acc += x_hat slice ph * w_hat slice ph^T
        const unsigned char *xb = xs + (ph & 1) * kBuf + lr * pitch + lh * 64;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (nb >= nv) break;
        half8_t xf[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) xf[0][rb] = *reinterpret_cast<const half8_t *>(xb + rb * 32 * pitch);
#pragma unroll
        for (int gl = 0; gl < G; ++gl) {
            const u32x4_t (&cur_set)[4] = ring[gl % 2];
            u32x4_t (&load_set)[4] = ring[(gl + 1) % 2];
            const unsigned char *xsrc = xb + gl * 128;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int t = kk + 1;              // the k-step whose x_hat fragments are read now; 4: first of the next group
                const int off = t < 4 ? t * 16 : 128;                  // (past the slice on its last group: unused)
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    xf[t % 2][rb] = *reinterpret_cast<const half8_t *>(xsrc + rb * 32 * pitch + off);
                if (kk == 1) load_unit(load_set);
                half8_t wf;
                __builtin_memcpy(&wf, &cur_set[kk], 16);
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    acc[nb][rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, xf[kk % 2][rb], acc[nb][rb], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 // 1 LDS read
                    if (kk == 1) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);    // 2 global loads
                }
            }
        }
      }
    };

#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[nb][rb][v] = 0.0f;

    // ---- the phases: iteration ph multiplies slice ph and quantizes slice ph + 1; iteration -1 only quantizes ----
    const bool multiply_first = ((wave >> 2) & 1) != 0;
    for (int ph = -1; ph < PHASES; ++ph) {
        if (ph >= 0 && has_block && multiply_first) product(ph);
        if (ph + 1 < PHASES) stage1(ph + 1);
        if (ph >= 0 && has_block && !multiply_first) product(ph);
        if (ph == -1) {
            // ---- every share of w_hat written? ----
            if (p.counter && tid == 0) {
                int ok = p.wait_ticks > 0;      // (a bound of zero: give up without looking -- how the tests reach the rebuild)
                const long long t0 = wall_clock64();
                while (ok && __hip_atomic_load(p.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                    if (wall_clock64() - t0 > p.wait_ticks) {
                        ok = 0;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(4);
                }
                if (!ok) __hip_atomic_fetch_add(p.timeouts, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_flag = ok;
            }
            if (p.counter && wave == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        __syncthreads();                         // slice ph + 1 of x_hat is complete, slice ph has been consumed
        if (ph == -1) {
            if (p.counter && !s_flag) {          // workgroup-uniform: the others are not resident; rebuild everything
                for (int64_t idx = tid; idx < pieces; idx += nthreads) {
                    fetch_piece<BITS, GT>(p, idx, pc);
                    finish_piece<BITS>(p, idx, pc);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
            if (has_block) load_unit(ring[0]);
        }
    }

    // ---- epilogue: as in otf_rows_kernel, one column block at a time ----
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
    if (nb >= nv) break;
    constexpr int kStageRow = 32 * static_cast<int>(sizeof(TOUT)) + 16;
    constexpr int kVec = 16 / static_cast<int>(sizeof(TOUT));
    constexpr int kPiecesPerRow = 32 / kVec;
    constexpr int kRowsPerInstr = 64 / kPiecesPerRow;
    TOUT *y = static_cast<TOUT *>(p.y);
    const TOUT *residual = static_cast<const TOUT *>(p.residual);
    const int cbk = wave + nb * W;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        float4 bv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[q] = *reinterpret_cast<const float4 *>(s_bias + cbk * 32 + 8 * q + 4 * lh);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int cl = 8 * q + 4 * lh;
            const float o0 = acc[nb][rb][4 * q] + bv[q].x, o1 = acc[nb][rb][4 * q + 1] + bv[q].y;
            const float o2 = acc[nb][rb][4 * q + 2] + bv[q].z, o3 = acc[nb][rb][4 * q + 3] + bv[q].w;
            unsigned char *dst = wave_lds + lr * kStageRow + cl * static_cast<int>(sizeof(TOUT));
            if constexpr (sizeof(TOUT) == 2) {
                const __half2 lo = __floats2half2_rn(o0, o1), hi = __floats2half2_rn(o2, o3);
                u32x2_t pk;
                pk[0] = *reinterpret_cast<const uint32_t *>(&lo);
                pk[1] = *reinterpret_cast<const uint32_t *>(&hi);
                *reinterpret_cast<u32x2_t *>(dst) = pk;
            } else {
                u32x4_t pk;
                pk[0] = __float_as_uint(o0); pk[1] = __float_as_uint(o1);
                pk[2] = __float_as_uint(o2); pk[3] = __float_as_uint(o3);
                *reinterpret_cast<u32x4_t *>(dst) = pk;
            }
        }
        __builtin_amdgcn_wave_barrier();
        const int col = cbk * 32 + (lane % kPiecesPerRow) * kVec;
#pragma unroll
        for (int i = 0; i < 32 / kRowsPerInstr; ++i) {
            const int r = i * kRowsPerInstr + lane / kPiecesPerRow;
            u32x4_store_t v = *reinterpret_cast<const u32x4_store_t *>(wave_lds + r * kStageRow + (lane % kPiecesPerRow) * 16);
            const int64_t grow = row_base + rb * 32 + r;
            if (grow < p.M) {
                if (residual || p.gelu)
                    post_ops16<TOUT>(v, residual ? residual + grow * p.N + col : nullptr, p.gelu != 0, kVec);
                store_streaming16(y + grow * p.N + col, v[0], v[1], v[2], v[3]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    }
}

// One counter per weight workspace.  Launches that share a counter word must never overlap (a workgroup derives its
// target from the value it finds); launches that share a weight workspace must never overlap either -- they would
// overwrite each other's w_hat -- so the workspace's address is the key: whatever the caller does with streams and
// graphs (two graphs captured on one stream and replayed on two, a destroyed stream whose handle is reused, the null
// stream's two flavours), overlapping launches count into different words as long as the caller keeps the rule it has
// to keep anyway.  The words live in device memory that is zero when the code object is loaded; the key -> word table
// is per device, open addressing from a hash of the address, never recycled (a word whose key left could still be
// counted into by a launch in flight): after 4096 distinct workspace addresses on a device further ones take the
// two-launch path (a model shares one workspace between its layers; the table is sized for processes that allocate
// and free workspaces all the time, such as a test suite).
constexpr int kCounterSlots = 4096;
__device__ unsigned long long g_rows_counters[kCounterSlots];
__device__ unsigned long long g_rows_timeouts;          // workgroups whose bounded wait ran out, ever

constexpr int kMaxDevices = 64;
std::mutex g_rows_mutex;
unsigned long long *g_counters_ptr[kMaxDevices];
unsigned long long *g_timeouts_ptr[kMaxDevices];
std::vector<const void *> g_slot_key[kMaxDevices];          // kCounterSlots keys per device, allocated on first use

}  // namespace

// Slot of `key` in a table of `slots` keys (nullptr = free): the key's own slot if it has one, else the first free
// one on its probe sequence (which it then owns), else -1.  Host logic only.
int rows_counter_slot(const void **table, int slots, const void *key)
{
    if (!key || slots <= 0) return -1;
    uint64_t h = reinterpret_cast<uintptr_t>(key) >> 8;          // (workspaces are at least 128-byte aligned)
    h ^= h >> 17;
    h *= 0x9E3779B97F4A7C15ull;
    h ^= h >> 29;
    const int start = static_cast<int>(h % static_cast<uint64_t>(slots));
    for (int i = 0; i < slots; ++i) {
        const int s = (start + i) % slots;
        if (table[s] == key) return s;
        if (table[s] == nullptr) {
            table[s] = key;
            return s;
        }
    }
    return -1;
}

namespace {

// Device address of the counter that belongs to weight workspace `key` on the current device; nullptr if none is left.
unsigned long long *counter_for(const void *key, unsigned long long **timeouts)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_rows_mutex);
    if (!g_counters_ptr[dev]) {
        void *ptr = nullptr, *tptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_rows_counters)) != hipSuccess || !ptr) return nullptr;
        if (hipGetSymbolAddress(&tptr, HIP_SYMBOL(g_rows_timeouts)) != hipSuccess || !tptr) return nullptr;
        g_counters_ptr[dev] = static_cast<unsigned long long *>(ptr);
        g_timeouts_ptr[dev] = static_cast<unsigned long long *>(tptr);
    }
    if (g_slot_key[dev].empty()) g_slot_key[dev].assign(kCounterSlots, nullptr);
    const int slot = rows_counter_slot(g_slot_key[dev].data(), kCounterSlots, key);
    if (slot < 0) return nullptr;            // more workspaces than counters: the caller falls back
    *timeouts = g_timeouts_ptr[dev];
    return g_counters_ptr[dev] + slot;
}

// Workgroups of `Kernel` (threads, dynamic LDS bytes) the current device holds at once.  A launch must not be larger:
// every workgroup waits for the weight shares of all the others, and those that are not resident write theirs only
// after a resident one has given up waiting (correct, but milliseconds late).  Asked once per device, kernel and LDS
// size; 0 if the runtime cannot tell.
template <auto Kernel>
int resident_workgroups(int threads, size_t smem)
{
    struct Entry { int dev; size_t smem; int blocks; };
    static std::mutex mutex;
    static std::vector<Entry> known;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(mutex);
    for (const Entry &e : known)
        if (e.dev == dev && e.smem == smem) return e.blocks;
    int per_cu = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(Kernel), threads, smem) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        per_cu = cus = 0;
    known.push_back({dev, smem, per_cu * cus});
    return per_cu * cus;
}

}  // namespace

// Compute units of the current device (256 when there is none to ask: the host-side predicates also run without a GPU).
int device_cus()
{
    static std::atomic<int> known[kMaxDevices];
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (const int c = known[dev].load(std::memory_order_relaxed)) return c;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
    known[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

namespace {

// Waves of otf_rows_kernel's workgroup: one per stage-1 tile (2 K / 64), for K = 768 half as many.
constexpr int rows_waves(int G) { return G == 12 ? 12 : 2 * G; }

size_t rows_lds_bytes(int N, int K, size_t out_size = 2)
{
    const int G = K / 64, W = rows_waves(G);
    return static_cast<size_t>(64) * (K * 2 + 16) + static_cast<size_t>(W) * rows_stage_bytes(2 * G / W, out_size) +
           64 * (2 * G + 1) * sizeof(float) + static_cast<size_t>(N) * sizeof(float);
}

// Workgroups to add to a launch of `tiles` row workgroups for the reconstruction of w_hat alone, given `spare` free
// places on the device: one per `threads` pieces (every thread one piece), if at least half as many are to be had and
// the row tiles fill at most half the device -- otherwise none, and the row workgroups share the reconstruction
// (with many row workgroups each one's share is small and hides under its load latency; helpers then cost 1 %).
int helper_workgroups(const RowsParams &p, int tiles, int spare, int threads)
{
    const int64_t pieces = static_cast<int64_t>(p.N) * p.G * 8;
    const int want = static_cast<int>((pieces + threads - 1) / threads);
    if (spare < tiles || spare * 2 < want) return 0;
    return spare < want ? spare : want;
}

// The launchers return false, having launched nothing, when the device would not hold the whole grid at once.
template <int BITS, typename TOUT, int G, int RING, int AHEAD>
bool launch_rows_g(const RowsParams &p, size_t smem, hipStream_t stream)
{
    constexpr int W = rows_waves(G);
    allow_dynamic_lds<otf_rows_kernel<BITS, TOUT, G, RING, AHEAD, W>>(160 * 1024 - 10 * 1024);
    const int tiles = (p.M + 63) / 64;
    const int cap = resident_workgroups<otf_rows_kernel<BITS, TOUT, G, RING, AHEAD, W>>(64 * W, smem);
    if (cap < tiles) return false;
    hipLaunchKernelGGL((otf_rows_kernel<BITS, TOUT, G, RING, AHEAD, W>), dim3(tiles + helper_workgroups(p, tiles, cap - tiles, 64 * W)),
                       dim3(64 * W), smem, stream, p);
    return true;
}

// Two fragment groups per wave (the one being multiplied and the next) and x_hat fragments read one k-step ahead:
// deeper pipelines (rings of three and four groups, reads two k-steps ahead) measured 2-5 % slower on the DeiT-S
// shapes -- the stream from L2 is bound by throughput, not latency.  Streaming stores for y and the MFMA / LDS /
// load interleave pinned with scheduling barriers are worth 7 % and 13 %.
template <int BITS, typename TOUT>
bool launch_rows(const RowsParams &p, size_t smem, hipStream_t stream)
{
    if (p.G == 3) return launch_rows_g<BITS, TOUT, 3, 2, 1>(p, smem, stream);
    if (p.G == 4) return launch_rows_g<BITS, TOUT, 4, 2, 1>(p, smem, stream);
    if (p.G == 12) {
        if constexpr (sizeof(TOUT) == 2) return launch_rows_g<BITS, TOUT, 12, 2, 1>(p, smem, stream);
        else return false;      // (fp32 outputs: the staging tiles do not fit beside a 64 x 768 x_hat tile)
    }
    return launch_rows_g<BITS, TOUT, 6, 2, 1>(p, smem, stream);
}

// The phased kernel's configurations: slices of G groups on 2 G waves, NB column blocks per wave.
//   K = 768 / 1536, N <= 384:  G = 6 (twelve waves), one block per wave
//   K = 3072,       N <= 768:  G = 4 (eight waves),  three blocks per wave
constexpr int kPhasedG = 6;
constexpr size_t phased_lds(int G, int NB) { return 2 * 64 * (64 * G * 2 + 16) + 32 * 2 * G * NB * sizeof(float); }

template <int BITS, typename TOUT, int G, int PHASES, int NB>
bool launch_phased_p(const RowsParams &p, hipStream_t stream)
{
    constexpr size_t lds = phased_lds(G, NB);
    allow_dynamic_lds<otf_rows_phased_kernel<BITS, TOUT, G, PHASES, NB>>(160 * 1024 - 10 * 1024);
    const int tiles = (p.M + 63) / 64;
    if (resident_workgroups<otf_rows_phased_kernel<BITS, TOUT, G, PHASES, NB>>(128 * G, lds) < tiles) return false;
    hipLaunchKernelGGL((otf_rows_phased_kernel<BITS, TOUT, G, PHASES, NB>), dim3(tiles), dim3(128 * G), lds, stream, p);
    return true;
}

template <int BITS, typename TOUT>
bool launch_phased(const RowsParams &p, int K, hipStream_t stream)
{
    if (K == 768) return launch_phased_p<BITS, TOUT, kPhasedG, 2, 1>(p, stream);
    if (K == 3072) return launch_phased_p<BITS, TOUT, 4, 12, 3>(p, stream);
    return launch_phased_p<BITS, TOUT, kPhasedG, 4, 1>(p, stream);
}

bool phased_shape(int64_t N, int64_t K)
{
    return ((K == 768 || K == 1536) && N <= 32 * 2 * kPhasedG) || (K == 3072 && N <= 32 * 8 * 3);
}

}  // namespace

bool otf_rows_is_phased(int64_t N, int64_t K) { return phased_shape(N, K); }

bool otf_rows_supported(int64_t M, int64_t N, int64_t K, bool layernorm)
{
    if (M < 512 || N < 32 || N % 32 != 0 || N > 16384) return false;
    // One workgroup per 64 rows, all of them resident at once: K = 192 leaves room for two per compute unit, longer
    // rows for one (registers: twelve or eight waves of ~165 VGPRs; LDS: 100 KB and more).
    const int64_t tiles = (M + 63) / 64;
    if (tiles > static_cast<int64_t>(device_cus()) * (K == 192 ? 2 : 1)) return false;
    if (phased_shape(N, K)) return !layernorm;
    if (K == 768) return rows_lds_bytes(static_cast<int>(N), 768) <= 160 * 1024 - 10 * 1024;      // (fp16 outputs only: launch_rows)
    if (K != 192 && K != 256 && K != 384) return false;
    return rows_lds_bytes(static_cast<int>(N), static_cast<int>(K)) <= 160 * 1024 - 10 * 1024;
}

bool otf_rows_pays(int64_t M, int64_t N, int64_t K, bool layernorm)
{
    if (!otf_rows_supported(M, N, K, layernorm) || tuning().gemm_kernel) return false;
    const char *e = tuning().rows;
    if (e) return e[0] != '0';
    if (phased_shape(N, K)) {
        // The phased kernel takes the same time for any number of row tiles up to the device's compute units (stage 1
        // of a whole row on one CU); the two launches it replaces spread stage 1 over all CUs and win while the grid
        // is small.  Crossover measured at 128 row tiles for K = 1536 and at 90 for K = 768 (256 CUs).
        const int64_t tiles = (M + 63) / 64;
        return tiles * (K == 768 ? 3 : 2) >= device_cus();
    }
    // otf_rows_kernel takes about 8 us + 23 ps per weight whatever the number of rows (every workgroup streams all of
    // w_hat); the two launches take about 12 us + 2.6 fs per multiply-add.  Fitted on N = 384 .. 1536, K = 192 .. 384,
    // M = 512 .. 12608: one launch from about 6 200 rows on for DeiT-S qkv, 6 900 for fc1, always for proj.
    const double weights = static_cast<double>(N) * static_cast<double>(K);
    return static_cast<double>(M) >= 8800.0 - 1.15e9 / weights;
}

int launch_otf_rows(const OtfRowsArgs &a, hipStream_t stream)
{
    RowsParams p{};
    p.x = static_cast<const __half *>(a.x);
    p.thr = a.a_thr, p.cb_a = a.a_cb, p.eps = a.eps;
    p.gamma = a.ln_weight, p.beta = a.ln_bias, p.ln_eps = a.ln_eps;
    p.pw = a.pw, p.cb_w = a.w_cb, p.wc = a.wc, p.ws = a.ws, p.wcs = a.wcs;
    p.w_blk = static_cast<__half *>(a.w_hat_ws);
    p.counter = counter_for(a.w_hat_ws, &p.timeouts);
    if (!p.counter) return kNotLaunched;     // more workspaces than counters: the caller takes the two-launch path
    p.wait_ticks = tuning().rows_wait_ticks;
    p.bias = a.bias, p.y = a.y, p.residual = a.residual, p.gelu = a.gelu ? 1 : 0;
    p.M = a.M, p.N = a.N, p.G = a.K / 64;
    bool launched;
    if (phased_shape(a.N, a.K)) {
        if (a.y_f16)
            launched = a.bits == 4   ? launch_phased<4, __half>(p, a.K, stream)
                       : a.bits == 3 ? launch_phased<3, __half>(p, a.K, stream)
                                     : launch_phased<2, __half>(p, a.K, stream);
        else
            launched = a.bits == 4   ? launch_phased<4, float>(p, a.K, stream)
                       : a.bits == 3 ? launch_phased<3, float>(p, a.K, stream)
                                     : launch_phased<2, float>(p, a.K, stream);
    } else {
        const size_t smem = rows_lds_bytes(a.N, a.K, a.y_f16 ? 2 : 4);
        if (a.y_f16)
            launched = a.bits == 4   ? launch_rows<4, __half>(p, smem, stream)
                       : a.bits == 3 ? launch_rows<3, __half>(p, smem, stream)
                                     : launch_rows<2, __half>(p, smem, stream);
        else
            launched = a.bits == 4   ? launch_rows<4, float>(p, smem, stream)
                       : a.bits == 3 ? launch_rows<3, float>(p, smem, stream)
                                     : launch_rows<2, float>(p, smem, stream);
    }
    return launched ? launch_status("arcq_linear_otf") : kNotLaunched;
}

}  // namespace arcq

// Host-side slot logic of the per-workspace counters, exposed so that it can be tested without a GPU: `table` is a
// caller-owned array of `slots` pointers, all NULL at first.
ARCQ_API int arcq_rows_counter_slot(const void **table, int slots, const void *key)
{
    return arcq::rows_counter_slot(table, slots, key);
}

// Diagnostic: how many workgroups of the one-launch layer kernels have, on the current device and since the library was
// loaded, given up waiting for the other workgroups' weight shares and rebuilt all of w_hat themselves (correct
// results, but each such launch is many times slower: the sign of a device shared with other work).  Synchronizes
// with the device (a blocking copy); -1 if the count cannot be read.
ARCQ_API long long arcq_rows_wait_timeouts(void)
{
    unsigned long long v = 0;
    if (hipMemcpyFromSymbol(&v, HIP_SYMBOL(arcq::g_rows_timeouts), sizeof(v), 0, hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return static_cast<long long>(v);
}
