// Stage-1 arithmetic shared by the stand-alone activation quantizer and the fused small-M layer kernel
// (semantics: EXT/arcq_activation_kernel.cu:24-184): per-workgroup lookup tables and the per-group routine
// that turns 64 inputs held in one lane's registers into mu, s, the codes and the reconstructed values.
#pragma once

#include "arcq_common.h"

namespace arcq {

constexpr int kMaxBuckets = 512;   // table entries 0 .. nb (nb <= 512); entry nb is reached by t == 8 only

// Bucket geometry: t in [-8, 8] maps to floor(f), f = t * scale + 8 * scale rounded to a multiple of 1/8; nb = 16 * scale
// buckets can hold a threshold.  The scale is the smallest of 4, 8, 16, 32 buckets per unit of t that separates every
// pair of thresholds (scale * smallest gap > 1), so the usual codebooks need a 65- or 129-entry table instead of 513.
// f is formed as 2^20 + f in one fma: in that binade a float's unit in the last place is 1/8, so the low mantissa bits
// of the result ARE 8 * f -- the byte offset of an 8-byte table entry once the three fraction bits are masked off.
// The map t -> bucket is monotone (fma and the mask are), which is all the code search needs.
constexpr float kBucketBias = 1048576.0f;      // 2^20
struct BucketScale { float scale, offset; int nb; };      // offset = 8 * scale + 2^20 (exact)

template <int BITS>
__device__ __forceinline__ BucketScale pick_bucket_scale(const float (&th)[(1 << BITS) - 1])
{
    constexpr int L = 1 << BITS;
    float gap = 16.0f;
#pragma unroll
    for (int i = 0; i + 1 < L - 1; ++i) gap = fminf(gap, th[i + 1] - th[i]);      // NaN gaps are ignored; checked later
    float scale = 32.0f;
    if (gap * 16.0f > 1.0f) scale = 16.0f;
    if (gap * 8.0f > 1.0f) scale = 8.0f;
    if (gap * 4.0f > 1.0f) scale = 4.0f;
    BucketScale q;
    q.scale = scale;
    q.offset = 8.0f * scale + kBucketBias;
    q.nb = static_cast<int>(16.0f * scale);
    return q;
}

// Bucket of a threshold: any float; -1 / nb flag a threshold outside [-8, 8).
__device__ __forceinline__ int bucket_of_threshold(float t, const BucketScale &q)
{
    const float f = __fmaf_rn(t, q.scale, q.offset);
    if (!(f >= kBucketBias)) return -1;         // below the table, or NaN
    if (f >= kBucketBias + static_cast<float>(q.nb)) return q.nb;
    return __float2int_rz(f - kBucketBias);     // exact difference
}

// Byte offset into the table of the bucket of t = d/s on the fast path: |t| <= 8, so f lies in [0, nb] <= 512 and the
// offset is bits 3..12 of the biased sum.
__device__ __forceinline__ uint32_t bucket_offset_of(float t, const BucketScale &q)
{
    return __float_as_uint(__fmaf_rn(t, q.scale, q.offset)) & 0x1ff8u;
}

struct Bucket { float thr; int base; };     // the threshold inside the bucket (+inf if none); thresholds in lower buckets
static_assert(sizeof(Bucket) == 8, "bucket_offset_of assumes 8-byte table entries");

template <int BITS>
__device__ __forceinline__ void load_quant_params(const float *__restrict__ thr, const float *__restrict__ cb,
                                                  float (&th)[(1 << BITS) - 1], float (&cbv)[1 << BITS])
{
    constexpr int L = 1 << BITS;
#pragma unroll
    for (int i = 0; i < L - 1; ++i) th[i] = thr[i];
#pragma unroll
    for (int c = 0; c < L; ++c) cbv[c] = cb[c];
}

// Table construction without barriers, by the `nt` threads numbered t = 0 .. nt-1 (nt a multiple of 64; the calling
// waves must be complete).  `lut` = codebook replicated per lane (lut[c*64 + lane], conflict-free), `table` = the
// threshold buckets.  Each participating wave reports through its own slot slow_slots[t / 64] whether the buckets
// are unusable (two thresholds in one bucket, a threshold outside [-8, 8), unsorted thresholds); the caller
// synchronizes and ORs the slots.
template <int BITS>
__device__ __forceinline__ void build_quant_tables_by(const float (&th)[(1 << BITS) - 1], const float (&cbv)[1 << BITS],
                                                      const BucketScale &q, float *lut, Bucket *table, int *slow_slots,
                                                      int t, int nt)
{
    constexpr int L = 1 << BITS;
    if (t < 64) {
#pragma unroll
        for (int c = 0; c < L; ++c) lut[c * 64 + t] = cbv[c];
    }
    int tb[L - 1];
    bool bad = false;
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        tb[i] = bucket_of_threshold(th[i], q);
        bad = bad || tb[i] < 0 || tb[i] >= q.nb;
    }
#pragma unroll
    for (int i = 0; i + 1 < L - 1; ++i) bad = bad || !(th[i] <= th[i + 1]);
    for (int b = t; b <= q.nb; b += nt) {
        int below = 0, upto = 0;   // thresholds in buckets < b, <= b
        float inside_thr = __int_as_float(0x7f800000);   // +inf: never exceeded
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            below += (tb[i] < b) ? 1 : 0;
            upto += (tb[i] <= b) ? 1 : 0;
            inside_thr = (tb[i] == b) ? th[i] : inside_thr;
        }
        bad = bad || (upto - below) > 1;
        Bucket e;
        e.base = below;
        e.thr = inside_thr;
        table[b] = e;
    }
    const bool any_bad = __any(bad);
    if ((t & 63) == 0) slow_slots[t >> 6] = any_bad ? 1 : 0;
}

// One group per lane, first half: xv holds the 64 inputs on entry and the residuals d_j = x_j - mu on exit.
// Needs no table, so it can run while other waves are still building them.
__device__ __forceinline__ void group_stats64(float (&xv)[64], float eps, float &mu_out, float &var_out, float &s_out)
{
    float mu = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; ++j) mu += xv[j];
    mu *= 0.015625f;                       // exact: /64
    float var = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
        xv[j] -= mu;                       // d_j
        var += xv[j] * xv[j];
    }
    mu_out = mu;
    var_out = var;
    s_out = sqrtf(var * 0.015625f + eps);
}

// Second half: xv holds the residuals on entry and cb[code_j] on exit.  The whole wave must call it (the fast/slow
// decision is wave-uniform).
template <int BITS, bool CODES>
__device__ __forceinline__ void group_codes64(float (&xv)[64], float mu, float var, float s,
                                              const float (&th)[(1 << BITS) - 1], const BucketScale &bq,
                                              const Bucket *table, const float *lut, bool table_ok, int lane,
                                              float &sum_out, uint32_t (&code)[CODES ? 64 : 1])
{
    constexpr int L = 1 << BITS;
    // Range in which d*y, the residuals and the corrections are exact or harmlessly rounded:
    // s normal and far from the ends, and no non-zero d_j small enough to push a residual
    // into the subnormals (|d_j| >= 2^-90 whenever |mu| >= 2^-66, or all d_j are zero).
    const bool lane_fast = (s >= 0x1p-60f) && (s <= 0x1p60f) && !(fabsf(mu) < 0x1p-66f && var > 0.0f);
    const bool fast = table_ok && __all(lane_fast);

    float sum_codes = 0.0f;
    if (fast) {
        const float y = 1.0f / s;
        const float ns = -s;
        const char *lut_lane = reinterpret_cast<const char *>(lut) + lane * 4;      // + 256 c: one shift-add per lookup
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            const float d = xv[j];
            float q = d * y;
            float e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);
            e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);        // == RN(d / s)
            const Bucket bk = *reinterpret_cast<const Bucket *>(reinterpret_cast<const char *>(table) + bucket_offset_of(q, bq));
            const uint32_t c = static_cast<uint32_t>(bk.base) + ((q > bk.thr) ? 1u : 0u);
            if constexpr (CODES) code[j] = c;
            const float v = *reinterpret_cast<const float *>(lut_lane + (c << 8));
            xv[j] = v;
            sum_codes += v;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            const float t = xv[j] / s;
            uint32_t c = 0;
            bool alive = true;
#pragma unroll
            for (int i = 0; i < L - 1; ++i) {   // while (c < L-1 && t > thr[c]) ++c
                alive = alive && (t > th[i]);
                c += alive ? 1u : 0u;
            }
            if constexpr (CODES) code[j] = c;
            const float v = lut[c * 64 + lane];
            xv[j] = v;
            sum_codes += v;
        }
    }
    sum_out = sum_codes;
}

// ---- two lanes per group -------------------------------------------------------------------------------------
// For launches too small to fill the chip the length of one lane's instruction chain is what counts.  Lanes 2i and
// 2i + 1 then share group i: the even lane holds inputs 0..31, the odd lane inputs 32..63.  The per-element work
// halves; the three group sums keep their serial left-to-right order by running in two phases (the even lane folds
// its half from 0, hands the partial sum to the odd lane, which folds its half on top; every lane executes both
// phases and the phase that is not its own is discarded), so every result bit is the one-lane routine's.
__device__ __forceinline__ float from_even_lane(float v)     // the pair's even lane's value, in both lanes
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xA0, 0xf, 0xf, false));    // quad_perm [0,0,2,2]
}
__device__ __forceinline__ float from_odd_lane(float v)      // the pair's odd lane's value, in both lanes
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xF5, 0xf, 0xf, false));    // quad_perm [1,1,3,3]
}

// Serial sum of the group's 64 values v_0 + v_1 + ... (from 0.0f, left to right), this lane holding its half.
__device__ __forceinline__ float pair_serial_sum(const float (&v)[32])
{
    float a = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) a += v[j];           // even lane: values 0..31
    float b = from_even_lane(a);
#pragma unroll
    for (int j = 0; j < 32; ++j) b += v[j];           // odd lane: ... + values 32..63
    return from_odd_lane(b);
}

// xv: this lane's 32 inputs on entry, the residuals d_j = x_j - mu on exit; mu, var, s as group_stats64, in both lanes.
__device__ __forceinline__ void group_stats32x2(float (&xv)[32], float eps, float &mu_out, float &var_out, float &s_out)
{
    const float mu = pair_serial_sum(xv) * 0.015625f;     // exact: /64
    float sq[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        xv[j] -= mu;
        sq[j] = xv[j] * xv[j];
    }
    const float var = pair_serial_sum(sq);
    mu_out = mu;
    var_out = var;
    s_out = sqrtf(var * 0.015625f + eps);
}

// xv: residuals on entry, cb[code_j] on exit; sum_out = the serial sum of all 64 cb[code_j], in both lanes.  The
// whole wave must call it (the fast/slow decision is wave-uniform).
template <int BITS>
__device__ __forceinline__ void group_codes32x2(float (&xv)[32], float mu, float var, float s,
                                                const float (&th)[(1 << BITS) - 1], const BucketScale &bq,
                                                const Bucket *table, const float *lut, bool table_ok, int lane,
                                                float &sum_out)
{
    constexpr int L = 1 << BITS;
    const bool lane_fast = (s >= 0x1p-60f) && (s <= 0x1p60f) && !(fabsf(mu) < 0x1p-66f && var > 0.0f);
    const bool fast = table_ok && __all(lane_fast);
    if (fast) {
        const float y = 1.0f / s;
        const float ns = -s;
        const char *lut_lane = reinterpret_cast<const char *>(lut) + lane * 4;      // + 256 c: one shift-add per lookup
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float d = xv[j];
            float q = d * y;
            float e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);
            e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);        // == RN(d / s)
            const Bucket bk = *reinterpret_cast<const Bucket *>(reinterpret_cast<const char *>(table) + bucket_offset_of(q, bq));
            const uint32_t c = static_cast<uint32_t>(bk.base) + ((q > bk.thr) ? 1u : 0u);
            xv[j] = *reinterpret_cast<const float *>(lut_lane + (c << 8));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float t = xv[j] / s;
            uint32_t c = 0;
            bool alive = true;
#pragma unroll
            for (int i = 0; i < L - 1; ++i) {   // while (c < L-1 && t > thr[c]) ++c
                alive = alive && (t > th[i]);
                c += alive ? 1u : 0u;
            }
            xv[j] = lut[c * 64 + lane];
        }
    }
    sum_out = pair_serial_sum(xv);
}

// The same with the thresholds of the compare-chain fallback read from LDS in a rolled loop (`th_lds`, L - 1 values)
// instead of held in registers: for callers that have no registers to keep them in (a GEMM's epilogue).  Same results.
template <int BITS>
__device__ __forceinline__ void group_codes32x2_lds(float (&xv)[32], float mu, float var, float s, const float *th_lds,
                                                    const BucketScale &bq, const Bucket *table, const float *lut,
                                                    bool table_ok, int lane, float &sum_out)
{
    constexpr int L = 1 << BITS;
    const bool lane_fast = (s >= 0x1p-60f) && (s <= 0x1p60f) && !(fabsf(mu) < 0x1p-66f && var > 0.0f);
    const bool fast = table_ok && __all(lane_fast);
    if (fast) {
        const float y = 1.0f / s;
        const float ns = -s;
        const char *lut_lane = reinterpret_cast<const char *>(lut) + lane * 4;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float d = xv[j];
            float q = d * y;
            float e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);
            e = __fmaf_rn(ns, q, d);
            q = __fmaf_rn(e, y, q);        // == RN(d / s)
            const Bucket bk = *reinterpret_cast<const Bucket *>(reinterpret_cast<const char *>(table) + bucket_offset_of(q, bq));
            const uint32_t c = static_cast<uint32_t>(bk.base) + ((q > bk.thr) ? 1u : 0u);
            xv[j] = *reinterpret_cast<const float *>(lut_lane + (c << 8));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; ++j) xv[j] = xv[j] / s;
#pragma unroll 1
        for (int j = 0; j < 32; ++j) {
            // (element j of a register array under a rolled loop: select it with a compare chain instead of indexing)
            float t = 0.0f;
#pragma unroll
            for (int q = 0; q < 32; ++q) t = (q == j) ? xv[q] : t;
            uint32_t c = 0;
            bool alive = true;
#pragma unroll 1
            for (int i = 0; i < L - 1; ++i) {   // while (c < L-1 && t > thr[c]) ++c
                alive = alive && (t > th_lds[i]);
                c += alive ? 1u : 0u;
            }
            const float v = lut[c * 64 + lane];
#pragma unroll
            for (int q = 0; q < 32; ++q) xv[q] = (q == j) ? v : xv[q];
        }
    }
    sum_out = pair_serial_sum(xv);
}

// ---- stage 1 of the NEXT layer inside a GEMM's epilogue ----------------------------------------------------------
// The block-layout GEMM kernels stage their outputs 32 rows x 64 fp16 columns at a time in a wave-private LDS tile
// (`pitch` bytes per row) -- one quantization group per row.  When the layer's output is only ever consumed quantized
// (fc1 -> GELU -> fc2) the wave quantizes the staged chunk right there, exactly as the consuming layer's stage 1 would
// have done on the stored tensor (two lanes per group, same arithmetic, same bits), and writes x_hat into the
// consumer's 32-row block layout.  The consumer's lookup tables live in LDS (built once per workgroup by
// next_quant_setup).
// LDS of the consumer's quantizer: [codebook per lane: L x 64 floats][buckets][per-wave flags: 64 bytes]
// [thresholds: 16 floats][bucket geometry: scale, offset, number of buckets].
constexpr int next_quant_lds_bytes(int bits) { return (1 << bits) * 64 * 4 + (kMaxBuckets + 64) * 8 + 64 + 64 + 16; }

// All `nthreads` threads of the workgroup call this (before a barrier that precedes the first epilogue): the
// consumer's lookup tables into `lds` (next_quant_lds_bytes(BITS) bytes, 16-byte aligned).
template <int BITS>
__device__ __forceinline__ void next_quant_setup(const float *__restrict__ thr, const float *__restrict__ cb,
                                                 unsigned char *lds, int tid, int nthreads)
{
    constexpr int L = 1 << BITS;
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(thr, cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    float *lut = reinterpret_cast<float *>(lds);
    Bucket *table = reinterpret_cast<Bucket *>(lut + L * 64);
    int *slots = reinterpret_cast<int *>(table + kMaxBuckets + 64);
    build_quant_tables_by<BITS>(th, cbv, bq, lut, table, slots, tid, nthreads);
    float *th_lds = reinterpret_cast<float *>(slots + 16);
    if (tid == 0) {
#pragma unroll
        for (int i = 0; i < L - 1; ++i) th_lds[i] = th[i];
        th_lds[16] = bq.scale;
        th_lds[17] = bq.offset;
        reinterpret_cast<int *>(th_lds)[18] = bq.nb;
    }
}

// One staged chunk (32 rows x 64 fp16 values, the rows `pitch` bytes apart) -> x_hat of the consuming layer.
// `gelu`: the exact GELU of the staged (rounded) values first, rounded to fp16 again.  dst_block = base of the chunk's
// 32-row block in the consumer's block layout, `rows` = rows of that block (32, or fewer for a last block),
// piece0 = index of the chunk's first 16-byte piece (column / 8).  The whole wave calls it.
template <int BITS>
__device__ __forceinline__ void next_quant_chunk(const unsigned char *lds, int nwaves,
                                                 const unsigned char *stage, int pitch, int lane, bool gelu, float eps,
                                                 __half *dst_block, int rows, int piece0)
{
    typedef uint32_t u32x4_nq __attribute__((ext_vector_type(4)));
    constexpr int L = 1 << BITS;
    const float *lut = reinterpret_cast<const float *>(lds);
    const Bucket *table = reinterpret_cast<const Bucket *>(lut + L * 64);
    const int *slots = reinterpret_cast<const int *>(table + kMaxBuckets + 64);
    const float *th_lds = reinterpret_cast<const float *>(slots + 16);
    BucketScale bq;
    bq.scale = th_lds[16];
    bq.offset = th_lds[17];
    bq.nb = reinterpret_cast<const int *>(th_lds)[18];
    const int r = lane >> 1, hf = lane & 1;
    float v[32];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4_nq q = *reinterpret_cast<const u32x4_nq *>(stage + r * pitch + hf * 64 + i * 16);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            v[8 * i + 2 * d] = __half2float(__ushort_as_half(static_cast<unsigned short>(q[d] & 0xffffu)));
            v[8 * i + 2 * d + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(q[d] >> 16)));
        }
    }
    if (gelu) {
#pragma unroll
        for (int j = 0; j < 32; ++j) v[j] = __half2float(__float2half_rn(gelu_f32(v[j])));
    }
    bool ok = true;
    for (int w = 0; w < nwaves; ++w) ok = ok && (slots[w] == 0);
    float mu, var, s, sum;
    group_stats32x2(v, eps, mu, var, s);
    group_codes32x2_lds<BITS>(v, mu, var, s, th_lds, bq, table, lut, ok, lane, sum);
    const float code_mean = sum * 0.015625f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t o[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int j = 8 * i + 2 * d;
            const __half2 h = __floats2half2_rn(fma_f32(s, v[j] - code_mean, mu), fma_f32(s, v[j + 1] - code_mean, mu));
            o[d] = *reinterpret_cast<const uint32_t *>(&h);
        }
        if (r < rows)
            store_writethrough16(dst_block + (static_cast<int64_t>(piece0 + hf * 4 + i) * rows + r) * 8, o[0], o[1], o[2], o[3]);
    }
}

}  // namespace arcq
