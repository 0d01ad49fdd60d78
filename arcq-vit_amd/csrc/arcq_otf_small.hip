// Whole on-the-fly layer (stage 1 + stages 2+3) in ONE launch, for a few hundred rows
// (FQ/arcq_packed_on_the_fly.py:137-161 end to end).
//
// At batch 1 every kernel of the layer costs about as much as an empty launch, so the number of launches is
// what matters.  A workgroup owns a tile of RT rows x 32 or 64 output columns.  It first quantizes the activations
// of its RT rows (all K/64 groups; one group per lane, the same arithmetic as the stand-alone stage-1 kernel,
// arcq_act_quant_core.h) and keeps x_hat as fp16 in LDS; the column tiles of a row tile repeat that work, on
// compute units that would otherwise idle.  Then it runs the split-K product of gemm_splitk_kernel: wave w
// multiplies groups w, w+8, ... against weights rebuilt from the packed codes, and the eight partial tiles are
// added in LDS in a fixed order.  Results are bit-identical to arcq_act_quant followed by arcq_linear_fused.
// The workgroups of column tile 0 also write x_hat to the caller's workspace, which keeps the entry point's contract.
#include "arcq_act_quant_core.h"
#include "arcq_gemm.h"

namespace arcq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kOsWaves = 8;
// Output columns per workgroup: 32 * CB (CB = 1 or 2); a row of a partial tile takes 32 * CB * 4 + 16 bytes.
__host__ __device__ constexpr int os_red_pitch(int cb) { return 32 * cb * 4 + 16; }
constexpr int kOsGroupPitch = 144;             // bytes per group of an x_hat row in LDS (128 + 16 pad)

__host__ __device__ inline int os_row_pitch(int G) { return G * kOsGroupPitch + 16; }

template <int BITS>
__device__ __forceinline__ void os_load_codes(const uint8_t *__restrict__ p, uint32_t (&w)[BITS])
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
__device__ __forceinline__ uint32_t os_code_at(const uint32_t (&w)[BITS], int q)
{
    const int bit = q * BITS;
    const int d = bit >> 5, sh = bit & 31;
    uint32_t v = w[d] >> sh;
    if (sh + BITS > 32) v |= w[d + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}

template <int BITS, int CB>
struct OsWeights {                  // what one wave needs of the weights for one group
    uint32_t codes[CB][BITS];       // 32 codes of this lane's weight row, per 32-column block
    float c[CB], s[CB], m[CB];
};

// The lane's E consecutive inputs (a whole group, or half of one when two lanes share a group): raw 16-byte loads
// (zeros when `valid` is false), converted later so that the loads can be in flight during the table setup.
template <typename TIN, int E> struct OsGroupRegs { u32x4_t raw[E * sizeof(TIN) / 16]; };

template <typename TIN, int E>
__device__ __forceinline__ void os_fetch_group(const TIN *__restrict__ src, bool valid, OsGroupRegs<TIN, E> &r)
{
    constexpr int n = E * sizeof(TIN) / 16;
#pragma unroll
    for (int i = 0; i < n; ++i)
        r.raw[i] = valid ? reinterpret_cast<const u32x4_t *>(src)[i] : u32x4_t{0u, 0u, 0u, 0u};
}

template <typename TIN, int E>
__device__ __forceinline__ void os_convert_group(const OsGroupRegs<TIN, E> &r, float (&xv)[E])
{
    if constexpr (sizeof(TIN) == 2) {
#pragma unroll
        for (int i = 0; i < E / 8; ++i)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t w = r.raw[i][d];
                xv[i * 8 + 2 * d] = __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
                xv[i * 8 + 2 * d + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
            }
    } else {
#pragma unroll
        for (int i = 0; i < E / 4; ++i)
#pragma unroll
            for (int d = 0; d < 4; ++d) xv[4 * i + d] = __uint_as_float(r.raw[i][d]);
    }
}

// RB = 32-row blocks per workgroup tile (1 or 2); LPG = lanes per quantization group in stage 1 (1 or 2).
template <typename TIN, int BITS, typename TOUT, int RB, int LPG, int CB>
__global__ void __launch_bounds__(kOsWaves * 64)
otf_small_kernel(const TIN *__restrict__ x, const float *__restrict__ a_thr, const float *__restrict__ a_cb,
                 const uint8_t *__restrict__ pw, const float *__restrict__ w_cb,
                 const float *__restrict__ wc, const float *__restrict__ ws, const float *__restrict__ wcs,
                 const float *__restrict__ bias, __half *__restrict__ x_hat_ws, TOUT *__restrict__ y,
                 int M, int N, int K, float eps, int tile_bytes, int partial_off,
                 const float *__restrict__ ln_w, const float *__restrict__ ln_b, float ln_eps, int ln_off,
                 const TOUT *residual, int gelu, const float *__restrict__ nx_thr, const float *__restrict__ nx_cb, int nx_off)
{
    constexpr int L = 1 << BITS;
    constexpr int RT = 32 * RB;
    constexpr int kOsCols = 32 * CB;
    constexpr int kOsRedPitch = os_red_pitch(CB);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // [x_hat tile | partial tiles] [activation LUT] [weight LUT] [buckets] [per-wave flags]; the partial tiles of
    // the reduction follow the x_hat tile (partial_off == tile_bytes) or, when K is too long for both, reuse its space
    // (partial_off == 0) after a barrier.
    unsigned char *xt = smem;
    unsigned char *partial = smem + partial_off;
    const int front = max(tile_bytes, partial_off + kOsWaves * RT * kOsRedPitch);
    float *a_lut = reinterpret_cast<float *>(smem + front);
    float *w_lut = a_lut + L * 64;
    Bucket *table = reinterpret_cast<Bucket *>(w_lut + L * 64);
    int *slow_slots = reinterpret_cast<int *>(table + kMaxBuckets + 64);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int lh = lane >> 5;
    const int m0 = blockIdx.y * RT, n0 = blockIdx.x * kOsCols;
    const int G = K / 64;
    const int row_pitch = os_row_pitch(G);
    const int64_t pcols = static_cast<int64_t>(K) * BITS / 8;

    // ---- weights of this wave's first group: requested now, used after stage 1 ---------------------------
    const uint8_t *w_src[CB];
    const float *wc_src[CB], *ws_src[CB], *wcs_src[CB];
#pragma unroll
    for (int j = 0; j < CB; ++j) {
        const int n = min(n0 + j * 32 + lr, N - 1);
        w_src[j] = pw + static_cast<int64_t>(n) * pcols + lh * (4 * BITS);
        wc_src[j] = wc + static_cast<int64_t>(n) * G;
        ws_src[j] = ws + static_cast<int64_t>(n) * G;
        wcs_src[j] = wcs + static_cast<int64_t>(n) * G;
    }
    auto fetch_w = [&](int g, OsWeights<BITS, CB> &o) {
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            os_load_codes<BITS>(w_src[j] + g * (8 * BITS), o.codes[j]);
            o.c[j] = wc_src[j][g];
            o.s[j] = ws_src[j][g];
            o.m[j] = wcs_src[j][g];
        }
    };
    OsWeights<BITS, CB> o0, o1;
    if (wave < G) fetch_w(wave, o0);

    // ---- stage 1: x_hat of the RT rows into LDS -----------------------------------------------------------
    // A wave tile is GPT consecutive groups of the row tile (group f = row f / G, group f % G), LPG lanes per group,
    // each lane holding EL consecutive inputs.  With two lanes per group the per-lane instruction chain, which is
    // what a launch this small waits for, is half as long (arcq_act_quant_core.h); it is used while the row tile is
    // at most eight such tiles (K <= 512 for 32 rows), i.e. while it does not add a round.
    // With a LayerNorm in front (ln_w != nullptr) a wave tile holds whole rows only (floor(slots / G) rows, the
    // remaining slots idle), so that a row's sums never leave the wave.
    constexpr int EL = 64 / LPG, SLOTS = 64 / LPG;
    const int groups = RT * G;
    const int gpt = ln_w ? (SLOTS / G) * G : SLOTS;      // groups per wave tile
    const int slot = lane / LPG;
    auto tile_group = [&](int t) { return slot < gpt ? t * gpt + slot : groups; };      // `groups`: this lane idles
    OsGroupRegs<TIN, EL> in;
    auto fetch_x = [&](int t) {
        const int f = tile_group(t);
        const int row = f / G, g = f - row * G;
        os_fetch_group<TIN, EL>(x + static_cast<int64_t>(min(m0 + row, M - 1)) * K + g * 64 + (lane % LPG) * EL,
                               f < groups && m0 + row < M, in);
    };
    float xv[EL];
    float mu = 0.0f, var = 0.0f, s = 0.0f;
    auto stats = [&]() {
        os_convert_group<TIN, EL>(in, xv);
    };
    // LayerNorm of the rows of tile t, on xv in place: arithmetic and summation order of the stand-alone LayerNorm +
    // stage-1 kernel (act_quant_rows_ln_kernel): every half group of 32 values is summed serially, a row's 2 G
    // partial sums are added in order, mean = sum / K, var = the same sum over (x - mean)^2, / K,
    // y = ((x - mean) * (1 / sqrt(var + eps))) * weight + bias, rounded to x's type.  The partial sums of a wave's
    // rows meet in a wave-private piece of LDS (LDS operations of one wave execute in order: no barrier needed).
    float *ln_part = reinterpret_cast<float *>(smem + ln_off) + wave * 128;
    auto layernorm = [&](int t) {
        constexpr int H = EL / 32;                    // half groups per lane
        const int f = tile_group(t);
        const bool act = f < groups;
        const int fl = act ? slot : 0;                // idle lanes read the first row's sums and write nothing
        const int rl = fl / G, g = fl - rl * G;
        const int base = rl * 2 * G;
        const int mine = base + 2 * g + (LPG == 2 ? (lane & 1) : 0);
        auto row_total = [&](const float (&ps)[H]) {
            if (act) {
#pragma unroll
                for (int h = 0; h < H; ++h) ln_part[mine + h] = ps[h];
            }
            __builtin_amdgcn_wave_barrier();
            float acc = 0.0f;
            for (int i = 0; i < 2 * G; ++i) acc += ln_part[base + i];
            __builtin_amdgcn_wave_barrier();
            return acc;
        };
        const float fk = static_cast<float>(K);
        const float4 *gp = reinterpret_cast<const float4 *>(ln_w + g * 64 + (lane % LPG) * EL);
        const float4 *bp = reinterpret_cast<const float4 *>(ln_b + g * 64 + (lane % LPG) * EL);
        // Half a group per lane: weight and bias are requested before the sums (64 registers); a whole group per lane
        // has no registers to spare and loads them where they are used.
        constexpr int PRE = LPG == 2 ? EL / 4 : 1;
        float4 gpre[PRE], bpre[PRE];
        if constexpr (LPG == 2) {
#pragma unroll
            for (int j4 = 0; j4 < PRE; ++j4) gpre[j4] = gp[j4], bpre[j4] = bp[j4];
        }
        float ps[H];
#pragma unroll
        for (int h = 0; h < H; ++h) {
            float a = 0.0f;
#pragma unroll
            for (int j = 0; j < 32; ++j) a += xv[32 * h + j];
            ps[h] = a;
        }
        const float mean = row_total(ps) / fk;
#pragma unroll
        for (int h = 0; h < H; ++h) {
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                xv[32 * h + j] -= mean;
                const float sq = xv[32 * h + j] * xv[32 * h + j];
                q += sq;
            }
            ps[h] = q;
        }
        const float var_row = row_total(ps) / fk;
        const float rstd = 1.0f / sqrtf(var_row + ln_eps);
#pragma unroll
        for (int j4 = 0; j4 < EL / 4; ++j4) {
            float4 gv, bv;
            if constexpr (LPG == 2) gv = gpre[j4], bv = bpre[j4];
            else gv = gp[j4], bv = bp[j4];
            const float g4[4] = {gv.x, gv.y, gv.z, gv.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float tt = xv[4 * j4 + e] * rstd;
                const float u = tt * g4[e];
                if constexpr (sizeof(TIN) == 2) xv[4 * j4 + e] = __half2float(__float2half_rn(u + b4[e]));
                else xv[4 * j4 + e] = u + b4[e];
            }
        }
    };
    // Wave w owns the tiles w, w + 8, ... of the row tile.  With fewer than eight tiles the waves without one build
    // the lookup tables while the others take their statistics, and one barrier joins the two halves; otherwise all
    // eight waves build the tables between the two halves of their first tile.
    const int n_tiles = (groups + gpt - 1) / gpt;
    const bool spare_waves = n_tiles < kOsWaves;
    const int tile_waves = spare_waves ? n_tiles : kOsWaves;
    const bool has_tile = wave < n_tiles;
    if (has_tile) fetch_x(wave);
    float th[L - 1], cbv[L];
    load_quant_params<BITS>(a_thr, a_cb, th, cbv);
    const BucketScale bq = pick_bucket_scale<BITS>(th);
    if (spare_waves && !has_tile)
        build_quant_tables_by<BITS>(th, cbv, bq, a_lut, table, slow_slots, tid - tile_waves * 64, (kOsWaves - tile_waves) * 64);
    if (wave == kOsWaves - 1) {
#pragma unroll
        for (int c = 0; c < L; ++c) w_lut[c * 64 + lane] = w_cb[c];
    }
    if (has_tile) {
        stats();
        if (wave + kOsWaves < n_tiles) fetch_x(wave + kOsWaves);      // the next tile's inputs, one round ahead
        if (ln_w) layernorm(wave);
        if constexpr (LPG == 1) group_stats64(xv, eps, mu, var, s);
        else group_stats32x2(xv, eps, mu, var, s);
    }
    if (!spare_waves) build_quant_tables_by<BITS>(th, cbv, bq, a_lut, table, slow_slots, tid, kOsWaves * 64);
    __syncthreads();
    const bool write_ws = (x_hat_ws != nullptr) && blockIdx.x == 0;
    bool table_ok = true;
    for (int w = 0; w < (spare_waves ? kOsWaves - tile_waves : kOsWaves); ++w) table_ok = table_ok && (slow_slots[w] == 0);
    // Quantize-the-output mode (nx_thr != nullptr: y receives stage 1 of the layer that consumes this one's output):
    // that layer's lookup tables are built by the waves without a stage-1 tile while the others run theirs, or, when
    // every wave has a tile, by all of them behind it.
    float *n_lut = reinterpret_cast<float *>(smem + nx_off);
    Bucket *n_table = reinterpret_cast<Bucket *>(n_lut + L * 64);
    int *n_slots = reinterpret_cast<int *>(n_table + kMaxBuckets + 64);
    const int n_builders = spare_waves ? kOsWaves - tile_waves : kOsWaves;
    auto build_next_tables = [&]() {
        float nth[L - 1], ncb[L];
        load_quant_params<BITS>(nx_thr, nx_cb, nth, ncb);
        const BucketScale nbq = pick_bucket_scale<BITS>(nth);
        build_quant_tables_by<BITS>(nth, ncb, nbq, n_lut, n_table, n_slots, tid - (kOsWaves - n_builders) * 64, n_builders * 64);
    };
    if (nx_thr && spare_waves && !has_tile) build_next_tables();
    for (int t = wave; t < n_tiles; t += kOsWaves) {
        if (t != wave) {                       // later tiles of this wave: their inputs were requested a round ago
            stats();
            if (t + kOsWaves < n_tiles) fetch_x(t + kOsWaves);
            if (ln_w) layernorm(t);
            if constexpr (LPG == 1) group_stats64(xv, eps, mu, var, s);
            else group_stats32x2(xv, eps, mu, var, s);
        }
        const int f = tile_group(t);
        const int row = f / G, g = f - row * G;
        const bool valid = f < groups && m0 + row < M;
        float sum_codes;
        if constexpr (LPG == 1) {
            uint32_t code[1];
            group_codes64<BITS, false>(xv, mu, var, s, th, bq, table, a_lut, table_ok, lane, sum_codes, code);
        } else {
            group_codes32x2<BITS>(xv, mu, var, s, th, bq, table, a_lut, table_ok, lane, sum_codes);
        }
        const float code_mean = sum_codes * 0.015625f;
        u32x4_t out[EL / 8];
#pragma unroll
        for (int i = 0; i < EL / 8; ++i)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const int j = i * 8 + 2 * d;
                const __half2 h = __floats2half2_rn(fma_f32(s, xv[j] - code_mean, mu), fma_f32(s, xv[j + 1] - code_mean, mu));
                out[i][d] = *reinterpret_cast<const uint32_t *>(&h);
            }
        const int part = (lane % LPG) * EL;      // first element of this lane inside its group
        if (f < groups) {
            unsigned char *dst = xt + row * row_pitch + g * kOsGroupPitch + part * 2;
#pragma unroll
            for (int i = 0; i < EL / 8; ++i) reinterpret_cast<u32x4_t *>(dst)[i] = out[i];
        }
        if (write_ws && valid) {
            u32x4_t *dst = reinterpret_cast<u32x4_t *>(x_hat_ws + static_cast<int64_t>(m0 + row) * K + g * 64 + part);
#pragma unroll
            for (int i = 0; i < EL / 8; ++i) dst[i] = out[i];
        }
    }
    if (nx_thr && !spare_waves) build_next_tables();
    __syncthreads();

    // The thread's outputs in the epilogue (E consecutive ones of a row) are known now: their bias and residual values
    // are requested here, so that the loads travel under the product instead of after it.
    constexpr int E = RT * kOsCols / (kOsWaves * 64);            // outputs per thread, consecutive in a row (8, 4 or 2)
    constexpr int TPR = kOsCols / E;                       // threads per row
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
    // ---- stages 2+3: split-K product, wave w takes groups w, w+8, ... --------------------------------------
    float16_t acc[RB][CB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const char *lut_lane = reinterpret_cast<const char *>(w_lut) + lane * 4;
    const unsigned char *a_lane = xt + lr * row_pitch + lh * 64;
    auto compute = [&](int g, const OsWeights<BITS, CB> &o) {
        float mg[CB];
#pragma unroll
        for (int j = 0; j < CB; ++j) mg[j] = o.m[j] * 0.015625f;       // S/64, exact
        const unsigned char *a_g = a_lane + g * kOsGroupPitch;
        float wv[CB][32];         // all table lookups are issued before the first is used
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int q = 0; q < 32; ++q)
                wv[j][q] = *reinterpret_cast<const float *>(lut_lane + (os_code_at<BITS>(o.codes[j], q) << 8));
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
                const half8_t af = *reinterpret_cast<const half8_t *>(a_g + i * 32 * row_pitch + kk * 16);
#pragma unroll
                for (int j = 0; j < CB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af, acc[i][j], 0, 0, 0);
            }
        }
    };
    for (int g = wave; g < G; g += 2 * kOsWaves) {
        if (g + kOsWaves < G) fetch_w(g + kOsWaves, o1);
        compute(g, o0);
        if (g + kOsWaves < G) {
            if (g + 2 * kOsWaves < G) fetch_w(g + 2 * kOsWaves, o0);
            compute(g + kOsWaves, o1);
        }
    }
    // ---- reduction over the waves in a fixed order, bias, output -------------------------------------------
    if (partial_off < tile_bytes) __syncthreads();      // the partial tiles reuse the x_hat tile: every wave is done reading it
    unsigned char *mine = partial + wave * (RT * kOsRedPitch);
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4_t v;
                v[0] = acc[i][j][4 * q]; v[1] = acc[i][j][4 * q + 1]; v[2] = acc[i][j][4 * q + 2]; v[3] = acc[i][j][4 * q + 3];
                *reinterpret_cast<f32x4_t *>(mine + (i * 32 + lr) * kOsRedPitch + (j * 32 + 8 * q + 4 * lh) * 4) = v;
            }
    __syncthreads();
    float sum[E];
#pragma unroll
    for (int e = 0; e < E; ++e) sum[e] = 0.0f;
    const int waves_used = min(kOsWaves, G);
    for (int w = 0; w < waves_used; ++w) {
        const unsigned char *src = partial + w * (RT * kOsRedPitch) + row * kOsRedPitch + col * 4;
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
    if constexpr (CB == 2 && sizeof(TOUT) == 2) {
        if (nx_thr) {          // workgroup-uniform; the launcher guarantees N % 64 == 0 (the tile is 32 rows x one group)
            // The tile's outputs, rounded (and post-processed) as they would have been stored, meet in LDS; wave 0 then
            // quantizes them as the consuming layer's stage 1 would -- two lanes per group -- and stores x_hat row-major.
            TOUT out[E];
#pragma unroll
            for (int e = 0; e < E; ++e)
                out[e] = post_op1<TOUT>(from_float<TOUT>(sum[e] + bv[e]), residual != nullptr, rv[e], gelu != 0);
            __syncthreads();                         // every thread is done reading the partial tiles
            unsigned char *yt = partial;             // [32 rows][128 + 16 bytes]
            *reinterpret_cast<u32x2_t *>(yt + row * 144 + col * 2) = *reinterpret_cast<const u32x2_t *>(out);
            __syncthreads();
            if (wave == 0) {
                float nth[L - 1], ncb[L];
                load_quant_params<BITS>(nx_thr, nx_cb, nth, ncb);
                const BucketScale nbq = pick_bucket_scale<BITS>(nth);
                bool n_ok = true;
                for (int w = 0; w < n_builders; ++w) n_ok = n_ok && (n_slots[w] == 0);
                const int r2 = lane >> 1, half = lane & 1;
                float v[32];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4_t q = *reinterpret_cast<const u32x4_t *>(yt + r2 * 144 + half * 64 + i * 16);
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        v[8 * i + 2 * d] = __half2float(__ushort_as_half(static_cast<unsigned short>(q[d] & 0xffffu)));
                        v[8 * i + 2 * d + 1] = __half2float(__ushort_as_half(static_cast<unsigned short>(q[d] >> 16)));
                    }
                }
                float nmu, nvar, ns, nsum;
                group_stats32x2(v, eps, nmu, nvar, ns);
                group_codes32x2<BITS>(v, nmu, nvar, ns, nth, nbq, n_table, n_lut, n_ok, lane, nsum);
                const float code_mean = nsum * 0.015625f;
                if (m0 + r2 < M) {
                    u32x4_t *dst = reinterpret_cast<u32x4_t *>(y + static_cast<int64_t>(m0 + r2) * N + n0 + half * 32);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        u32x4_t o;
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const int j = 8 * i + 2 * d;
                            const __half2 h = __floats2half2_rn(fma_f32(ns, v[j] - code_mean, nmu), fma_f32(ns, v[j + 1] - code_mean, nmu));
                            o[d] = *reinterpret_cast<const uint32_t *>(&h);
                        }
                        dst[i] = o;
                    }
                }
            }
            return;
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

template <typename TIN, int BITS, typename TOUT, int RB, int LPG, int CB>
static void launch_os(const OtfSmallArgs &a, hipStream_t stream)
{
    constexpr int L = 1 << BITS;
    constexpr int RT = 32 * RB;
    constexpr int kOsCols = 32 * CB;
    constexpr int kOsRedPitch = os_red_pitch(CB);
    const int G = a.K / 64;
    const int xhat_bytes = RT * os_row_pitch(G);
    const int partial_bytes = kOsWaves * RT * kOsRedPitch;
    const int tile_bytes = xhat_bytes;
    // (lookup tables, per-wave flags, and -- with a LayerNorm in front -- 128 floats per wave for the rows' partial sums)
    const size_t tables = 2 * L * 64 * sizeof(float) + (kMaxBuckets + 64) * sizeof(Bucket) + 64;
    const size_t ln_bytes = a.ln_weight ? kOsWaves * 128 * sizeof(float) : 0;
    // Both regions side by side while they fit 160 KB of LDS; else the partial tiles reuse the x_hat tile's space.
    const size_t nx_need = a.next_thr ? L * 64 * sizeof(float) + (kMaxBuckets + 64) * sizeof(Bucket) + 64 : 0;
    const int partial_off = (tile_bytes + partial_bytes + tables + ln_bytes + nx_need <= 160 * 1024) ? tile_bytes : 0;
    const size_t front = partial_off ? tile_bytes + partial_bytes : (tile_bytes > partial_bytes ? tile_bytes : partial_bytes);
    const int ln_off = static_cast<int>(front + tables);
    // (quantize-the-output mode: a second set of lookup tables, for the consuming layer's codebook)
    const size_t nx_bytes = a.next_thr ? L * 64 * sizeof(float) + (kMaxBuckets + 64) * sizeof(Bucket) + 64 : 0;
    const int nx_off = static_cast<int>(front + tables + ln_bytes);
    const size_t smem = front + tables + ln_bytes + nx_bytes;
    auto kernel = otf_small_kernel<TIN, BITS, TOUT, RB, LPG, CB>;
    allow_dynamic_lds<otf_small_kernel<TIN, BITS, TOUT, RB, LPG, CB>>(160 * 1024);      // (the size varies with K: allow the CU's whole LDS)
    const dim3 grid((a.N + kOsCols - 1) / kOsCols, (a.M + RT - 1) / RT);
    hipLaunchKernelGGL(kernel, grid, dim3(kOsWaves * 64), smem, stream, static_cast<const TIN *>(a.x), a.a_thr, a.a_cb,
                       a.pw, a.w_cb, a.wc, a.ws, a.wcs, a.bias, static_cast<__half *>(a.x_hat_ws),
                       static_cast<TOUT *>(a.y), a.M, a.N, a.K, a.eps, tile_bytes, partial_off, a.ln_weight, a.ln_bias,
                       a.ln_eps, ln_off, static_cast<const TOUT *>(a.residual), a.gelu ? 1 : 0, a.next_thr, a.next_cb, nx_off);
}

template <typename TIN, int BITS, typename TOUT>
static void launch_os_rb(const OtfSmallArgs &a, hipStream_t stream)
{
    // Two lanes per group while the 32-row tile is at most eight 32-group tiles: half the chain, no extra round.
    // 32-column tiles while their grid fits the chip in one wave of workgroups: half the weight rows to rebuild per wave
    // and half the reduction, at the price of twice as many workgroups repeating stage 1 (M = 197, K = 384:
    // N = 1152, 252 tiles, 8.9 -> 8.0 us; N = 384 8.7 -> 7.6; N = 1536, 336 tiles, 8.7-9.4 -> 10.0).  Bit-identical.
    // (quantizing the output for the next layer needs a whole group per tile row: 64 columns)
    const bool narrow = !a.next_thr && static_cast<int64_t>((a.N + 31) / 32) * ((a.M + 31) / 32) <= 256;
    if (32 * (a.K / 64) <= 8 * 32) {
        if (narrow) launch_os<TIN, BITS, TOUT, 1, 2, 1>(a, stream);
        else launch_os<TIN, BITS, TOUT, 1, 2, 2>(a, stream);
    } else {
        if (narrow) launch_os<TIN, BITS, TOUT, 1, 1, 1>(a, stream);
        else launch_os<TIN, BITS, TOUT, 1, 1, 2>(a, stream);
    }
}

template <typename TIN, typename TOUT>
static void launch_os_bits(const OtfSmallArgs &a, hipStream_t stream)
{
    if (a.bits == 4) launch_os_rb<TIN, 4, TOUT>(a, stream);
    else if (a.bits == 3) launch_os_rb<TIN, 3, TOUT>(a, stream);
    else launch_os_rb<TIN, 2, TOUT>(a, stream);
}

// Every column tile repeats the activation quantizer of its 32 rows (K / 64 groups each, one 64-group tile per wave
// and round).  Measured at 197 rows: one launch wins while that is a single round and the grid fits the chip in one
// wave of workgroups (K = 384: 10.6 us against 12.6; K = 768, N = 2304: 13.8 against 15.5) and loses beyond (K = 768,
// N = 3072, 336 workgroups: 23.4 against 17.3; K = 1536, three rounds: 23.7 against 19.7).  `any_supported` is what
// the kernel can run at all (the x_hat tile of 32 rows must fit LDS): ARCQ_OTF_FUSED=2 asks for that.
bool otf_small_supported(int64_t M, int64_t N, int64_t K, bool any_supported)
{
    if (!(M < 512 && K >= 64 && K % 64 == 0 && K <= 1536)) return false;
    if (any_supported || K <= 512) return true;
    return K <= 768 && ((N + 63) / 64) * ((M + 31) / 32) <= 256;
}

void launch_otf_small(const OtfSmallArgs &a, hipStream_t stream)
{
    if (a.x_f16) {
        if (a.y_f16) launch_os_bits<__half, __half>(a, stream);
        else launch_os_bits<__half, float>(a, stream);
    } else {
        if (a.y_f16) launch_os_bits<float, __half>(a, stream);
        else launch_os_bits<float, float>(a, stream);
    }
}

}  // namespace arcq
