// Shared host/device helpers for the ARCQ HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include "arcq_hip.h"

#define ARCQ_API extern "C" __attribute__((visibility("default")))

namespace arcq {

// Records a message for arcq_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Turns hipGetLastError() after a launch into the ABI's return value.
int launch_status(const char *what);

// Tuning switches from the environment (ARCQ_GEMM_KERNEL, ARCQ_OTF_FUSED, ARCQ_PAIR, ARCQ_ROWS), read once per process;
// arcq_reload_tuning() reads them again.  nullptr = not set.
struct Tuning {
    const char *gemm_kernel;   // "stream" | "slab" | "small" | "splitk" | "slab8" | "prebuilt"
    const char *otf_fused;     // "0" | "2"
    const char *pair;          // "0" | "1"
    const char *rows;          // "0" | "1": the one-launch row-stationary layer kernel off / wherever it can run
    long long rows_wait_ticks; // bound of that kernel's wait for the other workgroups, in ticks of the 100 MHz clock
};
constexpr long long kRowsWaitTicks = 50000;     // 0.5 ms
const Tuning &tuning();

__host__ __device__ inline bool bits_ok(int bits) { return bits == 2 || bits == 3 || bits == 4; }
__host__ __device__ inline int64_t packed_cols(int64_t length, int bits) { return (length * bits + 7) / 8; }
inline bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Code j of a row whose packed bytes start at `row` (EXT/arcq_pack_kernel.cu:8-20).
// The second byte is read only when the code really straddles, so the read
// never leaves the row.
__device__ __forceinline__ int get_code(const uint8_t *__restrict__ row, int64_t idx, int bits)
{
    const int64_t bit_offset = idx * bits;
    const int64_t byte_idx = bit_offset >> 3;
    const int shift = static_cast<int>(bit_offset & 7);
    unsigned v = static_cast<unsigned>(row[byte_idx]) >> shift;
    if (shift + bits > 8) v |= static_cast<unsigned>(row[byte_idx + 1]) << (8 - shift);
    return static_cast<int>(v & ((1u << bits) - 1u));
}

// Eight consecutive codes starting at a multiple of eight occupy exactly `BITS`
// bytes.  Returns them as one little-endian integer (code i at bit i*BITS).
template <int BITS>
__device__ __forceinline__ uint32_t load_codes8(const uint8_t *__restrict__ p)
{
    if constexpr (BITS == 4) {
        return *reinterpret_cast<const uint32_t *>(p);
    } else if constexpr (BITS == 2) {
        return *reinterpret_cast<const uint16_t *>(p);
    } else {
        return static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8) | (static_cast<uint32_t>(p[2]) << 16);
    }
}

// fma with the fp32 rounding made visible.  Without the barrier the compiler fuses a following
// float->half conversion into v_fma_mixlo_f16, which rounds the exact result once to fp16; the
// contract here (and what the reference's kernels do) is round to fp32, then round to fp16.
__device__ __forceinline__ float fma_f32(float a, float b, float c)
{
    float v = __fmaf_rn(a, b, c);
    asm("" : "+v"(v));   // not volatile: opaque to instruction selection, free for the scheduler to move
    return v;
}

// 16-byte store with the streaming ("nt") hint, for the GEMM output.  Plain stores leave the lines dirty in L2 and the
// launch ends only when all of them have been written back; streamed lines leave while the kernel still computes
// (measured: 10 % of the duration of a GEMM launch that writes 39 MB).  Stage 1 keeps plain stores for x_hat: streaming
// them shortens stage 1 by 1 us and lengthens the GEMM that follows by more, because it then misses L2 on x_hat.
typedef uint32_t u32x4_store_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_streaming16(void *p, uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    u32x4_store_t v;
    v[0] = a; v[1] = b; v[2] = c; v[3] = d;
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4_store_t *>(p));
}

// 16-byte store that writes through L2 (agent scope) and keeps the line there: for x_hat, which the GEMM launch that
// follows reads back.  The launch again has nothing to write back when it ends (stage 1: -0.8 us), and unlike a
// streamed line this one still hits L2 in the next launch.
__device__ __forceinline__ void store_writethrough16(void *p, uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    u32x4_store_t v;
    v[0] = a; v[1] = b; v[2] = c; v[3] = d;
    // The two wait states keep the next VALU instruction from overwriting the data registers while the store still
    // reads them (the compiler inserts them for its own wide stores; it does not look inside an asm statement).
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// Raises a kernel's dynamic LDS limit, once per device and kernel (the attribute belongs to the device's copy of
// the code object).  Kernel is the kernel's address as a template argument, so every kernel has its own record.
template <auto Kernel>
inline void allow_dynamic_lds(int bytes)
{
    static std::atomic<uint64_t> done{0};          // one bit per device index (mod 64: at worst a redundant call)
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t bit = uint64_t(1) << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return;
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    done.fetch_or(bit, std::memory_order_release);
}

// Order of the (row range, slab) tiles of a weight-stationary GEMM whose slabs are copied from a reconstructed
// weight matrix.  Workgroups are dealt to the 8 XCDs round-robin and every XCD takes a contiguous run of tile numbers;
// with the slab fastest a run covers all N / 128 slabs of one or two row ranges, so that the slabs sharing a range read
// x_hat through one L2 -- but once K spans several slab slices every pass over the rows copies the slab again, and
// N * K * 2 bytes of weights per XCD (6 MB for ViT-L qkv) do not stay in its 4 MB L2: measured at the L2, the launch
// then fetched 3.5 times the x_hat it needs.  Slabs are therefore dealt in groups whose weights fit half the L2
// (`group` slabs: 2 MB / (128 * K * 2), groups of equal size): a run then covers one group x several ranges, the
// re-copies hit L2, and x_hat is fetched once per group instead of once.  That trade is taken only where it saves
// traffic by this estimate: x_hat (M * K * 2 bytes) once more per additional group, against the weights
// (N * K * 2 bytes) once more per XCD and per pass after the first (`blocks_per_pass` = row blocks a workgroup
// multiplies per pass over K).  DeiT-B qkv / fc1: 58.8 -> 53.5 and 77.3 -> 68.5 us; ViT-L qkv / fc1: 1 % faster;
// ViT-L fc2 (K = 4096: x_hat is 413 MB) keeps the plain order, which is 2.4 % faster there.
__host__ __device__ inline int slab_group_size(int n_slabs, int K, int M, int blocks_per_range, int blocks_per_pass)
{
    const int64_t slab_bytes = int64_t(128) * K * 2;
    const int fit = static_cast<int>((int64_t(2) << 20) / slab_bytes);
    if (fit >= n_slabs) return n_slabs;
    const int passes = (blocks_per_range + blocks_per_pass - 1) / blocks_per_pass;
    if (fit < 1 || passes <= 1) return n_slabs;
    const int groups = (n_slabs + fit - 1) / fit;
    const int64_t extra_x = int64_t(M) * K * 2 * (groups - 1);
    const int64_t rereads_w = 8 * n_slabs * slab_bytes * (passes - 1);
    return extra_x < rereads_w ? (n_slabs + groups - 1) / groups : n_slabs;
}
__device__ __forceinline__ void tile_range_slab(int tile, int n_slabs, int row_ranges, int group, int &range, int &slab)
{
    if (group >= n_slabs) {
        range = tile / n_slabs;
        slab = tile - range * n_slabs;
        return;
    }
    const int per_group = group * row_ranges;       // tiles of a full group
    const int sg = tile / per_group;
    const int first = sg * group;
    const int size = min(group, n_slabs - first);
    const int rem = tile - sg * per_group;
    range = rem / size;
    slab = first + (rem - range * size);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(__half v) { return __half2float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_float<__half>(float v) { return __float2half_rn(v); }

// The exact (erf) GELU in fp32, (x * 0.5) * (1 + erf(x * sqrt(1/2))), with the fp32 rounding of the last product made
// visible: without the barrier the compiler may fuse that product with a following float->half conversion into one
// instruction that rounds the exact product once to fp16, which differs from round-to-fp32-then-fp16 (what an
// elementwise kernel computing in fp32 stores) on rare ties.
__device__ __forceinline__ float gelu_f32(float x)
{
    float v = (x * 0.5f) * (1.0f + erff(x * 0.70710678118654752440f));
    asm("" : "+v"(v));
    return v;
}

// Optional elementwise work on a GEMM's outputs after they have been rounded to the output type, each step rounding
// to that type again -- the values separate elementwise kernels on the stored tensor would produce:
//   gelu:     y = round(gelu(y)),  gelu(v) = (v * 0.5) * (1 + erf(v * sqrt(1/2)))    (the exact, erf-based GELU)
//   residual: y = round(y + r)     r [M,N] of the output type (e.g. the transformer block's skip connection)
// `v` holds 16 bytes of consecutive outputs of one row (8 fp16 or 4 fp32), `res` points at the residual values of the
// same positions (or is nullptr), of which the first `valid` may be read.
template <typename TOUT>
__device__ __forceinline__ void post_ops16(u32x4_store_t &v, const TOUT *res, bool gelu, int valid)
{
    constexpr int n = 16 / static_cast<int>(sizeof(TOUT));
    TOUT e[n];
    __builtin_memcpy(e, &v, 16);
    if (gelu) {
#pragma unroll
        for (int i = 0; i < n; ++i) {
            e[i] = from_float<TOUT>(gelu_f32(to_float(e[i])));
        }
    }
    if (res) {
        TOUT r[n];
        if (valid >= n && (reinterpret_cast<uintptr_t>(res) & 15) == 0) {
            const u32x4_store_t rv = *reinterpret_cast<const u32x4_store_t *>(res);
            __builtin_memcpy(r, &rv, 16);
        } else {
#pragma unroll
            for (int i = 0; i < n; ++i) r[i] = i < valid ? res[i] : from_float<TOUT>(0.0f);
        }
#pragma unroll
        for (int i = 0; i < n; ++i) e[i] = from_float<TOUT>(to_float(e[i]) + to_float(r[i]));
    }
    __builtin_memcpy(&v, e, 16);
}

// The same two steps on one output value (the small-M kernels, whose threads hold a few consecutive outputs each);
// `r` is the residual value, used when `has_res`.
template <typename TOUT>
__device__ __forceinline__ TOUT post_op1(TOUT v, bool has_res, TOUT r, bool gelu)
{
    if (gelu) v = from_float<TOUT>(gelu_f32(to_float(v)));
    if (has_res) v = from_float<TOUT>(to_float(v) + to_float(r));
    return v;
}

}  // namespace arcq
