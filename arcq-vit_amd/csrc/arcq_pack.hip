// Bit packing of ARCQ codes: LSB-first bitstream per row
// (layout: EXT/arcq_pack_kernel.cu:8-36).
#include "arcq_common.h"

namespace arcq {

// One thread per OUTPUT byte: gathers the (at most ceil(8/bits)+1) codes whose
// bits fall into that byte, so no read-modify-write and no pre-zeroed output.
__global__ void __launch_bounds__(256)
pack_codes_kernel(const int64_t *__restrict__ codes, uint8_t *__restrict__ packed,
                  int64_t rows, int64_t length, int64_t pcols, int bits)
{
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= rows * pcols) return;
    const int64_t row = idx / pcols;
    const int64_t b = idx - row * pcols;
    const int64_t *__restrict__ in = codes + row * length;
    const unsigned mask = (1u << bits) - 1u;
    const int64_t bit_lo = b * 8;
    int64_t j = bit_lo / bits;  // first code touching this byte
    unsigned out = 0;
    for (; j < length && j * bits < bit_lo + 8; ++j) {
        const unsigned c = static_cast<unsigned>(in[j]) & mask;
        const int64_t rel = j * bits - bit_lo;  // in (-bits, 8)
        out |= (rel >= 0) ? (c << rel) : (c >> (-rel));
    }
    packed[idx] = static_cast<uint8_t>(out & 0xffu);
}

template <typename OUT>
__global__ void __launch_bounds__(256)
unpack_codes_kernel(const uint8_t *__restrict__ packed, OUT *__restrict__ codes,
                    int64_t rows, int64_t length, int64_t pcols, int bits)
{
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= rows * length) return;
    const int64_t row = idx / length;
    const int64_t col = idx - row * length;
    codes[idx] = static_cast<OUT>(get_code(packed + row * pcols, col, bits));
}

static int check_pack_args(const char *fn, const void *a, const void *b, int64_t rows, int64_t length, int bits)
{
    if (!bits_ok(bits)) return fail(ARCQ_ERR_BITS, "%s: bits must be 2, 3, or 4", fn);
    if (rows < 0 || length < 0) return fail(ARCQ_ERR_SHAPE, "%s: negative size", fn);
    if (rows * length > 0 && (!a || !b)) return fail(ARCQ_ERR_NULL, "%s: NULL tensor pointer", fn);
    if (rows * length >= (int64_t(1) << 39)) return fail(ARCQ_ERR_SHAPE, "%s: tensor too large", fn);
    return ARCQ_OK;
}

}  // namespace arcq

using namespace arcq;

ARCQ_API int arcq_pack_codes(const int64_t *codes, uint8_t *packed, int64_t rows, int64_t length, int bits, void *stream)
{
    int rc = check_pack_args("arcq_pack_codes", codes, packed, rows, length, bits);
    if (rc != ARCQ_OK) return rc;
    const int64_t pcols = packed_cols(length, bits);
    const int64_t total = rows * pcols;
    if (total == 0) return ARCQ_OK;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    hipLaunchKernelGGL(pack_codes_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       codes, packed, rows, length, pcols, bits);
    return launch_status("arcq_pack_codes");
}

ARCQ_API int arcq_unpack_codes(const uint8_t *packed, int64_t *codes, int64_t rows, int64_t length, int bits, void *stream)
{
    int rc = check_pack_args("arcq_unpack_codes", packed, codes, rows, length, bits);
    if (rc != ARCQ_OK) return rc;
    const int64_t total = rows * length;
    if (total == 0) return ARCQ_OK;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    hipLaunchKernelGGL(unpack_codes_kernel<int64_t>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       packed, codes, rows, length, packed_cols(length, bits), bits);
    return launch_status("arcq_unpack_codes");
}

ARCQ_API int arcq_unpack_codes_u8(const uint8_t *packed, uint8_t *codes, int64_t rows, int64_t length, int bits, void *stream)
{
    int rc = check_pack_args("arcq_unpack_codes_u8", packed, codes, rows, length, bits);
    if (rc != ARCQ_OK) return rc;
    const int64_t total = rows * length;
    if (total == 0) return ARCQ_OK;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    hipLaunchKernelGGL(unpack_codes_kernel<uint8_t>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       packed, codes, rows, length, packed_cols(length, bits), bits);
    return launch_status("arcq_unpack_codes_u8");
}
