// widen_codes.hip -- repack 2-, 3-, 5- and 6-bit codes as 4- or 8-bit codes.
//
// A code keeps its value, so scales and biases stay as they are: the product
// over the repacked matrix is the product over the original one.  Used for
// transpose=false calls at the widths whose rows the column loaders of the
// [K, N] kernels cannot address (3-, 5- and 6-bit codes straddle words), and
// for 2-bit codes along with them: one pass over the packed matrix, then the
// 4- or 8-bit kernel.
//
// Packing on both sides is the little-endian bit stream of mx.quantize
// (python/src/ops.cpp:4738-4742): code i of a row at bits [i b, (i + 1) b).
#include "qmm_args.h"

namespace mlxrocm {

namespace {

// One thread repacks 32 codes: BITS words in, OBITS words out.
template <int BITS, int OBITS>
__global__ __launch_bounds__(256) void widen_codes_kernel(
    const uint32_t* src,
    uint32_t* dst,
    size_t blocks) {
  const size_t t = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= blocks) {
    return;
  }
  uint32_t in[BITS + 1];
#pragma unroll
  for (int j = 0; j < BITS; ++j) {
    in[j] = src[t * BITS + j];
  }
  in[BITS] = 0u;
  uint32_t out[OBITS];
#pragma unroll
  for (int j = 0; j < OBITS; ++j) {
    out[j] = 0u;
  }
  constexpr uint32_t kMask = (1u << BITS) - 1u;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int bit = i * BITS;
    const int word = bit / 32;
    const int shift = bit % 32;
    const uint64_t two = (static_cast<uint64_t>(in[word + 1]) << 32) | in[word];
    const uint32_t code = static_cast<uint32_t>(two >> shift) & kMask;
    const int obit = i * OBITS;
    out[obit / 32] |= code << (obit % 32); // OBITS divides 32: no straddling
  }
#pragma unroll
  for (int j = 0; j < OBITS; ++j) {
    dst[t * OBITS + j] = out[j];
  }
}

} // namespace

// The width the codes of `bits` bits are repacked to (0: none needed).
int widened_bits(int bits) {
  switch (bits) {
    case 2:
    case 3:
      return 4;
    case 5:
    case 6:
      return 8;
    default:
      return 0;
  }
}

// `codes` codes (a multiple of 32) from src to dst, which holds `dst_words`
// words.  Thread t reads words [t bits, (t + 1) bits) and writes words
// [t wide, (t + 1) wide), t < codes / 32: the last word read is
// codes / 32 * bits - 1 (the packed matrix has exactly that many), the last
// word written codes / 32 * wide - 1, checked against the region here.
int launch_widen_codes(
    const uint32_t* src, uint32_t* dst, size_t dst_words, size_t codes, int bits, hipStream_t s) {
  const size_t blocks = codes / 32;
  const size_t grid = (blocks + 255) / 256;
  if (codes % 32 != 0 || grid > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] cannot repack %zu codes of %d bits", codes, bits);
  }
  const size_t wide = static_cast<size_t>(widened_bits(bits));
  if (wide == 0 || blocks > SIZE_MAX / 8 / sizeof(uint32_t) || blocks * wide > dst_words) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[qmm] repacking %zu codes of %d bits writes %zu words; the region holds %zu",
        codes, bits, blocks * wide, dst_words);
  }
  const unsigned g = static_cast<unsigned>(grid);
  MLXROCM_REHEARSE("widen_codes(%d->%d)", bits, widened_bits(bits));
  switch (bits) {
    case 2:
      widen_codes_kernel<2, 4><<<g, 256, 0, s>>>(src, dst, blocks);
      break;
    case 3:
      widen_codes_kernel<3, 4><<<g, 256, 0, s>>>(src, dst, blocks);
      break;
    case 5:
      widen_codes_kernel<5, 8><<<g, 256, 0, s>>>(src, dst, blocks);
      break;
    case 6:
      widen_codes_kernel<6, 8><<<g, 256, 0, s>>>(src, dst, blocks);
      break;
    default:
      return fail(MLXROCM_INVALID_ARGUMENT, "[qmm] no wider packing for %d-bit codes", bits);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

} // namespace mlxrocm
