// mfma_dequant.h -- pieces shared by the matrix-core kernels: the 16x16x32 MFMA
// wrappers, packed converts and the dequantization of packed codes two at a
// time.
#pragma once

#include <type_traits>
#include <utility>

#include "common.h"

namespace mlxrocm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

template <typename T>
__device__ __forceinline__ floatx4 mfma16(const uint4& a, const uint4& b, const floatx4& c);

template <>
__device__ __forceinline__ floatx4
mfma16<bf16_t>(const uint4& a, const uint4& b, const floatx4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <>
__device__ __forceinline__ floatx4
mfma16<f16_t>(const uint4& a, const uint4& b, const floatx4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(
      __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Two floats -> two T in one dword (lo in the low half), round to nearest even;
// the vector convert selects the packed hardware convert.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef T Tx2 __attribute__((ext_vector_type(2)));
  const floatx2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, Tx2));
}

// Code i (0..31) of the 32 codes held in BITS consecutive dwords.
template <int BITS>
__device__ __forceinline__ uint32_t code32(const uint32_t (&w)[BITS], int i) {
  const int bit = i * BITS;
  const int word = bit >> 5;
  const int sh = bit & 31;
  uint32_t v = w[word] >> sh;
  if (sh + BITS > 32) {
    v |= w[word + 1] << (32 - sh);
  }
  return v & ((1u << BITS) - 1u);
}

// Dequantization of the 32 codes held in BITS consecutive dwords, two codes at
// a time so that the work can be spread between MFMAs: pair<Q>() returns
// elements 2Q and 2Q+1 as fma(s, code, b) in fp32, rounded once to T and packed.
template <typename T, int BITS>
struct PairDequant {
  uint32_t lo, hi; // 4-bit: codes 0,2,4,6 / 1,3,5,7 of the current dword as bytes
  floatx2 flo, fhi; // 4-bit: two of those bytes each, converted

  // 4-bit codes are converted two at a time with the fp8 convert: a byte 0..15
  // read as an OCP e4m3 number is exactly code * 2^-9 (the format is linear
  // through its subnormals and first binade), so fma(512 s, code / 512, b) is
  // the same real product, and the same rounding, as fma(s, code, b).
  static constexpr float kCodeScale = BITS == 4 ? 512.0f : 1.0f;

  // low_part: return v - T(v) instead of v (the second term of the split of an
  // fp32 weight into two T values); wave-uniform.  `s` is kCodeScale times the
  // group's scale.
  template <int Q>
  __device__ __forceinline__ uint32_t
  pair(const uint32_t (&w)[BITS], float s, float b, bool low_part = false) {
    float c0, c1;
    if constexpr (BITS == 4) {
      constexpr int d = Q / 4;
      constexpr int j = Q % 4;
      if constexpr (j == 0) {
        lo = w[d] & 0x0f0f0f0fu;
        hi = (w[d] >> 4) & 0x0f0f0f0fu;
      }
      if constexpr (j % 2 == 0) {
        flo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(lo), j == 2);
        fhi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(hi), j == 2);
      }
      c0 = flo[j % 2];
      c1 = fhi[j % 2];
    } else if constexpr (BITS == 8) {
      constexpr int d = Q / 2;
      constexpr int j = Q % 2;
      c0 = static_cast<float>((w[d] >> (16 * j)) & 0xffu);
      c1 = static_cast<float>((w[d] >> (16 * j + 8)) & 0xffu);
    } else {
      c0 = static_cast<float>(code32<BITS>(w, 2 * Q));
      c1 = static_cast<float>(code32<BITS>(w, 2 * Q + 1));
    }
    float v0 = fmaf(s, c0, b);
    float v1 = fmaf(s, c1, b);
    if (low_part) {
      v0 -= static_cast<float>(static_cast<T>(v0));
      v1 -= static_cast<float>(static_cast<T>(v1));
    }
    return pack2<T>(v0, v1);
  }
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// The floating-point modes in the same shape: 32 codes of one row of W in four
// (e2m1) or eight (e4m3) consecutive dwords, pair<Q>() returns elements 2Q and
// 2Q+1 times their group's scale, packed as T.  Every such product is exact in
// bf16 and f16 (at most 4 significant bits times a power of two, or 2 times 4).
//   FP == 1: e2m1 codes, one power-of-two scale `s` for all 32 (mxfp4)
//   FP == 2: e4m3 codes, one power-of-two scale `s` for all 32 (mxfp8)
//   FP == 3: e2m1 codes, scale `s` for codes 0..15 and `b` for 16..31 (nvfp4)
// With a power-of-two scale the hardware convert applies it: one instruction
// per pair.  The e4m3 bytes 0x7f / 0xff, which the quantizer never writes, are
// NaN to that convert.
template <typename T, int FP>
struct FpPairDequant {
  static constexpr float kCodeScale = 1.0f;
  static constexpr int kWords = FP == 2 ? 8 : 4;

  template <int Q>
  __device__ __forceinline__ uint32_t
  pair(const uint32_t (&w)[kWords], float s, float b, bool = false) {
    if constexpr (FP == 1) {
      if constexpr (std::is_same<T, bf16_t>::value) {
        return __builtin_bit_cast(
            uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[Q / 4], s, Q % 4));
      } else {
        return __builtin_bit_cast(
            uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[Q / 4], s, Q % 4));
      }
    } else if constexpr (FP == 2) {
      if constexpr (std::is_same<T, bf16_t>::value) {
        return __builtin_bit_cast(
            uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[Q / 2], s, Q % 2 == 1));
      } else {
        return __builtin_bit_cast(
            uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[Q / 2], s, Q % 2 == 1));
      }
    } else {
      const floatx2 v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[Q / 4], 1.0f, Q % 4);
      const float sc = Q < 8 ? s : b;
      return pack2<T>(v[0] * sc, v[1] * sc);
    }
  }
};

template <typename T, int FP, int... Q>
__device__ __forceinline__ void dequant32_fp_impl(
    const uint32_t (&w)[FpPairDequant<T, FP>::kWords],
    float s,
    float b,
    uint32_t (&out)[16],
    std::integer_sequence<int, Q...>) {
  FpPairDequant<T, FP> dq;
  ((out[Q] = dq.template pair<Q>(w, s, b)), ...);
}

template <typename T, int FP>
__device__ __forceinline__ void dequant32_fp(
    const uint32_t (&w)[FpPairDequant<T, FP>::kWords],
    float s,
    float b,
    uint32_t (&out)[16]) {
  dequant32_fp_impl<T, FP>(w, s, b, out, std::make_integer_sequence<int, 16>{});
}

// Dequantization of a 4 (k) x 8 (n) block of a [K, N] weight matrix whose codes
// run along n: w holds, row by row, the BITS / 4 words with the 8 codes of each
// of the 4 rows, s / b the rows' scale and bias.  pair<Q>() returns column
// Q / 2, rows 2 (Q % 2) and 2 (Q % 2) + 1, rounded to T and packed: two
// neighbours along k, which is how the LDS tile wants them.
template <typename T, int BITS>
struct ColDequant {
  static_assert(BITS == 4 || BITS == 8, "columns of 4- and 8-bit codes");
  uint32_t lo[4], hi[4]; // 4-bit: even / odd columns of a row as bytes

  template <int Q>
  __device__ __forceinline__ uint32_t
  pair(const uint32_t (&w)[BITS], const float (&s)[4], const float (&b)[4]) {
    constexpr int i = Q / 2;      // column 0..7
    constexpr int j0 = 2 * (Q % 2); // first of the two rows
    float c0, c1;
    if constexpr (BITS == 4) {
      if constexpr (i == 0) {
        lo[j0] = w[j0] & 0x0f0f0f0fu;
        lo[j0 + 1] = w[j0 + 1] & 0x0f0f0f0fu;
        asm("" : "+v"(lo[j0]));
        asm("" : "+v"(lo[j0 + 1]));
      }
      if constexpr (i == 1) {
        hi[j0] = (w[j0] >> 4) & 0x0f0f0f0fu;
        hi[j0 + 1] = (w[j0 + 1] >> 4) & 0x0f0f0f0fu;
        asm("" : "+v"(hi[j0]));
        asm("" : "+v"(hi[j0 + 1]));
      }
      constexpr int sh = 8 * (i / 2);
      if constexpr (i % 2 == 0) {
        c0 = static_cast<float>((lo[j0] >> sh) & 0xffu);
        c1 = static_cast<float>((lo[j0 + 1] >> sh) & 0xffu);
      } else {
        c0 = static_cast<float>((hi[j0] >> sh) & 0xffu);
        c1 = static_cast<float>((hi[j0 + 1] >> sh) & 0xffu);
      }
    } else {
      constexpr int word = i / 4;
      constexpr int sh = 8 * (i % 4);
      c0 = static_cast<float>((w[2 * j0 + word] >> sh) & 0xffu);
      c1 = static_cast<float>((w[2 * (j0 + 1) + word] >> sh) & 0xffu);
    }
    return pack2<T>(fmaf(s[j0], c0, b[j0]), fmaf(s[j0 + 1], c1, b[j0 + 1]));
  }
};

template <typename T, int BITS, int... Q>
__device__ __forceinline__ void dequant_cols_impl(
    const uint32_t (&w)[BITS],
    const float (&s)[4],
    const float (&b)[4],
    uint32_t (&out)[16],
    std::integer_sequence<int, Q...>) {
  ColDequant<T, BITS> dq;
  ((out[Q] = dq.template pair<Q>(w, s, b)), ...);
}

// The whole 4 x 8 block in one go (prologue): out[2 i], out[2 i + 1] hold rows
// 0..3 of column i.
template <typename T, int BITS>
__device__ __forceinline__ void dequant_cols(
    const uint32_t (&w)[BITS],
    const float (&s)[4],
    const float (&b)[4],
    uint32_t (&out)[16]) {
  dequant_cols_impl<T, BITS>(w, s, b, out, std::make_integer_sequence<int, 16>{});
}

template <typename T, int BITS, int... Q>
__device__ __forceinline__ void dequant32_impl(
    const uint32_t (&w)[BITS],
    float s,
    float b,
    uint32_t (&out)[16],
    std::integer_sequence<int, Q...>) {
  PairDequant<T, BITS> dq;
  const float sc = s * PairDequant<T, BITS>::kCodeScale;
  ((out[Q] = dq.template pair<Q>(w, sc, b)), ...);
}

// 32 codes -> 32 elements of T in one go (prologue).
template <typename T, int BITS>
__device__ __forceinline__ void dequant32(
    const uint32_t (&w)[BITS],
    float s,
    float b,
    uint32_t (&out)[16]) {
  dequant32_impl<T, BITS>(w, s, b, out, std::make_integer_sequence<int, 16>{});
}

} // namespace mlxrocm
