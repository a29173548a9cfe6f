// quantize.hip -- affine group-wise quantize / dequantize for gfx950.
//
// Both kernels are HBM-bound streaming kernels.  A lane owns one "unit" of 8
// consecutive elements: 8 codes are exactly BITS bytes of the packed stream for
// every supported width, so a unit never shares a byte with its neighbour even
// when 3/5/6-bit codes straddle uint32 words.  A quantization group is GS/8
// adjacent lanes of one wavefront; its min/max is a butterfly over those lanes.
//
// The arithmetic follows the CPU backend operation by operation (fp32 division,
// rint, clamp; scale/bias rounded to T only when stored) so that packed words,
// scales and biases are bit-identical to mlx/backend/cpu/quantized.cpp:1148-1211.
// The file must be compiled without FMA contraction.
#include "common.h"

namespace mlxrocm {

namespace {

constexpr int kQuantBlock = 256;

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(kQuantBlock) void affine_quantize_kernel(
    const T* __restrict__ w,
    uint8_t* __restrict__ out,
    T* __restrict__ scales,
    T* __restrict__ biases,
    size_t n_units) {
  constexpr int LPG = GS / 8; // lanes per group
  constexpr bool kStage = !(BITS == 4 || BITS == 8);
  __shared__ uint32_t stage[kStage ? (kQuantBlock * BITS) / 4 : 1];

  const size_t block_first = static_cast<size_t>(blockIdx.x) * kQuantBlock;
  const size_t u = block_first + threadIdx.x;
  const bool active = u < n_units;

  float v[8];
  if (active) {
    load8<T>(w + u * 8, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = 0.0f;
    }
  }

  // std::max / std::min semantics: keep the accumulator unless strictly beaten.
  float w_max = v[0];
  float w_min = v[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    w_max = (w_max < v[i]) ? v[i] : w_max;
    w_min = (v[i] < w_min) ? v[i] : w_min;
  }
#pragma unroll
  for (int off = LPG / 2; off > 0; off >>= 1) {
    const float o_max = __shfl_xor(w_max, off, 64);
    const float o_min = __shfl_xor(w_min, off, 64);
    w_max = (w_max < o_max) ? o_max : w_max;
    w_min = (o_min < w_min) ? o_min : w_min;
  }

  constexpr float n_bins = static_cast<float>((1 << BITS) - 1);
  constexpr float eps = 1e-7f;
  const bool mask = fabsf(w_min) > fabsf(w_max);
  float scale = (w_max - w_min) / n_bins;
  scale = (scale < eps) ? eps : scale;
  scale = mask ? scale : -scale;
  const float edge = mask ? w_min : w_max;
  const float q0 = rintf(edge / scale);
  float bias = 0.0f;
  if (q0 != 0.0f) {
    scale = edge / q0;
    bias = edge;
  }

  // The eight quotients (v - bias) / scale share their divisor.  The correctly
  // rounded fp32 division is a reciprocal refined once, then per numerator
  // q = a r, two residual corrections q += (a - scale q) r -- the compiler's own
  // expansion without its range scaling, which only acts on operands far outside
  // what occurs here (|scale| in [1e-7, 1e38), quotients far from overflow; a
  // numerator small enough to be scaled gives a quotient that rounds to 0 either
  // way).  Groups with a non-finite edge take the plain division.
  uint64_t packed = 0;
  const bool regular = fabsf(edge) < 3.0e38f && fabsf(scale) >= 1e-7f; // false for NaN
  if (regular) {
    float r = __builtin_amdgcn_rcpf(scale);
    r = __builtin_fmaf(__builtin_fmaf(-scale, r, 1.0f), r, r);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float a = v[i] - bias;
      float q = a * r;
      q = __builtin_fmaf(__builtin_fmaf(-scale, q, a), r, q);
      q = __builtin_fmaf(__builtin_fmaf(-scale, q, a), r, q);
      q = rintf(q);
      q = (q < 0.0f) ? 0.0f : q;
      q = (n_bins < q) ? n_bins : q;
      packed |= static_cast<uint64_t>(static_cast<uint32_t>(q)) << (i * BITS);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float q = rintf((v[i] - bias) / scale);
      q = (q < 0.0f) ? 0.0f : q;
      q = (n_bins < q) ? n_bins : q;
      packed |= static_cast<uint64_t>(static_cast<uint32_t>(q)) << (i * BITS);
    }
  }

  if (active && (threadIdx.x % LPG) == 0) {
    const size_t g = u / LPG;
    scales[g] = from_f32<T>(scale);
    biases[g] = from_f32<T>(bias);
  }

  if constexpr (BITS == 4) {
    if (active) {
      reinterpret_cast<uint32_t*>(out)[u] = static_cast<uint32_t>(packed);
    }
  } else if constexpr (BITS == 8) {
    if (active) {
      reinterpret_cast<uint2*>(out)[u] = make_uint2(
          static_cast<uint32_t>(packed), static_cast<uint32_t>(packed >> 32));
    }
  } else {
    // Stage the block's bytes in LDS, then write whole dwords, coalesced.
    uint8_t* sb = reinterpret_cast<uint8_t*>(stage) + threadIdx.x * BITS;
#pragma unroll
    for (int i = 0; i < BITS; ++i) {
      sb[i] = static_cast<uint8_t>(packed >> (8 * i));
    }
    __syncthreads();
    const size_t remaining = n_units > block_first ? n_units - block_first : 0;
    const int units_here =
        remaining < kQuantBlock ? static_cast<int>(remaining) : kQuantBlock;
    // units_here is a multiple of LPG >= 4, so the byte count is a multiple of 4
    const int words_here = units_here * BITS / 4;
    uint32_t* out32 = reinterpret_cast<uint32_t*>(out) +
        static_cast<size_t>(blockIdx.x) * (kQuantBlock * BITS / 4);
    for (int i = threadIdx.x; i < words_here; i += kQuantBlock) {
      out32[i] = stage[i];
    }
  }
}

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(kQuantBlock) void affine_dequantize_kernel(
    const uint8_t* __restrict__ wq,
    const T* __restrict__ scales,
    const T* __restrict__ biases,
    T* __restrict__ out,
    size_t n_units) {
  const size_t u =
      static_cast<size_t>(blockIdx.x) * kQuantBlock + threadIdx.x;
  if (u >= n_units) {
    return;
  }
  const uint64_t unit = load_unit<BITS>(wq, u);
  const size_t g = (u * 8) / GS;
  const float s = to_f32(scales[g]);
  const float b = to_f32(biases[g]);
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // Multiply, then Add, each rounded to T (mlx/ops.cpp:5322-5323).
    const float q = static_cast<float>(unit_code<BITS>(unit, i));
    const float prod = round_to<T>(q * s);
    v[i] = prod + b;
  }
  store8<T>(out + u * 8, v);
}

int check_common(
    const void* a,
    const void* b,
    const void* c,
    const void* d,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype,
    const char* who) {
  if (!valid_bits(bits)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the requested number of bits %d is not supported; "
        "supported bits are 2, 3, 4, 5, 6 and 8",
        who,
        bits);
  }
  if (!valid_group(group_size)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the requested group size %d is not supported; "
        "supported group sizes are 32, 64 and 128",
        who,
        group_size);
  }
  if (!valid_dtype(dtype)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown dtype %d", who, dtype);
  }
  if (n_elems % static_cast<size_t>(group_size) != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] element count %zu is not a multiple of the group size %d",
        who,
        n_elems,
        group_size);
  }
  if (n_elems != 0 && (!a || !b || !c || !d)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] null device pointer", who);
  }
  if (n_elems / 8 / kQuantBlock >= 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[%s] %zu elements exceed the grid", who, n_elems);
  }
  return MLXROCM_OK;
}

} // namespace

} // namespace mlxrocm

using namespace mlxrocm;

extern "C" int mlxrocm_affine_quantize(
    const void* w,
    uint32_t* wq,
    void* scales,
    void* biases,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_affine_quantize");
  int rc = check_common(
      w, wq, scales, biases, n_elems, group_size, bits, dtype, "quantize");
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  const size_t n_units = n_elems / 8;
  const unsigned blocks =
      static_cast<unsigned>((n_units + kQuantBlock - 1) / kQuantBlock);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(group_size, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        affine_quantize_kernel<T, B, G><<<blocks, kQuantBlock, 0, s>>>(
            static_cast<const T*>(w),
            reinterpret_cast<uint8_t*>(wq),
            static_cast<T*>(scales),
            static_cast<T*>(biases),
            n_units);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  });
}

extern "C" int mlxrocm_affine_dequantize(
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_affine_dequantize");
  int rc = check_common(
      wq, scales, biases, out, n_elems, group_size, bits, dtype, "dequantize");
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  const size_t n_units = n_elems / 8;
  const unsigned blocks =
      static_cast<unsigned>((n_units + kQuantBlock - 1) / kQuantBlock);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(group_size, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        affine_dequantize_kernel<T, B, G><<<blocks, kQuantBlock, 0, s>>>(
            reinterpret_cast<const uint8_t*>(wq),
            static_cast<const T*>(scales),
            static_cast<const T*>(biases),
            static_cast<T*>(out),
            n_units);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  });
}
