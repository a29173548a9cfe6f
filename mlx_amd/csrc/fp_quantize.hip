// fp_quantize.hip -- the floating-point quantization modes of mx.quantize /
// mx.dequantize (mxfp4, mxfp8, nvfp4) and the quantize-dequantize of
// activations that qqmm applies.  HBM-bound elementwise kernels.
//
// Parity target: the CPU path.  mx.quantize in these modes is, on the CPU, a
// graph of generic ops evaluated in the element type T
// (mlx/ops.cpp:5128-5190); the kernel performs the same operations in the same
// order with every intermediate rounded to T:
//   scales = max(abs(group)) / T(maxval)
//   groups of 16:  scales = to_fp8(scales);  q = w / from_fp8(scales) (in T)
//   groups of 32:  e = round(log2(scales)) (both in T);  q = w / 2^e (in T);
//                  scales = uint8(e + 127)
//   4-bit: code = argmin |q - lut| (first minimum); 8-bit: code = to_fp8(q)
// The argmin over the sixteen e2m1 values is evaluated with seven thresholds:
// the two candidates next to q differ from it by exactly representable amounts
// (or, below 0.25, by amounts whose rounding cannot change the comparison), so
// the rounded distances of the op graph order the candidates as the real ones do
// and a tie goes to the smaller index, i.e. the smaller magnitude; +0 (index 0)
// beats -0 (index 8), so a value that rounds to zero gets code 0 whatever its
// sign.
// mx.dequantize (mlx/ops.cpp:5399-5446): T(code value) * scale in T -- an exact
// product in all three element types.
// Quantize-dequantize of activations: fp_quantize_dequantize<T>
// (mlx/backend/cpu/quantized.cpp:1049-1128), fp32 arithmetic, e2m1 ties to the
// even mantissa.
// nvfp4 with a tensor-wide scale (`global_scale`, one float on the device): the
// CPU path has no such mode, so these kernels follow the CUDA backend's
// arithmetic (mlx/backend/cuda/quantized/fp_quantize.cuh:73-145, 147-215,
// 548-592), all in fp32:
//   scale_enc = 448 * 6 / global_scale
//   byte      = to_fp8(max(abs(group)) / 6 * scale_enc)
//   code      = e2m1 nearest, ties to even, of w * (scale_enc / from_fp8(byte))
//   dequantize:          code value * (from_fp8(byte) * (global_scale / (448 * 6)))
//   quantize-dequantize: code value * (from_fp8(byte) * (1 / scale_enc))
// A group of zeros gets the byte 0 and, through 0 * inf, the code of a NaN
// (+6); it decodes to zeros.
#include "common.h"

namespace mlxrocm {

namespace {

constexpr int kFpBlock = 256;

// mlx/backend/cpu/unary_ops.h:120-146
__device__ __forceinline__ uint32_t to_fp8_bits(float f) {
  const uint32_t fp8_max = 543u << 21;
  const uint32_t denorm_mask = 141u << 23;
  uint32_t f_bits = __float_as_uint(f);
  const uint32_t sign = f_bits & 0x80000000u;
  f_bits ^= sign;
  const uint32_t low = __float_as_uint(__uint_as_float(f_bits) + __uint_as_float(denorm_mask));
  const uint32_t result_low = (low - denorm_mask) & 0xffu;
  const uint32_t mant_odd = (f_bits >> 20) & 1u;
  const uint32_t high = f_bits + ((static_cast<uint32_t>(7 - 127) << 23) + 0x7FFFFu) + mant_odd;
  const uint32_t result_high = (high >> 20) & 0xffu;
  uint32_t result = f_bits < (121u << 23) ? result_low : result_high;
  result = f_bits >= fp8_max ? 0x7Eu : result;
  return result | (sign >> 24);
}

// mlx/backend/cpu/unary_ops.h:154-170: exponent bias 7, subnormals, no special codes
__device__ __forceinline__ float from_fp8_bits(uint32_t x) {
  const uint32_t e = (x >> 3) & 0xFu;
  const uint32_t m = x & 7u;
  const float mag = e == 0 ? static_cast<float>(m) * 0.001953125f /* 2^-9 */
                           : __uint_as_float(((e + 120u) << 23) | (m << 20));
  return (x & 0x80u) ? -mag : mag;
}

__device__ __forceinline__ float fp4_value(uint32_t c) {
  const uint32_t mag = c & 7u;
  // 0, .5, 1, 1.5, 2, 3, 4, 6
  const float v = mag < 2 ? 0.5f * static_cast<float>(mag)
                          : __uint_as_float((mag << 22) + (126u << 23));
  return (c & 8u) ? -v : v;
}

// argmin over the e2m1 table, first minimum: nearest value, ties to the smaller
// magnitude, zero always as code 0; NaN (every comparison false) as code 0.
__device__ __forceinline__ uint32_t fp4_nearest_first(float q) {
  const float a = fabsf(q);
  if (!(a > 0.25f)) {
    return 0u;
  }
  const uint32_t mag = a <= 0.75f ? 1u
      : a <= 1.25f ? 2u
      : a <= 1.75f ? 3u
      : a <= 2.5f ? 4u
      : a <= 3.5f ? 5u
      : a <= 5.0f ? 6u : 7u;
  return mag | (q < 0.0f ? 8u : 0u);
}

// mlx/backend/cpu/quantized.cpp:1063-1091: ties to the even mantissa
__device__ __forceinline__ uint32_t fp4_nearest_even(float x) {
  if (x != x) {
    return 7u;
  }
  const uint32_t sign = (__float_as_uint(x) >> 31) << 3;
  const float a = fabsf(x);
  const uint32_t bits = a > 5.0f ? 7u
      : a >= 3.5f ? 6u
      : a > 2.5f ? 5u
      : a >= 1.75f ? 4u
      : a > 1.25f ? 3u
      : a >= 0.75f ? 2u
      : a > 0.25f ? 1u : 0u;
  return bits | sign;
}

// Mantissa bits of the float next to sqrt(2) (0x3FB504F3), and how far from it
// the mantissa of a scale has to be for round(log2(scale)) to be decided without
// evaluating the logarithm: 4096 steps of 2^-23 are 4.9e-4 in m, 5e-4 in log2(m).
constexpr uint32_t kSqrt2Mant = 0x3504F3u;
constexpr uint32_t kTieMargin = 4096u;

// float log2, correctly rounded up to double rounding (evaluated in double)
__device__ __forceinline__ float log2_rn(float x) {
  return static_cast<float>(log2(static_cast<double>(x)));
}

// Maximum over the `lanes` (2 or 4) adjacent lanes that share a group.
__device__ __forceinline__ float group_max(float m, int lanes) {
  m = fmaxf(m, __shfl_xor(m, 1, 64));
  if (lanes == 4) {
    m = fmaxf(m, __shfl_xor(m, 2, 64));
  }
  return m;
}

// One thread: 8 consecutive elements.  GS is 16 (nvfp4) or 32; BITS 4 or 8.
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(kFpBlock) void fp_quantize_kernel(
    const T* w, uint8_t* wq, uint8_t* scales, size_t n_units) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  constexpr int kLanes = GS / 8;
  float v[8];
  const bool live = u < n_units;
  if (live) {
    load8<T>(w + u * 8, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = 0.0f;
    }
  }
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    m = fmaxf(m, fabsf(v[i]));
  }
  m = group_max(m, kLanes);
  constexpr float kMaxVal = BITS == 4 ? 6.0f : 448.0f;
  const float s = round_to<T>(m / kMaxVal);
  float q[8];
  uint32_t scale_byte;
  if constexpr (GS == 16) {
    scale_byte = to_fp8_bits(s);
    const float sv = round_to<T>(from_fp8_bits(scale_byte));
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q[i] = round_to<T>(v[i] / sv);
    }
  } else {
    float e = 0.0f;
    if (s != 0.0f) {
      const float l = round_to<T>(log2_rn(s));
      e = round_to<T>(rintf(l));
      e = round_to<T>(static_cast<float>(static_cast<int>(e)));
    }
    const float p = round_to<T>(ldexpf(1.0f, static_cast<int>(e))); // 2^e, exact in float
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q[i] = round_to<T>(v[i] / p);
    }
    scale_byte = static_cast<uint32_t>(static_cast<int>(round_to<T>(e + 127.0f))) & 0xffu;
  }
  if (!live) {
    return;
  }
  if ((u % kLanes) == 0) {
    scales[u / kLanes] = static_cast<uint8_t>(scale_byte);
  }
  if constexpr (BITS == 4) {
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      word |= fp4_nearest_first(q[i]) << (4 * i);
    }
    reinterpret_cast<uint32_t*>(wq)[u] = word;
  } else {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo |= to_fp8_bits(q[i]) << (8 * i);
      hi |= to_fp8_bits(q[4 + i]) << (8 * i);
    }
    reinterpret_cast<uint2*>(wq)[u] = make_uint2(lo, hi);
  }
}

// The scale of group `g` as a value of T (mlx/ops.cpp:5431-5440).
template <typename T, int GS>
__device__ __forceinline__ float fp_scale_value(uint32_t s) {
  if constexpr (GS == 16) {
    return round_to<T>(from_fp8_bits(s));
  } else {
    const float e = round_to<T>(round_to<T>(static_cast<float>(s)) - 127.0f);
    return round_to<T>(ldexpf(1.0f, static_cast<int>(e)));
  }
}

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(kFpBlock) void fp_dequantize_kernel(
    const uint8_t* wq, const uint8_t* scales, T* out, size_t n_units) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  if (u >= n_units) {
    return;
  }
  const float s = fp_scale_value<T, GS>(scales[u * 8 / GS]);
  float v[8];
  if constexpr (BITS == 4) {
    const uint32_t word = reinterpret_cast<const uint32_t*>(wq)[u];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = fp4_value((word >> (4 * i)) & 0xFu) * s;
    }
  } else {
    const uint2 words = reinterpret_cast<const uint2*>(wq)[u];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = round_to<T>(from_fp8_bits((words.x >> (8 * i)) & 0xffu)) * s;
      v[4 + i] = round_to<T>(from_fp8_bits((words.y >> (8 * i)) & 0xffu)) * s;
    }
  }
  store8<T>(out + u * 8, v);
}

// mlx/backend/cpu/quantized.cpp:1094-1128, fp32 arithmetic throughout.
// CODES: write the codes and the scale byte (wq, scales) instead of the
// dequantized elements (out): the operand the block-scaled matrix instruction
// multiplies as it is.
template <typename T, int GS, int BITS, bool CODES = false>
__global__ __launch_bounds__(kFpBlock) void fp_quantize_dequantize_kernel(
    const T* w, T* out, size_t n_units, uint8_t* wq = nullptr, uint8_t* scales = nullptr) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  constexpr int kLanes = GS / 8;
  float v[8];
  const bool live = u < n_units;
  if (live) {
    load8<T>(w + u * 8, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = 0.0f;
    }
  }
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    m = fmaxf(m, fabsf(v[i]));
  }
  m = group_max(m, kLanes);
  float scale = m / (BITS == 4 ? 6.0f : 448.0f);
  uint32_t scale_byte;
  float recip = 0.0f;
  bool exact_recip = false;
  if constexpr (GS == 16) {
    scale_byte = to_fp8_bits(scale);
    scale = from_fp8_bits(scale_byte);
  } else {
    // to_fp8_e8m0 (:1049-1061): round(log2(scale)) half away from zero, clamped;
    // log2(0) = -inf clamps to -127, which decodes to 2^-127
    int n;
    const uint32_t sbits = __float_as_uint(scale);
    const uint32_t mant = sbits & 0x7fffffu;
    if (sbits - 0x00800000u < 0x7e000000u &&
        (mant < kSqrt2Mant - kTieMargin || mant > kSqrt2Mant + kTieMargin)) {
      // a normal number 2^e m below 2^126, m in [1, 2), away from sqrt(2):
      // log2 = e + log2(m) rounds to e below sqrt(2) and to e + 1 above, whatever
      // the sign of e.  Evaluating log2 in float moves it by less than 2^-16; the
      // margin keeps log2(m) 5e-4 away from one half.  The reciprocal of
      // 2^n, |n| <= 126, is a normal float.
      n = static_cast<int>(sbits >> 23) - 127 + (mant > kSqrt2Mant ? 1 : 0);
      recip = __uint_as_float(static_cast<uint32_t>(127 - n) << 23);
      exact_recip = true;
    } else if (!(scale == scale) || fabsf(scale) == INFINITY) {
      n = 128; // code 0xFF: decodes to NaN as a bfloat16 pattern
    } else if (scale <= 0.0f) {
      n = -127;
    } else {
      n = static_cast<int>(roundf(log2_rn(scale)));
      n = n < -127 ? -127 : (n > 127 ? 127 : n);
    }
    const uint32_t s8 = static_cast<uint32_t>(n + 127);
    scale = __uint_as_float((s8 == 0 ? 0x40u : (s8 << 7)) << 16);
    scale_byte = s8;
  }
  if (!live) {
    return;
  }
  // The scale of an MX mode is a power of two: multiplying by its reciprocal is
  // the same single rounding as the reference's division.
  if (exact_recip) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] *= recip;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = scale == 0.0f ? 0.0f : v[i] / scale;
    }
  }
  if constexpr (CODES) {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float w_el = v[i];
      if constexpr (BITS == 8) {
        const uint32_t c = to_fp8_bits(w_el);
        if (i < 4) {
          lo |= c << (8 * i);
        } else {
          hi |= c << (8 * (i - 4));
        }
      } else {
        lo |= fp4_nearest_even(w_el) << (4 * i);
      }
    }
    if constexpr (BITS == 8) {
      reinterpret_cast<uint2*>(wq)[u] = make_uint2(lo, hi);
    } else {
      reinterpret_cast<uint32_t*>(wq)[u] = lo;
    }
    if (u % kLanes == 0) {
      scales[u / kLanes] = static_cast<uint8_t>(scale_byte);
    }
  } else {
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float w_el = v[i];
      const float val = BITS == 8 ? from_fp8_bits(to_fp8_bits(w_el))
                                  : fp4_value(fp4_nearest_even(w_el));
      o[i] = scale * val;
    }
    store8<T>(out + u * 8, o);
  }
}

constexpr float kNvfp4Span = 448.0f * 6.0f;

// One thread: 8 consecutive elements, two threads per group of 16.
// OUT == 0: codes and scale bytes; OUT == 1: the dequantized elements.
template <typename T, int OUT>
__global__ __launch_bounds__(kFpBlock) void nvfp4_global_quantize_kernel(
    const T* w, const float* global_scale, uint8_t* wq, uint8_t* scales, T* out, size_t n_units) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  const float scale_enc = kNvfp4Span / *global_scale;
  float v[8];
  const bool live = u < n_units;
  if (live) {
    load8<T>(w + u * 8, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = 0.0f;
    }
  }
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    m = fmaxf(m, fabsf(v[i]));
  }
  m = group_max(m, 2);
  float scale_dec_b = m / 6.0f;
  scale_dec_b *= scale_enc;
  const uint32_t scale_byte = to_fp8_bits(scale_dec_b);
  const float sv = from_fp8_bits(scale_byte);
  const float scale_enc_b = scale_enc / sv;
  if (!live) {
    return;
  }
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    word |= fp4_nearest_even(v[i] * scale_enc_b) << (4 * i);
  }
  if constexpr (OUT == 0) {
    reinterpret_cast<uint32_t*>(wq)[u] = word;
    if ((u & 1) == 0) {
      scales[u / 2] = static_cast<uint8_t>(scale_byte);
    }
  } else {
    const float scale_dec = sv * (1.0f / scale_enc);
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      o[i] = fp4_value((word >> (4 * i)) & 0xFu) * scale_dec;
    }
    store8<T>(out + u * 8, o);
  }
}

template <typename T>
__global__ __launch_bounds__(kFpBlock) void nvfp4_global_dequantize_kernel(
    const uint8_t* wq, const uint8_t* scales, const float* global_scale, T* out, size_t n_units) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  if (u >= n_units) {
    return;
  }
  const float inv_scale_enc = *global_scale / kNvfp4Span;
  const float s = from_fp8_bits(scales[u / 2]) * inv_scale_enc;
  const uint32_t word = reinterpret_cast<const uint32_t*>(wq)[u];
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    v[i] = s * fp4_value((word >> (4 * i)) & 0xFu);
  }
  store8<T>(out + u * 8, v);
}

// mx.to_fp8 / mx.from_fp8 (fast::ConvertFP8, mlx/backend/cpu/quantized.cpp:1282-1320
// with detail::ToFP8 / FromFP8, mlx/backend/cpu/unary_ops.h:120-174).  One thread:
// 8 consecutive elements; the tail of a length that is not a multiple of 8
// element by element.
template <typename T>
__global__ __launch_bounds__(kFpBlock) void to_fp8_kernel(const T* x, uint8_t* out, size_t n) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  const size_t first = u * 8;
  if (first >= n) {
    return;
  }
  if (first + 8 <= n) {
    float v[8];
    load8<T>(x + first, v);
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo |= to_fp8_bits(v[i]) << (8 * i);
      hi |= to_fp8_bits(v[4 + i]) << (8 * i);
    }
    *reinterpret_cast<uint2*>(out + first) = make_uint2(lo, hi);
  } else {
    for (size_t i = first; i < n; ++i) {
      out[i] = static_cast<uint8_t>(to_fp8_bits(to_f32(x[i])));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kFpBlock) void from_fp8_kernel(const uint8_t* x, T* out, size_t n) {
  const size_t u = static_cast<size_t>(blockIdx.x) * kFpBlock + threadIdx.x;
  const size_t first = u * 8;
  if (first >= n) {
    return;
  }
  if (first + 8 <= n) {
    const uint2 words = *reinterpret_cast<const uint2*>(x + first);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = from_fp8_bits((words.x >> (8 * i)) & 0xffu);
      v[4 + i] = from_fp8_bits((words.y >> (8 * i)) & 0xffu);
    }
    store8<T>(out + first, v);
  } else {
    for (size_t i = first; i < n; ++i) {
      out[i] = from_f32<T>(from_fp8_bits(x[i]));
    }
  }
}

int check_mode(const char* who, int mode, int dtype, size_t n_elems) {
  if (mode != MLXROCM_MXFP4 && mode != MLXROCM_MXFP8 && mode != MLXROCM_NVFP4) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown quantization mode %d", who, mode);
  }
  if (!valid_dtype(dtype)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown dtype %d", who, dtype);
  }
  const size_t gs = mode == MLXROCM_NVFP4 ? 16 : 32;
  if (n_elems % gs != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the number of elements %zu is not a multiple of the group size %zu", who, n_elems, gs);
  }
  return MLXROCM_OK;
}

template <typename F>
int dispatch_mode(int mode, F&& fn) {
  switch (mode) {
    case MLXROCM_MXFP4:
      return fn(IntC<32>{}, IntC<4>{});
    case MLXROCM_MXFP8:
      return fn(IntC<32>{}, IntC<8>{});
    default:
      return fn(IntC<16>{}, IntC<4>{});
  }
}

} // namespace

} // namespace mlxrocm

using namespace mlxrocm;

extern "C" int mlxrocm_fp_quantize(
    const void* w,
    uint32_t* wq,
    uint8_t* scales,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_quantize");
  int rc = check_mode("quantize", mode, dtype, n_elems);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!w || !wq || !scales) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(wq) & 7u)) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize] operand pointers must be 16-byte aligned");
  }
  const size_t n_units = n_elems / 8;
  const size_t blocks = (n_units + kFpBlock - 1) / kFpBlock;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize] %zu elements exceed the grid", n_elems);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_mode(mode, [&](auto gval, auto bval) {
      constexpr int G = decltype(gval)::value;
      constexpr int B = decltype(bval)::value;
      fp_quantize_kernel<T, G, B><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
          static_cast<const T*>(w), reinterpret_cast<uint8_t*>(wq), scales, n_units);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  });
}

extern "C" int mlxrocm_fp_dequantize(
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_dequantize");
  int rc = check_mode("dequantize", mode, dtype, n_elems);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!wq || !scales || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[dequantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(out) & 15u) || (reinterpret_cast<uintptr_t>(wq) & 7u)) {
    return fail(MLXROCM_UNSUPPORTED, "[dequantize] operand pointers must be 16-byte aligned");
  }
  const size_t n_units = n_elems / 8;
  const size_t blocks = (n_units + kFpBlock - 1) / kFpBlock;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[dequantize] %zu elements exceed the grid", n_elems);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_mode(mode, [&](auto gval, auto bval) {
      constexpr int G = decltype(gval)::value;
      constexpr int B = decltype(bval)::value;
      fp_dequantize_kernel<T, G, B><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
          reinterpret_cast<const uint8_t*>(wq), scales, static_cast<T*>(out), n_units);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  });
}

namespace mlxrocm {

// x -> codes and scale bytes by the rules of fp_quantize_dequantize (what qqmm
// applies to its first operand).  n_elems a multiple of the group size.
int fp_quantize_activations(
    const void* x, void* codes, uint8_t* scales, size_t n_elems, int mode, int dtype, hipStream_t s) {
  const size_t n_units = n_elems / 8;
  const size_t blocks = (n_units + kFpBlock - 1) / kFpBlock;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[qqmm] %zu elements exceed the grid", n_elems);
  }
  MLXROCM_REHEARSE("fp_quantize_activations");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_mode(mode, [&](auto gval, auto bval) {
      constexpr int G = decltype(gval)::value;
      constexpr int B = decltype(bval)::value;
      fp_quantize_dequantize_kernel<T, G, B, true><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
          static_cast<const T*>(x), nullptr, n_units, static_cast<uint8_t*>(codes), scales);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  });
}

} // namespace mlxrocm

extern "C" int mlxrocm_fp_quantize_dequantize(
    const void* x,
    void* out,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_quantize_dequantize");
  int rc = check_mode("quantize_dequantize", mode, dtype, n_elems);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!x || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantize_dequantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(out) & 15u)) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize_dequantize] operand pointers must be 16-byte aligned");
  }
  const size_t n_units = n_elems / 8;
  const size_t blocks = (n_units + kFpBlock - 1) / kFpBlock;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize_dequantize] %zu elements exceed the grid", n_elems);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  MLXROCM_REHEARSE("fp_quantize_dequantize");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_mode(mode, [&](auto gval, auto bval) {
      constexpr int G = decltype(gval)::value;
      constexpr int B = decltype(bval)::value;
      fp_quantize_dequantize_kernel<T, G, B><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
          static_cast<const T*>(x), static_cast<T*>(out), n_units);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  });
}

namespace {

// Shared argument checks of the nvfp4 entry points that take a tensor-wide scale.
int check_global(const char* who, int dtype, size_t n_elems, const void* global_scale, size_t* blocks) {
  int rc = check_mode(who, MLXROCM_NVFP4, dtype, n_elems);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (global_scale == nullptr || (reinterpret_cast<uintptr_t>(global_scale) & 3u) != 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] global_scale must point at one float32 on the device", who);
  }
  *blocks = (n_elems / 8 + kFpBlock - 1) / kFpBlock;
  if (*blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[%s] %zu elements exceed the grid", who, n_elems);
  }
  return MLXROCM_OK;
}

} // namespace

extern "C" int mlxrocm_nvfp4_quantize_global(
    const void* w,
    const float* global_scale,
    uint32_t* wq,
    uint8_t* scales,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_nvfp4_quantize_global");
  size_t blocks = 0;
  int rc = check_global("quantize", dtype, n_elems, global_scale, &blocks);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!w || !wq || !scales) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(wq) & 7u)) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize] operand pointers must be 16-byte aligned");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    nvfp4_global_quantize_kernel<T, 0><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
        static_cast<const T*>(w), global_scale, reinterpret_cast<uint8_t*>(wq), scales, nullptr,
        n_elems / 8);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}

extern "C" int mlxrocm_nvfp4_dequantize_global(
    const uint32_t* wq,
    const uint8_t* scales,
    const float* global_scale,
    void* out,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_nvfp4_dequantize_global");
  size_t blocks = 0;
  int rc = check_global("dequantize", dtype, n_elems, global_scale, &blocks);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!wq || !scales || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[dequantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(out) & 15u) || (reinterpret_cast<uintptr_t>(wq) & 7u)) {
    return fail(MLXROCM_UNSUPPORTED, "[dequantize] operand pointers must be 16-byte aligned");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    nvfp4_global_dequantize_kernel<T><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
        reinterpret_cast<const uint8_t*>(wq), scales, global_scale, static_cast<T*>(out),
        n_elems / 8);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}

extern "C" int mlxrocm_nvfp4_quantize_dequantize_global(
    const void* x,
    const float* global_scale,
    void* out,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_nvfp4_quantize_dequantize_global");
  size_t blocks = 0;
  int rc = check_global("quantize_dequantize", dtype, n_elems, global_scale, &blocks);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  if (!x || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantize_dequantize] null device pointer");
  }
  if ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(out) & 15u)) {
    return fail(MLXROCM_UNSUPPORTED, "[quantize_dequantize] operand pointers must be 16-byte aligned");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  MLXROCM_REHEARSE("nvfp4_global_quantize_dequantize");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    nvfp4_global_quantize_kernel<T, 1><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
        static_cast<const T*>(x), global_scale, nullptr, nullptr, static_cast<T*>(out),
        n_elems / 8);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}

namespace {

int check_convert(
    const char* who, const void* wide, const void* bytes, size_t n, int dtype, size_t* blocks) {
  if (!valid_dtype(dtype)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown dtype %d", who, dtype);
  }
  *blocks = ((n + 7) / 8 + kFpBlock - 1) / kFpBlock;
  if (n == 0) {
    return MLXROCM_OK;
  }
  if (!wide || !bytes) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] null device pointer", who);
  }
  if ((reinterpret_cast<uintptr_t>(wide) & 15u) || (reinterpret_cast<uintptr_t>(bytes) & 7u)) {
    return fail(MLXROCM_UNSUPPORTED, "[%s] operand pointers must be 16-byte aligned", who);
  }
  if (*blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[%s] %zu elements exceed the grid", who, n);
  }
  return MLXROCM_OK;
}

} // namespace

extern "C" int mlxrocm_to_fp8(
    const void* x, uint8_t* out, size_t n_elems, int dtype, mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_to_fp8");
  size_t blocks = 0;
  int rc = check_convert("to_fp8", x, out, n_elems, dtype, &blocks);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    to_fp8_kernel<T><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
        static_cast<const T*>(x), out, n_elems);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}

extern "C" int mlxrocm_from_fp8(
    const uint8_t* x, void* out, size_t n_elems, int dtype, mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_from_fp8");
  size_t blocks = 0;
  int rc = check_convert("from_fp8", out, x, n_elems, dtype, &blocks);
  if (rc != MLXROCM_OK || n_elems == 0) {
    return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    from_fp8_kernel<T><<<static_cast<unsigned>(blocks), kFpBlock, 0, s>>>(
        x, static_cast<T*>(out), n_elems);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}
