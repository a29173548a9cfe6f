/*
 * fp_qref.c -- CPU restatement of MLX's floating-point quantization modes
 * (mxfp4, mxfp8, nvfp4): quantize, dequantize, the quantized matmul and the
 * quantize-dequantize of activations that qqmm applies.
 *
 * TEST INFRASTRUCTURE ONLY, like affine_qref.c: tests, the smoke check and the
 * benchmark's cpu_baseline leg may link it; the product library never does.
 *
 * Modes: 0 = mxfp4 (4-bit e2m1 codes, groups of 32, e8m0 scales),
 *        1 = mxfp8 (8-bit e4m3 codes, groups of 32, e8m0 scales),
 *        2 = nvfp4 (4-bit e2m1 codes, groups of 16, e4m3 scales; no global scale).
 *
 * How each function is pinned:
 *   fpq_to_fp8 / fpq_from_fp8   all 256 codes and sampled / exhaustive-in-range
 *                               floats against the reference's detail::ToFP8 /
 *                               FromFP8 compiled in the reference translation
 *                               unit (mlx/backend/cpu/unary_ops.h:120-174)
 *   fpq_qmm                     byte-for-byte against the reference's fp_qmm_t /
 *                               fp_qmm (mlx/backend/cpu/quantized.cpp:449-530)
 *                               through fp_qmm_dispatch_transpose<T, gs, bits>
 *                               of the same translation unit
 *   fpq_e8m0 / fpq_e2m1,
 *   fpq_quantize_dequantize     the scalar helpers to_fp8_e8m0 / to_fp4_e2m1 of
 *                               the translation unit (:1049-1092) value by value;
 *                               the loop over groups (:1094-1128) takes MLX arrays
 *                               and cannot be called, it is restated line by line
 *   fpq_dequantize              the op graph of mlx/ops.cpp:5341-5460 has no
 *                               callable function; every product it forms (an
 *                               e2m1 or e4m3 value times a power of two or an
 *                               e4m3 scale) is exact in all three element types,
 *                               so it is pinned by the exact real value, the nibble
 *                               order of python/tests/test_quantized.py:41-95 and
 *                               fpq_qmm == x @ dequantize(w).T in fp64
 *   fpq_quantize                PARITY UNPINNED for exact bits: on the CPU
 *                               mx.quantize in these modes is a graph of generic
 *                               ops evaluated in the element type
 *                               (mlx/ops.cpp:5128-5190), restated here op by op
 *                               with every intermediate rounded to that type; no
 *                               function of the reference computes it, so no
 *                               reference run backs the restatement.  What is
 *                               checked: the known-answer cases of the reference's
 *                               tests (values on the e2m1 / e4m3 grid round-trip
 *                               exactly, python/tests/test_quantized.py:41-181),
 *                               nearest-value and error-bound properties, and
 *                               agreement with the translation unit's own fp32
 *                               rules (to_fp8_e8m0 / to_fp4_e2m1) away from ties.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "affine_qref.h"
#include "fp_qref.h"

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Element load / store and the rounding step of the software half types
 * (every operator evaluates in float and rounds back, mlx/types/half_types.h). */
static inline float ld(const void* p, size_t i, int dtype) {
  switch (dtype) {
    case QREF_F32:
      return ((const float*)p)[i];
    case QREF_F16:
      return qref_f16_to_f32(((const uint16_t*)p)[i]);
    default:
      return qref_bf16_to_f32(((const uint16_t*)p)[i]);
  }
}
static inline void st(void* p, size_t i, int dtype, float v) {
  switch (dtype) {
    case QREF_F32:
      ((float*)p)[i] = v;
      break;
    case QREF_F16:
      ((uint16_t*)p)[i] = qref_f16_from_f32(v);
      break;
    default:
      ((uint16_t*)p)[i] = qref_bf16_from_f32(v);
      break;
  }
}
static inline float rnd(float v, int dtype) {
  switch (dtype) {
    case QREF_F32:
      return v;
    case QREF_F16:
      return qref_f16_to_f32(qref_f16_from_f32(v));
    default:
      return qref_bf16_to_f32(qref_bf16_from_f32(v));
  }
}

static const float kFp4Lut[16] = {+0.0f, +0.5f, +1.0f, +1.5f, +2.0f, +3.0f, +4.0f, +6.0f,
                                  -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

int fpq_group_size(int mode) {
  return mode == FPQ_NVFP4 ? 16 : 32;
}
int fpq_bits(int mode) {
  return mode == FPQ_MXFP8 ? 8 : 4;
}

/* mlx/backend/cpu/unary_ops.h:120-146 (ToFP8): float -> e4m3, round to nearest
 * even, saturating at 0x7E (448); the sign is carried over. */
uint8_t fpq_to_fp8(float f) {
  const uint32_t fp8_max = 543u << 21;
  const uint32_t denorm_mask = 141u << 23;
  uint32_t f_bits = f32_bits(f);
  const uint32_t sign = f_bits & 0x80000000u;
  f_bits ^= sign;
  const uint32_t f_bits_low = f32_bits(bits_f32(f_bits) + bits_f32(denorm_mask));
  const uint8_t result_low = (uint8_t)(f_bits_low - denorm_mask);
  const uint8_t mant_odd = (uint8_t)((f_bits >> 20) & 1u);
  uint32_t f_bits_high = f_bits + (((uint32_t)(7 - 127) << 23) + 0x7FFFFu);
  f_bits_high += mant_odd;
  const uint8_t result_high = (uint8_t)(f_bits_high >> 20);
  uint8_t result = f_bits < (121u << 23) ? result_low : result_high;
  if (f_bits >= fp8_max) {
    result = 0x7E;
  }
  return (uint8_t)(result | (uint8_t)(sign >> 24));
}

/* mlx/backend/cpu/unary_ops.h:154-170 (FromFP8): the low seven bits shifted into
 * a binary16 pattern, times 256; the sign applied afterwards. */
float fpq_from_fp8(uint8_t x) {
  const uint16_t v = (uint16_t)((uint16_t)(x & 127u) << 7);
  const float out = qref_f16_to_f32(v) * 256.0f;
  return (x & 128u) ? -out : out;
}

/* mlx/backend/cpu/quantized.cpp:49-62 (dequantize_scale<T, group_size>): e4m3
 * for groups of 16; otherwise the bfloat16 whose bits are s << 7, i.e.
 * 2^(s - 127), with s == 0 mapped to 0x40 (2^-127 as a bfloat16 subnormal). */
static inline float scale_value(uint8_t s, int mode, int dtype) {
  if (mode == FPQ_NVFP4) {
    return rnd(fpq_from_fp8(s), dtype);
  }
  const uint16_t b = s == 0 ? 0x40 : (uint16_t)((uint16_t)s << 7);
  return rnd(qref_bf16_to_f32(b), dtype);
}

/* mlx/backend/cpu/quantized.cpp:1049-1061 */
uint8_t fpq_e8m0(float x) {
  if (!isfinite(x)) {
    return 0xFF;
  }
  if (x < 0.0f) {
    return 0x00;
  }
  const float le = log2f(x);
  int n = (int)roundf(le);
  n = n < -127 ? -127 : n;
  n = n > 127 ? 127 : n;
  return (uint8_t)(n + 127);
}

/* mlx/backend/cpu/quantized.cpp:1063-1091: nearest e2m1 value, ties to the even
 * mantissa. */
uint8_t fpq_e2m1(float x) {
  if (isnan(x)) {
    return 0x7;
  }
  const uint8_t sign_bit = signbit(x) ? 0x8 : 0x0;
  x = fabsf(x);
  uint8_t bits;
  if (x > 5.0f) {
    bits = 0x7;
  } else if (x >= 3.5f) {
    bits = 0x6;
  } else if (x > 2.5f) {
    bits = 0x5;
  } else if (x >= 1.75f) {
    bits = 0x4;
  } else if (x > 1.25f) {
    bits = 0x3;
  } else if (x >= 0.75f) {
    bits = 0x2;
  } else if (x > 0.25f) {
    bits = 0x1;
  } else {
    bits = 0x0;
  }
  return (uint8_t)(bits | sign_bit);
}

/* mlx/backend/cpu/quantized.cpp:1094-1128 (fp_quantize_dequantize<T>): what
 * QQMatmul::eval_cpu (:1322-1356) applies to x before the matmul.  fp32 math. */
int fpq_quantize_dequantize(const void* w, void* out, size_t n, int mode, int dtype) {
  if (mode < 0 || mode > 2 || dtype < 0 || dtype > 2) {
    return -1;
  }
  const int gs = fpq_group_size(mode);
  const int bits = fpq_bits(mode);
  if (n % (size_t)gs != 0) {
    return -1;
  }
  for (size_t g = 0; g < n / (size_t)gs; ++g) {
    const size_t idx = g * (size_t)gs;
    float scale = -INFINITY;
    for (int j = 0; j < gs; ++j) {
      const float a = fabsf(ld(w, idx + j, dtype));
      scale = scale > a ? scale : a; /* std::max(scale, a) */
    }
    scale /= bits == 4 ? 6.0f : 448.0f;
    if (gs == 16) {
      scale = fpq_from_fp8(fpq_to_fp8(scale));
    } else {
      const uint8_t s = fpq_e8m0(scale);
      scale = qref_bf16_to_f32(s == 0 ? 0x40 : (uint16_t)((uint16_t)s << 7));
    }
    for (int j = 0; j < gs; ++j) {
      const float w_el = scale == 0 ? 0.0f : ld(w, idx + j, dtype) / scale;
      float output;
      if (bits == 8) {
        output = fpq_from_fp8(fpq_to_fp8(w_el));
      } else {
        output = kFp4Lut[fpq_e2m1(w_el)];
      }
      st(out, idx + j, dtype, scale * output);
    }
  }
  return 0;
}

/* mlx/ops.cpp:5128-5190: the fallback of fp_quantize, op by op.  `T` below is
 * the element type of w; a value "in T" has been rounded to it.
 *   wq     = reshape(w, {-1, group_size})
 *   scales = max(abs(wq), -1) / T(maxval)                         (in T)
 * groups of 16 (no global scale: scale_encode = float32 1.0):
 *   scales = to_fp8(scales * 1.0f)                 (the product is float32)
 *   wq     = (wq / from_fp8(scales, T)) * 1.0f     (division in T, then float32)
 * groups of 32:
 *   scales = where(scales == 0, 0, int32(round(log2(scales))))    (in T)
 *   wq     = wq / power(T(2), scales)                             (in T)
 *   scales = uint8(scales + 127)
 * 4-bit:  code = argmin(abs(wq - T(lut)))  (in T for groups of 32, float32 for
 *         groups of 16; the first minimum wins), code j of a word at bit 4 j
 * 8-bit:  code = to_fp8(wq), four per word
 * round() is rint (mlx/backend/cpu/unary_ops.h:53), log2 is std::log2 on the
 * value widened to float (mlx/backend/cpu/simd/base_simd.h:137-144).  log2 is
 * evaluated in double here and rounded to float: glibc's and any other correct
 * float log2 give the same float except where the double result lies within a
 * few 1e-9 ulp of a rounding boundary. */
int fpq_quantize(const void* w, uint32_t* wq, uint8_t* scales, size_t n, int mode, int dtype) {
  if (mode < 0 || mode > 2 || dtype < 0 || dtype > 2) {
    return -1;
  }
  const int gs = fpq_group_size(mode);
  const int bits = fpq_bits(mode);
  if (n % (size_t)gs != 0 || (n * (size_t)bits) % 32 != 0) {
    return -1;
  }
  const float maxval = bits == 4 ? 6.0f : 448.0f;
  uint8_t* bytes = (uint8_t*)wq;
  memset(bytes, 0, n * (size_t)bits / 8);
  for (size_t g = 0; g < n / (size_t)gs; ++g) {
    const size_t idx = g * (size_t)gs;
    float m = 0.0f; /* max of abs: exact; NaN propagates as in std::max folds */
    for (int j = 0; j < gs; ++j) {
      const float a = fabsf(ld(w, idx + j, dtype));
      m = (a > m || isnan(a)) ? a : m;
    }
    float s = rnd(m / maxval, dtype);
    float q[32];
    int arg_in_t; /* whether wq - lut is rounded to T */
    if (gs == 16) {
      const uint8_t code = fpq_to_fp8(s);
      scales[g] = code;
      const float sv = rnd(fpq_from_fp8(code), dtype);
      for (int j = 0; j < gs; ++j) {
        q[j] = rnd(ld(w, idx + j, dtype) / sv, dtype);
      }
      arg_in_t = 0;
    } else {
      float e; /* the exponent as a value of T */
      if (s == 0.0f) {
        e = 0.0f;
      } else {
        const float l = rnd((float)log2((double)s), dtype);
        e = rnd(rintf(l), dtype);
        e = (float)(int32_t)e; /* astype(int32), then back into T by where() */
        e = rnd(e, dtype);
      }
      const float p = rnd(powf(2.0f, e), dtype);
      for (int j = 0; j < gs; ++j) {
        q[j] = rnd(ld(w, idx + j, dtype) / p, dtype);
      }
      const float biased = rnd(e + 127.0f, dtype);
      scales[g] = (uint8_t)(int32_t)biased; /* astype(uint8) of a float */
      arg_in_t = 1;
    }
    for (int j = 0; j < gs; ++j) {
      const size_t at = idx + j;
      if (bits == 8) {
        bytes[at] = fpq_to_fp8(q[j]);
        continue;
      }
      int best = 0;
      float best_d = 0.0f;
      for (int c = 0; c < 16; ++c) {
        float d = q[j] - kFp4Lut[c]; /* lut values are exact in T */
        if (arg_in_t) {
          d = rnd(d, dtype);
        }
        d = fabsf(d);
        if (c == 0 || d < best_d) {
          best = c;
          best_d = d;
        }
      }
      bytes[at / 2] |= (uint8_t)(best << (4 * (at & 1)));
    }
  }
  return 0;
}

/* mlx/ops.cpp:5399-5446: value = T(code value) * scale in T, where the scale is
 * from_fp8(s, T) * T(1) for groups of 16 and power(T(2), T(s) - T(127)) for
 * groups of 32.  4-bit codes: byte b of the packed stream holds elements 2 b
 * (low nibble) and 2 b + 1 (high nibble). */
int fpq_dequantize(
    const uint32_t* wq, const uint8_t* scales, void* out, size_t n, int mode, int dtype) {
  if (mode < 0 || mode > 2 || dtype < 0 || dtype > 2) {
    return -1;
  }
  const int gs = fpq_group_size(mode);
  const int bits = fpq_bits(mode);
  if (n % (size_t)gs != 0) {
    return -1;
  }
  const uint8_t* bytes = (const uint8_t*)wq;
  for (size_t i = 0; i < n; ++i) {
    float v;
    if (bits == 4) {
      v = kFp4Lut[(bytes[i / 2] >> (4 * (i & 1))) & 0xF];
    } else {
      v = rnd(fpq_from_fp8(bytes[i]), dtype);
    }
    const uint8_t sc = scales[i / (size_t)gs];
    float s;
    if (gs == 16) {
      s = rnd(rnd(fpq_from_fp8(sc), dtype) * 1.0f, dtype);
    } else {
      const float e = rnd(rnd((float)sc, dtype) - 127.0f, dtype);
      s = rnd(powf(2.0f, e), dtype);
    }
    st(out, i, dtype, v * s);
  }
  return 0;
}

/* mlx/backend/cpu/quantized.cpp:449-530 (fp_qmm, fp_qmm_t; the scalar forms are
 * what runs on x86, where simd::max_size<T> == 1): every product and sum is
 * rounded to T.
 *   transposed: w [N, K bits / 32], scales [N, K / gs]:
 *     y[m, n] = sum_g scale * (sum_{k in g} x[m, k] * T(code value))
 *   otherwise:  w [K, N bits / 32], scales [K, N / gs]:
 *     y[m, n] += (x[m, k] * scale) * T(code value), k ascending */
int fpq_qmm(
    void* result, const void* x, const uint32_t* w, const uint8_t* scales, int M, int N, int K,
    int mode, int transposed_w, int dtype) {
  if (mode < 0 || mode > 2 || dtype < 0 || dtype > 2) {
    return -1;
  }
  const int gs = fpq_group_size(mode);
  const int bits = fpq_bits(mode);
  const uint8_t* wb = (const uint8_t*)w;
  if (transposed_w) {
    if (K % gs != 0) {
      return -1;
    }
    for (int m = 0; m < M; ++m) {
      const uint8_t* w_local = wb;
      const uint8_t* s_local = scales;
      for (int n = 0; n < N; ++n) {
        float sum = 0.0f;
        size_t xi = (size_t)m * K;
        for (int k = 0; k < K; k += gs) {
          const float scale = scale_value(*s_local++, mode, dtype);
          float gsum = 0.0f;
          if (bits == 4) {
            for (int kw = 0; kw < gs / 2; ++kw) {
              gsum = rnd(gsum + rnd(ld(x, xi++, dtype) * kFp4Lut[w_local[0] & 0xF], dtype), dtype);
              gsum = rnd(
                  gsum + rnd(ld(x, xi++, dtype) * kFp4Lut[(w_local[0] >> 4) & 0xF], dtype), dtype);
              w_local++;
            }
          } else {
            for (int kw = 0; kw < gs; ++kw) {
              const float c = rnd(fpq_from_fp8(w_local[0]), dtype);
              gsum = rnd(gsum + rnd(ld(x, xi++, dtype) * c, dtype), dtype);
              w_local++;
            }
          }
          sum = rnd(sum + rnd(scale * gsum, dtype), dtype);
        }
        st(result, (size_t)m * N + n, dtype, sum);
      }
    }
    return 0;
  }
  if (N % gs != 0) {
    return -1;
  }
  for (int m = 0; m < M; ++m) {
    const uint8_t* w_local = wb;
    const uint8_t* s_local = scales;
    for (int n = 0; n < N; ++n) {
      st(result, (size_t)m * N + n, dtype, 0.0f);
    }
    for (int k = 0; k < K; ++k) {
      const float xi = ld(x, (size_t)m * K + k, dtype);
      size_t at = (size_t)m * N;
      for (int n = 0; n < N; n += gs) {
        const float scale = scale_value(*s_local++, mode, dtype);
        const float xs = rnd(xi * scale, dtype);
        if (bits == 4) {
          for (int ng = 0; ng < gs / 2; ++ng) {
            float r = ld(result, at, dtype);
            st(result, at++, dtype, r + rnd(xs * kFp4Lut[w_local[0] & 0xF], dtype));
            r = ld(result, at, dtype);
            st(result, at++, dtype, r + rnd(xs * kFp4Lut[(w_local[0] >> 4) & 0xF], dtype));
            w_local++;
          }
        } else {
          for (int ng = 0; ng < gs; ++ng) {
            const float c = rnd(fpq_from_fp8(w_local[0]), dtype);
            const float r = ld(result, at, dtype);
            st(result, at++, dtype, r + rnd(xs * c, dtype));
            w_local++;
          }
        }
      }
    }
  }
  return 0;
}
