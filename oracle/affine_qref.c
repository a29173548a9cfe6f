/*
 * affine_qref.c -- CPU restatement of MLX's affine group-wise quantization path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity oracle: tests, the smoke
 * check and the cpu_baseline leg of the benchmark may link it; the product
 * library never does.  Every function names the reference lines it follows
 * (paths relative to the reference checkout).
 *
 * How each function is pinned (what a wrong restatement would fail):
 *   qref_f16_* / qref_bf16_*  exhaustive / randomized comparison with the
 *                             reference's own soft-float types compiled from
 *                             mlx/types/{fp16,bf16}.h (tests/test_oracle_vs_ref.py)
 *   qref_quantize             byte-for-byte against the reference's quantize<T,U>
 *                             (same test), committed golden vectors produced by
 *                             it, closed-form special cases, ramp test of
 *                             tests/ops_tests.cpp:3376-3395
 *   qref_qmm                  byte-for-byte against the reference's
 *                             _qmm_dispatch_typed<T> + golden vectors + fp64
 *                             GEMM on dequantized weights
 *   qref_dequantize           no callable reference function exists on the CPU
 *                             (the reference composes generic ops,
 *                             mlx/ops.cpp:5284-5326); pinned by: inverse of the
 *                             reference packer on every (bits, group) pair,
 *                             extract_bits masks, exact zero round trip
 *                             (python/tests/test_quantized.py:33-39), the
 *                             |w - w_hat| <= |scale| bound (:22-31) and the GGUF
 *                             d*q+m known-answer layout (python/tests/test_load.py:203-281)
 *   qref_qmm_batched /
 *   qref_gather_qmm           brute force: equal to per-problem qref_qmm calls;
 *                             equal to gather of dense fp64 products
 *
 * Element types: 0 = float32, 1 = float16, 2 = bfloat16.  On x86 the reference
 * computes float16/bfloat16 arithmetic with software types whose every binary
 * operator evaluates in float and rounds the result back to the 16-bit type
 * (mlx/types/half_types.h:16-21,33-38; mlx/types/bf16.h:68-101;
 * mlx/types/fp16.h binop macros).  rnd() below is that rounding step.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "affine_qref.h"

#define QREF_INLINE static inline __attribute__((always_inline))

QREF_INLINE uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
QREF_INLINE float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* mlx/types/bf16.h:42-58: NaN -> 0x7FC0, otherwise round-to-nearest-even by
 * adding 0x7FFF + lsb and keeping the upper half. */
uint16_t qref_bf16_from_f32(float x) {
  if (isnan(x)) {
    return 0x7FC0;
  }
  uint32_t u = f32_bits(x);
  u += ((u >> 16) & 1u) + 0x7FFFu;
  return (uint16_t)(u >> 16);
}

/* mlx/types/bf16.h:61-69 */
float qref_bf16_to_f32(uint16_t b) {
  return bits_f32((uint32_t)b << 16);
}

/* mlx/types/fp16.h:41-88.  The reference uses the "magic addition" conversion;
 * what it computes is IEEE binary32 -> binary16 with round-to-nearest-even,
 * overflow to infinity, gradual underflow, and NaN -> sign | 0x7D00.  This is a
 * direct bit-level statement of that function. */
uint16_t qref_f16_from_f32(float x) {
  uint32_t u = f32_bits(x);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) {
    return (uint16_t)(sign | 0x7D00u);
  }
  if (mag >= 0x47800000u) { /* >= 65536: inf (65520..65535.99 handled below) */
    return (uint16_t)(sign | 0x7C00u);
  }
  int32_t exp = (int32_t)(mag >> 23) - 127;
  uint32_t man = mag & 0x007FFFFFu;
  if (exp < -25) {
    return sign; /* below half of the smallest subnormal: rounds to zero */
  }
  uint32_t sig; /* significand to be shifted, with implicit bit */
  int shift;    /* bits to drop */
  uint32_t base;
  if (exp < -14) {
    /* subnormal half: value = sig * 2^(exp-23), target unit 2^-24 */
    sig = man | 0x00800000u;
    shift = -exp - 1; /* 14..24 */
    base = 0;
  } else {
    sig = man;
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
  }
  uint32_t kept = sig >> shift;
  uint32_t rem = sig & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) {
    kept += 1; /* may carry into the exponent, which is the right answer */
  }
  return (uint16_t)(sign | (base + kept));
}

/* mlx/types/fp16.h:90-118: exact widening of binary16 to binary32. */
float qref_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    /* zero / subnormal: man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-8f;
    return bits_f32(f32_bits(v) | sign);
  }
  if (exp == 31) {
    return bits_f32(sign | 0x7F800000u | (man << 13));
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

QREF_INLINE float ld(const void* p, size_t i, const int dt) {
  if (dt == QREF_F32) {
    return ((const float*)p)[i];
  } else if (dt == QREF_F16) {
    return qref_f16_to_f32(((const uint16_t*)p)[i]);
  } else {
    return qref_bf16_to_f32(((const uint16_t*)p)[i]);
  }
}

QREF_INLINE void st(void* p, size_t i, float v, const int dt) {
  if (dt == QREF_F32) {
    ((float*)p)[i] = v;
  } else if (dt == QREF_F16) {
    ((uint16_t*)p)[i] = qref_f16_from_f32(v);
  } else {
    ((uint16_t*)p)[i] = qref_bf16_from_f32(v);
  }
}

/* Result of one arithmetic operator evaluated in element type dt. */
QREF_INLINE float rnd(float v, const int dt) {
  if (dt == QREF_F32) {
    return v;
  } else if (dt == QREF_F16) {
    return qref_f16_to_f32(qref_f16_from_f32(v));
  } else {
    return qref_bf16_to_f32(qref_bf16_from_f32(v));
  }
}

/* mlx/backend/common/quantized.h:5-7 */
QREF_INLINE int pack_factor(int bits, int wsize) {
  return (bits == 3 || bits == 5) ? 8 : (bits == 6 ? 4 : wsize / bits);
}

/* mlx/backend/common/quantized.h:9-12 */
QREF_INLINE int bytes_per_pack(int bits, int wsize) {
  int pow2 = (bits & (bits - 1)) == 0;
  return pow2 ? (wsize / 8) : (bits == 5 ? 5 : 3);
}

int qref_pack_factor(int bits, int wsize) {
  return pack_factor(bits, wsize);
}
int qref_bytes_per_pack(int bits, int wsize) {
  return bytes_per_pack(bits, wsize);
}

/* mlx/backend/cpu/quantized.cpp:64-94: the byte masks of one 3/5/6-bit pack. */
QREF_INLINE void extract_bits(const uint8_t* in, int* out, const int bits) {
  if (bits == 3) {
    out[0] = in[0] & 0x7;
    out[1] = (in[0] & 0x38) >> 3;
    out[2] = ((in[0] & 0xc0) >> 6) + ((in[1] & 0x1) << 2);
    out[3] = (in[1] & 0xe) >> 1;
    out[4] = (in[1] & 0x70) >> 4;
    out[5] = ((in[1] & 0x80) >> 7) + ((in[2] & 0x3) << 1);
    out[6] = (in[2] & 0x1c) >> 2;
    out[7] = (in[2] & 0xe0) >> 5;
  } else if (bits == 5) {
    out[0] = in[0] & 0x1f;
    out[1] = ((in[0] & 0xe0) >> 5) + ((in[1] & 0x3) << 3);
    out[2] = (in[1] & 0x7c) >> 2;
    out[3] = ((in[1] & 0x80) >> 7) + ((in[2] & 0xf) << 1);
    out[4] = ((in[2] & 0xf0) >> 4) + ((in[3] & 0x1) << 4);
    out[5] = (in[3] & 0x3e) >> 1;
    out[6] = ((in[3] & 0xc0) >> 6) + ((in[4] & 0x7) << 2);
    out[7] = (in[4] & 0xf8) >> 3;
  } else { /* 6 */
    out[0] = in[0] & 0x3f;
    out[1] = ((in[0] >> 6) & 0x03) + ((in[1] & 0x0f) << 2);
    out[2] = ((in[1] >> 4) & 0x0f) + ((in[2] & 0x03) << 4);
    out[3] = (in[2] >> 2) & 0x3f;
  }
}

/* ------------------------------------------------------------------------ */
/* quantize<T,U>: mlx/backend/cpu/quantized.cpp:1148-1211                    */
/* ------------------------------------------------------------------------ */
QREF_INLINE void quantize_impl(
    const void* w,
    uint8_t* out,
    void* scales,
    void* biases,
    int bits,
    int group_size,
    size_t w_size,
    const int dt) {
  float n_bins = (float)((1 << bits) - 1);
  float eps = 1e-7f;

  int pow2 = (bits & (bits - 1)) == 0;
  int el_per_int = pack_factor(bits, 32);
  int bpp = bytes_per_pack(bits, 8);
  int int_per_group = group_size * bpp / el_per_int;
  size_t n_groups = w_size / (size_t)group_size;
  uint32_t* out32 = (uint32_t*)out;

  for (size_t i = 0; i < n_groups; ++i) {
    size_t w_idx = i * (size_t)group_size;
    float w_min = INFINITY;
    float w_max = -INFINITY;
    for (int j = 0; j < group_size; ++j) {
      float v = ld(w, w_idx + j, dt);
      w_max = (w_max < v) ? v : w_max; /* std::max(w_max, v) */
      w_min = (v < w_min) ? v : w_min; /* std::min(w_min, v) */
    }
    int mask = fabsf(w_min) > fabsf(w_max);
    float scale = (w_max - w_min) / n_bins;
    scale = (scale < eps) ? eps : scale; /* std::max(scale, eps) */
    scale = mask ? scale : -scale;

    float edge = mask ? w_min : w_max;
    float q0 = rintf(edge / scale);
    float bias = 0;
    if (q0 != 0) {
      scale = edge / q0;
      bias = edge;
    }
    size_t out_idx = i * (size_t)int_per_group;
    for (int j = 0; j < int_per_group / bpp; ++j) {
      uint64_t out_el = 0;
      for (int k = 0; k < el_per_int; ++k) {
        float w_el = ld(w, w_idx + (size_t)j * el_per_int + k, dt);
        w_el = rintf((w_el - bias) / scale);
        /* std::min(std::max(w_el, 0.0f), n_bins) */
        w_el = (w_el < 0.0f) ? 0.0f : w_el;
        w_el = (n_bins < w_el) ? n_bins : w_el;
        out_el |= (uint64_t)w_el << (k * bits);
      }
      if (pow2) {
        out32[out_idx + j] = (uint32_t)out_el;
      } else {
        for (int byte = 0; byte < bpp; ++byte) {
          out[out_idx + (size_t)bpp * j + byte] =
              (uint8_t)((out_el >> (8 * byte)) & 0xff);
        }
      }
    }
    st(scales, i, scale, dt);
    st(biases, i, bias, dt);
  }
}

int qref_quantize(
    const void* w,
    void* out,
    void* scales,
    void* biases,
    int bits,
    int group_size,
    size_t w_size,
    int dtype) {
  if (!(bits == 2 || bits == 3 || bits == 4 || bits == 5 || bits == 6 ||
        bits == 8) ||
      !(group_size == 32 || group_size == 64 || group_size == 128)) {
    return -1;
  }
  switch (dtype) {
    case QREF_F32:
      quantize_impl(w, out, scales, biases, bits, group_size, w_size, QREF_F32);
      return 0;
    case QREF_F16:
      quantize_impl(w, out, scales, biases, bits, group_size, w_size, QREF_F16);
      return 0;
    case QREF_BF16:
      quantize_impl(
          w, out, scales, biases, bits, group_size, w_size, QREF_BF16);
      return 0;
    default:
      return -1;
  }
}

/* ------------------------------------------------------------------------ */
/* dequantize: the op graph of mlx/ops.cpp:5284-5326.  The codes of the whole */
/* array form one little-endian bit stream (element e at bit e*bits,          */
/* :5294-5317); the affine step is Multiply then Add as two separately        */
/* rounded operations in scales' dtype (:5322-5323; uint32 x T promotes to T, */
/* mlx/dtype.cpp:35-48).                                                      */
/* ------------------------------------------------------------------------ */
QREF_INLINE uint32_t code_at(const uint32_t* wq, size_t e, int bits) {
  size_t bit = e * (size_t)bits;
  size_t word = bit >> 5;
  int sh = (int)(bit & 31);
  uint64_t v = wq[word];
  if (sh + bits > 32) {
    v |= (uint64_t)wq[word + 1] << 32;
  }
  return (uint32_t)((v >> sh) & ((1u << bits) - 1u));
}

QREF_INLINE void dequantize_impl(
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    size_t n_elems,
    int group_size,
    int bits,
    const int dt) {
  for (size_t e = 0; e < n_elems; ++e) {
    size_t g = e / (size_t)group_size;
    float q = rnd((float)code_at(wq, e, bits), dt); /* astype(T) */
    float s = ld(scales, g, dt);
    float b = ld(biases, g, dt);
    float v = rnd(q * s, dt);
    v = rnd(v + b, dt);
    st(out, e, v, dt);
  }
}

int qref_dequantize(
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype) {
  switch (dtype) {
    case QREF_F32:
      dequantize_impl(
          wq, scales, biases, out, n_elems, group_size, bits, QREF_F32);
      return 0;
    case QREF_F16:
      dequantize_impl(
          wq, scales, biases, out, n_elems, group_size, bits, QREF_F16);
      return 0;
    case QREF_BF16:
      dequantize_impl(
          wq, scales, biases, out, n_elems, group_size, bits, QREF_BF16);
      return 0;
    default:
      return -1;
  }
}

/* ------------------------------------------------------------------------ */
/* _qmm_t<T,bits,group_size>: mlx/backend/cpu/quantized.cpp:154-212          */
/* (the path x86 takes: simd::max_size<T> == 1, :286-307)                     */
/* ------------------------------------------------------------------------ */
QREF_INLINE void qmm_t_impl(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int group_size,
    const int bits,
    const int dt) {
  const int bitmask = (1 << bits) - 1;
  const int pf = pack_factor(bits, 8);
  const int bpp = bytes_per_pack(bits, 8);
  const int packs_in_group = group_size / pf;
  const int odd = (bits == 3 || bits == 5 || bits == 6);

  size_t r = 0;
  for (int m = 0; m < M; m++) {
    const uint8_t* w_local = (const uint8_t*)w;
    size_t sb = 0;
    for (int n = 0; n < N; n++) {
      size_t xk = (size_t)m * K;
      float sum = 0;
      for (int k = 0; k < K; k += group_size) {
        float scale = ld(scales, sb, dt);
        float bias = ld(biases, sb, dt);
        sb++;
        for (int kw = 0; kw < packs_in_group; kw++) {
          if (odd) {
            int wl[8];
            extract_bits(w_local, wl, bits);
            for (int p = 0; p < pf; p++) {
              float wv = rnd(rnd(scale * (float)wl[p], dt) + bias, dt);
              sum = rnd(sum + rnd(ld(x, xk + p, dt) * wv, dt), dt);
            }
            w_local += bpp;
            xk += pf;
          } else {
            uint8_t wi = *w_local++;
            for (int p = 0; p < pf; p++) {
              float wv =
                  rnd(rnd(scale * (float)(wi & bitmask), dt) + bias, dt);
              sum = rnd(sum + rnd(ld(x, xk, dt) * wv, dt), dt);
              xk++;
              if (bits != 8) {
                wi >>= bits;
              }
            }
          }
        }
      }
      st(result, r++, sum, dt);
    }
  }
}

/* ------------------------------------------------------------------------ */
/* _qmm<T,bits,group_size>: mlx/backend/cpu/quantized.cpp:96-152             */
/* (w is [K, N*bits/32], scales/biases [K, N/group_size])                     */
/* ------------------------------------------------------------------------ */
QREF_INLINE void qmm_n_impl(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int group_size,
    const int bits,
    const int dt) {
  const int bitmask = (1 << bits) - 1;
  const int pf = pack_factor(bits, 8);
  const int bpp = bytes_per_pack(bits, 8);
  const int packs_in_group = group_size / pf;
  const int odd = (bits == 3 || bits == 5 || bits == 6);

  for (int m = 0; m < M; m++) {
    const uint8_t* w_local = (const uint8_t*)w;
    size_t sb = 0;
    size_t row = (size_t)m * N;
    for (int n = 0; n < N; n++) {
      st(result, row + n, 0.0f, dt);
    }
    for (int k = 0; k < K; k++) {
      size_t rl = row;
      float xi = ld(x, (size_t)m * K + k, dt);
      for (int n = 0; n < N; n += group_size) {
        float scale = ld(scales, sb, dt);
        float bias = ld(biases, sb, dt);
        sb++;
        for (int ng = 0; ng < packs_in_group; ng++) {
          if (odd) {
            int wl[8];
            extract_bits(w_local, wl, bits);
            for (int p = 0; p < pf; p++) {
              float wv = rnd(rnd(scale * (float)wl[p], dt) + bias, dt);
              float acc = ld(result, rl, dt);
              st(result, rl, acc + rnd(xi * wv, dt), dt);
              rl++;
            }
            w_local += bpp;
          } else {
            uint8_t wi = *w_local++;
            for (int p = 0; p < pf; p++) {
              float wv =
                  rnd(rnd(scale * (float)(wi & bitmask), dt) + bias, dt);
              float acc = ld(result, rl, dt);
              st(result, rl, acc + rnd(xi * wv, dt), dt);
              rl++;
              if (bits != 8) {
                wi >>= bits;
              }
            }
          }
        }
      }
    }
  }
}

/* Dispatch on bits so the inner loops see a constant (the reference
 * instantiates templates per bits/group, :309-381). */
#define QREF_BITS_SWITCH(FN, DT)                                              \
  switch (bits) {                                                             \
    case 2:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 2, DT);           \
      break;                                                                  \
    case 3:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 3, DT);           \
      break;                                                                  \
    case 4:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 4, DT);           \
      break;                                                                  \
    case 5:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 5, DT);           \
      break;                                                                  \
    case 6:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 6, DT);           \
      break;                                                                  \
    case 8:                                                                   \
      FN(result, x, w, scales, biases, M, N, K, group_size, 8, DT);           \
      break;                                                                  \
    default:                                                                  \
      return -1;                                                              \
  }

#define QREF_DEFINE_QMM(NAME, DT)                                    \
  static int NAME(                                                   \
      void* result,                                                  \
      const void* x,                                                 \
      const uint32_t* w,                                             \
      const void* scales,                                            \
      const void* biases,                                            \
      int M,                                                         \
      int N,                                                         \
      int K,                                                         \
      int group_size,                                                \
      int bits,                                                      \
      int transposed_w) {                                            \
    if (transposed_w) {                                              \
      QREF_BITS_SWITCH(qmm_t_impl, DT)                               \
    } else {                                                         \
      QREF_BITS_SWITCH(qmm_n_impl, DT)                               \
    }                                                                \
    return 0;                                                        \
  }

QREF_DEFINE_QMM(qmm_f32, QREF_F32)
QREF_DEFINE_QMM(qmm_f16, QREF_F16)
QREF_DEFINE_QMM(qmm_bf16, QREF_BF16)

/* _qmm_dispatch_typed<T> (pointer overload):
 * mlx/backend/cpu/quantized.cpp:340-381 */
int qref_qmm(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int group_size,
    int bits,
    int transposed_w,
    int dtype) {
  if (!(group_size == 32 || group_size == 64 || group_size == 128)) {
    return -1;
  }
  switch (dtype) {
    case QREF_F32:
      return qmm_f32(
          result, x, w, scales, biases, M, N, K, group_size, bits,
          transposed_w);
    case QREF_F16:
      return qmm_f16(
          result, x, w, scales, biases, M, N, K, group_size, bits,
          transposed_w);
    case QREF_BF16:
      return qmm_bf16(
          result, x, w, scales, biases, M, N, K, group_size, bits,
          transposed_w);
    default:
      return -1;
  }
}

static size_t elem_size(int dtype) {
  return dtype == QREF_F32 ? 4 : 2;
}

/* _qmm_dispatch_typed<T> (array overload) batch loop:
 * mlx/backend/cpu/quantized.cpp:383-419.  Strides are in elements; a weight
 * stride of 0 is the "w.ndim() == 2" broadcast of :396-397. */
int qref_qmm_batched(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int batch,
    size_t x_batch_stride,
    size_t w_batch_stride,
    size_t sb_batch_stride,
    int group_size,
    int bits,
    int transposed_w,
    int dtype) {
  size_t es = elem_size(dtype);
  for (int i = 0; i < batch; i++) {
    int rc = qref_qmm(
        (char*)result + (size_t)i * M * N * es,
        (const char*)x + (size_t)i * x_batch_stride * es,
        w + (size_t)i * w_batch_stride,
        (const char*)scales + (size_t)i * sb_batch_stride * es,
        (const char*)biases + (size_t)i * sb_batch_stride * es,
        M,
        N,
        K,
        group_size,
        bits,
        transposed_w,
        dtype);
    if (rc != 0) {
      return rc;
    }
  }
  return 0;
}

/* _bs_qmm_dispatch_typed<T>: mlx/backend/cpu/quantized.cpp:700-747.
 * out[i] = qmm(x[lhs[i]], w[rhs[i]]); indices are flat batch indices. */
int qref_gather_qmm(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    int n_indices,
    int M,
    int N,
    int K,
    size_t x_batch_stride,
    size_t w_batch_stride,
    size_t sb_batch_stride,
    int group_size,
    int bits,
    int transposed_w,
    int dtype) {
  size_t es = elem_size(dtype);
  for (int i = 0; i < n_indices; i++) {
    size_t x_idx = lhs_indices[i];
    size_t w_idx = rhs_indices[i];
    int rc = qref_qmm(
        (char*)result + (size_t)i * M * N * es,
        (const char*)x + x_idx * x_batch_stride * es,
        w + w_idx * w_batch_stride,
        (const char*)scales + w_idx * sb_batch_stride * es,
        (const char*)biases + w_idx * sb_batch_stride * es,
        M,
        N,
        K,
        group_size,
        bits,
        transposed_w,
        dtype);
    if (rc != 0) {
      return rc;
    }
  }
  return 0;
}
