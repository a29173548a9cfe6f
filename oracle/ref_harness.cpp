// ref_harness.cpp -- builds the reference's own CPU implementation of the
// affine quantized path into oracle/_ref/libmlx_cpu_qref.so.
//
// TEST INFRASTRUCTURE ONLY.  Nothing of the reference is copied: this file
// includes mlx/backend/cpu/quantized.cpp where it lies in the reference
// checkout (include path given on the command line by oracle/build.py) as one
// translation unit and exposes its raw-pointer templates through a C
// interface.  Every array-based function of that file is dead-stripped
// (--gc-sections + export map), so no other MLX object is needed.
//
//   ref_quantize -> mlx::core::quantize<T,U>          cpu/quantized.cpp:1148
//   ref_qmm      -> _qmm_dispatch_typed<T> (pointers) cpu/quantized.cpp:340
//   ref_*16_*    -> _MLX_Float16 / _MLX_BFloat16      mlx/types/{fp16,bf16}.h
//   ref_to_fp8 / ref_from_fp8 -> detail::ToFP8 / FromFP8  cpu/unary_ops.h:120-174
//   ref_e8m0 / ref_e2m1 -> to_fp8_e8m0 / to_fp4_e2m1   cpu/quantized.cpp:1049-1091
//   ref_fp_qmm   -> fp_qmm_dispatch_transpose<T, gs, bits> cpu/quantized.cpp:603
#include "mlx/backend/cpu/quantized.cpp"

#define REF_EXPORT extern "C" __attribute__((visibility("default")))

using namespace mlx::core;

REF_EXPORT int ref_simd_max_size(int dtype) {
  switch (dtype) {
    case 0:
      return simd::max_size<float>;
    case 1:
      return simd::max_size<float16_t>;
    default:
      return simd::max_size<bfloat16_t>;
  }
}

REF_EXPORT uint16_t ref_bf16_from_f32(float x) {
  return bfloat16_t(x).bits_;
}
REF_EXPORT float ref_bf16_to_f32(uint16_t b) {
  bfloat16_t v;
  v.bits_ = b;
  return static_cast<float>(v);
}
REF_EXPORT uint16_t ref_f16_from_f32(float x) {
  return float16_t(x).bits_;
}
REF_EXPORT float ref_f16_to_f32(uint16_t b) {
  float16_t v;
  v.bits_ = b;
  return static_cast<float>(v);
}

template <typename T>
static void quantize_any(
    const void* w,
    void* out,
    void* scales,
    void* biases,
    int bits,
    int group_size,
    size_t w_size) {
  // Same U selection as fast::Quantize::eval_cpu (cpu/quantized.cpp:1251-1274)
  if (is_power_of_2(bits)) {
    quantize<T, uint32_t>(
        (const T*)w, (uint32_t*)out, (T*)scales, (T*)biases, bits, group_size,
        w_size);
  } else {
    quantize<T, uint8_t>(
        (const T*)w, (uint8_t*)out, (T*)scales, (T*)biases, bits, group_size,
        w_size);
  }
}

REF_EXPORT int ref_quantize(
    const void* w,
    void* out,
    void* scales,
    void* biases,
    int bits,
    int group_size,
    size_t w_size,
    int dtype) {
  switch (dtype) {
    case 0:
      quantize_any<float>(w, out, scales, biases, bits, group_size, w_size);
      return 0;
    case 1:
      quantize_any<float16_t>(w, out, scales, biases, bits, group_size, w_size);
      return 0;
    case 2:
      quantize_any<bfloat16_t>(
          w, out, scales, biases, bits, group_size, w_size);
      return 0;
    default:
      return -1;
  }
}

REF_EXPORT int ref_qmm(
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
  try {
    switch (dtype) {
      case 0:
        _qmm_dispatch_typed<float>(
            (float*)result, (const float*)x, w, (const float*)scales,
            (const float*)biases, M, N, K, group_size, bits, transposed_w);
        return 0;
      case 1:
        _qmm_dispatch_typed<float16_t>(
            (float16_t*)result, (const float16_t*)x, w,
            (const float16_t*)scales, (const float16_t*)biases, M, N, K,
            group_size, bits, transposed_w);
        return 0;
      case 2:
        _qmm_dispatch_typed<bfloat16_t>(
            (bfloat16_t*)result, (const bfloat16_t*)x, w,
            (const bfloat16_t*)scales, (const bfloat16_t*)biases, M, N, K,
            group_size, bits, transposed_w);
        return 0;
      default:
        return -1;
    }
  } catch (const std::exception&) {
    return -1;
  }
}

REF_EXPORT uint8_t ref_to_fp8(float x) {
  return detail::ToFP8{}(x);
}
REF_EXPORT float ref_from_fp8(uint8_t x) {
  return detail::FromFP8{}(x);
}
REF_EXPORT uint8_t ref_e8m0(float x) {
  return to_fp8_e8m0(x);
}
REF_EXPORT uint8_t ref_e2m1(float x) {
  return to_fp4_e2m1(x);
}

template <typename T>
static void fp_qmm_any(
    void* result, const void* x, const uint32_t* w, const uint8_t* scales, int M, int N, int K,
    int mode, bool transposed_w) {
  // the three instantiations of fp_qmm_dispatch_typed (cpu/quantized.cpp:648-662)
  if (mode == 1) {
    fp_qmm_dispatch_transpose<T, 32, 8>((T*)result, (const T*)x, w, scales, M, N, K, transposed_w);
  } else if (mode == 0) {
    fp_qmm_dispatch_transpose<T, 32, 4>((T*)result, (const T*)x, w, scales, M, N, K, transposed_w);
  } else {
    fp_qmm_dispatch_transpose<T, 16, 4>((T*)result, (const T*)x, w, scales, M, N, K, transposed_w);
  }
}

// mode: 0 mxfp4, 1 mxfp8, 2 nvfp4
REF_EXPORT int ref_fp_qmm(
    void* result,
    const void* x,
    const uint32_t* w,
    const uint8_t* scales,
    int M,
    int N,
    int K,
    int mode,
    int transposed_w,
    int dtype) {
  if (mode < 0 || mode > 2) {
    return -1;
  }
  switch (dtype) {
    case 0:
      fp_qmm_any<float>(result, x, w, scales, M, N, K, mode, transposed_w);
      return 0;
    case 1:
      fp_qmm_any<float16_t>(result, x, w, scales, M, N, K, mode, transposed_w);
      return 0;
    case 2:
      fp_qmm_any<bfloat16_t>(result, x, w, scales, M, N, K, mode, transposed_w);
      return 0;
    default:
      return -1;
  }
}
