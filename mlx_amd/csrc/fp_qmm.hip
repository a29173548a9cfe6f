// fp_qmm.hip -- quantized_matmul / gather_qmm for the floating-point modes
// (mxfp4, mxfp8, nvfp4): w holds e2m1 or e4m3 codes, scales one byte per group
// (e8m0, or e4m3 for groups of 16), no biases.
//
//   y[m, n] = sum_g scale[n, g] * sum_{k in g} x[m, k] * value(code[n, k])
//
// (mlx/backend/cpu/quantized.cpp:449-530).  The CPU evaluates every product and
// sum in the element type; here x and the code values are widened to fp32, the
// sums run in fp32 and the result is rounded once -- closer to the exact product.
//
// transpose=true: a streaming kernel (HBM-bound for few rows of x).  A lane
// owns 16 bytes of a packed row per step -- whole 1 KiB pieces of one row per
// wavefront instruction, as in the affine decode kernels -- and up to four rows
// of x per pass; more rows of x repeat the pass (the weights are re-read once
// per four rows: a functional floor for prefill, not a tile GEMM).
// transpose=false: one thread per eight output columns, k ascending.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

__device__ __forceinline__ float e4m3_value(uint32_t x) {
  const uint32_t e = (x >> 3) & 0xFu;
  const uint32_t m = x & 7u;
  const float mag = e == 0 ? static_cast<float>(m) * 0.001953125f
                           : __uint_as_float(((e + 120u) << 23) | (m << 20));
  return (x & 0x80u) ? -mag : mag;
}

__device__ __forceinline__ float e2m1_value(uint32_t c) {
  const uint32_t mag = c & 7u;
  const float v = mag < 2 ? 0.5f * static_cast<float>(mag)
                          : __uint_as_float((mag << 22) + (126u << 23));
  return (c & 8u) ? -v : v;
}

// mlx/backend/cpu/quantized.cpp:49-62 (dequantize_scale)
template <int GS>
__device__ __forceinline__ float scale_value(uint32_t s) {
  if constexpr (GS == 16) {
    return e4m3_value(s);
  } else {
    return __uint_as_float((s == 0 ? 0x40u : (s << 7)) << 16);
  }
}

struct FpProblem {
  const uint8_t* x;
  const uint8_t* w;
  const uint8_t* scales;
  uint8_t* out;
  bool valid;
};

__device__ __forceinline__ FpProblem fp_resolve(const QmmArgs& a, int l, size_t esize) {
  FpProblem p;
  int64_t xb = l;
  int64_t wb = l;
  p.valid = true;
  if (a.lhs_indices != nullptr) {
    const uint32_t xi = a.lhs_indices[l];
    const uint32_t wi = a.rhs_indices[l];
    p.valid = xi < static_cast<uint32_t>(a.x_batches) && wi < static_cast<uint32_t>(a.n_experts);
    xb = p.valid ? xi : 0;
    wb = p.valid ? wi : 0;
  }
  p.x = static_cast<const uint8_t*>(a.x) + xb * a.x_batch_stride * esize;
  p.w = reinterpret_cast<const uint8_t*>(a.w + wb * a.w_batch_stride);
  p.scales = static_cast<const uint8_t*>(a.scales) + wb * a.sb_batch_stride;
  p.out = static_cast<uint8_t*>(a.out) +
      static_cast<int64_t>(l) * a.M * static_cast<int64_t>(a.N) * esize;
  return p;
}

constexpr int kFpRowsPerWave = 2;
constexpr int kFpWaves = 4;
constexpr int kFpRowBlock = 4; // rows of x per pass

// K % (128 / BITS) == 0: a lane's 16 bytes never straddle the end of a row.
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(64 * kFpWaves) void fp_qmv_kernel(const QmmArgs a) {
  constexpr int kCodes = 128 / BITS; // codes per lane and step: 32 or 16
  constexpr int kGroups = kCodes / GS > 0 ? kCodes / GS : 1;
  constexpr int kPerGroup = kCodes / kGroups;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const FpProblem p = fp_resolve(a, blockIdx.z, sizeof(T));
  const int K = a.K;
  const int N = a.N;
  const int m0 = blockIdx.y * kFpRowBlock;
  const int rows = a.M - m0 < kFpRowBlock ? a.M - m0 : kFpRowBlock;
  const int n0 = (blockIdx.x * kFpWaves + wave) * kFpRowsPerWave;
  const size_t row_bytes = static_cast<size_t>(K) * BITS / 8;
  const int groups = K / GS;
  const T* x = reinterpret_cast<const T*>(p.x);

  float acc[kFpRowsPerWave][kFpRowBlock];
#pragma unroll
  for (int r = 0; r < kFpRowsPerWave; ++r) {
#pragma unroll
    for (int m = 0; m < kFpRowBlock; ++m) {
      acc[r][m] = 0.0f;
    }
  }
  for (int k0 = lane * kCodes; k0 < K; k0 += 64 * kCodes) {
    // this lane's slice of every row of x, as floats
    float xs[kFpRowBlock][kCodes];
#pragma unroll
    for (int m = 0; m < kFpRowBlock; ++m) {
      if (m < rows) {
#pragma unroll
        for (int j = 0; j < kCodes; j += 8) {
          float v[8];
          load8<T>(x + static_cast<size_t>(m0 + m) * K + k0 + j, v);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            xs[m][j + i] = v[i];
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < kCodes; ++j) {
          xs[m][j] = 0.0f;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kFpRowsPerWave; ++r) {
      const int n = n0 + r < N ? n0 + r : N - 1; // clamp: stay in bounds
      const uint4 wv = *reinterpret_cast<const uint4*>(
          p.w + static_cast<size_t>(n) * row_bytes + static_cast<size_t>(k0) * BITS / 8);
      const uint32_t words[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        const float s = scale_value<GS>(p.scales[static_cast<size_t>(n) * groups + k0 / GS + g]);
        float part[kFpRowBlock];
#pragma unroll
        for (int m = 0; m < kFpRowBlock; ++m) {
          part[m] = 0.0f;
        }
#pragma unroll
        for (int j = 0; j < kPerGroup; ++j) {
          const int c = g * kPerGroup + j; // code index inside the lane's slice
          float v;
          if constexpr (BITS == 4) {
            v = e2m1_value((words[c / 8] >> (4 * (c % 8))) & 0xFu);
          } else {
            v = e4m3_value((words[c / 4] >> (8 * (c % 4))) & 0xffu);
          }
#pragma unroll
          for (int m = 0; m < kFpRowBlock; ++m) {
            part[m] = fmaf(xs[m][c], v, part[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < kFpRowBlock; ++m) {
          acc[r][m] = fmaf(s, part[m], acc[r][m]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kFpRowsPerWave; ++r) {
#pragma unroll
    for (int m = 0; m < kFpRowBlock; ++m) {
      const float y = wave_sum(acc[r][m]);
      if (lane == 0 && m < rows && n0 + r < N) {
        reinterpret_cast<T*>(p.out)[static_cast<size_t>(m0 + m) * N + n0 + r] =
            from_f32<T>(p.valid ? y : 0.0f);
      }
    }
  }
}

// transpose=true, any K that is a multiple of the group size: one thread per
// output element (nvfp4 rows whose length is an odd multiple of 16).
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void fp_qmm_naive_t_kernel(const QmmArgs a) {
  const FpProblem p = fp_resolve(a, blockIdx.z, sizeof(T));
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  if (n >= a.N) {
    return;
  }
  const int K = a.K;
  const T* x = reinterpret_cast<const T*>(p.x) + static_cast<size_t>(m) * K;
  const uint8_t* w = p.w + static_cast<size_t>(n) * (static_cast<size_t>(K) * BITS / 8);
  const uint8_t* sc = p.scales + static_cast<size_t>(n) * (K / GS);
  float acc = 0.0f;
  for (int g = 0; g < K / GS; ++g) {
    float part = 0.0f;
    for (int j = 0; j < GS; ++j) {
      const int k = g * GS + j;
      float v;
      if constexpr (BITS == 4) {
        v = e2m1_value((w[k / 2] >> (4 * (k & 1))) & 0xFu);
      } else {
        v = e4m3_value(w[k]);
      }
      part = fmaf(to_f32(x[k]), v, part);
    }
    acc = fmaf(scale_value<GS>(sc[g]), part, acc);
  }
  reinterpret_cast<T*>(p.out)[static_cast<size_t>(m) * a.N + n] = from_f32<T>(p.valid ? acc : 0.0f);
}

// transpose=false: w [K, N bits / 32], scales [K, N / GS].  One thread per 8
// output columns of one row of x; N % 8 == 0 (N is a multiple of the group size).
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void fp_qmm_n_kernel(const QmmArgs a) {
  const FpProblem p = fp_resolve(a, blockIdx.z, sizeof(T));
  const int c8 = blockIdx.x * 256 + threadIdx.x; // block of 8 columns
  const int m = blockIdx.y;
  const int N = a.N;
  if (c8 * 8 >= N) {
    return;
  }
  const int K = a.K;
  const T* x = reinterpret_cast<const T*>(p.x) + static_cast<size_t>(m) * K;
  const size_t row_bytes = static_cast<size_t>(N) * BITS / 8;
  const int groups = N / GS;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    acc[i] = 0.0f;
  }
  for (int k = 0; k < K; ++k) {
    const float xs = to_f32(x[k]) * scale_value<GS>(p.scales[static_cast<size_t>(k) * groups + c8 * 8 / GS]);
    const uint8_t* w = p.w + static_cast<size_t>(k) * row_bytes;
    if constexpr (BITS == 4) {
      const uint32_t word = reinterpret_cast<const uint32_t*>(w)[c8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[i] = fmaf(xs, e2m1_value((word >> (4 * i)) & 0xFu), acc[i]);
      }
    } else {
      const uint2 words = reinterpret_cast<const uint2*>(w)[c8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = fmaf(xs, e4m3_value((words.x >> (8 * i)) & 0xffu), acc[i]);
        acc[4 + i] = fmaf(xs, e4m3_value((words.y >> (8 * i)) & 0xffu), acc[4 + i]);
      }
    }
  }
  T* y = reinterpret_cast<T*>(p.out) + static_cast<size_t>(m) * N + c8 * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    y[i] = from_f32<T>(p.valid ? acc[i] : 0.0f);
  }
}

template <typename F>
int dispatch_fp_mode(int mode, F&& fn) {
  switch (mode) {
    case MLXROCM_MXFP4:
      return fn(IntC<32>{}, IntC<4>{});
    case MLXROCM_MXFP8:
      return fn(IntC<32>{}, IntC<8>{});
    default:
      return fn(IntC<16>{}, IntC<4>{});
  }
}

int fp_check(const char* who, int M, int N, int K, int L, int mode, int dtype, int transpose) {
  if (mode != MLXROCM_MXFP4 && mode != MLXROCM_MXFP8 && mode != MLXROCM_NVFP4) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown quantization mode %d", who, mode);
  }
  if (!valid_dtype(dtype)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown dtype %d", who, dtype);
  }
  if (M < 0 || N < 0 || K < 0 || L < 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] negative dimension", who);
  }
  const int gs = mode == MLXROCM_NVFP4 ? 16 : 32;
  const int quantized_axis = transpose ? K : N;
  if (quantized_axis % gs != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the quantized dimension %d is not a multiple of group_size=%d (transpose=%d)", who,
        quantized_axis, gs, transpose);
  }
  return MLXROCM_OK;
}

// L problems (batch entries or index pairs), at most 65535 per launch.
int fp_launch(const QmmArgs& a, int mode, int dtype, bool transpose, hipStream_t s) {
  if (a.L > 65535 || a.M > 65535 * kFpRowBlock) {
    return fail(MLXROCM_UNSUPPORTED, "[quantized_matmul] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_fp_mode(mode, [&](auto gval, auto bval) {
      constexpr int G = decltype(gval)::value;
      constexpr int B = decltype(bval)::value;
      if (!transpose) {
        MLXROCM_REHEARSE("fp_qmm_n");
        const dim3 grid((a.N / 8 + 255) / 256, a.M, a.L);
        fp_qmm_n_kernel<T, G, B><<<grid, 256, 0, s>>>(a);
      } else if (a.K % (128 / B) == 0) {
        MLXROCM_REHEARSE("fp_qmv");
        const int rows_per_wg = kFpWaves * kFpRowsPerWave;
        const dim3 grid(
            (a.N + rows_per_wg - 1) / rows_per_wg, (a.M + kFpRowBlock - 1) / kFpRowBlock, a.L);
        fp_qmv_kernel<T, G, B><<<grid, 64 * kFpWaves, 0, s>>>(a);
      } else {
        MLXROCM_REHEARSE("fp_qmm_naive_t");
        const dim3 grid((a.N + 255) / 256, a.M, a.L);
        fp_qmm_naive_t_kernel<T, G, B><<<grid, 256, 0, s>>>(a);
      }
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  });
}

bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

} // namespace

} // namespace mlxrocm

using namespace mlxrocm;

extern "C" int mlxrocm_fp_qmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t scales_batch_stride,
    int mode,
    int dtype,
    int transpose,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_qmm");
  int rc = fp_check("quantized_matmul", M, N, K, L, mode, dtype, transpose);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * L == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(out, static_cast<size_t>(M) * N * L * dtype_size(dtype), s);
  }
  if (!x || !wq || !scales || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantized_matmul] null device pointer");
  }
  if (x_batch_stride < 0 || w_batch_stride < 0 || scales_batch_stride < 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantized_matmul] negative stride");
  }
  const int64_t x_vec = 16 / static_cast<int64_t>(dtype_size(dtype));
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out) ||
      (L > 1 && (x_batch_stride % x_vec != 0 || w_batch_stride % 4 != 0))) {
    return fail(MLXROCM_UNSUPPORTED, "[quantized_matmul] operands must keep 16-byte alignment");
  }
  QmmArgs a{};
  a.x = x;
  a.w = wq;
  a.scales = scales;
  a.biases = nullptr;
  a.out = out;
  a.M = M;
  a.N = N;
  a.K = K;
  a.L = L;
  a.x_batch_stride = x_batch_stride;
  a.w_batch_stride = w_batch_stride;
  a.sb_batch_stride = scales_batch_stride;
  a.x_batches = L;
  a.n_experts = L;
  return fp_launch(a, mode, dtype, transpose != 0, s);
}

extern "C" int mlxrocm_fp_gather_qmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    void* out,
    int M,
    int N,
    int K,
    int n_indices,
    int x_batches,
    int n_experts,
    int64_t x_batch_stride,
    int64_t w_expert_stride,
    int64_t scales_expert_stride,
    int mode,
    int dtype,
    int transpose,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_gather_qmm");
  int rc = fp_check("gather_qmm", M, N, K, n_indices, mode, dtype, transpose);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * n_indices == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(out, static_cast<size_t>(M) * N * n_indices * dtype_size(dtype), s);
  }
  if (!x || !wq || !scales || !out || !lhs_indices || !rhs_indices) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qmm] null device pointer");
  }
  if (x_batches <= 0 || n_experts <= 0 || x_batch_stride < 0 || w_expert_stride < 0 ||
      scales_expert_stride < 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qmm] invalid batch description");
  }
  const int64_t x_vec = 16 / static_cast<int64_t>(dtype_size(dtype));
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out) || x_batch_stride % x_vec != 0 ||
      w_expert_stride % 4 != 0) {
    return fail(MLXROCM_UNSUPPORTED, "[gather_qmm] operands must keep 16-byte alignment");
  }
  constexpr int kMaxZ = 65535;
  for (int first = 0; first < n_indices; first += kMaxZ) {
    QmmArgs a{};
    a.x = x;
    a.w = wq;
    a.scales = scales;
    a.out = static_cast<char*>(out) + static_cast<size_t>(first) * M * N * dtype_size(dtype);
    a.M = M;
    a.N = N;
    a.K = K;
    a.L = n_indices - first < kMaxZ ? n_indices - first : kMaxZ;
    a.x_batch_stride = x_batch_stride;
    a.w_batch_stride = w_expert_stride;
    a.sb_batch_stride = scales_expert_stride;
    a.lhs_indices = lhs_indices + first;
    a.rhs_indices = rhs_indices + first;
    a.x_batches = x_batches;
    a.n_experts = n_experts;
    rc = fp_launch(a, mode, dtype, transpose != 0, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
  }
  return MLXROCM_OK;
}
