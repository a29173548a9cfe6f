// qmm_generic.hip -- width-agnostic quantized matmul kernels (any bits, group,
// dtype).  They are the functional floor under the MFMA kernels: every shape
// the operator accepts runs here when no specialised kernel applies.
//
//   qmv_generic : transpose=true, small M.  One wavefront per output row n;
//                 lanes stride over 8-code units of the row, so the packed row
//                 is read exactly once per launch row block, fully coalesced.
//                 y = sum_g ( s_g * sum_k x_k q_k  +  b_g * sum_k x_k ), fp32.
//   qmm_naive   : one thread per output element (transpose=true) or per 8
//                 adjacent outputs (transpose=false, the w [K, N] layout of
//                 mlx/backend/cpu/quantized.cpp:96-152).
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kRowsPerPass = 4; // x rows handled by one wave pass

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(256) void qmv_generic_kernel(const QmmArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = blockIdx.x * 4 + wave;
  const int m0 = blockIdx.y * kRowsPerPass;
  const int l = blockIdx.z;
  if (n >= a.N) {
    return; // whole wavefront leaves together; no block barrier below
  }
  const QmmProblem<T> p = resolve_problem<T>(a, l);
  const int K = a.K;
  const int groups = K / GS;
  const uint8_t* wrow = p.w + static_cast<size_t>(n) * (K / 8) * BITS;
  const T* srow = p.scales + static_cast<size_t>(n) * groups;
  const T* brow = p.biases + static_cast<size_t>(n) * groups;

  float acc[kRowsPerPass];
#pragma unroll
  for (int i = 0; i < kRowsPerPass; ++i) {
    acc[i] = 0.0f;
  }

  if (p.valid) {
    for (int u = lane; u < K / 8; u += kWaveSize) {
      const uint64_t unit = load_unit<BITS>(wrow, u);
      const int g = (u * 8) / GS;
      const float s = to_f32(srow[g]);
      const float b = to_f32(brow[g]);
      float q[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        q[i] = static_cast<float>(unit_code<BITS>(unit, i));
      }
#pragma unroll
      for (int mi = 0; mi < kRowsPerPass; ++mi) {
        if (m0 + mi < a.M) {
          float xv[8];
          load8<T>(p.x + static_cast<size_t>(m0 + mi) * K + u * 8, xv);
          float dot = 0.0f;
          float sx = 0.0f;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            dot = fmaf(xv[i], q[i], dot);
            sx += xv[i];
          }
          acc[mi] = fmaf(s, dot, acc[mi]);
          acc[mi] = fmaf(b, sx, acc[mi]);
        }
      }
    }
  }

#pragma unroll
  for (int mi = 0; mi < kRowsPerPass; ++mi) {
    const float total = wave_sum(acc[mi]);
    if (lane == 0 && m0 + mi < a.M) {
      p.out[static_cast<size_t>(m0 + mi) * a.N + n] = from_f32<T>(total);
    }
  }
}

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(256) void qmm_naive_t_kernel(const QmmArgs a) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  const int l = blockIdx.z;
  if (n >= a.N) {
    return;
  }
  const QmmProblem<T> p = resolve_problem<T>(a, l);
  const int K = a.K;
  const int groups = K / GS;
  float acc = 0.0f;
  if (p.valid) {
    const uint8_t* wrow = p.w + static_cast<size_t>(n) * (K / 8) * BITS;
    const T* srow = p.scales + static_cast<size_t>(n) * groups;
    const T* brow = p.biases + static_cast<size_t>(n) * groups;
    const T* xrow = p.x + static_cast<size_t>(m) * K;
    for (int u = 0; u < K / 8; ++u) {
      const uint64_t unit = load_unit<BITS>(wrow, u);
      const int g = (u * 8) / GS;
      const float s = to_f32(srow[g]);
      const float b = to_f32(brow[g]);
      float xv[8];
      load8<T>(xrow + u * 8, xv);
      float dot = 0.0f;
      float sx = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        dot = fmaf(xv[i], static_cast<float>(unit_code<BITS>(unit, i)), dot);
        sx += xv[i];
      }
      acc = fmaf(s, dot, acc);
      acc = fmaf(b, sx, acc);
    }
  }
  p.out[static_cast<size_t>(m) * a.N + n] = from_f32<T>(acc);
}

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(256) void qmm_naive_n_kernel(const QmmArgs a) {
  // w [K, N*BITS/32], scales/biases [K, N/GS]; a thread owns outputs
  // [8*un, 8*un + 8) of row m.
  const int un = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  const int l = blockIdx.z;
  if (un >= a.N / 8) {
    return;
  }
  const QmmProblem<T> p = resolve_problem<T>(a, l);
  const int K = a.K;
  const int N = a.N;
  const int groups = N / GS;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    acc[i] = 0.0f;
  }
  if (p.valid) {
    const T* xrow = p.x + static_cast<size_t>(m) * K;
    const int g = (un * 8) / GS;
    for (int k = 0; k < K; ++k) {
      const uint8_t* wrow = p.w + static_cast<size_t>(k) * (N / 8) * BITS;
      const uint64_t unit = load_unit<BITS>(wrow, un);
      const float s = to_f32(p.scales[static_cast<size_t>(k) * groups + g]);
      const float b = to_f32(p.biases[static_cast<size_t>(k) * groups + g]);
      const float xk = to_f32(xrow[k]);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float wv =
            fmaf(s, static_cast<float>(unit_code<BITS>(unit, i)), b);
        acc[i] = fmaf(xk, wv, acc[i]);
      }
    }
  }
  store8<T>(p.out + static_cast<size_t>(m) * N + un * 8, acc);
}

__global__ __launch_bounds__(256) void zero_fill_kernel(uint16_t* p, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) {
    p[i] = 0;
  }
}

} // namespace

// Zero `bytes` (a multiple of 2) of device memory with a kernel rather than a
// memset node, so the call can be captured into a HIP graph.  Only degenerate
// K == 0 products come here.
int launch_zero_fill(void* p, size_t bytes, hipStream_t s) {
  MLXROCM_REHEARSE("zero_fill");
  const size_t n = bytes / 2;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  zero_fill_kernel<<<blocks, 256, 0, s>>>(static_cast<uint16_t*>(p), n);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

int launch_qmv_generic(
    const QmmArgs& a,
    int gs,
    int bits,
    int dtype,
    hipStream_t s) {
  const dim3 grid(
      (a.N + 3) / 4, (a.M + kRowsPerPass - 1) / kRowsPerPass, a.L);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  MLXROCM_REHEARSE("qmv_generic");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(gs, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        qmv_generic_kernel<T, B, G><<<grid, 256, 0, s>>>(a);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  });
}

int launch_qmm_naive(
    const QmmArgs& a,
    int gs,
    int bits,
    int dtype,
    bool transpose,
    hipStream_t s) {
  constexpr int kMaxRows = 65535; // one grid row per row of x
  if (a.M > kMaxRows && a.lhs_indices == nullptr && a.L <= kMaxRows) {
    // more rows of x than a grid is deep: one problem at a time, in slices of rows
    const size_t esize = dtype_size(dtype);
    for (int l = 0; l < a.L; ++l) {
      for (int m0 = 0; m0 < a.M; m0 += kMaxRows) {
        QmmArgs part = a;
        part.L = 1;
        part.M = a.M - m0 < kMaxRows ? a.M - m0 : kMaxRows;
        part.x = static_cast<const char*>(a.x) +
            (static_cast<size_t>(l) * a.x_batch_stride + static_cast<size_t>(m0) * a.K) * esize;
        part.w = a.w + static_cast<size_t>(l) * a.w_batch_stride;
        part.scales = static_cast<const char*>(a.scales) +
            static_cast<size_t>(l) * a.sb_batch_stride * esize;
        part.biases = static_cast<const char*>(a.biases) +
            static_cast<size_t>(l) * a.sb_batch_stride * esize;
        part.out = static_cast<char*>(a.out) +
            (static_cast<size_t>(l) * a.M + m0) * static_cast<size_t>(a.N) * esize;
        const int rc = launch_qmm_naive(part, gs, bits, dtype, transpose, s);
        if (rc != MLXROCM_OK) {
          return rc;
        }
      }
    }
    return MLXROCM_OK;
  }
  const int cols = transpose ? a.N : a.N / 8;
  const dim3 grid((cols + 255) / 256, a.M, a.L);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  MLXROCM_REHEARSE(transpose ? "qmm_naive_t" : "qmm_naive_n");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(gs, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        if (transpose) {
          qmm_naive_t_kernel<T, B, G><<<grid, 256, 0, s>>>(a);
        } else {
          qmm_naive_n_kernel<T, B, G><<<grid, 256, 0, s>>>(a);
        }
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  });
}

} // namespace mlxrocm
