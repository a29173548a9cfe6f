// qmm_mfma.hip -- prefill GEMM (transpose=true, large M) for 16-bit element
// types and every code width, on the gfx950 matrix cores.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T
//
// A workgroup of 256 threads (2 x 2 wavefronts) owns a 256 (M) x 128 (N) tile of
// y and walks K in steps of 64.  Per step:
//   * the x tile (256 x 64) and the packed W tile (128 rows x 64 codes) are
//     fetched into registers while the previous step's MFMAs run;
//   * W is dequantized exactly once per workgroup -- thread (n, h) expands the
//     32 codes [32h, 32h+32) of row n with one scale/bias pair (a K-step never
//     holds more than one group per 32 codes) as fp32 fma(s, code, b), rounds to
//     T and stores them to LDS, so the 256 rows of x reuse every weight;
//   * each wavefront computes a 64 (N) x 128 (M) block of y^T with
//     v_mfma_f32_32x32x16: A operand = W rows, B operand = x rows, so that a lane
//     ends up with 4 consecutive n of one m -- an 8-byte store of y.
// LDS rows are 64 elements + 8 of padding (144 bytes), which makes the 16-byte
// fragment reads of 16 consecutive rows hit 64 distinct banks.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 256;
constexpr int kBN = 128;
constexpr int kBK = 64;
constexpr int kLdsStride = kBK + 8; // elements per LDS row
constexpr int kThreads = 256;

template <typename T>
__device__ __forceinline__ floatx16 mfma32(const uint4& a, const uint4& b, const floatx16& c);

template <>
__device__ __forceinline__ floatx16
mfma32<bf16_t>(const uint4& a, const uint4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
      __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <>
__device__ __forceinline__ floatx16
mfma32<f16_t>(const uint4& a, const uint4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(
      __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  union {
    T h[2];
    uint32_t u;
  } r;
  r.h[0] = static_cast<T>(lo);
  r.h[1] = static_cast<T>(hi);
  return r.u;
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

// 32 codes -> 32 elements of T: fma(s, code, b) in fp32, one rounding to T.
template <typename T, int BITS>
__device__ __forceinline__ void dequant32(
    const uint32_t (&w)[BITS],
    float s,
    float b,
    uint32_t (&out)[16]) {
  if constexpr (BITS == 4) {
    // nibbles -> bytes first, so that every convert is a cvt_f32_ubyteN
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t lo = w[d] & 0x0f0f0f0fu;        // codes 0,2,4,6
      const uint32_t hi = (w[d] >> 4) & 0x0f0f0f0fu; // codes 1,3,5,7
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float c0 = static_cast<float>((lo >> (8 * j)) & 0xffu);
        const float c1 = static_cast<float>((hi >> (8 * j)) & 0xffu);
        out[4 * d + j] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
      }
    }
  } else if constexpr (BITS == 8) {
#pragma unroll
    for (int d = 0; d < 8; ++d) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float c0 = static_cast<float>((w[d] >> (16 * j)) & 0xffu);
        const float c1 = static_cast<float>((w[d] >> (16 * j + 8)) & 0xffu);
        out[2 * d + j] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float c0 = static_cast<float>(code32<BITS>(w, 2 * i));
      const float c1 = static_cast<float>(code32<BITS>(w, 2 * i + 1));
      out[i] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
    }
  }
}

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(kThreads) void qmm_t_mfma_kernel(const QmmArgs a) {
  __shared__ __attribute__((aligned(16))) T xs[kBM * kLdsStride];
  __shared__ __attribute__((aligned(16))) T ws[kBN * kLdsStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wn = wave & 1;  // which 64 columns (n) of the tile
  const int wm = wave >> 1; // which 128 rows (m) of the tile
  const int M = a.M;
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kBN;
  const int m0 = blockIdx.y * kBM;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.z);

  const int groups = K / GS;
  const int row_words = K / 32 * BITS;

  // ---- loader roles ----
  // x: thread covers 16-byte chunk (tid % 8) of rows tid/8 + 32 i, i < 8.
  const int xc = tid & 7;
  const int xr = tid >> 3;
  // W: thread (wr, wh) covers codes [32 wh, 32 wh + 32) of tile row wr.
  const int wr = tid >> 1;
  const int wh = tid & 1;
  const int w_row = (n0 + wr < N) ? n0 + wr : N - 1; // clamp: loads stay in bounds
  const uint32_t* wsrc = reinterpret_cast<const uint32_t*>(p.w) +
      static_cast<size_t>(w_row) * row_words + wh * BITS;
  const T* ssrc = p.scales + static_cast<size_t>(w_row) * groups;
  const T* bsrc = p.biases + static_cast<size_t>(w_row) * groups;

  uint4 xreg[8];
  uint32_t wreg[BITS];
  float sreg, breg;

  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int m = m0 + xr + 32 * i;
      xreg[i] = make_uint4(0, 0, 0, 0);
      if (m < M) {
        xreg[i] = *reinterpret_cast<const uint4*>(p.x + static_cast<size_t>(m) * K + k0 + xc * 8);
      }
    }
    const uint32_t* wp = wsrc + (k0 / 32) * BITS;
#pragma unroll
    for (int j = 0; j < BITS; ++j) {
      wreg[j] = wp[j];
    }
    const int g = (k0 + 32 * wh) / GS;
    sreg = to_f32(ssrc[g]);
    breg = to_f32(bsrc[g]);
  };

  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      *reinterpret_cast<uint4*>(&xs[(xr + 32 * i) * kLdsStride + xc * 8]) = xreg[i];
    }
    uint32_t dq[16];
    dequant32<T, BITS>(wreg, sreg, breg, dq);
    uint4* dst = reinterpret_cast<uint4*>(&ws[wr * kLdsStride + wh * 32]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dst[j] = make_uint4(dq[4 * j], dq[4 * j + 1], dq[4 * j + 2], dq[4 * j + 3]);
    }
  };

  // ---- accumulators: 2 (n) x 4 (m) tiles of 32 x 32 ----
  floatx16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }

  const int fr = lane & 31; // fragment row inside a 32-row MFMA tile
  const int fk = lane >> 5; // which 8 of the 16 k of an MFMA step
  const T* wfrag = &ws[(wn * 64 + fr) * kLdsStride + fk * 8];
  const T* xfrag = &xs[(wm * 128 + fr) * kLdsStride + fk * 8];

  load_tile(0);
  for (int k0 = 0; k0 < K; k0 += kBK) {
    __syncthreads(); // the previous step's fragment reads are done
    store_tile();
    __syncthreads();
    if (k0 + kBK < K) {
      load_tile(k0 + kBK);
    }
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      uint4 af[2];
      uint4 bf[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *reinterpret_cast<const uint4*>(wfrag + i * 32 * kLdsStride + kk * 16);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bf[j] = *reinterpret_cast<const uint4*>(xfrag + j * 32 * kLdsStride + kk * 16);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = mfma32<T>(af[i], bf[j], acc[i][j]);
        }
      }
    }
  }

  // ---- epilogue: D[n][m] tiles; register r of lane (col, half) holds
  // n = 8 (r / 4) + 4 half + r % 4, m = col.  Four consecutive n -> one 8-byte
  // store of y[m][n .. n+3].
  const int col = lane & 31;
  const int half = lane >> 5;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + wm * 128 + j * 32 + col;
    if (m >= M) {
      continue;
    }
    T* yrow = p.out + static_cast<size_t>(m) * N;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + i * 32 + 8 * q + 4 * half;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = p.valid ? acc[i][j][4 * q + e] : 0.0f;
        }
        if (n + 3 < N && (N % 4) == 0) {
          uint2 packed;
          packed.x = pack2<T>(v[0], v[1]);
          packed.y = pack2<T>(v[2], v[3]);
          *reinterpret_cast<uint2*>(yrow + n) = packed;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < N) {
              yrow[n + e] = from_f32<T>(v[e]);
            }
          }
        }
      }
    }
  }
}

} // namespace

bool qmm_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  (void)gs;
  (void)bits;
  if (!transpose || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  return a.K % kBK == 0 && a.K >= kBK;
}

int launch_qmm_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const dim3 grid((a.N + kBN - 1) / kBN, (a.M + kBM - 1) / kBM, a.L);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(gs, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        qmm_t_mfma_kernel<T, B, G><<<grid, kThreads, 0, s>>>(a);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
