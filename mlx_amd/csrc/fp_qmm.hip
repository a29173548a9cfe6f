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
// per four rows: a functional floor for prefill, not a tile GEMM).  For the
// 16-bit element types the codes are widened two at a time by the hardware's
// fp4 / fp8 converts (v_cvt_scalef32_pk_{bf16,f16}_{fp4,fp8} with scale 1: both
// formats are exact in bf16 and f16) and multiplied with v_dot2_f32_{bf16,f16};
// the group's scale is applied to the partial sum, once per group.
// transpose=false: one thread per eight output columns, k ascending.
#include <type_traits>

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

// Factor of the fp32 sums: weights quantized with a tensor-wide scale (nvfp4
// only; mlx/backend/cuda/quantized/qmm/qmv.cu:163-165), 1 otherwise.
template <int GS>
__device__ __forceinline__ float fp_out_factor(const QmmArgs& a) {
  if constexpr (GS == 16) {
    if (a.out_scale != nullptr) {
      return *a.out_scale / (448.0f * 6.0f);
    }
  }
  return 1.0f;
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
  const float out_factor = fp_out_factor<GS>(a);
#pragma unroll
  for (int r = 0; r < kFpRowsPerWave; ++r) {
#pragma unroll
    for (int m = 0; m < kFpRowBlock; ++m) {
      const float y = wave_sum(acc[r][m]) * out_factor;
      if (lane == 0 && m < rows && n0 + r < N) {
        reinterpret_cast<T*>(p.out)[static_cast<size_t>(m0 + m) * N + n0 + r] =
            from_f32<T>(p.valid ? y : 0.0f);
      }
    }
  }
}

typedef __bf16 fp_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 fp_f16x2 __attribute__((ext_vector_type(2)));

// Codes -> pairs of T, packed in a dword (first code in the low half), and the
// two-element dot product with fp32 accumulation.
template <typename T>
struct FpWiden;

template <>
struct FpWiden<bf16_t> {
  // the eight e2m1 codes of a word: byte b holds codes 2 b (low nibble), 2 b + 1
  static __device__ __forceinline__ void fp4(uint32_t w, uint32_t (&p)[4]) {
    p[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 0));
    p[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 1));
    p[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 2));
    p[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 3));
  }
  // the four e4m3 codes of a word
  static __device__ __forceinline__ void fp8(uint32_t w, uint32_t (&p)[2]) {
    p[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
    p[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(
        __builtin_bit_cast(fp_bf16x2, a), __builtin_bit_cast(fp_bf16x2, b), c, false);
  }
};

template <>
struct FpWiden<f16_t> {
  static __device__ __forceinline__ void fp4(uint32_t w, uint32_t (&p)[4]) {
    p[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0));
    p[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1));
    p[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2));
    p[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3));
  }
  static __device__ __forceinline__ void fp8(uint32_t w, uint32_t (&p)[2]) {
    p[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
    p[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(
        __builtin_bit_cast(fp_f16x2, a), __builtin_bit_cast(fp_f16x2, b), c, false);
  }
};

// An e4m3 byte whose low seven bits are all ones: NaN to the hardware convert,
// +-480 to the reference's decoder (mlx/backend/cpu/quantized.cpp FromFP8, which
// has no special codes).  The quantizer never writes it (it saturates at 448).
__device__ __forceinline__ bool has_e4m3_top_code(uint32_t w) {
  return (((w & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u) != 0;
}

template <typename T>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  const T a = from_f32<T>(lo);
  const T b = from_f32<T>(hi);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, a)) |
      (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, b)) << 16);
}

// 16-byte load of data that is read exactly once: nontemporal, so the stream
// does not displace x and the scales from the caches.
__device__ __forceinline__ uint4 load_once(const uint8_t* p) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

constexpr int kFp16Waves = 4;

// 16-bit element types, K % (128 / BITS) == 0.  MB rows of x per pass (1, 2 or
// 4), RPW rows of w per wavefront.
// XL: the workgroup's four wavefronts work on the same codes of different rows of
// W, so the step's slice of x (MB rows x 64 lanes x kCodes elements) is fetched
// once per workgroup into LDS -- piece j of lane l at ((m P + j) 64 + l) 16 bytes,
// so that 16-byte reads of neighbouring lanes hit every bank once -- instead of
// once per wavefront from the caches: with four rows of x those re-reads were
// four times the bytes of the weights and set the kernel's time.
template <typename T, int GS, int BITS, int MB, int RPW, bool XL = false>
__global__ __launch_bounds__(64 * kFp16Waves) void fp_qmv16_kernel(const QmmArgs a) {
  constexpr int kCodes = 128 / BITS; // codes per lane and step: 32 or 16
  constexpr int kPairs = kCodes / 2;
  constexpr int kPieces = kPairs / 4; // 16-byte pieces of x per lane, row and step
  constexpr int kGroups = kCodes / GS > 0 ? kCodes / GS : 1;
  constexpr int kPairsPerGroup = kPairs / kGroups;
  __shared__ __attribute__((aligned(16))) uint4 xs[XL ? MB * kPieces * 64 : 1];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const FpProblem p = fp_resolve(a, blockIdx.z, sizeof(T));
  const int K = a.K;
  const int N = a.N;
  const int m0 = blockIdx.y * MB;
  const int n0 = (blockIdx.x * kFp16Waves + wave) * RPW;
  if constexpr (!XL) {
    if (n0 >= N) {
      return;
    }
  }
  const size_t row_bytes = static_cast<size_t>(K) * BITS / 8;
  const int groups = K / GS;
  const T* x = reinterpret_cast<const T*>(p.x);

  float acc[RPW][MB];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      acc[r][m] = 0.0f;
    }
  }
  const uint8_t* wrow[RPW];
  const uint8_t* srow[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int n = n0 + r < N ? n0 + r : N - 1; // clamp: stay in bounds
    wrow[r] = p.w + static_cast<size_t>(n) * row_bytes;
    srow[r] = p.scales + static_cast<size_t>(n) * groups;
  }
  // The codes and scale bytes of a step are fetched one step ahead of their use,
  // so that a wavefront always has two steps' loads in flight.  A lane whose
  // codes lie past K fetches nothing and multiplies zero codes.
  uint4 wv_next[RPW];
  uint32_t sb_next[RPW][kGroups];
  auto fetch_w = [&](int kb) {
    const int kf = kb + lane * kCodes;
    const bool in_range = kf < K;
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      wv_next[r] = in_range ? load_once(wrow[r] + static_cast<size_t>(kf) * BITS / 8)
                            : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        sb_next[r][g] = in_range ? srow[r][kf / GS + g] : 0x7fu;
      }
    }
  };
  fetch_w(0);
  // every lane takes every step (the staged form has barriers inside)
  for (int kbase = 0; kbase < K; kbase += 64 * kCodes) {
    const int k0 = kbase + lane * kCodes;
    const bool live = k0 < K;
    if constexpr (!XL) {
      if (!live) {
        break; // no barriers here, and the lanes past K stay past K
      }
    }
    uint4 wv[RPW];
    uint32_t sb[RPW][kGroups];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      wv[r] = wv_next[r];
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        sb[r][g] = sb_next[r][g];
      }
    }
    fetch_w(kbase + 64 * kCodes);
    // this lane's slice of the rows of x, as pairs
    uint32_t xr[MB][kPairs];
    if constexpr (XL) {
      __syncthreads(); // the previous step's slice has been read
      // the slice is MB rows of 64 kPieces pieces; thread t takes pieces t, t + 256, ..
      for (int i = threadIdx.x; i < MB * 64 * kPieces; i += 64 * kFp16Waves) {
        const int m = i / (64 * kPieces);
        const int piece = i % (64 * kPieces); // along k: lane piece / kPieces, its piece % kPieces
        const int row = m0 + m < a.M ? m0 + m : a.M - 1;
        const int k = kbase + piece * 8;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (k < K) {
          v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K + k);
        }
        xs[(m * kPieces + piece % kPieces) * 64 + piece / kPieces] = v;
      }
      __syncthreads();
#pragma unroll
      for (int m = 0; m < MB; ++m) {
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
          const uint4 v = xs[(m * kPieces + j) * 64 + lane];
          xr[m][4 * j + 0] = v.x;
          xr[m][4 * j + 1] = v.y;
          xr[m][4 * j + 2] = v.z;
          xr[m][4 * j + 3] = v.w;
        }
      }
    } else {
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const int row = m0 + m < a.M ? m0 + m : a.M - 1;
        const uint4* src = reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K + k0);
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
          const uint4 v = src[j];
          xr[m][4 * j + 0] = v.x;
          xr[m][4 * j + 1] = v.y;
          xr[m][4 * j + 2] = v.z;
          xr[m][4 * j + 3] = v.w;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const uint32_t words[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
      uint32_t pr[kPairs];
      if constexpr (BITS == 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t q[4];
          FpWiden<T>::fp4(words[i], q);
          pr[4 * i + 0] = q[0];
          pr[4 * i + 1] = q[1];
          pr[4 * i + 2] = q[2];
          pr[4 * i + 3] = q[3];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t q[2];
          FpWiden<T>::fp8(words[i], q);
          if (has_e4m3_top_code(words[i])) {
            q[0] = pack_pair<T>(e4m3_value(words[i] & 0xffu), e4m3_value((words[i] >> 8) & 0xffu));
            q[1] = pack_pair<T>(e4m3_value((words[i] >> 16) & 0xffu), e4m3_value(words[i] >> 24));
          }
          pr[2 * i + 0] = q[0];
          pr[2 * i + 1] = q[1];
        }
      }
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        const float s = scale_value<GS>(sb[r][g]);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
          float part = 0.0f;
#pragma unroll
          for (int j = 0; j < kPairsPerGroup; ++j) {
            part = FpWiden<T>::dot2(xr[m][g * kPairsPerGroup + j], pr[g * kPairsPerGroup + j], part);
          }
          acc[r][m] = fmaf(s, part, acc[r][m]);
        }
      }
    }
  }
  const float out_factor = fp_out_factor<GS>(a);
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float y = wave_sum(acc[r][m]) * out_factor;
      if (lane == 0 && m0 + m < a.M && n0 + r < N) {
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
  acc *= fp_out_factor<GS>(a);
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

// From this many rows of x on, 16-bit problems with transpose=true run on the
// matrix-core tile kernel (one pass over W, K split into ranges while the tiles
// do not fill the chip) instead of one streaming pass per four rows.  bf16
// [M, 4096] x [14336, 4096], mxfp4 / mxfp8 / nvfp4: streaming 30 / 35 / 35 us at
// 8 rows (two passes); the tile kernel with its scale pre-pass 37 / 39 / 40 us at
// 9 rows, 39 / 41 / 43 at 64, 70 / 73 / 75 at 512.
constexpr int kFpTileMinM = 9;

// The tile kernel addresses its operands with 32-bit byte offsets.
bool fp_tile_applies(int M, int N, int K, int L, int mode, int dtype, bool transpose) {
  const int bits = mode == MLXROCM_MXFP8 ? 8 : 4;
  const uint64_t limit = uint64_t{1} << 32;
  return transpose && dtype != MLXROCM_FLOAT32 && M >= kFpTileMinM && K % 64 == 0 && K >= 64 &&
      L >= 1 && static_cast<uint64_t>(N) * K * bits / 8 < limit &&
      static_cast<uint64_t>(M) * K * 2 < limit && static_cast<uint64_t>(M) * N * 2 < limit &&
      static_cast<uint64_t>(N) * (K / 32) * 4 < limit;
}

size_t fp_image_bytes(int N, int K, int batches) {
  return (static_cast<size_t>(batches) * N * (K / 32) * 4 + 255) / 256 * 256;
}

// ranges of K for a launch whose tiles do not fill the compute units
int fp_k_splits(int M, int N, int K, int L) {
  return (static_cast<int64_t>(M) * N) % 4 == 0 ? qmm_mfma_k_splits(M, N, K, L) : 1;
}

size_t fp_tile_workspace(int M, int N, int K, int L, int batches) {
  const int splits = fp_k_splits(M, N, K, L);
  const size_t planes = splits > 1 ? static_cast<size_t>(M) * N * splits * sizeof(float) : 0;
  return fp_image_bytes(N, K, batches) + planes;
}

// L problems (batch entries or index pairs), at most 65535 per launch.
int fp_launch(const QmmArgs& a, int mode, int dtype, bool transpose, hipStream_t s) {
  constexpr int kMaxRows = 65535; // the kernels below use up to one grid row per row of x
  if (a.M > kMaxRows && a.lhs_indices == nullptr && a.L <= 65535) {
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
        part.scales = static_cast<const uint8_t*>(a.scales) +
            static_cast<size_t>(l) * a.sb_batch_stride;
        part.out = static_cast<char*>(a.out) +
            (static_cast<size_t>(l) * a.M + m0) * static_cast<size_t>(a.N) * esize;
        const int rc = fp_launch(part, mode, dtype, transpose, s);
        if (rc != MLXROCM_OK) {
          return rc;
        }
      }
    }
    return MLXROCM_OK;
  }
  if (a.L > 65535 || a.M > kMaxRows) {
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
      } else if (a.K % (128 / B) == 0 && !std::is_same_v<T, float>) {
        if constexpr (!std::is_same_v<T, float>) {
          // Two rows of w per wavefront: with four or eight, measured at
          // [14336, 4096], 2..8 rows of x took the same time or longer (fewer
          // wavefronts); what sets the time with several rows of x is the rate of
          // v_dot2 (a quarter of the plain vector rate), not the bytes.
          constexpr int kRows = 2;
          const int mb = a.M == 1 ? 1 : (a.M == 2 ? 2 : 4);
          MLXROCM_REHEARSE("fp_qmv16(mb=%d)", mb);
          const int rows_per_wg = kFp16Waves * kRows;
          const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, (a.M + mb - 1) / mb, a.L);
          if (mb == 1) {
            fp_qmv16_kernel<T, G, B, 1, kRows, false><<<grid, 64 * kFp16Waves, 0, s>>>(a);
          } else if (mb == 2) {
            fp_qmv16_kernel<T, G, B, 2, kRows, true><<<grid, 64 * kFp16Waves, 0, s>>>(a);
          } else {
            fp_qmv16_kernel<T, G, B, 4, kRows, true><<<grid, 64 * kFp16Waves, 0, s>>>(a);
          }
        }
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

namespace {

int fp_qmm_entry(
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
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream,
    const float* out_scale = nullptr) {
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
  // [K, N] weights with a K that is not a multiple of 16 bytes: the kernel of that
  // case reads x element by element, and a stack of such matrices cannot have an
  // aligned stride
  const bool x_by_elements = transpose == 0 && K % x_vec != 0;
  // packed rows that are not whole 16-byte pieces are read by the byte
  const int64_t row_bits = static_cast<int64_t>(transpose ? K : N) * (mode == MLXROCM_MXFP8 ? 8 : 4);
  const bool w_by_bytes = row_bits % 128 != 0;
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out) ||
      (L > 1 && ((!x_by_elements && x_batch_stride % x_vec != 0) ||
                 (!w_by_bytes && w_batch_stride % 4 != 0)))) {
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
  a.out_scale = out_scale;
  if (fp_tile_applies(M, N, K, L, mode, dtype, transpose != 0)) {
    const int batches = scales_batch_stride != 0 ? L : 1;
    const size_t need = fp_tile_workspace(M, N, K, L, batches);
    if (workspace == nullptr || workspace_bytes < need ||
        (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
      return fail(
          MLXROCM_INVALID_ARGUMENT,
          "[quantized_matmul] this shape needs a 16-byte aligned workspace of %zu bytes "
          "(mlxrocm_fp_qmm_workspace_size); got %zu",
          need, workspace_bytes);
    }
    rc = fp_scale_image_for_qmm_t(
        scales, workspace, N, K, batches, scales_batch_stride, mode, dtype, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    a.scales = workspace;
    a.biases = workspace;
    a.sb_transposed = 2;
    // elements of T between the images of two batch entries
    a.sb_batch_stride = batches > 1 ? static_cast<int64_t>(N) * (K / 32) * 2 : 0;
    const int splits = fp_k_splits(M, N, K, L);
    if (splits <= 1) {
      return launch_qmm_mfma_fp(a, mode, dtype, 1, s);
    }
    void* partial = static_cast<char*>(workspace) + fp_image_bytes(N, K, batches);
    a.out = partial;
    rc = launch_qmm_mfma_fp(a, mode, dtype, splits, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    return reduce_k_splits(partial, out, static_cast<size_t>(M) * N, splits, dtype, s);
  }
  return fp_launch(a, mode, dtype, transpose != 0, s);
}

// From this many rows of x on, qqmm in the MX modes multiplies the codes of both
// operands on the block-scaled matrix instruction; below, x is quantized and
// dequantized in its own type and takes the kernels of quantized_matmul.
constexpr int kQqNativeMinM = 16;

// 4-bit codes: the instruction's sums are exact (products of two e2m1 numbers
// have few bits), results equal the fp32-accumulated ones bit for bit on the
// test shapes.  8-bit codes: inside a 128-code step the hardware aligns the
// products to the largest and keeps about 17 bits below it (measured: errors of
// 8e-6 of sum |x w|, against 1e-7 for fp32 accumulation) -- far below the
// rounding of a 16-bit result, but visible in a float32 one, so float32 problems
// stay on the fp32-accumulating kernels.
bool qq_native(int M, int N, int K, int mode, int dtype) {
  return M >= kQqNativeMinM && qq_mfma_supported(M, N, K, mode) &&
      (mode == MLXROCM_MXFP4 || dtype != MLXROCM_FLOAT32);
}

size_t round256(size_t n) {
  return (n + 255) / 256 * 256;
}

} // namespace

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
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_qmm");
  return fp_qmm_entry(
      x, wq, scales, out, M, N, K, L, x_batch_stride, w_batch_stride, scales_batch_stride, mode,
      dtype, transpose, workspace, workspace_bytes, stream);
}

extern "C" size_t mlxrocm_fp_qqmm_workspace_size(int M, int N, int K, int mode, int dtype) {
  if (fp_check("qqmm", M, N, K, 1, mode, dtype, 1) != MLXROCM_OK ||
      static_cast<int64_t>(M) * N == 0 || K == 0) {
    return 0;
  }
  if (qq_native(M, N, K, mode, dtype)) {
    const int bits = mode == MLXROCM_MXFP8 ? 8 : 4;
    return round256(static_cast<size_t>(M) * K * bits / 8) + round256(static_cast<size_t>(M) * K / 32);
  }
  return round256(static_cast<size_t>(M) * K * dtype_size(dtype)) +
      mlxrocm_fp_qmm_workspace_size(M, N, K, 1, 0, mode, dtype, 1);
}

extern "C" int mlxrocm_fp_qqmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    int M,
    int N,
    int K,
    int mode,
    int dtype,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_qqmm");
  int rc = fp_check("qqmm", M, N, K, 1, mode, dtype, 1);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(out, static_cast<size_t>(M) * N * dtype_size(dtype), s);
  }
  if (!x || !wq || !scales || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qqmm] null device pointer");
  }
  const size_t need = mlxrocm_fp_qqmm_workspace_size(M, N, K, mode, dtype);
  if (workspace == nullptr || workspace_bytes < need ||
      (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[qqmm] needs a 256-byte aligned workspace of %zu bytes (mlxrocm_fp_qqmm_workspace_size); "
        "got %zu",
        need, workspace_bytes);
  }
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out)) {
    return fail(MLXROCM_UNSUPPORTED, "[qqmm] operands must keep 16-byte alignment");
  }
  const size_t n_elems = static_cast<size_t>(M) * K;
  if (qq_native(M, N, K, mode, dtype)) {
    const int bits = mode == MLXROCM_MXFP8 ? 8 : 4;
    void* codes = workspace;
    uint8_t* xs = static_cast<uint8_t*>(workspace) + round256(n_elems * bits / 8);
    rc = fp_quantize_activations(x, codes, xs, n_elems, mode, dtype, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    return launch_qq_mfma(codes, xs, wq, scales, out, M, N, K, mode, dtype, s);
  }
  // x_hat in the element type, then the product with the quantized w
  rc = mlxrocm_fp_quantize_dequantize(x, workspace, n_elems, mode, dtype, stream);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  const size_t xhat_bytes = round256(n_elems * dtype_size(dtype));
  return fp_qmm_entry(
      workspace, wq, scales, out, M, N, K, 1, 0, 0, 0, mode, dtype, 1,
      static_cast<char*>(workspace) + xhat_bytes, workspace_bytes - xhat_bytes, stream);
}

namespace {

// Stand-ins for device pointers in a rehearsal: aligned, never dereferenced.
void* fake_pointer(int which) {
  return reinterpret_cast<void*>(uintptr_t{1} << 40 | static_cast<uintptr_t>(which) << 32);
}

} // namespace

extern "C" int mlxrocm_fp_qmm_plan(
    int M,
    int N,
    int K,
    int L,
    int batched_weights,
    int mode,
    int dtype,
    int transpose,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes) {
  RehearsalScope rehearsal(plan, plan_bytes);
  const int64_t w_stride = batched_weights ? int64_t{1} << 28 : 0;
  return fp_qmm_entry(
      fake_pointer(0), static_cast<const uint32_t*>(fake_pointer(1)),
      static_cast<const uint8_t*>(fake_pointer(2)), fake_pointer(3), M, N, K, L,
      static_cast<int64_t>(M) * K, w_stride, w_stride, mode, dtype, transpose,
      workspace_bytes != 0 ? fake_pointer(4) : nullptr, workspace_bytes, nullptr);
}

extern "C" int mlxrocm_fp_qqmm_plan(
    int M,
    int N,
    int K,
    int mode,
    int dtype,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes) {
  RehearsalScope rehearsal(plan, plan_bytes);
  return mlxrocm_fp_qqmm(
      fake_pointer(0), static_cast<const uint32_t*>(fake_pointer(1)),
      static_cast<const uint8_t*>(fake_pointer(2)), fake_pointer(3), M, N, K, mode, dtype,
      workspace_bytes != 0 ? fake_pointer(4) : nullptr, workspace_bytes, nullptr);
}

extern "C" size_t mlxrocm_fp_qmm_workspace_size(
    int M, int N, int K, int L, int batched_weights, int mode, int dtype, int transpose) {
  if (fp_check("quantized_matmul", M, N, K, L, mode, dtype, transpose) != MLXROCM_OK ||
      static_cast<int64_t>(M) * N * L == 0 || K == 0) {
    return 0;
  }
  if (!fp_tile_applies(M, N, K, L, mode, dtype, transpose != 0)) {
    return 0;
  }
  return fp_tile_workspace(M, N, K, L, batched_weights ? L : 1);
}

namespace {

// A gather with one row of x per index pair and many pairs per expert is sorted
// by expert (gather_group.hip) and multiplied by the tile kernel once per group
// of up to 256 pairs, so that every expert's weights are read once for all the
// rows routed to it, instead of one streaming product per pair.  The sort, the
// scale images of the experts and the kernel's ramp cost about four products of
// one pair per expert.  The kernel addresses x, an expert's codes and its scale
// image with 32-bit byte offsets.
bool fp_group_gather(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int x_batches,
    int64_t x_batch_stride,
    int mode,
    int dtype,
    bool transpose) {
  if (M != 1 || !transpose || dtype == MLXROCM_FLOAT32 || K % 64 != 0 || K < 64) {
    return false;
  }
  if (n_indices < 32 || static_cast<int64_t>(n_indices) < int64_t{4} * n_experts) {
    return false;
  }
  const uint64_t bits = mode == MLXROCM_MXFP8 ? 8 : 4;
  const uint64_t limit = uint64_t{1} << 32;
  if ((static_cast<uint64_t>(x_batches) * static_cast<uint64_t>(x_batch_stride) + K) * 2 >= limit ||
      static_cast<uint64_t>(N) * K * bits / 8 >= limit ||
      static_cast<uint64_t>(N) * (K / 32) * 4 >= limit) {
    return false;
  }
  if (gather_group_max_tiles(n_indices, n_experts, kGroupLargeTile) > 65535 || n_experts > 65535) {
    return false;
  }
  return gather_group_workspace_bytes(n_indices, n_experts) > 0;
}

// Grouping tables, then the scale images of the experts (one when they share
// their scales).
size_t fp_group_gather_bytes(int N, int K, int n_indices, int n_experts, int images) {
  return gather_group_workspace_bytes(n_indices, n_experts) + fp_image_bytes(N, K, images);
}

int fp_gather_entry(
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
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream,
    const float* out_scale) {
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
  const bool x_by_elements = transpose == 0 && K % x_vec != 0; // as in quantized_matmul
  const int64_t row_bits = static_cast<int64_t>(transpose ? K : N) * (mode == MLXROCM_MXFP8 ? 8 : 4);
  const bool w_by_bytes = row_bits % 128 != 0;
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out) ||
      (!x_by_elements && x_batch_stride % x_vec != 0) ||
      (!w_by_bytes && w_expert_stride % 4 != 0)) {
    return fail(MLXROCM_UNSUPPORTED, "[gather_qmm] operands must keep 16-byte alignment");
  }
  const int images = scales_expert_stride != 0 ? n_experts : 1;
  if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0 &&
      fp_group_gather(
          M, N, K, n_indices, n_experts, x_batches, x_batch_stride, mode, dtype, transpose != 0) &&
      workspace_bytes >= fp_group_gather_bytes(N, K, n_indices, n_experts, images)) {
    QmmArgs a{};
    a.x = x;
    a.w = wq;
    a.out = out;
    a.M = M;
    a.N = N;
    a.K = K;
    a.L = n_indices;
    a.x_batch_stride = x_batch_stride;
    a.w_batch_stride = w_expert_stride;
    a.lhs_indices = lhs_indices;
    a.rhs_indices = rhs_indices;
    a.x_batches = x_batches;
    a.n_experts = n_experts;
    a.out_scale = out_scale;
    // pairs with an index out of range are zero-filled by the grouping kernels
    rc = launch_gather_group(a, dtype, kGroupLargeTile, workspace, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    void* image = static_cast<char*>(workspace) + gather_group_workspace_bytes(n_indices, n_experts);
    rc = fp_scale_image_for_qmm_t(
        scales, image, N, K, images, scales_expert_stride, mode, dtype, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    a.scales = image;
    a.biases = image;
    a.sb_transposed = 2;
    // elements of T between the images of two experts
    a.sb_batch_stride = images > 1 ? static_cast<int64_t>(N) * (K / 32) * 2 : 0;
    return launch_qmm_mfma_fp_grouped(a, mode, dtype, s);
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
    a.out_scale = out_scale;
    rc = fp_launch(a, mode, dtype, transpose != 0, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
  }
  return MLXROCM_OK;
}

// The two tensor-wide scales of nvfp4: both or neither, and only in that mode.
int check_global_scales(const char* who, int mode, const float* gx, const float* gw) {
  if ((gx == nullptr) != (gw == nullptr)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] For nvfp4 mode, either both global_scale_x and global_scale_w must be provided, "
        "or neither.", who);
  }
  if (gx != nullptr && mode != MLXROCM_NVFP4) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] Global scale is only supported for 'nvfp4' mode.", who);
  }
  if ((reinterpret_cast<uintptr_t>(gx) & 3u) != 0 || (reinterpret_cast<uintptr_t>(gw) & 3u) != 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] a global scale must point at one float32", who);
  }
  return MLXROCM_OK;
}

} // namespace

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
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_gather_qmm");
  return fp_gather_entry(
      x, wq, scales, lhs_indices, rhs_indices, out, M, N, K, n_indices, x_batches, n_experts,
      x_batch_stride, w_expert_stride, scales_expert_stride, mode, dtype, transpose, workspace,
      workspace_bytes, stream, nullptr);
}

extern "C" size_t mlxrocm_fp_gather_qmm_workspace_size(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int batched_scales,
    int mode,
    int dtype,
    int transpose) {
  if (fp_check("gather_qmm", M, N, K, n_indices, mode, dtype, transpose) != MLXROCM_OK ||
      n_experts <= 0) {
    return 0;
  }
  // x is assumed to be within reach of 32-bit offsets; a call whose x is not
  // leaves the workspace unused
  if (!fp_group_gather(M, N, K, n_indices, n_experts, 1, 0, mode, dtype, transpose != 0)) {
    return 0;
  }
  return fp_group_gather_bytes(N, K, n_indices, n_experts, batched_scales ? n_experts : 1);
}

extern "C" size_t mlxrocm_fp_gather_qqmm_workspace_size(
    int M, int N, int K, int n_indices, int x_batches, int n_experts, int batched_scales, int mode,
    int dtype) {
  if (!valid_dtype(dtype) || M <= 0 || K <= 0 || x_batches <= 0) {
    return 0;
  }
  return round256(static_cast<size_t>(x_batches) * M * K * dtype_size(dtype)) +
      mlxrocm_fp_gather_qmm_workspace_size(
             M, N, K, n_indices, n_experts, batched_scales, mode, dtype, 1);
}

extern "C" int mlxrocm_fp_gather_qqmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    const float* global_scale_x,
    const float* global_scale_w,
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
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_fp_gather_qqmm");
  int rc = fp_check("gather_qqmm", M, N, K, n_indices, mode, dtype, 1);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  rc = check_global_scales("gather_qqmm", mode, global_scale_x, global_scale_w);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * n_indices == 0) {
    return MLXROCM_OK;
  }
  if (K == 0) {
    return launch_zero_fill(
        out, static_cast<size_t>(M) * N * n_indices * dtype_size(dtype),
        static_cast<hipStream_t>(stream));
  }
  if (!x) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qqmm] null device pointer");
  }
  const int64_t rows_elems = static_cast<int64_t>(M) * K;
  if (x_batches <= 0 || x_batch_stride < rows_elems) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qqmm] invalid batch description");
  }
  const size_t xhat_bytes = round256(static_cast<size_t>(x_batches) * M * K * dtype_size(dtype));
  const size_t need = mlxrocm_fp_gather_qqmm_workspace_size(
      M, N, K, n_indices, x_batches, n_experts, scales_expert_stride != 0, mode, dtype);
  if (workspace == nullptr || workspace_bytes < need ||
      (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[gather_qqmm] needs a 256-byte aligned workspace of %zu bytes "
        "(mlxrocm_fp_gather_qqmm_workspace_size); got %zu",
        need, workspace_bytes);
  }
  // x_hat: every matrix of x quantized and dequantized in its own type, packed
  const size_t esize = dtype_size(dtype);
  const bool packed = x_batch_stride == rows_elems;
  const int calls = packed ? 1 : x_batches;
  const size_t per_call = static_cast<size_t>(rows_elems) * (packed ? x_batches : 1);
  for (int b = 0; b < calls; ++b) {
    const char* src = static_cast<const char*>(x) + static_cast<size_t>(b) * x_batch_stride * esize;
    char* dst = static_cast<char*>(workspace) + static_cast<size_t>(b) * rows_elems * esize;
    rc = global_scale_x != nullptr
        ? mlxrocm_nvfp4_quantize_dequantize_global(src, global_scale_x, dst, per_call, dtype, stream)
        : mlxrocm_fp_quantize_dequantize(src, dst, per_call, mode, dtype, stream);
    if (rc != MLXROCM_OK) {
      return rc;
    }
  }
  return fp_gather_entry(
      workspace, wq, scales, lhs_indices, rhs_indices, out, M, N, K, n_indices, x_batches,
      n_experts, rows_elems, w_expert_stride, scales_expert_stride, mode, dtype, 1,
      static_cast<char*>(workspace) + xhat_bytes, workspace_bytes - xhat_bytes, stream,
      global_scale_w);
}

extern "C" int mlxrocm_nvfp4_qqmm_global(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    const float* global_scale_x,
    const float* global_scale_w,
    void* out,
    int M,
    int N,
    int K,
    int dtype,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_nvfp4_qqmm_global");
  const int mode = MLXROCM_NVFP4;
  int rc = fp_check("qqmm", M, N, K, 1, mode, dtype, 1);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (global_scale_x == nullptr || global_scale_w == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qqmm] both global scales must be given");
  }
  rc = check_global_scales("qqmm", mode, global_scale_x, global_scale_w);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(out, static_cast<size_t>(M) * N * dtype_size(dtype), s);
  }
  if (!x || !wq || !scales || !out) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qqmm] null device pointer");
  }
  const size_t need = mlxrocm_fp_qqmm_workspace_size(M, N, K, mode, dtype);
  if (workspace == nullptr || workspace_bytes < need ||
      (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[qqmm] needs a 256-byte aligned workspace of %zu bytes (mlxrocm_fp_qqmm_workspace_size); "
        "got %zu",
        need, workspace_bytes);
  }
  if (!aligned16(x) || !aligned16(wq) || !aligned16(out)) {
    return fail(MLXROCM_UNSUPPORTED, "[qqmm] operands must keep 16-byte alignment");
  }
  const size_t n_elems = static_cast<size_t>(M) * K;
  rc = mlxrocm_nvfp4_quantize_dequantize_global(x, global_scale_x, workspace, n_elems, dtype, stream);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  const size_t xhat_bytes = round256(n_elems * dtype_size(dtype));
  return fp_qmm_entry(
      workspace, wq, scales, out, M, N, K, 1, 0, 0, 0, mode, dtype, 1,
      static_cast<char*>(workspace) + xhat_bytes, workspace_bytes - xhat_bytes, stream,
      global_scale_w);
}
