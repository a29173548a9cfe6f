// qmv_n.hip -- transpose=false with 1..4 rows of x (the reference's "qvm"):
//
//   y[M, N] = x[M, K] * dequant(W)[K, N],  W packed along n, groups along n.
//
// Every weight is used once per row of x, so this is a streaming kernel over the
// packed rows of W.  A lane owns 8 bytes of a packed row (16 codes at 4 bits, 8 at
// 8 bits: one dwordx2 load, inside one quantization group for every group size)
// and keeps one fp32 accumulator per code and row of x; a wavefront therefore
// covers 512 contiguous bytes of a row per load instruction and 1024 / 512
// columns of y.  K is cut twice: a workgroup owns a range of 64 rows, its four
// wavefronts take rows k, k+4, ... of it (sixteen rows each, every load issued
// before the first is used, and before x is staged) and are added through LDS;
// workgroups along blockIdx.y take the ranges and write fp32 planes that
// reduce_planes adds up (one range: written to y directly).  The planes cost
// K N / 16 bytes of extra traffic each way, against K N bits / 8 of weights.
// Per row and lane the affine part is applied to x, not to the codes:
//   acc[j] += q[j] * (x[k] * s) ;  bsum += x[k] * b ;  y[j] = acc[j] + bsum.
// x reaches the lanes through an fp32 image of the workgroup's K range in LDS
// (wave-uniform addresses: broadcast reads).
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kNThreads = 256;
constexpr int kNWaves = 4;
constexpr int kNUnroll = 16;                   // rows of W in flight per wavefront
constexpr int kNRange = kNWaves * kNUnroll;    // rows of K per workgroup

template <int BITS>
__device__ __forceinline__ void codes_to_float(const uint2 w, float (&q)[64 / BITS]) {
  if constexpr (BITS == 8) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t v = h == 0 ? w.x : w.y;
      q[4 * h + 0] = static_cast<float>(v & 0xffu);
      q[4 * h + 1] = static_cast<float>((v >> 8) & 0xffu);
      q[4 * h + 2] = static_cast<float>((v >> 16) & 0xffu);
      q[4 * h + 3] = static_cast<float>(v >> 24);
    }
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t v = h == 0 ? w.x : w.y;
      // even and odd nibbles as bytes, then byte -> float conversions
      const uint32_t lo = v & 0x0f0f0f0fu;
      const uint32_t hi = (v >> 4) & 0x0f0f0f0fu;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        q[8 * h + 2 * b + 0] = static_cast<float>((lo >> (8 * b)) & 0xffu);
        q[8 * h + 2 * b + 1] = static_cast<float>((hi >> (8 * b)) & 0xffu);
      }
    }
  }
}

__device__ __forceinline__ uint2 load_once8(const uint8_t* p) {
  typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
  const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
  return make_uint2(v.x, v.y);
}

// MR: rows of x held in registers (M <= MR).  `partial`: fp32 planes of
// [L, M, N] per K range when gridDim.y > 1, else null (y is written directly).
template <typename T, int BITS, int MR>
__global__ __launch_bounds__(kNThreads) void qmv_n_kernel(
    const QmmArgs a,
    const int gs_shift,
    float* __restrict__ partial) {
  constexpr int kCodes = 64 / BITS;
  constexpr int kWaveCols = 64 * kCodes;
  __shared__ float xs[MR][kNRange];
  __shared__ float red[kNWaves - 1][MR][kWaveCols];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int N = a.N;
  const int K = a.K;
  const int M = a.M;
  const int l = blockIdx.z;
  const QmmProblem<T> p = resolve_problem<T>(a, l);

  const int k_begin = blockIdx.y * kNRange;
  const int k_end = k_begin + kNRange < K ? k_begin + kNRange : K;
  const int rows = k_end - k_begin;

  const int n0 = blockIdx.x * kWaveCols + lane * kCodes;
  const bool live = n0 < N; // N is a multiple of 32 and kCodes divides 32
  const int nc = live ? n0 : 0;
  const int groups = N >> gs_shift;
  const int g = nc >> gs_shift;
  const size_t row_bytes = static_cast<size_t>(N) / 8 * BITS;
  const uint8_t* wcol = p.w + static_cast<size_t>(nc) / 8 * BITS;

  // rows k_begin + wave + 4 u of the range: every load first
  uint2 wv[kNUnroll];
  T sv[kNUnroll], bv[kNUnroll];
#pragma unroll
  for (int u = 0; u < kNUnroll; ++u) {
    const int r = wave + u * kNWaves;
    const int k = k_begin + (r < rows ? r : rows - 1); // clamp: stay in bounds
    wv[u] = load_once8(wcol + static_cast<size_t>(k) * row_bytes);
    sv[u] = p.scales[static_cast<size_t>(k) * groups + g];
    bv[u] = p.biases[static_cast<size_t>(k) * groups + g];
  }

  // x image of the range, fp32, zero for rows of x beyond M and rows past K
  for (int i = tid; i < MR * kNRange; i += kNThreads) {
    const int m = i / kNRange;
    const int r = i % kNRange;
    float v = 0.0f;
    if (m < M && r < rows) {
      v = to_f32(p.x[static_cast<size_t>(m) * K + k_begin + r]);
    }
    xs[m][r] = v;
  }
  __syncthreads();

  float acc[MR][kCodes];
  float bsum[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    bsum[m] = 0.0f;
#pragma unroll
    for (int j = 0; j < kCodes; ++j) {
      acc[m][j] = 0.0f;
    }
  }
#pragma unroll
  for (int u = 0; u < kNUnroll; ++u) {
    const int r = wave + u * kNWaves; // x is zero for rows past the range's end
    float q[kCodes];
    codes_to_float<BITS>(wv[u], q);
    const float s = to_f32(sv[u]);
    const float b = to_f32(bv[u]);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float x = xs[m][r];
      const float xsc = x * s;
      bsum[m] = fmaf(x, b, bsum[m]);
#pragma unroll
      for (int j = 0; j < kCodes; ++j) {
        acc[m][j] = fmaf(q[j], xsc, acc[m][j]);
      }
    }
  }

  // waves 1..3 -> LDS, wave 0 adds and writes
  if (wave > 0) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
#pragma unroll
      for (int j = 0; j < kCodes; ++j) {
        // column-major over the lanes: conflict-free
        red[wave - 1][m][j * 64 + lane] = acc[m][j] + bsum[m];
      }
    }
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      if (m < M) {
        float y[kCodes];
#pragma unroll
        for (int j = 0; j < kCodes; ++j) {
          y[j] = acc[m][j] + bsum[m];
#pragma unroll
          for (int w = 0; w < kNWaves - 1; ++w) {
            y[j] += red[w][m][j * 64 + lane];
          }
        }
        if (partial != nullptr) {
          float* dst = partial +
              ((static_cast<size_t>(blockIdx.y) * a.L + l) * M + m) * static_cast<size_t>(N) + n0;
#pragma unroll
          for (int j = 0; j < kCodes; j += 4) {
            *reinterpret_cast<float4*>(dst + j) = make_float4(y[j], y[j + 1], y[j + 2], y[j + 3]);
          }
        } else {
          T* dst = p.out + static_cast<size_t>(m) * N + n0;
#pragma unroll
          for (int j = 0; j < kCodes; ++j) {
            dst[j] = from_f32<T>(y[j]);
          }
        }
      }
    }
  }
}

// y = sum of `splits` fp32 planes of n elements (n % 4 == 0).  Sixteen threads
// of a workgroup share a group of four outputs and walk the planes sixteen
// apart, four loads in flight each, so that hundreds of planes of a small y
// still fill the memory pipeline; LDS adds the sixteen partial sums.
template <typename TO>
__global__ __launch_bounds__(256) void reduce_planes_kernel(
    const float* __restrict__ partial,
    TO* __restrict__ out,
    const size_t n,
    const int splits) {
  __shared__ float4 red[16][16];
  const int c = threadIdx.x & 15;
  const int pg = threadIdx.x >> 4;
  const size_t i = (static_cast<size_t>(blockIdx.x) * 16 + c) * 4;
  const bool live = i < n;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (live) {
    for (int z = pg; z < splits; z += 64) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int zz = z + 16 * u;
        v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (zz < splits) {
          v[u] = *reinterpret_cast<const float4*>(partial + static_cast<size_t>(zz) * n + i);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc.x += v[u].x;
        acc.y += v[u].y;
        acc.z += v[u].z;
        acc.w += v[u].w;
      }
    }
  }
  red[pg][c] = acc;
  __syncthreads();
  if (pg == 0 && live) {
#pragma unroll
    for (int g = 1; g < 16; ++g) {
      const float4 v = red[g][c];
      acc.x += v.x;
      acc.y += v.y;
      acc.z += v.z;
      acc.w += v.w;
    }
    out[i + 0] = from_f32<TO>(acc.x);
    out[i + 1] = from_f32<TO>(acc.y);
    out[i + 2] = from_f32<TO>(acc.z);
    out[i + 3] = from_f32<TO>(acc.w);
  }
}

} // namespace

int reduce_planes(const float* partial, void* out, size_t n, int splits, int dtype, hipStream_t s) {
  const size_t blocks = (n / 4 + 15) / 16;
  if (n % 4 != 0 || blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] output of %zu elements does not fit the plane reduction", n);
  }
  MLXROCM_REHEARSE("reduce_planes(%d)", splits);
  const unsigned g = static_cast<unsigned>(blocks);
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    reduce_planes_kernel<T><<<g, 256, 0, s>>>(partial, static_cast<T*>(out), n, splits);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
}

bool qmv_n_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  (void)gs;
  (void)dtype;
  if (a.M < 1 || a.M > 4 || !(bits == 4 || bits == 8) || a.lhs_indices != nullptr ||
      a.L > 65535) {
    return false;
  }
  // the K ranges are a grid dimension, and their fp32 planes (K N M / 16 bytes)
  // stay below 256 MiB of scratch
  const long splits = (static_cast<long>(a.K) + kNRange - 1) / kNRange;
  const long plane = static_cast<long>(a.L) * a.M * a.N;
  return splits <= 65535 && splits * plane <= (64L << 20);
}

QmvNPlan qmv_n_plan(const QmmArgs& a, int bits) {
  (void)bits;
  QmvNPlan pl;
  pl.range = kNRange;
  pl.splits = (a.K + kNRange - 1) / kNRange;
  return pl;
}

int launch_qmv_n(const QmmArgs& a, int gs, int bits, int dtype, float* partial, hipStream_t s) {
  const QmvNPlan pl = qmv_n_plan(a, bits);
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const int wave_cols = 64 * (64 / bits);
  const dim3 grid((a.N + wave_cols - 1) / wave_cols, pl.splits, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] K=%d needs too many ranges", a.K);
  }
  if (pl.splits > 1 && partial == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qmv] the K ranges need a partial buffer");
  }
  MLXROCM_REHEARSE("qmv_n(rows=%d,ranges=%d)", a.M, pl.splits);
  float* part = pl.splits > 1 ? partial : nullptr;
  auto go = [&](auto tval, auto bval, auto mval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int MR = decltype(mval)::value;
    qmv_n_kernel<T, B, MR><<<grid, kNThreads, 0, s>>>(a, gs_shift, part);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  };
  auto by_m = [&](auto tval, auto bval) -> int {
    if (a.M == 1) {
      return go(tval, bval, IntC<1>{});
    }
    if (a.M == 2) {
      return go(tval, bval, IntC<2>{});
    }
    return go(tval, bval, IntC<4>{});
  };
  return dispatch_dtype(dtype, [&](auto tval) {
    return bits == 4 ? by_m(tval, IntC<4>{}) : by_m(tval, IntC<8>{});
  });
}

} // namespace mlxrocm
