// qmv_f32.hip -- decode GEMV (transpose=true) in plain fp32 arithmetic, every
// code width and element type, one to four rows of x: the streaming kernel for
// float32 operands and for the 16-bit types at widths 2/3/5/6.
//
// A lane owns 32 consecutive codes of a row (= `bits` whole dwords for every
// width, and never more than one quantization group), so a wavefront covers a
// "chunk" of 2048 codes with `bits` dword loads per lane whose addresses are
// contiguous across the lanes.  The K axis is split over KW wavefronts of the
// workgroup, CPW chunks each; every wavefront keeps its slices of x in
// registers (fetched once, straight from global memory: x is small and shared by
// every workgroup, so it stays in the caches) and walks over kRowsInFlight rows
// of W at a time with all their loads issued before the first is consumed.  Per
// lane and chunk the affine part is applied once: y += s * dot(q, x) + b * sum(x).
// Lanes are added with DPP / permutes, k-waves through LDS.
#include "mfma_dequant.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kF32ChunkCodes = 64 * 32;
constexpr int kF32RowsInFlight = 4;
constexpr int kF32Threads = 256;

// 32 consecutive elements of x as floats.
__device__ __forceinline__ void load_x32(const float* src, float (&out)[32]) {
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const float4 v = *reinterpret_cast<const float4*>(src + 4 * u);
    out[4 * u + 0] = v.x;
    out[4 * u + 1] = v.y;
    out[4 * u + 2] = v.z;
    out[4 * u + 3] = v.w;
  }
}
template <typename T>
__device__ __forceinline__ void load_x32(const T* src, float (&out)[32]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    union {
      uint4 v;
      T h[8];
    } r;
    r.v = *reinterpret_cast<const uint4*>(src + 8 * u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      out[8 * u + e] = to_f32(r.h[e]);
    }
  }
}

template <typename T, int BITS, int MROWS, int CPW, int KW>
__global__ __launch_bounds__(kF32Threads) void qmv_f32_kernel(const QmmArgs a, const int gs_shift) {
  constexpr int RW = kF32Threads / 64 / KW; // row-waves per workgroup
  __shared__ float red[kF32Threads / 64][kF32RowsInFlight][MROWS];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kw = wave % KW;
  const int rw = wave / KW;
  const int K = a.K;
  const int N = a.N;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);
  const int groups = K >> gs_shift;
  const int row_words = K / 32 * BITS;

  // this lane's codes of chunk c: k in [k_of(c), k_of(c) + 32)
  int kpos[CPW];
  bool live[CPW];
#pragma unroll
  for (int c = 0; c < CPW; ++c) {
    const int k = (kw * CPW + c) * kF32ChunkCodes + lane * 32;
    live[c] = k < K; // K is a multiple of 32
    kpos[c] = live[c] ? k : 0;
  }
  // x slices and their sums
  float xr[MROWS][CPW][32];
  float sx[MROWS][CPW];
#pragma unroll
  for (int m = 0; m < MROWS; ++m) {
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      load_x32(p.x + static_cast<size_t>(m < a.M ? m : 0) * K + kpos[c], xr[m][c]);
      float s = 0.0f;
#pragma unroll
      for (int e = 0; e < 32; ++e) {
        if (!live[c] || m >= a.M) {
          xr[m][c][e] = 0.0f;
        }
        s += xr[m][c][e];
      }
      sx[m][c] = s;
    }
  }

  const int rows_per_wg = RW * kF32RowsInFlight;
  const int row0 = blockIdx.x * rows_per_wg + rw * kF32RowsInFlight;
  uint32_t wv[kF32RowsInFlight][CPW][BITS];
  T sv[kF32RowsInFlight][CPW], bv[kF32RowsInFlight][CPW];
#pragma unroll
  for (int r = 0; r < kF32RowsInFlight; ++r) {
    const int row = row0 + r < N ? row0 + r : N - 1; // clamp: stay in bounds
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const int g = kpos[c] >> gs_shift;
      sv[r][c] = p.scales[static_cast<size_t>(row) * groups + g];
      bv[r][c] = p.biases[static_cast<size_t>(row) * groups + g];
    }
  }
#pragma unroll
  for (int r = 0; r < kF32RowsInFlight; ++r) {
    const int row = row0 + r < N ? row0 + r : N - 1;
    const uint32_t* wrow = reinterpret_cast<const uint32_t*>(p.w) +
        static_cast<size_t>(row) * row_words;
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const uint32_t* src = wrow + kpos[c] / 32 * BITS;
#pragma unroll
      for (int j = 0; j < BITS; ++j) {
        wv[r][c][j] = __builtin_nontemporal_load(src + j);
      }
    }
  }

  float y[kF32RowsInFlight][MROWS];
#pragma unroll
  for (int r = 0; r < kF32RowsInFlight; ++r) {
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      y[r][m] = 0.0f;
    }
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      float dot[MROWS];
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        dot[m] = 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 32; ++e) {
        const float q = static_cast<float>(code32<BITS>(wv[r][c], e));
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          dot[m] = fmaf(q, xr[m][c][e], dot[m]);
        }
      }
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        y[r][m] = fmaf(to_f32(sv[r][c]), dot[m], y[r][m]);
        y[r][m] = fmaf(to_f32(bv[r][c]), sx[m][c], y[r][m]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < kF32RowsInFlight; ++r) {
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const float total = wave_sum(y[r][m]);
      if (lane == 0) {
        red[wave][r][m] = total;
      }
    }
  }
  __syncthreads();
  if (tid < RW * kF32RowsInFlight * MROWS) {
    const int m = tid % MROWS;
    const int r = (tid / MROWS) % kF32RowsInFlight;
    const int w = tid / (MROWS * kF32RowsInFlight);
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < KW; ++k) {
      total += red[w * KW + k][r][m];
    }
    const int row = blockIdx.x * rows_per_wg + w * kF32RowsInFlight + r;
    if (row < N && m < a.M) {
      p.out[static_cast<size_t>(m) * N + row] = from_f32<T>(p.valid ? total : 0.0f);
    }
  }
}

struct F32Plan {
  int kw; // 0: not covered
  int cpw;
};

F32Plan f32_plan(int K) {
  const int need = (K + kF32ChunkCodes - 1) / kF32ChunkCodes;
  F32Plan pl{0, 0};
  if (need <= 1) {
    pl = {1, 1};
  } else if (need <= 2) {
    pl = {1, 2};
  } else if (need <= 4) {
    pl = {2, 2};
  } else if (need <= 8) {
    pl = {4, 2};
  }
  return pl;
}

} // namespace

// Rows of x in one launch: one for every K up to 16384; two to four while a
// lane keeps a single 32-code slice of each row of x (K <= 8192).
bool qmv_f32_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  (void)gs;
  (void)bits;
  (void)dtype;
  if (a.M < 1 || a.M > 4) {
    return false;
  }
  const F32Plan pl = f32_plan(a.K);
  if (pl.kw == 0) {
    return false; // K > 16384
  }
  return a.M == 1 || (a.K + kF32ChunkCodes - 1) / kF32ChunkCodes <= 4;
}

int launch_qmv_f32(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  F32Plan pl = f32_plan(a.K);
  if (pl.kw == 0 || a.M < 1 || a.M > 4) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] M=%d K=%d is not covered by the fp32 GEMV", a.M, a.K);
  }
  if (a.M > 1) {
    // one chunk per wave: the registers go to the rows of x
    const int need = (a.K + kF32ChunkCodes - 1) / kF32ChunkCodes;
    if (need > 4) {
      return fail(MLXROCM_UNSUPPORTED, "[qmv] K=%d is not covered by the fp32 GEMV at M=%d", a.K, a.M);
    }
    pl.cpw = 1;
    pl.kw = need <= 1 ? 1 : (need <= 2 ? 2 : 4);
  }
  MLXROCM_REHEARSE("qmv_f32");
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const int rows_per_wg = (kF32Threads / 64 / pl.kw) * kF32RowsInFlight;
  const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] batch=%d exceeds the grid", a.L);
  }
  auto go = [&](auto tval, auto bval, auto mval, auto cval, auto kval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int M = decltype(mval)::value;
    constexpr int C = decltype(cval)::value;
    constexpr int KWv = decltype(kval)::value;
    qmv_f32_kernel<T, B, M, C, KWv><<<grid, kF32Threads, 0, s>>>(a, gs_shift);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  };
  auto by_plan = [&](auto tval, auto bval, auto mval) -> int {
    if (pl.cpw == 1) {
      if (pl.kw == 1) {
        return go(tval, bval, mval, IntC<1>{}, IntC<1>{});
      }
      if (pl.kw == 2) {
        return go(tval, bval, mval, IntC<1>{}, IntC<2>{});
      }
      return go(tval, bval, mval, IntC<1>{}, IntC<4>{});
    }
    if constexpr (decltype(mval)::value == 1) {
      if (pl.kw == 1) {
        return go(tval, bval, mval, IntC<2>{}, IntC<1>{});
      }
      if (pl.kw == 2) {
        return go(tval, bval, mval, IntC<2>{}, IntC<2>{});
      }
      return go(tval, bval, mval, IntC<2>{}, IntC<4>{});
    }
    return fail(MLXROCM_UNSUPPORTED, "[qmv] no fp32 GEMV plan for M=%d K=%d", a.M, a.K);
  };
  return dispatch_dtype(dtype, [&](auto tval) {
    return dispatch_bits(bits, [&](auto bval) {
      if (a.M == 1) {
        return by_plan(tval, bval, IntC<1>{});
      }
      if (a.M == 2) {
        return by_plan(tval, bval, IntC<2>{});
      }
      return by_plan(tval, bval, IntC<4>{});
    });
  });
}

} // namespace mlxrocm
