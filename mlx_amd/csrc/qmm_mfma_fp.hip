// qmm_mfma_fp.hip -- the prefill tile kernel for the floating-point modes
// (mxfp4 / mxfp8 / nvfp4, 16-bit element types, transpose=true).  The kernel is
// the affine one with another code-to-element step (FpPairDequant); its scales
// come from a pair image built here first: [K / 32][N] dwords, the scale of
// codes 0..15 of the 32 in the low half and of codes 16..31 in the high half,
// both already decoded to the element type (the same value twice for the modes
// with one scale per 32).
#include "qmm_mfma_tile.h"

namespace mlxrocm {

namespace {

// one byte -> the scale as an element of T (mlx/backend/cpu/quantized.cpp:49-62)
template <typename T, bool E4M3>
__device__ __forceinline__ uint32_t scale_bits(uint32_t s) {
  float v;
  if constexpr (E4M3) {
    const uint32_t e = (s >> 3) & 0xFu;
    const uint32_t m = s & 7u;
    v = e == 0 ? static_cast<float>(m) * 0.001953125f
               : __uint_as_float(((e + 120u) << 23) | (m << 20));
    v = (s & 0x80u) ? -v : v;
  } else {
    v = __uint_as_float((s == 0 ? 0x40u : (s << 7)) << 16);
  }
  return __builtin_bit_cast(uint16_t, from_f32<T>(v));
}

// scales [N][G * PER] bytes (PER scales per 32 codes: 1 or 2) -> out [G][N]
// dwords.  32 x 32 tiles through LDS: read along a row's groups, written along n.
template <typename T, int PER>
__global__ __launch_bounds__(256) void fp_scale_image_kernel(
    const uint8_t* scales, uint32_t* out, int N, int G, int64_t src_stride) {
  __shared__ uint32_t tile[32][33];
  const int l = blockIdx.z;
  const uint8_t* sc = scales + l * src_stride;
  uint32_t* dst = out + static_cast<size_t>(l) * N * G;
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5; // 0..7
  const int g0 = blockIdx.x * 32;
  const int n0 = blockIdx.y * 32;
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int n = n0 + r;
    const int g = g0 + tx;
    if (n < N && g < G) {
      const uint8_t* at = sc + (static_cast<size_t>(n) * G + g) * PER;
      uint32_t lo, hi;
      if constexpr (PER == 2) {
        lo = scale_bits<T, true>(at[0]);
        hi = scale_bits<T, true>(at[1]);
      } else {
        lo = hi = scale_bits<T, false>(at[0]);
      }
      tile[r][tx] = lo | (hi << 16);
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int g = g0 + r;
    const int n = n0 + tx;
    if (n < N && g < G) {
      dst[static_cast<size_t>(g) * N + n] = tile[tx][r];
    }
  }
}

// The same image four scale bytes per load: a workgroup takes 32 rows x 128
// bytes of scales (128 groups, or 64 with two scales per 32 codes) through LDS.
// Rows of scales must be whole dwords (G * PER % 4 == 0) and 4-byte aligned.
template <typename T, int PER>
__global__ __launch_bounds__(256) void fp_scale_image_wide_kernel(
    const uint8_t* scales, uint32_t* out, int N, int G, int64_t src_stride) {
  constexpr int kGroups = 128 / PER; // groups per workgroup
  __shared__ uint32_t tile[32][kGroups + 1];
  const int l = blockIdx.z;
  const uint8_t* sc = scales + l * src_stride;
  uint32_t* dst = out + static_cast<size_t>(l) * N * G;
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5; // 0..7
  const int g0 = blockIdx.x * kGroups;
  const int n0 = blockIdx.y * 32;
  const int row_bytes = G * PER;
  const int c = g0 * PER + 4 * tx; // first of this thread's four bytes in a row
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int n = n0 + r;
    if (n < N && c < row_bytes) { // whole dwords: c + 3 < row_bytes as well
      const uint32_t v =
          *reinterpret_cast<const uint32_t*>(sc + static_cast<size_t>(n) * row_bytes + c);
      if constexpr (PER == 2) {
        tile[r][2 * tx] = scale_bits<T, true>(v & 0xffu) | (scale_bits<T, true>((v >> 8) & 0xffu) << 16);
        tile[r][2 * tx + 1] =
            scale_bits<T, true>((v >> 16) & 0xffu) | (scale_bits<T, true>(v >> 24) << 16);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t b = scale_bits<T, false>((v >> (8 * j)) & 0xffu);
          tile[r][4 * tx + j] = b | (b << 16);
        }
      }
    }
  }
  __syncthreads();
  for (int r = ty; r < kGroups; r += 8) {
    const int g = g0 + r;
    const int n = n0 + tx;
    if (n < N && g < G) {
      dst[static_cast<size_t>(g) * N + n] = tile[tx][r];
    }
  }
}

} // namespace

// `mode`: mlxrocm_fp_mode.  out: batches * (K / 32) * N dwords.
int fp_scale_image_for_qmm_t(
    const uint8_t* scales,
    void* out,
    int N,
    int K,
    int batches,
    int64_t src_stride,
    int mode,
    int dtype,
    hipStream_t s) {
  const int G = K / 32;
  const dim3 grid((G + 31) / 32, (N + 31) / 32, batches);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] N=%d or batch=%d exceed the grid", N, batches);
  }
  MLXROCM_REHEARSE("fp_scale_image");
  uint32_t* dst = static_cast<uint32_t*>(out);
  const int per = mode == MLXROCM_NVFP4 ? 2 : 1;
  if ((G * per) % 4 == 0 && (reinterpret_cast<uintptr_t>(scales) & 3u) == 0 && src_stride % 4 == 0) {
    // whole dwords of scale bytes per row: four bytes per load
    const int groups_per_block = 128 / per;
    const dim3 wide((G + groups_per_block - 1) / groups_per_block, (N + 31) / 32, batches);
    if (dtype == MLXROCM_BFLOAT16) {
      if (per == 2) {
        fp_scale_image_wide_kernel<bf16_t, 2><<<wide, 256, 0, s>>>(scales, dst, N, G, src_stride);
      } else {
        fp_scale_image_wide_kernel<bf16_t, 1><<<wide, 256, 0, s>>>(scales, dst, N, G, src_stride);
      }
    } else {
      if (per == 2) {
        fp_scale_image_wide_kernel<f16_t, 2><<<wide, 256, 0, s>>>(scales, dst, N, G, src_stride);
      } else {
        fp_scale_image_wide_kernel<f16_t, 1><<<wide, 256, 0, s>>>(scales, dst, N, G, src_stride);
      }
    }
    MLXROCM_HIP_TRY(hipGetLastError());
    return MLXROCM_OK;
  }
  if (dtype == MLXROCM_BFLOAT16) {
    if (mode == MLXROCM_NVFP4) {
      fp_scale_image_kernel<bf16_t, 2><<<grid, 256, 0, s>>>(scales, dst, N, G, src_stride);
    } else {
      fp_scale_image_kernel<bf16_t, 1><<<grid, 256, 0, s>>>(scales, dst, N, G, src_stride);
    }
  } else {
    if (mode == MLXROCM_NVFP4) {
      fp_scale_image_kernel<f16_t, 2><<<grid, 256, 0, s>>>(scales, dst, N, G, src_stride);
    } else {
      fp_scale_image_kernel<f16_t, 1><<<grid, 256, 0, s>>>(scales, dst, N, G, src_stride);
    }
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// a.scales: the image above (a.sb_transposed == 2); K % 64 == 0.  k_splits > 1:
// K is cut into that many ranges and a.out points at as many fp32 planes of
// M x N, which reduce_k_splits adds up.
int launch_qmm_mfma_fp(const QmmArgs& a, int mode, int dtype, int k_splits, hipStream_t s) {
  if (k_splits > 1) {
    constexpr int kNT = 7;
    MLXROCM_REHEARSE("fp_qmm_t_tile(ksplit=%d)", k_splits);
    const dim3 grid((a.N + 32 * kNT - 1) / (32 * kNT), (a.M + kBM - 1) / kBM, k_splits);
    auto split = [&](auto tval) -> int {
      using T = decltype(tval);
      switch (mode) {
        case MLXROCM_MXFP4:
          return launch_variant<T, T, float, 4, kNT, false, false, true, 1>(a, 5, grid, s, k_splits);
        case MLXROCM_MXFP8:
          return launch_variant<T, T, float, 8, kNT, false, false, true, 2>(a, 5, grid, s, k_splits);
        default:
          return launch_variant<T, T, float, 4, kNT, false, false, true, 3>(a, 5, grid, s, k_splits);
      }
    };
    return dtype == MLXROCM_BFLOAT16 ? split(bf16_t{}) : split(f16_t{});
  }
  const int nt = choose_nt(a.M, a.N, a.L);
  MLXROCM_REHEARSE("fp_qmm_t_tile(nt=%d)", nt);
  const dim3 grid((a.N + 32 * nt - 1) / (32 * nt), (a.M + kBM - 1) / kBM, a.L);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    auto with_nt = [&](auto ntval) -> int {
      constexpr int NT = decltype(ntval)::value;
      switch (mode) {
        case MLXROCM_MXFP4:
          return launch_variant<T, T, T, 4, NT, false, false, true, 1>(a, 5, grid, s);
        case MLXROCM_MXFP8:
          return launch_variant<T, T, T, 8, NT, false, false, true, 2>(a, 5, grid, s);
        default:
          return launch_variant<T, T, T, 4, NT, false, false, true, 3>(a, 5, grid, s);
      }
    };
    switch (nt) {
      case 5:
        return with_nt(IntC<5>{});
      case 6:
        return with_nt(IntC<6>{});
      default:
        return with_nt(IntC<7>{});
    }
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

// Gather grouped by expert (M == 1 per index pair): `a` carries the tile list of
// launch_gather_group and the scale images of all experts (a.sb_batch_stride
// elements apart, 0 when the experts share one); one grid row per possible tile,
// rows past the device-side tile count exit at once.
int launch_qmm_mfma_fp_grouped(const QmmArgs& a, int mode, int dtype, hipStream_t s) {
  MLXROCM_REHEARSE("fp_qmm_t_tile_grouped");
  constexpr int kNT = 7;
  const dim3 grid(
      (a.N + 32 * kNT - 1) / (32 * kNT), gather_group_max_tiles(a.L, a.n_experts, kGroupLargeTile), 1);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    switch (mode) {
      case MLXROCM_MXFP4:
        return launch_variant<T, T, T, 4, kNT, true, false, true, 1>(a, 5, grid, s);
      case MLXROCM_MXFP8:
        return launch_variant<T, T, T, 8, kNT, true, false, true, 2>(a, 5, grid, s);
      default:
        return launch_variant<T, T, T, 4, kNT, true, false, true, 3>(a, 5, grid, s);
    }
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
