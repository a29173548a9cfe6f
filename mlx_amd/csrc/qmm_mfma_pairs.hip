// qmm_mfma_pairs.hip -- the prefill tile kernel reading scales and biases from
// the pair image: [K / group][N] dwords, scale in the low half and bias in the
// high half (16-bit types).  The lanes of a wavefront own consecutive rows of W,
// so one coalesced dword load per thread and K-step fetches both values; with
// two images it took two 16-bit loads, and with the caller's [N][K / group]
// layout every lane of such a load touched a cache line of its own (15 % of the
// kernel's time).  A load instruction costs the issuing wavefront about as much
// as four matrix instructions here whatever its size, so the count matters.
#include "qmm_mfma_tile.h"

namespace mlxrocm {

namespace {

// 32 x 32 tiles through LDS: read along the groups of a row (contiguous in the
// caller's [N][G] arrays), written along n.
template <typename T>
__global__ __launch_bounds__(256) void interleave_sb_kernel(
    const T* scales,
    const T* biases,
    uint32_t* out,
    int N,
    int G,
    int64_t src_stride) {
  __shared__ uint32_t tile[32][33];
  const int l = blockIdx.z;
  const T* sc = scales + l * src_stride;
  const T* bi = biases + l * src_stride;
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
      const size_t at = static_cast<size_t>(n) * G + g;
      const uint32_t lo = __builtin_bit_cast(uint16_t, sc[at]);
      const uint32_t hi = __builtin_bit_cast(uint16_t, bi[at]);
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

} // namespace

int interleave_sb_for_qmm_t(
    const void* scales,
    const void* biases,
    void* out,
    int N,
    int G,
    int batches,
    int64_t src_stride,
    hipStream_t s) {
  const dim3 grid((G + 31) / 32, (N + 31) / 32, batches);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] N=%d or batch=%d exceed the grid", N, batches);
  }
  MLXROCM_REHEARSE("interleave_sb");
  // the kernel only moves 16-bit patterns: one instantiation serves both types
  interleave_sb_kernel<uint16_t><<<grid, 256, 0, s>>>(
      static_cast<const uint16_t*>(scales), static_cast<const uint16_t*>(biases),
      static_cast<uint32_t*>(out), N, G, src_stride);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// a.scales: the pair image (a.sb_transposed == 2).
int launch_qmm_mfma_pairs(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const int gs_shift = shift_of(gs);
  const int nt = choose_nt(a.M, a.N, a.L);
  MLXROCM_REHEARSE("qmm_t_tile(nt=%d,pairs)", nt);
  const dim3 grid((a.N + 32 * nt - 1) / (32 * nt), (a.M + kBM - 1) / kBM, a.L);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      switch (nt) {
        case 5:
          return launch_variant<T, T, T, B, 5, false, false, true>(a, gs_shift, grid, s);
        case 6:
          return launch_variant<T, T, T, B, 6, false, false, true>(a, gs_shift, grid, s);
        default:
          return launch_variant<T, T, T, B, 7, false, false, true>(a, gs_shift, grid, s);
      }
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

// K cut into k_splits ranges: `a.out` points at k_splits fp32 planes of M x N.
int launch_qmm_mfma_ksplit_pairs(
    const QmmArgs& a, int gs, int bits, int dtype, int k_splits, hipStream_t s) {
  constexpr int kNT = 7;
  const int gs_shift = shift_of(gs);
  MLXROCM_REHEARSE("qmm_t_tile(ksplit=%d,pairs)", k_splits);
  const dim3 grid((a.N + 32 * kNT - 1) / (32 * kNT), (a.M + kBM - 1) / kBM, k_splits);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      return launch_variant<T, T, float, B, kNT, false, false, true>(a, gs_shift, grid, s, k_splits);
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
