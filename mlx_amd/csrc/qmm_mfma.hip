// qmm_mfma.hip -- launchers of the prefill tile kernel (qmm_mfma_tile.h):
// transpose=true with the caller's scale layout or the two transposed images,
// split K, float32 through split bf16 operands, [K, N] weights, grouped gathers.
// The launches that read the (scale, bias) pair image are in qmm_mfma_pairs.hip.
#include "qmm_mfma_tile.h"

namespace mlxrocm {

bool qmm_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  (void)gs;
  if (dtype == MLXROCM_FLOAT32) {
    return false;
  }
  if (!transpose && !(bits == 4 || bits == 8)) {
    return false; // [K, N] weights: the column loader reads whole words per 8 codes
  }
  return a.K % kBK == 0 && a.K >= kBK;
}

namespace {

// [K, N] weights (transpose=false), 4- or 8-bit; TO = float when K is split.
template <typename T, typename TO, int NT>
int launch_wn(const QmmArgs& a, int gs_shift, int bits, dim3 grid, hipStream_t s, int k_splits) {
  if (bits == 4) {
    return launch_variant<T, T, TO, 4, NT, false, true>(a, gs_shift, grid, s, k_splits);
  }
  return launch_variant<T, T, TO, 8, NT, false, true>(a, gs_shift, grid, s, k_splits);
}

} // namespace

namespace {

// [K][G] -> [G][K] for scales and biases (blockIdx.z: which of the two, then
// which batch entry), 32 x 32 tiles through LDS.
template <typename T>
__global__ __launch_bounds__(256) void transpose_sb_kernel(
    const T* scales,
    const T* biases,
    T* out,
    int K,
    int G,
    int64_t src_stride) {
  __shared__ T tile[32][33];
  const int which = blockIdx.z & 1;
  const int l = blockIdx.z >> 1;
  const T* src = (which == 0 ? scales : biases) + l * src_stride;
  T* dst = out + (static_cast<size_t>(l) * 2 + which) * K * G;
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5; // 0..7
  const int g0 = blockIdx.x * 32;
  const int k0 = blockIdx.y * 32;
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int k = k0 + r;
    const int g = g0 + tx;
    if (k < K && g < G) {
      tile[r][tx] = src[static_cast<size_t>(k) * G + g];
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int g = g0 + r;
    const int k = k0 + tx;
    if (k < K && g < G) {
      dst[static_cast<size_t>(g) * K + k] = tile[tx][r];
    }
  }
}

} // namespace

// Scratch bytes of the transposed scale / bias image of `batches` weight matrices.
size_t qmm_n_sb_bytes(int K, int G, int batches, int dtype) {
  return static_cast<size_t>(2) * batches * K * G * dtype_size(dtype);
}

// out: per batch entry the [G][K] scales followed by the [G][K] biases.
int transpose_sb_for_qmm_n(
    const void* scales,
    const void* biases,
    void* out,
    int K,
    int G,
    int batches,
    int64_t src_stride,
    int dtype,
    hipStream_t s) {
  const dim3 grid((G + 31) / 32, (K + 31) / 32, 2 * batches);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] K=%d or batch=%d exceed the grid", K, batches);
  }
  MLXROCM_REHEARSE("transpose_sb");
  if (dtype == MLXROCM_FLOAT32) {
    transpose_sb_kernel<float><<<grid, 256, 0, s>>>(
        static_cast<const float*>(scales), static_cast<const float*>(biases),
        static_cast<float*>(out), K, G, src_stride);
  } else if (dtype == MLXROCM_BFLOAT16) {
    transpose_sb_kernel<bf16_t><<<grid, 256, 0, s>>>(
        static_cast<const bf16_t*>(scales), static_cast<const bf16_t*>(biases),
        static_cast<bf16_t*>(out), K, G, src_stride);
  } else {
    transpose_sb_kernel<f16_t><<<grid, 256, 0, s>>>(
        static_cast<const f16_t*>(scales), static_cast<const f16_t*>(biases),
        static_cast<f16_t*>(out), K, G, src_stride);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// transpose=false on the matrix cores: same tiles, column loader for W.  a.scales
// / a.biases point at the transposed images made by transpose_sb_for_qmm_n.
int launch_qmm_mfma_n(const QmmArgs& a, int gs, int bits, int dtype, int k_splits, hipStream_t s) {
  const int gs_shift = shift_of(gs);
  MLXROCM_REHEARSE("qmm_n_tile(ksplit=%d)", k_splits);
  if (k_splits > 1) {
    const dim3 grid((a.N + 32 * 6 - 1) / (32 * 6), (a.M + kBM - 1) / kBM, k_splits);
    return dtype == MLXROCM_BFLOAT16
        ? launch_wn<bf16_t, float, 6>(a, gs_shift, bits, grid, s, k_splits)
        : launch_wn<f16_t, float, 6>(a, gs_shift, bits, grid, s, k_splits);
  }
  int nt = choose_nt(a.M, a.N, a.L);
  nt = nt > 6 ? 6 : nt; // the column loader's registers leave room for 6 x 32 columns
  const dim3 grid((a.N + 32 * nt - 1) / (32 * nt), (a.M + kBM - 1) / kBM, a.L);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return nt == 5 ? launch_wn<T, T, 5>(a, gs_shift, bits, grid, s, 1)
                   : launch_wn<T, T, 6>(a, gs_shift, bits, grid, s, 1);
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

int launch_qmm_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const int gs_shift = shift_of(gs);
  // (128-wide tiles, which would make x [2048, .] x W [4096, .] exactly one round
  // of 256 workgroups, were measured and are not offered: a K-step costs nearly
  // the same whatever the tile's width -- the x tile, the barrier and the
  // dequantization work per thread do not shrink with it -- so 4096 x 4096 went
  // from 83 to 82 us at 2048 rows and from 292 to 338 us at 8192)
  const int nt = choose_nt(a.M, a.N, a.L);
  MLXROCM_REHEARSE("qmm_t_tile(nt=%d)", nt);
  const dim3 grid((a.N + 32 * nt - 1) / (32 * nt), (a.M + kBM - 1) / kBM, a.L);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      switch (nt) {
        case 5:
          return launch_variant<T, T, T, B, 5, false>(a, gs_shift, grid, s);
        case 6:
          return launch_variant<T, T, T, B, 6, false>(a, gs_shift, grid, s);
        default:
          return launch_variant<T, T, T, B, 7, false>(a, gs_shift, grid, s);
      }
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

// How many ranges to cut K into so that a launch with few tiles still fills the
// compute units (1 = no split): only for a single problem, and every range
// keeps at least eight steps.
int qmm_mfma_k_splits(int M, int N, int K, int L) {
  if (L != 1) {
    return 1;
  }
  const long cus = compute_units();
  const long tiles = static_cast<long>((M + kBM - 1) / kBM) * ((N + 32 * 7 - 1) / (32 * 7));
  const long steps = K / kBK;
  long s = cus / tiles;
  if (s > steps / 8) {
    s = steps / 8;
  }
  // (up to 16 ranges: a narrow N over a long K -- 3584 x 18944, 128 rows: 45.6 us
  // against 57.5 with at most 8, 2048 x 8192: 26.7 against 32.7)
  if (s > 16) {
    s = 16;
  }
  return s < 2 ? 1 : static_cast<int>(s);
}

// 16-bit operands with K cut into k_splits ranges: `a.out` points at k_splits
// fp32 planes of M x N (reduce_k_splits adds them up into y).
int launch_qmm_mfma_ksplit(
    const QmmArgs& a,
    int gs,
    int bits,
    int dtype,
    int k_splits,
    hipStream_t s) {
  constexpr int kNT = 7;
  const int gs_shift = shift_of(gs);
  const dim3 grid((a.N + 32 * kNT - 1) / (32 * kNT), (a.M + kBM - 1) / kBM, k_splits);
  MLXROCM_REHEARSE("qmm_t_tile(ksplit=%d)", k_splits);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      return launch_variant<T, T, float, B, kNT, false>(a, gs_shift, grid, s, k_splits);
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

namespace {

template <typename TO>
__global__ __launch_bounds__(256) void reduce_k_splits_kernel(
    const float* partial,
    TO* out,
    size_t n,
    int k_splits) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i >= n) {
    return;
  }
  if (i + 4 <= n) {
    float4 acc = *reinterpret_cast<const float4*>(partial + i);
    for (int z = 1; z < k_splits; ++z) {
      const float4 v = *reinterpret_cast<const float4*>(partial + z * n + i);
      acc.x += v.x;
      acc.y += v.y;
      acc.z += v.z;
      acc.w += v.w;
    }
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<float4*>(out + i) = acc;
    } else {
      uint2 packed;
      packed.x = pack2<TO>(acc.x, acc.y);
      packed.y = pack2<TO>(acc.z, acc.w);
      *reinterpret_cast<uint2*>(out + i) = packed;
    }
  } else {
    for (size_t e = i; e < n; ++e) {
      float acc = 0.0f;
      for (int z = 0; z < k_splits; ++z) {
        acc += partial[z * n + e];
      }
      out[e] = static_cast<TO>(acc);
    }
  }
}

} // namespace

// y = sum of the k_splits fp32 planes (n = M * N elements each, a multiple of 4
// apart); y must be 16-byte aligned.
int reduce_k_splits(const void* partial, void* out, size_t n, int k_splits, int dtype, hipStream_t s) {
  const size_t blocks = (n / 4 + 1 + 255) / 256;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] output too large for the split-K reduction");
  }
  MLXROCM_REHEARSE("reduce_k_splits(%d)", k_splits);
  const float* p = static_cast<const float*>(partial);
  const unsigned g = static_cast<unsigned>(blocks);
  if (dtype == MLXROCM_FLOAT32) {
    reduce_k_splits_kernel<float><<<g, 256, 0, s>>>(p, static_cast<float*>(out), n, k_splits);
  } else if (dtype == MLXROCM_BFLOAT16) {
    reduce_k_splits_kernel<bf16_t><<<g, 256, 0, s>>>(p, static_cast<bf16_t*>(out), n, k_splits);
  } else {
    reduce_k_splits_kernel<f16_t><<<g, 256, 0, s>>>(p, static_cast<f16_t*>(out), n, k_splits);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// fp32 operands: `a.x` already points at the [hi | lo | hi] bf16 image of x
// (split_x_for_mfma) and a.x_batch_stride counts its elements (M * 3 K).
int launch_qmm_mfma_split(const QmmArgs& a, int gs, int bits, hipStream_t s, int k_splits) {
  // six column blocks: with fp32 scales and the weight split, seven spill
  // registers to scratch memory (measured 620 against 415 us at 1024 x 11008 x 4096)
  constexpr int kNT = 6;
  const int gs_shift = shift_of(gs);
  const dim3 grid(
      (a.N + 32 * kNT - 1) / (32 * kNT), (a.M + kBM - 1) / kBM, k_splits > 1 ? k_splits : a.L);
  MLXROCM_REHEARSE("qmm_t_tile_split_fp32(ksplit=%d)", k_splits);
  return dispatch_bits(bits, [&](auto bval) {
    constexpr int B = decltype(bval)::value;
    return launch_variant<bf16_t, float, float, B, kNT, false>(a, gs_shift, grid, s, k_splits);
  });
}

namespace {

// 8 consecutive fp32 of x -> 8 bf16 high parts and 8 bf16 low parts, written to
// blocks 0/2 and 1 of the element's group of three 64-wide blocks.
__global__ __launch_bounds__(256) void split_x_kernel(
    const float* x,
    bf16_t* xs,
    size_t rows,
    int K) {
  const size_t unit = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t units_per_row = static_cast<size_t>(K) / 8;
  if (unit >= rows * units_per_row) {
    return;
  }
  const size_t row = unit / units_per_row;
  const int k = static_cast<int>(unit - row * units_per_row) * 8;
  const float4 v0 = *reinterpret_cast<const float4*>(x + row * K + k);
  const float4 v1 = *reinterpret_cast<const float4*>(x + row * K + k + 4);
  const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
  uint32_t hi[4], lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float h0 = static_cast<float>(static_cast<bf16_t>(v[2 * i]));
    const float h1 = static_cast<float>(static_cast<bf16_t>(v[2 * i + 1]));
    hi[i] = pack2<bf16_t>(v[2 * i], v[2 * i + 1]);
    lo[i] = pack2<bf16_t>(v[2 * i] - h0, v[2 * i + 1] - h1);
  }
  bf16_t* dst = xs + row * (3 * static_cast<size_t>(K)) + static_cast<size_t>(k / 64) * 192 + k % 64;
  const uint4 h = make_uint4(hi[0], hi[1], hi[2], hi[3]);
  *reinterpret_cast<uint4*>(dst) = h;
  *reinterpret_cast<uint4*>(dst + 64) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
  *reinterpret_cast<uint4*>(dst + 128) = h;
}

} // namespace

size_t split_x_bytes(size_t rows, int K) {
  return rows * 3 * static_cast<size_t>(K) * sizeof(bf16_t);
}

int split_x_for_mfma(const void* x, void* xs, size_t rows, int K, hipStream_t s) {
  const size_t units = rows * (static_cast<size_t>(K) / 8);
  const size_t blocks = (units + 255) / 256;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] x is too large to split");
  }
  MLXROCM_REHEARSE("split_x");
  split_x_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(
      static_cast<const float*>(x), static_cast<bf16_t*>(xs), rows, K);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// Gather grouped by expert: `a` carries the tile list; one grid row per
// possible tile, rows past the device-side tile count exit at once.
int launch_qmm_mfma_grouped(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  MLXROCM_REHEARSE("qmm_t_tile_grouped");
  constexpr int kNT = 7;
  const int gs_shift = shift_of(gs);
  const dim3 grid(
      (a.N + 32 * kNT - 1) / (32 * kNT), gather_group_max_tiles(a.L, a.n_experts, kGroupLargeTile), 1);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      return launch_variant<T, T, T, B, kNT, true>(a, gs_shift, grid, s);
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

// The same for [K, N] weights (transpose=false): a.scales / a.biases point at
// the transposed images of all experts (transpose_sb_for_qmm_n), a.sb_batch_stride
// is the distance between two experts' images.
int launch_qmm_mfma_grouped_n(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  MLXROCM_REHEARSE("qmm_n_tile_grouped");
  constexpr int kNT = 6;
  const int gs_shift = shift_of(gs);
  const dim3 grid(
      (a.N + 32 * kNT - 1) / (32 * kNT), gather_group_max_tiles(a.L, a.n_experts, kGroupLargeTile), 1);
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    if (bits == 4) {
      return launch_variant<T, T, T, 4, kNT, true, true>(a, gs_shift, grid, s);
    }
    return launch_variant<T, T, T, 8, kNT, true, true>(a, gs_shift, grid, s);
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
