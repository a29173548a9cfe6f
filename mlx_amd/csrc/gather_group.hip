// gather_group.hip -- groups the index pairs of a GatherQMM call by expert so
// that the matrix-core GEMM reads every expert's weights once for all the rows
// routed to it (the reference loops over the pairs one GEMV at a time,
// mlx/backend/cpu/quantized.cpp:700-747; the Metal backend groups sorted runs,
// mlx/backend/metal/quantized.cpp:1905-1923).
//
// Three small kernels fill a caller-provided workspace (one workgroup does all
// three steps in a single launch when there are at most 16384 pairs):
//   count    a histogram per workgroup in LDS, then one global atomic per
//            workgroup and expert into counts[expert] (one global atomic per
//            pair serializes on the few counters, worst for sorted indices);
//            pairs with an index out of range are left out and their output
//            rows are zero-filled here;
//   plan     one workgroup: exclusive scan of the counts -> first sorted
//            position of every expert, and the list of tiles {expert, first
//            position, rows} of up to tile_rows rows (256 for the tile GEMM, 32
//            for the few-row kernel when the groups are small); the tile count
//            stays on the device;
//   scatter  perm[position] = pair: rank inside the workgroup from an LDS
//            counter, the workgroup's base from one atomic on a per-expert cursor.
// The order inside an expert's run is arbitrary; every output row depends on
// its own x row only, so the result does not depend on it.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kMaxExperts = 4096; // plan kernel keeps the counts in LDS

template <typename T>
__global__ __launch_bounds__(256) void group_count_kernel(
    const uint32_t* lhs,
    const uint32_t* rhs,
    int n_indices,
    int x_batches,
    int n_experts,
    int32_t* counts,
    T* out,
    int N) {
  __shared__ int32_t hist[kMaxExperts];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    hist[e] = 0;
  }
  __syncthreads();
  const int l = blockIdx.x * blockDim.x + threadIdx.x;
  if (l < n_indices) {
    const uint32_t xi = lhs[l];
    const uint32_t wi = rhs[l];
    if (xi < static_cast<uint32_t>(x_batches) && wi < static_cast<uint32_t>(n_experts)) {
      atomicAdd(&hist[wi], 1);
    } else {
      T* row = out + static_cast<size_t>(l) * N;
      for (int n = 0; n < N; ++n) {
        row[n] = static_cast<T>(0.0f);
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    if (hist[e] != 0) {
      atomicAdd(&counts[e], hist[e]);
    }
  }
}

__global__ __launch_bounds__(256) void group_plan_kernel(
    int n_experts,
    int tile_rows,
    const int32_t* counts,
    int32_t* offsets,
    int32_t* tiles,
    int32_t* n_tiles) {
  __shared__ int32_t cnt[kMaxExperts];
  __shared__ int32_t first_pos[kMaxExperts];
  __shared__ int32_t first_tile[kMaxExperts];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    cnt[e] = counts[e];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int pos = 0;
    int tile = 0;
    for (int e = 0; e < n_experts; ++e) {
      first_pos[e] = pos;
      first_tile[e] = tile;
      pos += cnt[e];
      tile += (cnt[e] + tile_rows - 1) / tile_rows;
    }
    n_tiles[0] = tile;
    n_tiles[1] = pos; // pairs with both indices in range
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    offsets[e] = first_pos[e];
    const int c = cnt[e];
    int t = first_tile[e];
    for (int r = 0; r < c; r += tile_rows, ++t) {
      tiles[3 * t + 0] = e;
      tiles[3 * t + 1] = first_pos[e] + r;
      tiles[3 * t + 2] = (c - r < tile_rows) ? c - r : tile_rows;
    }
  }
}

__global__ __launch_bounds__(256) void group_scatter_kernel(
    const uint32_t* lhs,
    const uint32_t* rhs,
    int n_indices,
    int x_batches,
    int n_experts,
    const int32_t* offsets,
    int32_t* cursor,
    int32_t* perm) {
  __shared__ int32_t hist[kMaxExperts]; // pairs of this workgroup per expert, then its base
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    hist[e] = 0;
  }
  __syncthreads();
  const int l = blockIdx.x * blockDim.x + threadIdx.x;
  bool live = false;
  uint32_t wi = 0;
  int rank = 0;
  if (l < n_indices) {
    const uint32_t xi = lhs[l];
    wi = rhs[l];
    live = xi < static_cast<uint32_t>(x_batches) && wi < static_cast<uint32_t>(n_experts);
    if (live) {
      rank = atomicAdd(&hist[wi], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    const int c = hist[e];
    if (c != 0) {
      hist[e] = atomicAdd(&cursor[e], c);
    }
  }
  __syncthreads();
  if (live) {
    perm[offsets[wi] + hist[wi] + rank] = l;
  }
}

// All three steps in one workgroup, for calls with so few pairs that four
// launches cost more than the work: counts, scan and cursors stay in LDS, no
// global atomics, nothing to clear beforehand.
constexpr int kFusedThreads = 1024;
constexpr int kFusedMaxPairs = 16384;

template <typename T>
__global__ __launch_bounds__(kFusedThreads) void group_fused_kernel(
    const uint32_t* lhs,
    const uint32_t* rhs,
    int n_indices,
    int x_batches,
    int n_experts,
    int tile_rows,
    int32_t* offsets,
    int32_t* tiles,
    int32_t* n_tiles,
    int32_t* perm,
    T* out,
    int N) {
  __shared__ int32_t cnt[kMaxExperts];
  __shared__ int32_t first_pos[kMaxExperts];
  __shared__ int32_t first_tile[kMaxExperts]; // later: the scatter cursor
  for (int e = threadIdx.x; e < n_experts; e += kFusedThreads) {
    cnt[e] = 0;
  }
  __syncthreads();
  for (int l = threadIdx.x; l < n_indices; l += kFusedThreads) {
    const uint32_t xi = lhs[l];
    const uint32_t wi = rhs[l];
    if (xi < static_cast<uint32_t>(x_batches) && wi < static_cast<uint32_t>(n_experts)) {
      atomicAdd(&cnt[wi], 1);
    } else {
      T* row = out + static_cast<size_t>(l) * N;
      for (int n = 0; n < N; ++n) {
        row[n] = static_cast<T>(0.0f);
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int pos = 0;
    int tile = 0;
    for (int e = 0; e < n_experts; ++e) {
      first_pos[e] = pos;
      first_tile[e] = tile;
      pos += cnt[e];
      tile += (cnt[e] + tile_rows - 1) / tile_rows;
    }
    n_tiles[0] = tile;
    n_tiles[1] = pos; // pairs with both indices in range
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += kFusedThreads) {
    offsets[e] = first_pos[e];
    const int c = cnt[e];
    int t = first_tile[e];
    for (int r = 0; r < c; r += tile_rows, ++t) {
      tiles[3 * t + 0] = e;
      tiles[3 * t + 1] = first_pos[e] + r;
      tiles[3 * t + 2] = (c - r < tile_rows) ? c - r : tile_rows;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += kFusedThreads) {
    first_tile[e] = 0;
  }
  __syncthreads();
  for (int l = threadIdx.x; l < n_indices; l += kFusedThreads) {
    const uint32_t xi = lhs[l];
    const uint32_t wi = rhs[l];
    if (xi < static_cast<uint32_t>(x_batches) && wi < static_cast<uint32_t>(n_experts)) {
      const int rank = atomicAdd(&first_tile[wi], 1);
      perm[first_pos[wi] + rank] = l;
    }
  }
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* p, int n, int32_t v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    p[i] = v;
  }
}

size_t align_up(size_t v, size_t a) {
  return (v + a - 1) / a * a;
}

} // namespace

int gather_group_max_tiles(int n_indices, int n_experts, int tile_rows) {
  // every expert may end on a partial tile
  return (n_indices + tile_rows - 1) / tile_rows + n_experts;
}

size_t gather_group_workspace_bytes(int n_indices, int n_experts) {
  if (n_indices <= 0 || n_experts <= 0 || n_experts > kMaxExperts) {
    return 0;
  }
  const size_t ints = static_cast<size_t>(3) * n_experts + 4 +
      static_cast<size_t>(3) * gather_group_max_tiles(n_indices, n_experts, kGroupSmallTile) +
      n_indices; // sized for the smaller tile
  return align_up(ints * sizeof(int32_t), 256);
}

void bind_gather_group(QmmArgs& a, int tile_rows, void* workspace) {
  const int E = a.n_experts;
  int32_t* ws = static_cast<int32_t*>(workspace);
  int32_t* n_tiles = ws + 3 * E;
  int32_t* tiles = n_tiles + 4;
  a.group_tiles = tiles;
  a.group_perm = tiles + 3 * gather_group_max_tiles(a.L, E, tile_rows);
  a.group_ntiles = n_tiles;
  a.group_tile_rows = tile_rows;
}

// Fills the workspace and points the grouped-mode fields of `a` into it.
int launch_gather_group(QmmArgs& a, int dtype, int tile_rows, void* workspace, hipStream_t s) {
  const int E = a.n_experts;
  const int n = a.L;
  int32_t* ws = static_cast<int32_t*>(workspace);
  int32_t* counts = ws;
  int32_t* cursor = counts + E;
  int32_t* offsets = cursor + E;
  int32_t* n_tiles = offsets + E;
  int32_t* tiles = n_tiles + 4;
  int32_t* perm = tiles + 3 * gather_group_max_tiles(n, E, tile_rows);

  a.group_tiles = tiles;
  a.group_perm = perm;
  a.group_ntiles = n_tiles;
  MLXROCM_REHEARSE(n <= kFusedMaxPairs ? "gather_group(fused)" : "gather_group(3 kernels)");
  a.group_tile_rows = tile_rows;
  if (n <= kFusedMaxPairs) {
    if (dtype == MLXROCM_BFLOAT16) {
      group_fused_kernel<bf16_t><<<1, kFusedThreads, 0, s>>>(
          a.lhs_indices, a.rhs_indices, n, a.x_batches, E, tile_rows, offsets, tiles, n_tiles,
          perm, static_cast<bf16_t*>(a.out), a.N);
    } else {
      group_fused_kernel<f16_t><<<1, kFusedThreads, 0, s>>>(
          a.lhs_indices, a.rhs_indices, n, a.x_batches, E, tile_rows, offsets, tiles, n_tiles,
          perm, static_cast<f16_t*>(a.out), a.N);
    }
    MLXROCM_HIP_TRY(hipGetLastError());
    return MLXROCM_OK;
  }

  // counts and cursors start at zero (a fill kernel, so that the sequence can be
  // captured into a graph)
  fill_i32_kernel<<<(2 * E + 255) / 256, 256, 0, s>>>(counts, 2 * E, 0);
  MLXROCM_HIP_TRY(hipGetLastError());
  const int blocks = (n + 255) / 256;
  if (dtype == MLXROCM_BFLOAT16) {
    group_count_kernel<bf16_t><<<blocks, 256, 0, s>>>(
        a.lhs_indices, a.rhs_indices, n, a.x_batches, E, counts,
        static_cast<bf16_t*>(a.out), a.N);
  } else {
    group_count_kernel<f16_t><<<blocks, 256, 0, s>>>(
        a.lhs_indices, a.rhs_indices, n, a.x_batches, E, counts,
        static_cast<f16_t*>(a.out), a.N);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  group_plan_kernel<<<1, 256, 0, s>>>(E, tile_rows, counts, offsets, tiles, n_tiles);
  MLXROCM_HIP_TRY(hipGetLastError());
  group_scatter_kernel<<<blocks, 256, 0, s>>>(
      a.lhs_indices, a.rhs_indices, n, a.x_batches, E, offsets, cursor, perm);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

} // namespace mlxrocm
