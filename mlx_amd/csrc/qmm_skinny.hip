// qmm_skinny.hip -- transpose=true products with 17..32 rows of x for 16-bit
// element types, and small expert groups of a gather (tiles of up to 32 rows).
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T
//
// The weights are read once and the work is bound by that stream, so the
// kernel is built around full-line coalesced fetches of the packed rows:
// a workgroup of 256 threads (4 wavefronts) owns 64 rows of W and walks K in
// steps of 128 codes (52 KiB of LDS, so three workgroups share a compute unit
// and hide each other's barrier and LDS latencies).  Per step
//   * every thread fetches one 32-code piece (four consecutive lanes cover the
//     128 codes of a row; consecutive steps use up the rest of the cache line),
//     three steps ahead of its use;
//   * the pieces are dequantized (fp32 fma(s, code, b), one rounding to T) into
//     the idle LDS stage, next to the x tile of the step (M rows x 256);
//   * wavefront w multiplies rows [16 w, 16 w + 16) of the tile with
//     v_mfma_f32_16x16x32 (A = W rows, B = x rows), fp32 accumulators.
// LDS rows are 128 elements + 8 of padding (272 bytes): the 16-byte fragment
// reads of 16 consecutive rows fall on distinct banks.
#include "mfma_dequant.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kSkBN = 64;
constexpr int kSkBK = 128;
constexpr int kSkStride = kSkBK + 8; // elements per LDS row
constexpr int kSkThreads = 256;
constexpr int kSkAhead = 3; // packed-W fetch distance in steps

template <int MROWS>
constexpr size_t skinny_smem_bytes() {
  return static_cast<size_t>(2) * (kSkBN + MROWS) * kSkStride * 2;
}

// MROWS: rows of x staged per step (16 or 32; M <= MROWS).
// GROUPED: blockIdx.y walks the 32-row tile list of a gather grouped by expert
// (one x row per index pair, fetched and written back through the permutation).
template <typename T, int BITS, int MROWS, bool GROUPED>
__global__ __launch_bounds__(kSkThreads) void qmm_skinny_kernel(const QmmArgs a, const int gs_shift) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int kMRows = MROWS;
  constexpr int MT = MROWS > 16 ? 2 : 1;
  constexpr int kWTile = kSkBN * kSkStride; // elements
  constexpr int kXTile = kMRows * kSkStride;
  constexpr int kStage = kWTile + kXTile;
  T* lds = reinterpret_cast<T*>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kSkBN;
  int M = a.M;
  int row0 = 0; // grouped: first sorted position of the tile
  QmmProblem<T> p;
  if constexpr (GROUPED) {
    const int tile = blockIdx.y;
    if (tile >= *a.group_ntiles) {
      return; // the grid covers the worst-case tile count
    }
    const int e = a.group_tiles[3 * tile];
    row0 = a.group_tiles[3 * tile + 1];
    M = a.group_tiles[3 * tile + 2];
    p.x = static_cast<const T*>(a.x);
    p.w = reinterpret_cast<const uint8_t*>(a.w + static_cast<int64_t>(e) * a.w_batch_stride);
    p.scales = static_cast<const T*>(a.scales) + static_cast<int64_t>(e) * a.sb_batch_stride;
    p.biases = static_cast<const T*>(a.biases) + static_cast<int64_t>(e) * a.sb_batch_stride;
    p.out = static_cast<T*>(a.out);
    p.valid = true;
  } else {
    p = resolve_problem<T>(a, blockIdx.y);
  }

  const int groups = K >> gs_shift;
  const int row_words = K / 32 * BITS;
  const int nk = K / kSkBK;

  // ---- loader roles ----
  // W: thread covers piece (tid % 4) -- codes [32 piece, 32 piece + 32) of the
  // step -- of tile row tid / 4.
  constexpr int kPieces = kSkBK / 32;              // pieces per row and step
  constexpr int kWRows = kSkThreads / kPieces;     // rows covered by one pass
  constexpr int kWPasses = kSkBN / kWRows;         // 1
  const int piece = tid % kPieces;
  const int wr0 = tid / kPieces;
  const uint32_t* wsrc[kWPasses];
  const T* ssrc[kWPasses];
  const T* bsrc[kWPasses];
#pragma unroll
  for (int h = 0; h < kWPasses; ++h) {
    const int n = n0 + wr0 + kWRows * h;
    const int row = n < N ? n : N - 1; // clamp: loads stay in bounds
    wsrc[h] = reinterpret_cast<const uint32_t*>(p.w) + static_cast<size_t>(row) * row_words +
        piece * BITS;
    ssrc[h] = p.scales + static_cast<size_t>(row) * groups;
    bsrc[h] = p.biases + static_cast<size_t>(row) * groups;
  }
  // x: 16 sixteen-byte pieces per row and step; thread covers piece (tid % 16)
  // of rows tid / 16 + 16 i.  Rows past M reread row M - 1 (never stored).
  // (named registers: small arrays indexed inside lambdas end up in scratch)
  constexpr int kXPieces = kSkBK / 8;
  constexpr int kXRows = kSkThreads / kXPieces;    // rows covered by one pass
  constexpr int kXLoads = kMRows / kXRows;         // 1 or 2
  static_assert(kXLoads >= 1 && kXLoads <= 4, "x staging shape");
  const int xpiece = tid % kXPieces;
  const int xr0 = tid / kXPieces;
  auto x_row_off = [&](int i) {
    const int m = xr0 + kXRows * i;
    const int mc = m < M ? m : M - 1;
    if constexpr (GROUPED) {
      const uint32_t pair = static_cast<uint32_t>(a.group_perm[row0 + mc]);
      return a.lhs_indices[pair] * static_cast<uint32_t>(a.x_batch_stride) + xpiece * 8;
    } else {
      return static_cast<uint32_t>(mc) * static_cast<uint32_t>(K) + xpiece * 8;
    }
  };
  const uint32_t xoff0 = x_row_off(0);
  const uint32_t xoff1 = x_row_off(1);
  const uint32_t xoff2 = x_row_off(2);
  const uint32_t xoff3 = x_row_off(3);
  // x of the next kSkAhead steps: ring slot s, row block i -> xq<s><i>
  uint4 xq00, xq01, xq02, xq03, xq10, xq11, xq12, xq13, xq20, xq21, xq22, xq23;

  // packed W, scales and biases of the next kSkAhead steps
  uint32_t wq[kSkAhead][kWPasses][BITS];
  T sq[kSkAhead][kWPasses], bq[kSkAhead][kWPasses];
  auto fetch_w = [&](int slot, int step) {
    const int st = step < nk ? step : nk - 1; // past the end: refetch, never used
#pragma unroll
    for (int h = 0; h < kWPasses; ++h) {
      const uint32_t* wp = wsrc[h] + st * (kSkBK / 32) * BITS;
#pragma unroll
      for (int j = 0; j < BITS; ++j) {
        wq[slot][h][j] = wp[j];
      }
      const int g = (st * kSkBK + 32 * piece) >> gs_shift;
      sq[slot][h] = ssrc[h][g];
      bq[slot][h] = bsrc[h][g];
    }
  };
#define SKINNY_FETCH_X(slot, step)                                               \
  do {                                                                           \
    const int st__ = (step) < nk ? (step) : nk - 1;                              \
    xq##slot##0 = *reinterpret_cast<const uint4*>(p.x + xoff0 + st__ * kSkBK);   \
    if constexpr (kXLoads > 1) {                                                 \
      xq##slot##1 = *reinterpret_cast<const uint4*>(p.x + xoff1 + st__ * kSkBK); \
    }                                                                            \
    if constexpr (kXLoads > 2) {                                                 \
      xq##slot##2 = *reinterpret_cast<const uint4*>(p.x + xoff2 + st__ * kSkBK); \
      xq##slot##3 = *reinterpret_cast<const uint4*>(p.x + xoff3 + st__ * kSkBK); \
    }                                                                            \
  } while (0)

#define SKINNY_STORE_X(stage, slot)                                              \
  do {                                                                           \
    T* xs__ = lds + (stage) * kStage + kWTile;                                   \
    *reinterpret_cast<uint4*>(&xs__[(xr0 + 0 * kXRows) * kSkStride + xpiece * 8]) = xq##slot##0; \
    if constexpr (kXLoads > 1) {                                                 \
      *reinterpret_cast<uint4*>(&xs__[(xr0 + 1 * kXRows) * kSkStride + xpiece * 8]) = xq##slot##1; \
    }                                                                            \
    if constexpr (kXLoads > 2) {                                                 \
      *reinterpret_cast<uint4*>(&xs__[(xr0 + 2 * kXRows) * kSkStride + xpiece * 8]) = xq##slot##2; \
      *reinterpret_cast<uint4*>(&xs__[(xr0 + 3 * kXRows) * kSkStride + xpiece * 8]) = xq##slot##3; \
    }                                                                            \
  } while (0)

  auto store_w = [&](int stage, int slot) {
    T* ws = lds + stage * kStage;
#pragma unroll
    for (int h = 0; h < kWPasses; ++h) {
      uint32_t dq[16];
      dequant32<T, BITS>(wq[slot][h], to_f32(sq[slot][h]), to_f32(bq[slot][h]), dq);
      uint4* dst = reinterpret_cast<uint4*>(&ws[(wr0 + kWRows * h) * kSkStride + piece * 32]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dst[j] = make_uint4(dq[4 * j], dq[4 * j + 1], dq[4 * j + 2], dq[4 * j + 3]);
      }
    }
  };

  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      acc[t][r] = 0.0f;
    }
  }
  const int fi = lane & 15;
  const int fk = lane >> 4;
  const int afrag = (wave * 16 + fi) * kSkStride + fk * 8;
  const int bfrag = kWTile + (fi % kMRows) * kSkStride + fk * 8;
  auto mfma_tile = [&](int stage) {
    const T* base = lds + stage * kStage;
#pragma unroll
    for (int s = 0; s < kSkBK / 32; ++s) {
      const uint4 af = *reinterpret_cast<const uint4*>(base + afrag + s * 32);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const uint4 bf =
            *reinterpret_cast<const uint4*>(base + bfrag + t * 16 * kSkStride + s * 32);
        acc[t] = mfma16<T>(af, bf, acc[t]);
      }
    }
  };

  // ---- pipeline: registers hold the packed W and the x of steps t+1 .. t+3,
  // LDS stage t%2 feeds the matrix cores; one barrier per step.  The register
  // ring is indexed at compile time: the loop runs in rounds of kSkAhead steps.
  static_assert(kSkAhead == 3, "the rounds below are written out for three steps");
  fetch_w(0, 0);
  SKINNY_FETCH_X(0, 0);
  fetch_w(1, 1);
  SKINNY_FETCH_X(1, 1);
  fetch_w(2, 2);
  SKINNY_FETCH_X(2, 2);
  SKINNY_STORE_X(0, 0);
  store_w(0, 0);
  fetch_w(0, kSkAhead);
  SKINNY_FETCH_X(0, kSkAhead);
  __syncthreads();
  // Step t, whose successor t + 1 sits in ring slot `nx` (= (t + 1) % 3).  The
  // fetches are clamped to the last step and what the last step stores is never
  // read, so the step has no branch.
#define SKINNY_STEP(t, nx)                                                       \
  {                                                                              \
    const int cur__ = (t) & 1;                                                   \
    SKINNY_STORE_X(cur__ ^ 1, nx);                                               \
    store_w(cur__ ^ 1, nx);                                                      \
    fetch_w(nx, (t) + 1 + kSkAhead);                                             \
    SKINNY_FETCH_X(nx, (t) + 1 + kSkAhead);                                      \
    mfma_tile(cur__);                                                            \
    __syncthreads();                                                             \
  }
  int t0 = 0;
  for (; t0 + kSkAhead <= nk; t0 += kSkAhead) {
    SKINNY_STEP(t0, 1)
    SKINNY_STEP(t0 + 1, 2)
    SKINNY_STEP(t0 + 2, 0)
  }
  if (t0 < nk) {
    SKINNY_STEP(t0, 1)
  }
  if (t0 + 1 < nk) {
    SKINNY_STEP(t0 + 1, 2)
  }
#undef SKINNY_STEP
#undef SKINNY_FETCH_X
#undef SKINNY_STORE_X

  // ---- epilogue: lane (col, quad) holds y[m = 16 t + col][n = 4 quad + r].
  const int col = lane & 15;
  const int quad = lane >> 4;
  const int n = n0 + wave * 16 + 4 * quad;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + col;
    if (m >= M) {
      continue;
    }
    const size_t orow =
        GROUPED ? static_cast<size_t>(a.group_perm[row0 + m]) : static_cast<size_t>(m);
    T* yrow = p.out + orow * N;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = p.valid ? acc[t][r] : 0.0f;
    }
    if (n + 3 < N && (N % 4) == 0) {
      uint2 packed;
      packed.x = pack2<T>(v[0], v[1]);
      packed.y = pack2<T>(v[2], v[3]);
      *reinterpret_cast<uint2*>(yrow + n) = packed;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n + r < N) {
          yrow[n + r] = from_f32<T>(v[r]);
        }
      }
    }
  }
}

} // namespace

bool qmm_skinny_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  (void)gs;
  (void)bits;
  if (!transpose || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  if (a.M < 1 || a.M > 32) {
    return false;
  }
  // whole steps of 128 codes; 32-bit element offsets into x
  if (a.K % kSkBK != 0 || a.K < kSkBK) {
    return false;
  }
  return static_cast<int64_t>(a.M) * a.K < (int64_t{1} << 32);
}

int launch_qmm_skinny(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const dim3 grid((a.N + kSkBN - 1) / kSkBN, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] batch=%d exceeds the grid", a.L);
  }
  MLXROCM_REHEARSE("qmm_skinny");
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      auto go = [&](auto mrv) -> int {
        constexpr int MR = decltype(mrv)::value;
        constexpr size_t smem = skinny_smem_bytes<MR>();
        auto kern = qmm_skinny_kernel<T, B, MR, false>;
        static bool configured = false; // per instantiation
        if (!configured) {
          MLXROCM_HIP_TRY(hipFuncSetAttribute(
              reinterpret_cast<const void*>(kern),
              hipFuncAttributeMaxDynamicSharedMemorySize,
              static_cast<int>(smem)));
          configured = true;
        }
        kern<<<grid, kSkThreads, smem, s>>>(a, gs_shift);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      };
      return a.M <= 16 ? go(IntC<16>{}) : go(IntC<32>{});
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

// Gather grouped by expert in 32-row tiles: `a` carries the tile list; one grid
// row per possible tile, rows past the device-side tile count exit at once.
int launch_qmm_skinny_grouped(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const dim3 grid(
      (a.N + kSkBN - 1) / kSkBN, gather_group_max_tiles(a.L, a.n_experts, kGroupSmallTile));
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[gather_qmm] %d index pairs exceed the grid", a.L);
  }
  MLXROCM_REHEARSE("qmm_skinny_grouped");
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      constexpr size_t smem = skinny_smem_bytes<kGroupSmallTile>();
      auto kern = qmm_skinny_kernel<T, B, kGroupSmallTile, true>;
      static bool configured = false; // per instantiation
      if (!configured) {
        MLXROCM_HIP_TRY(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern),
            hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(smem)));
        configured = true;
      }
      kern<<<grid, kSkThreads, smem, s>>>(a, gs_shift);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
