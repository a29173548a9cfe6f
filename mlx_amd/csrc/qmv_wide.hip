// qmv_wide.hip -- transpose=true products with up to 16 rows of x for 16-bit
// element types (batched decode, small expert groups) on the matrix cores.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T,   M <= 16
//
// The weight stream bounds the work, so the kernel is shaped for many
// independent wavefronts that each stream packed codes straight into MFMA
// operands -- no LDS round trip for the weights and no workgroup barrier in the
// loop:
//   * a workgroup of 8 wavefronts owns 16 rows of W; wavefront w takes the
//     128-code steps w, w + 8, w + 16, ... of K;
//   * in a step, lane (i = lane % 16, kb = lane / 16) fetches the 32 codes
//     [32 kb, 32 kb + 32) of row i (4 lanes cover 128 codes of a row; the
//     neighbouring wavefront fetches the other half of a 4-bit row's cache
//     line), dequantizes them (fp32 fma(s, code, b), one rounding to T) and uses
//     them as the A operands of four v_mfma_f32_16x16x32: MFMA q multiplies the
//     codes 32 kb + 8 q .. + 8 of every lane.  Any assignment of k to the
//     MFMA's reduction slots is valid as long as the x operand uses the same
//     one, and x goes through a small wavefront-private LDS tile from which
//     each lane picks exactly those elements;
//   * fetches run four steps ahead of their use;
//   * the eight partial tiles are summed through LDS at the end.
#include "mfma_dequant.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kWdRows = 16;    // rows of W per workgroup
constexpr int kWdWaves = 8;    // wavefronts per workgroup, interleaved over K
constexpr int kWdStep = 128;   // codes of a row per step
constexpr int kWdAhead = 4;    // fetch distance in steps
constexpr int kWdXStride = kWdStep + 8; // elements per row of the staged x tile
constexpr int kWdThreads = kWdWaves * 64;

template <int MROWS>
constexpr size_t wide_smem_bytes() {
  // per wavefront: two x tiles; reused for the final reduction (8 x 64 x 16 B)
  constexpr size_t x = static_cast<size_t>(kWdWaves) * 2 * MROWS * kWdXStride * 2;
  constexpr size_t red = static_cast<size_t>(kWdWaves) * 64 * 16;
  return x > red ? x : red;
}

// MROWS: rows of x staged per step (8 or 16, M <= MROWS); with 8 the MFMA's
// 16-row x operand reads every staged row twice and the upper half of the
// result is dropped.
template <typename T, int BITS, int MROWS>
__global__ __launch_bounds__(kWdThreads) void qmv_wide_kernel(const QmmArgs a, const int gs_shift) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int kXLoads = MROWS / 4; // 16-byte loads per lane and step for x
  constexpr int kXTile = MROWS * kWdXStride;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int M = a.M;
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kWdRows;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  const int groups = K >> gs_shift;
  const int nsteps = K / kWdStep;
  // this wavefront's steps: wave, wave + 8, ...; it has `mine` of them
  const int mine = (nsteps - wave + kWdWaves - 1) / kWdWaves;

  const int fi = lane & 15;
  const int fk = lane >> 4;
  const int row = (n0 + fi < N) ? n0 + fi : N - 1; // clamp: loads stay in bounds
  const uint32_t* wsrc = reinterpret_cast<const uint32_t*>(p.w) +
      static_cast<size_t>(row) * (K / 32 * BITS) + fk * BITS;
  const T* ssrc = p.scales + static_cast<size_t>(row) * groups;
  const T* bsrc = p.biases + static_cast<size_t>(row) * groups;
  // x: lane covers 16-byte piece (lane % 16) of rows lane / 16 + 4 i.  Rows past
  // M reread row M - 1 (their results are never stored).
  const int xpiece = lane & 15;
  const int xr = lane >> 4;
  auto x_off = [&](int i) {
    const int m = xr + 4 * i;
    return static_cast<uint32_t>(m < M ? m : M - 1) * static_cast<uint32_t>(K) + xpiece * 8;
  };
  const uint32_t xoff0 = x_off(0);
  const uint32_t xoff1 = x_off(1);
  const uint32_t xoff2 = x_off(2);
  const uint32_t xoff3 = x_off(3);

  T* xlds = reinterpret_cast<T*>(smem) + wave * 2 * kXTile; // wavefront-private
  const int xst = xr * kWdXStride + xpiece * 8;               // staging position
  const int xfr = (fi % MROWS) * kWdXStride + fk * 32;        // fragment position

  // ring of kWdAhead steps in flight (named registers: arrays indexed through
  // macros end up in scratch memory)
  uint32_t w0[BITS], w1[BITS], w2[BITS], w3[BITS];
  T s0, s1, s2, s3, b0, b1, b2, b3;
  uint4 x00, x01, x02, x03, x10, x11, x12, x13, x20, x21, x22, x23, x30, x31, x32, x33;

  // fetch own step number j (clamped to the last own step: past the end the
  // same data is fetched again and never used)
#define WIDE_FETCH(slot, j)                                                      \
  do {                                                                           \
    const int jj__ = (j) < mine ? (j) : mine - 1;                                \
    const int k0__ = (jj__ * kWdWaves + wave) * kWdStep;                         \
    const uint32_t* wp__ = wsrc + (k0__ / 32) * BITS;                            \
    _Pragma("unroll") for (int q__ = 0; q__ < BITS; ++q__) {                     \
      w##slot[q__] = wp__[q__];                                                  \
    }                                                                            \
    const int g__ = (k0__ + 32 * fk) >> gs_shift;                                \
    s##slot = ssrc[g__];                                                         \
    b##slot = bsrc[g__];                                                         \
    x##slot##0 = *reinterpret_cast<const uint4*>(p.x + xoff0 + k0__);            \
    x##slot##1 = *reinterpret_cast<const uint4*>(p.x + xoff1 + k0__);            \
    if constexpr (kXLoads > 2) {                                                 \
      x##slot##2 = *reinterpret_cast<const uint4*>(p.x + xoff2 + k0__);          \
      x##slot##3 = *reinterpret_cast<const uint4*>(p.x + xoff3 + k0__);          \
    }                                                                            \
  } while (0)

  floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};

  // consume ring slot `slot` (own step j, LDS buffer j % 2)
#define WIDE_CONSUME(slot, j)                                                    \
  do {                                                                           \
    T* xt__ = xlds + ((j) & 1) * kXTile;                                         \
    *reinterpret_cast<uint4*>(xt__ + xst) = x##slot##0;                          \
    *reinterpret_cast<uint4*>(xt__ + xst + 4 * kWdXStride) = x##slot##1;         \
    if constexpr (kXLoads > 2) {                                                 \
      *reinterpret_cast<uint4*>(xt__ + xst + 8 * kWdXStride) = x##slot##2;       \
      *reinterpret_cast<uint4*>(xt__ + xst + 12 * kWdXStride) = x##slot##3;      \
    }                                                                            \
    /* the tile is private to this wavefront, whose lanes run in lockstep: no   \
       barrier instruction, only an ordering point for the compiler */          \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                       \
    __builtin_amdgcn_wave_barrier();                                             \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                       \
    uint32_t dq__[16];                                                           \
    dequant32<T, BITS>(w##slot, to_f32(s##slot), to_f32(b##slot), dq__);         \
    _Pragma("unroll") for (int q__ = 0; q__ < 4; ++q__) {                        \
      const uint4 af__ = make_uint4(                                             \
          dq__[4 * q__], dq__[4 * q__ + 1], dq__[4 * q__ + 2], dq__[4 * q__ + 3]); \
      const uint4 bf__ = *reinterpret_cast<const uint4*>(xt__ + xfr + 8 * q__);  \
      acc = mfma16<T>(af__, bf__, acc);                                          \
    }                                                                            \
  } while (0)

  if (mine > 0) {
    WIDE_FETCH(0, 0);
    if (mine > 1) {
      WIDE_FETCH(1, 1);
    }
    if (mine > 2) {
      WIDE_FETCH(2, 2);
    }
    if (mine > 3) {
      WIDE_FETCH(3, 3);
    }
    for (int j = 0; j < mine; j += kWdAhead) {
      WIDE_CONSUME(0, j);
      if (j + 4 < mine) {
        WIDE_FETCH(0, j + 4);
      }
      if (j + 1 < mine) {
        WIDE_CONSUME(1, j + 1);
        if (j + 5 < mine) {
          WIDE_FETCH(1, j + 5);
        }
      }
      if (j + 2 < mine) {
        WIDE_CONSUME(2, j + 2);
        if (j + 6 < mine) {
          WIDE_FETCH(2, j + 6);
        }
      }
      if (j + 3 < mine) {
        WIDE_CONSUME(3, j + 3);
        if (j + 7 < mine) {
          WIDE_FETCH(3, j + 7);
        }
      }
    }
  }
#undef WIDE_FETCH
#undef WIDE_CONSUME

  // ---- sum the eight partial tiles: lane l of every wavefront holds
  // y[m = l % 16][n = 4 (l / 16) + r], r = 0..3.
  __syncthreads(); // all wavefronts are done with their x tiles
  floatx4* red = reinterpret_cast<floatx4*>(smem);
  red[wave * 64 + lane] = acc;
  __syncthreads();
  if (wave == 0) {
    floatx4 total = red[lane];
#pragma unroll
    for (int w = 1; w < kWdWaves; ++w) {
      const floatx4 v = red[w * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        total[r] += v[r];
      }
    }
    const int m = lane & 15;
    const int n = n0 + 4 * (lane >> 4);
    if (m < M) {
      T* yrow = p.out + static_cast<size_t>(m) * N;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] = p.valid ? total[r] : 0.0f;
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
}

} // namespace

bool qmv_wide_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  (void)gs;
  (void)bits;
  if (!transpose || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  if (a.M < 1 || a.M > 16) {
    return false;
  }
  // whole steps of 128 codes; 32-bit element offsets into x
  if (a.K % kWdStep != 0 || a.K < kWdStep) {
    return false;
  }
  return static_cast<int64_t>(a.M) * a.K < (int64_t{1} << 32);
}

int launch_qmv_wide(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const dim3 grid((a.N + kWdRows - 1) / kWdRows, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] batch=%d exceeds the grid", a.L);
  }
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      constexpr int B = decltype(bval)::value;
      auto go = [&](auto mrv) -> int {
        constexpr int MR = decltype(mrv)::value;
        qmv_wide_kernel<T, B, MR><<<grid, kWdThreads, wide_smem_bytes<MR>(), s>>>(a, gs_shift);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      };
      return a.M <= 8 ? go(IntC<8>{}) : go(IntC<16>{});
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
