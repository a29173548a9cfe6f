// qmv_wide.hip -- transpose=true products with up to 16 rows of x for 16-bit
// element types (batched decode, small expert groups, odd code widths) on the
// matrix cores.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T,   M <= 16
//
// The weight stream bounds the work, so the kernel is shaped for many
// independent wavefronts that each stream packed codes straight into MFMA
// operands -- no LDS round trip for the weights and no workgroup barrier in the
// loop:
//   * a workgroup of 8 wavefronts owns 16 rows of W; wavefront w takes the
//     256-code steps w, w + 8, w + 16, ... of K;
//   * in a step, lane l fetches piece l / 8 (32 codes) of rows l % 8 and
//     l % 8 + 8: eight consecutive lanes cover 256 consecutive codes of a row,
//     whole cache lines for 4-bit codes and wider.  The MFMA wants lane
//     (i = l % 16, kb = l / 16) to hold codes of row i, so each lane keeps the
//     piece of its own row and swaps the other with lane l ^ 8 (one DPP rotate
//     per dword): it ends up with the 64 codes [64 kb, 64 kb + 64) of row i;
//   * those are dequantized (fp32 fma(s, code, b), one rounding to T) and used
//     as the A operands of eight v_mfma_f32_16x16x32: MFMA q multiplies the
//     codes 64 kb + 8 q .. + 8 of every lane.  Any assignment of k to the MFMA's
//     reduction slots is valid as long as the x operand uses the same one, and x
//     goes through a small wavefront-private LDS tile from which each lane picks
//     exactly those elements;
//   * the last step may be partial (K is a multiple of 32, not of 256): x is
//     staged as zero past K and the weight fetches are clamped into the row;
//   * fetches run kAhead steps ahead of their use;
//   * the eight partial tiles are summed through LDS at the end.
#include "mfma_dequant.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kWdRows = 16;    // rows of W per workgroup
constexpr int kWdWaves = 8;    // wavefronts per workgroup, interleaved over K
constexpr int kWdStep = 256;   // codes of a row per step
constexpr int kWdXStride = kWdStep + 8; // elements per row of the staged x tile
constexpr int kWdThreads = kWdWaves * 64;

template <int MROWS>
constexpr size_t wide_smem_bytes() {
  // per wavefront: one x tile; reused for the final reduction (8 x 64 x 16 B)
  constexpr size_t x = static_cast<size_t>(kWdWaves) * MROWS * kWdXStride * 2;
  constexpr size_t red = static_cast<size_t>(kWdWaves) * 64 * 16;
  return x > red ? x : red;
}

// value of lane (l ^ 8): a rotation by 8 inside each row of 16 lanes
__device__ __forceinline__ uint32_t swap8(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
      0, static_cast<int>(v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
}

// MROWS: rows of x staged per step (8 or 16, M <= MROWS); with 8 the MFMA's
// 16-row x operand reads every staged row twice and the upper half of the
// result is dropped.
template <typename T, int BITS, int MROWS>
__global__ __launch_bounds__(kWdThreads) void qmv_wide_kernel(const QmmArgs a, const int gs_shift) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int kXLoads = MROWS / 2; // 16-byte loads per lane and step for x
  constexpr int kXTile = MROWS * kWdXStride;
  constexpr int kAhead = 2; // fetch distance in steps (registers are what limits occupancy)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int M = a.M;
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kWdRows;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  const int groups = K >> gs_shift;
  const int pieces = K / 32;                       // 32-code pieces per row
  const int nsteps = (K + kWdStep - 1) / kWdStep;
  // this wavefront's steps: wave, wave + 8, ...; it has `mine` of them
  const int mine = nsteps > wave ? (nsteps - wave + kWdWaves - 1) / kWdWaves : 0;

  // fetch role: piece (lane / 8) of rows lane % 8 and lane % 8 + 8
  const int pc = lane >> 3;
  const uint32_t* wrow[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int n = n0 + (lane & 7) + 8 * h;
    wrow[h] = reinterpret_cast<const uint32_t*>(p.w) +
        static_cast<size_t>(n < N ? n : N - 1) * (K / 32 * BITS); // clamp: stay in bounds
  }
  // MFMA role: row i = lane % 16, codes [64 kb, 64 kb + 64) of the step
  const int fi = lane & 15;
  const int fk = lane >> 4;
  const bool upper = (lane & 8) != 0; // rows 8..15 came with the second fetch
  const int frow = (n0 + fi < N) ? n0 + fi : N - 1;
  const T* ssrc = p.scales + static_cast<size_t>(frow) * groups;
  const T* bsrc = p.biases + static_cast<size_t>(frow) * groups;
  // x: lane covers 16-byte piece (lane % 32) of rows lane / 32 + 2 i.  Rows past
  // M reread row M - 1 (their results are never stored).
  const int xpiece = lane & 31;
  const int xr = lane >> 5;
  uint32_t xoff[kXLoads];
#pragma unroll
  for (int i = 0; i < kXLoads; ++i) {
    const int m = xr + 2 * i;
    xoff[i] = static_cast<uint32_t>(m < M ? m : M - 1) * static_cast<uint32_t>(K);
  }

  T* xlds = reinterpret_cast<T*>(smem) + wave * kXTile; // wavefront-private
  const int xst = xr * kWdXStride + xpiece * 8;           // staging position
  const int xfr = (fi % MROWS) * kWdXStride + fk * 64;    // fragment position

  // one step in flight
  struct Step {
    uint32_t w[2][BITS];
    T s[2], b[2];
    uint4 x[kXLoads];
  };
  auto fetch = [&](Step& st, int j) {
    const int k0 = (j * kWdWaves + wave) * kWdStep;
    // pieces past the end of the row (partial last step) reread the last piece;
    // x is zero there
    const int piece = (k0 / 32 + pc < pieces) ? k0 / 32 + pc : pieces - 1;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t* wp = wrow[h] + piece * BITS;
#pragma unroll
      for (int q = 0; q < BITS; ++q) {
        st.w[h][q] = wp[q];
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int k = k0 + 64 * fk + 32 * h;
      const int g = (k < K ? k : K - 1) >> gs_shift;
      st.s[h] = ssrc[g];
      st.b[h] = bsrc[g];
    }
    const int kx = k0 + 8 * xpiece;
    const bool live = kx < K;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      st.x[i] = make_uint4(0u, 0u, 0u, 0u);
      if (live) {
        st.x[i] = *reinterpret_cast<const uint4*>(p.x + xoff[i] + kx);
      }
    }
  };

  floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};

  auto consume = [&](Step& st) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      *reinterpret_cast<uint4*>(xlds + xst + 2 * i * kWdXStride) = st.x[i];
    }
    // The tile is private to this wavefront, whose lanes run in lockstep and
    // whose LDS operations complete in order: no barrier instruction, only an
    // ordering point for the compiler.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // keep the piece of this lane's row, swap the other one with lane ^ 8
    uint32_t lo[BITS], hi[BITS];
#pragma unroll
    for (int q = 0; q < BITS; ++q) {
      const uint32_t own = upper ? st.w[1][q] : st.w[0][q];   // row i, piece 2 kb + upper
      const uint32_t give = upper ? st.w[0][q] : st.w[1][q];  // row i ^ 8, same piece
      const uint32_t got = swap8(give);                       // row i, piece 2 kb + !upper
      lo[q] = upper ? got : own;
      hi[q] = upper ? own : got;
    }
    // one 32-code piece at a time, to keep few registers live
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint32_t dq[16];
      dequant32<T, BITS>(h == 0 ? lo : hi, to_f32(st.s[h]), to_f32(st.b[h]), dq);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 af = make_uint4(dq[4 * q], dq[4 * q + 1], dq[4 * q + 2], dq[4 * q + 3]);
        const uint4 bf = *reinterpret_cast<const uint4*>(xlds + xfr + 32 * h + 8 * q);
        acc = mfma16<T>(af, bf, acc);
      }
    }
    // the next step's x stores must not overtake these reads in the compiler's
    // schedule (the hardware keeps LDS operations of a wavefront in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  Step s0, s1, s2;
  if (mine > 0) {
    fetch(s0, 0);
    if (mine > 1) {
      fetch(s1, 1);
    }
    if constexpr (kAhead == 3) {
      if (mine > 2) {
        fetch(s2, 2);
      }
    }
    for (int j = 0; j < mine; j += kAhead) {
      consume(s0);
      if (j + kAhead < mine) {
        fetch(s0, j + kAhead);
      }
      if (j + 1 < mine) {
        consume(s1);
        if (j + 1 + kAhead < mine) {
          fetch(s1, j + 1 + kAhead);
        }
      }
      if constexpr (kAhead == 3) {
        if (j + 2 < mine) {
          consume(s2);
          if (j + 2 + kAhead < mine) {
            fetch(s2, j + 2 + kAhead);
          }
        }
      }
    }
  }

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
  // 32-code pieces (any K the operator accepts); 32-bit element offsets into x
  if (a.K % 32 != 0 || a.K < 32) {
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
  MLXROCM_REHEARSE("qmv_wide");
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
