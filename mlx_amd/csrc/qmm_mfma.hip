// qmm_mfma.hip -- prefill GEMM (transpose=true, large M) for 16-bit element
// types and every code width, on the gfx950 matrix cores.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T
//
// A workgroup of 512 threads (8 wavefronts: 2 along M x 4 along N) owns a
// 256 (M) x 256 (N) tile of y and walks K in steps of 64 through two LDS stages
// (2 x 72 KiB).  Per step:
//   * the x tile (256 x 64) and the packed W tile (256 rows x 64 codes) of the
//     step after next are fetched into registers;
//   * W is dequantized exactly once per workgroup -- thread (n, h) expands the
//     32 codes [32h, 32h+32) of row n with one scale/bias pair (a K-step never
//     holds more than one group per 32 codes) as fp32 fma(s, code, b), rounds to
//     T and stores them to the idle LDS stage while the matrix cores work on
//     the other one, so the 256 rows of x reuse every weight;
//   * each wavefront computes a 64 (N) x 128 (M) block of y^T with
//     v_mfma_f32_32x32x16: A operand = W rows, B operand = x rows, so that a lane
//     ends up with 4 consecutive n of one m -- an 8-byte store of y.
// LDS rows are 64 elements + 8 of padding (144 bytes), which makes the 16-byte
// fragment reads of 16 consecutive rows hit 64 distinct banks.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 256;
constexpr int kBN = 256;
constexpr int kBK = 64;
constexpr int kLdsStride = kBK + 8; // elements per LDS row
constexpr int kThreads = 512;

template <typename T>
__device__ __forceinline__ floatx16 mfma32(const uint4& a, const uint4& b, const floatx16& c);

template <>
__device__ __forceinline__ floatx16
mfma32<bf16_t>(const uint4& a, const uint4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
      __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <>
__device__ __forceinline__ floatx16
mfma32<f16_t>(const uint4& a, const uint4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(
      __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

typedef float floatx2 __attribute__((ext_vector_type(2)));

// Two floats -> two T in one dword (lo in the low half), round to nearest even;
// the vector convert selects the packed hardware convert.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef T Tx2 __attribute__((ext_vector_type(2)));
  const floatx2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, Tx2));
}

// Code i (0..31) of the 32 codes held in BITS consecutive dwords.
template <int BITS>
__device__ __forceinline__ uint32_t code32(const uint32_t (&w)[BITS], int i) {
  const int bit = i * BITS;
  const int word = bit >> 5;
  const int sh = bit & 31;
  uint32_t v = w[word] >> sh;
  if (sh + BITS > 32) {
    v |= w[word + 1] << (32 - sh);
  }
  return v & ((1u << BITS) - 1u);
}

// 32 codes -> 32 elements of T: fma(s, code, b) in fp32, one rounding to T.
template <typename T, int BITS>
__device__ __forceinline__ void dequant32(
    const uint32_t (&w)[BITS],
    float s,
    float b,
    uint32_t (&out)[16]) {
  if constexpr (BITS == 4) {
    // nibbles -> bytes first, so that every convert is a cvt_f32_ubyteN
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t lo = w[d] & 0x0f0f0f0fu;        // codes 0,2,4,6
      uint32_t hi = (w[d] >> 4) & 0x0f0f0f0fu; // codes 1,3,5,7
      // keep the byte form: otherwise the shifts are folded back into one
      // bit-field extract per code
      asm volatile("" : "+v"(lo), "+v"(hi));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float c0 = static_cast<float>((lo >> (8 * j)) & 0xffu);
        const float c1 = static_cast<float>((hi >> (8 * j)) & 0xffu);
        out[4 * d + j] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
      }
    }
  } else if constexpr (BITS == 8) {
#pragma unroll
    for (int d = 0; d < 8; ++d) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float c0 = static_cast<float>((w[d] >> (16 * j)) & 0xffu);
        const float c1 = static_cast<float>((w[d] >> (16 * j + 8)) & 0xffu);
        out[2 * d + j] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float c0 = static_cast<float>(code32<BITS>(w, 2 * i));
      const float c1 = static_cast<float>(code32<BITS>(w, 2 * i + 1));
      out[i] = pack2<T>(fmaf(s, c0, b), fmaf(s, c1, b));
    }
  }
}

template <typename T, int BITS, int GS>
__global__ __launch_bounds__(kThreads) void qmm_t_mfma_kernel(const QmmArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // two stages, each an x tile followed by a W tile
  constexpr int kXTile = kBM * kLdsStride; // elements
  constexpr int kWTile = kBN * kLdsStride;
  constexpr int kStage = kXTile + kWTile;
  T* lds = reinterpret_cast<T*>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 3;  // which 64 columns (n) of the tile
  const int wm = wave >> 2; // which 128 rows (m) of the tile
  const int M = a.M;
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kBN;
  const int m0 = blockIdx.y * kBM;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.z);

  const int groups = K / GS;
  const int row_words = K / 32 * BITS;

  // ---- loader roles ----
  // x: thread covers 16-byte chunk (tid % 8) of rows tid/8 + 64 i, i < 4.
  const int xc = tid & 7;
  const int xr = tid >> 3;
  // W: thread (wr, wh) covers codes [32 wh, 32 wh + 32) of tile row wr.
  const int wr = tid >> 1;
  const int wh = tid & 1;
  const int w_row = (n0 + wr < N) ? n0 + wr : N - 1; // clamp: loads stay in bounds
  const uint32_t* wsrc = reinterpret_cast<const uint32_t*>(p.w) +
      static_cast<size_t>(w_row) * row_words + wh * BITS;
  const T* ssrc = p.scales + static_cast<size_t>(w_row) * groups;
  const T* bsrc = p.biases + static_cast<size_t>(w_row) * groups;
  // Rows of x past M are never stored, so they may read any valid row: the
  // loads then need no predicate.  32-bit element offsets from p.x.
  uint32_t xoff0, xoff1, xoff2, xoff3;
  {
    auto row_off = [&](int i) {
      const int m = m0 + xr + 64 * i;
      return static_cast<uint32_t>(m < M ? m : M - 1) * static_cast<uint32_t>(K) + xc * 8;
    };
    xoff0 = row_off(0);
    xoff1 = row_off(1);
    xoff2 = row_off(2);
    xoff3 = row_off(3);
  }

  // registers of the tile in flight
  uint4 xq0, xq1, xq2, xq3;
  uint32_t wreg[BITS];
  T sreg, breg; // converted when used, so the loads are not waited for early

#define QMM_LOAD_TILE(k0)                                                        \
  do {                                                                           \
    xq0 = *reinterpret_cast<const uint4*>(p.x + xoff0 + (k0));                   \
    xq1 = *reinterpret_cast<const uint4*>(p.x + xoff1 + (k0));                   \
    xq2 = *reinterpret_cast<const uint4*>(p.x + xoff2 + (k0));                   \
    xq3 = *reinterpret_cast<const uint4*>(p.x + xoff3 + (k0));                   \
    const uint32_t* wp__ = wsrc + ((k0) / 32) * BITS;                            \
    _Pragma("unroll") for (int j__ = 0; j__ < BITS; ++j__) {                     \
      wreg[j__] = wp__[j__];                                                     \
    }                                                                            \
    const int g__ = ((k0) + 32 * wh) / GS;                                       \
    sreg = ssrc[g__];                                                            \
    breg = bsrc[g__];                                                            \
  } while (0)

#define QMM_STORE_TILE(stage)                                                    \
  do {                                                                           \
    T* xs__ = lds + (stage) * kStage;                                            \
    T* ws__ = xs__ + kXTile;                                                     \
    *reinterpret_cast<uint4*>(&xs__[(xr + 0) * kLdsStride + xc * 8]) = xq0;      \
    *reinterpret_cast<uint4*>(&xs__[(xr + 64) * kLdsStride + xc * 8]) = xq1;     \
    *reinterpret_cast<uint4*>(&xs__[(xr + 128) * kLdsStride + xc * 8]) = xq2;    \
    *reinterpret_cast<uint4*>(&xs__[(xr + 192) * kLdsStride + xc * 8]) = xq3;    \
    uint32_t dq__[16];                                                           \
    dequant32<T, BITS>(wreg, to_f32(sreg), to_f32(breg), dq__);                  \
    uint4* dst__ = reinterpret_cast<uint4*>(&ws__[wr * kLdsStride + wh * 32]);   \
    _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                        \
      dst__[j__] = make_uint4(                                                   \
          dq__[4 * j__], dq__[4 * j__ + 1], dq__[4 * j__ + 2], dq__[4 * j__ + 3]); \
    }                                                                            \
  } while (0)

  // ---- accumulators: 2 (n) x 4 (m) tiles of 32 x 32 ----
  floatx16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }

  const int fr = lane & 31; // fragment row inside a 32-row MFMA tile
  const int fk = lane >> 5; // which 8 of the 16 k of an MFMA step
  const int xfrag_off = (wm * 128 + fr) * kLdsStride + fk * 8;
  const int wfrag_off = kXTile + (wn * 64 + fr) * kLdsStride + fk * 8;

  auto mfma_tile = [&](int stage) {
    const T* xfrag = lds + stage * kStage + xfrag_off;
    const T* wfrag = lds + stage * kStage + wfrag_off;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      uint4 af[2];
      uint4 bf[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *reinterpret_cast<const uint4*>(wfrag + i * 32 * kLdsStride + kk * 16);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bf[j] = *reinterpret_cast<const uint4*>(xfrag + j * 32 * kLdsStride + kk * 16);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = mfma32<T>(af[i], bf[j], acc[i][j]);
        }
      }
    }
  };

  // ---- software pipeline: registers hold tile t+1 while LDS stage t%2 feeds
  // the matrix cores.  The two wavefronts that share a SIMD (wm = 0 and 1)
  // work in opposite phases: while one issues the MFMAs of tile t, the other
  // dequantizes and stores its share of tile t+1 and fetches tile t+2, so the
  // matrix pipe and the vector ALU of a SIMD are busy at the same time.  Tile
  // t+1 is complete after both phases; stage (t+1)%2 was last read in step t-1.
  const int nk = K / kBK;
  QMM_LOAD_TILE(0);
  QMM_STORE_TILE(0);
  if (nk > 1) {
    QMM_LOAD_TILE(kBK);
  }
  __syncthreads();
  // wm = 0: compute(t), store(t+1), compute(t+1), ...
  // wm = 1: store(1), compute(0), store(2), compute(1), ...
  // with a barrier after every phase; both sides execute 2 nk + 1 barriers.
#define QMM_MEM_PHASE(ts)                                                        \
  do {                                                                           \
    const int ts__ = (ts);                                                       \
    if (ts__ < nk) {                                                             \
      QMM_STORE_TILE(ts__ & 1);                                                  \
    }                                                                            \
    /* unconditional: past the end the last tile is fetched again and never     \
       stored, which keeps the loaded registers free of a select */             \
    const int tl__ = ts__ + 1 < nk ? ts__ + 1 : nk - 1;                          \
    QMM_LOAD_TILE(tl__ * kBK);                                                   \
  } while (0)

  if (wm == 1) {
    QMM_MEM_PHASE(1);
    __syncthreads();
  }
  for (int t = 0; t < nk; ++t) {
    __builtin_amdgcn_s_setprio(1);
    mfma_tile(t & 1);
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();
    QMM_MEM_PHASE(t + 1 + wm);
    __syncthreads();
  }
  if (wm == 0) {
    __syncthreads();
  }
#undef QMM_MEM_PHASE

  // ---- epilogue: D[n][m] tiles; register r of lane (col, half) holds
  // n = 8 (r / 4) + 4 half + r % 4, m = col.  Four consecutive n -> one 8-byte
  // store of y[m][n .. n+3].
  const int col = lane & 31;
  const int half = lane >> 5;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + wm * 128 + j * 32 + col;
    if (m >= M) {
      continue;
    }
    T* yrow = p.out + static_cast<size_t>(m) * N;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + i * 32 + 8 * q + 4 * half;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = p.valid ? acc[i][j][4 * q + e] : 0.0f;
        }
        if (n + 3 < N && (N % 4) == 0) {
          uint2 packed;
          packed.x = pack2<T>(v[0], v[1]);
          packed.y = pack2<T>(v[2], v[3]);
          *reinterpret_cast<uint2*>(yrow + n) = packed;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < N) {
              yrow[n + e] = from_f32<T>(v[e]);
            }
          }
        }
      }
    }
  }
}

#undef QMM_LOAD_TILE
#undef QMM_STORE_TILE

constexpr size_t kQmmSmemBytes =
    static_cast<size_t>(2) * (kBM + kBN) * kLdsStride * 2; // two stages, 16-bit

} // namespace

bool qmm_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  (void)gs;
  (void)bits;
  if (!transpose || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  return a.K % kBK == 0 && a.K >= kBK;
}

int launch_qmm_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const dim3 grid((a.N + kBN - 1) / kBN, (a.M + kBM - 1) / kBM, a.L);
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    return dispatch_bits(bits, [&](auto bval) {
      return dispatch_group(gs, [&](auto gval) {
        constexpr int B = decltype(bval)::value;
        constexpr int G = decltype(gval)::value;
        auto kern = qmm_t_mfma_kernel<T, B, G>;
        static bool configured = false; // per instantiation
        if (!configured) {
          MLXROCM_HIP_TRY(hipFuncSetAttribute(
              reinterpret_cast<const void*>(kern),
              hipFuncAttributeMaxDynamicSharedMemorySize,
              static_cast<int>(kQmmSmemBytes)));
          configured = true;
        }
        kern<<<grid, kThreads, kQmmSmemBytes, s>>>(a);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      });
    });
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
