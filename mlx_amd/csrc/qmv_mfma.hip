// qmv_mfma.hip -- decode GEMV (transpose=true, M <= 8) for 16-bit element
// types and 4/8-bit codes, written for gfx950.
//
// The kernel is an HBM streaming kernel: every packed weight, scale and bias is
// read exactly once, and all loads of a wave's K-block are issued before the
// first one is consumed.  The arithmetic rides on the matrix cores so that the
// vector ALU only has to widen codes:
//
//   * A workgroup owns 32 output rows: two sub-tiles of 16 rows.  With
//     v_mfma_f32_16x16x32 lane (n = lane % 16, kb = lane / 16) supplies the B
//     operand of row n; the four kb lanes together hold one "unit" of U <= 64
//     consecutive codes of that row, which never crosses a quantization group.
//   * Codes become MFMA B operands without arithmetic: a 4-bit code c is OR-ed
//     into the mantissa of the constant 128.0 (bf16) / 1024.0 (f16), giving
//     exactly OFFSET + c; 8-bit codes are converted with cvt_f32_ubyte (bf16) or
//     a byte permute into 1024.0 (f16).
//   * x is the MFMA A operand (its M <= 8 rows are rows of the 16-row A), staged
//     per wave in LDS in the k-order the code expansion produces, and read once
//     for both sub-tiles.  Per unit and lane the MFMA yields
//     P[m][n] = sum_k x[m][k] * (OFFSET + c[n][k]) in fp32.
//   * y[m][n] = sum_g scale[n][g] * P_g[m][n] + (bias[n][g] - OFFSET*scale[n][g])
//     * sum_{k in g} x[m][k]; the group sums of x are computed while staging.
//
// Wave w of a workgroup takes the K-blocks w, w+W, ...; partial results are
// reduced through LDS.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTileN = 32;        // output rows per workgroup
constexpr int kSubTiles = 2;      // 16-row MFMA tiles per wave
constexpr int kUnitsPerBlock = 8; // units a wave loads at once

template <typename T>
struct Mma;

template <>
struct Mma<bf16_t> {
  static constexpr uint32_t kMagic4 = 0x43004300u; // 128.0 | 128.0
  static constexpr float kOffset4 = 128.0f;
  static constexpr float kOffset8 = 0.0f;
  static __device__ __forceinline__ floatx4
  mfma(const uint4& a, const uint4& b, const floatx4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // 8 bytes -> 8 bf16 in natural order (every value 0..255 is exact in bf16).
  static __device__ __forceinline__ uint4 widen8(uint32_t w0, uint32_t w1) {
    union {
      bf16_t h[8];
      uint4 u;
    } r;
    r.h[0] = static_cast<bf16_t>(static_cast<float>(w0 & 0xffu));
    r.h[1] = static_cast<bf16_t>(static_cast<float>((w0 >> 8) & 0xffu));
    r.h[2] = static_cast<bf16_t>(static_cast<float>((w0 >> 16) & 0xffu));
    r.h[3] = static_cast<bf16_t>(static_cast<float>(w0 >> 24));
    r.h[4] = static_cast<bf16_t>(static_cast<float>(w1 & 0xffu));
    r.h[5] = static_cast<bf16_t>(static_cast<float>((w1 >> 8) & 0xffu));
    r.h[6] = static_cast<bf16_t>(static_cast<float>((w1 >> 16) & 0xffu));
    r.h[7] = static_cast<bf16_t>(static_cast<float>(w1 >> 24));
    return r.u;
  }
  static __device__ __forceinline__ float dot_ones(uint32_t pair, float acc) {
    const bf16x2 ones = {static_cast<__bf16>(1.0f), static_cast<__bf16>(1.0f)};
    return __builtin_amdgcn_fdot2_f32_bf16(
        __builtin_bit_cast(bf16x2, pair), ones, acc, false);
  }
  static __device__ __forceinline__ float widen_scalar(uint32_t h) {
    return __uint_as_float(h << 16);
  }
};

template <>
struct Mma<f16_t> {
  static constexpr uint32_t kMagic4 = 0x64006400u; // 1024.0 | 1024.0
  static constexpr float kOffset4 = 1024.0f;
  static constexpr float kOffset8 = 1024.0f;
  static __device__ __forceinline__ floatx4
  mfma(const uint4& a, const uint4& b, const floatx4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  // byte c -> f16 bits 0x64cc = 1024 + c, two per dword, natural order.
  static __device__ __forceinline__ uint4 widen8(uint32_t w0, uint32_t w1) {
    constexpr uint32_t hi = 0x64646464u;
    // perm selector bytes: 0-3 pick from the second operand, 4-7 from the first
    return make_uint4(
        __builtin_amdgcn_perm(hi, w0, 0x04010400u),
        __builtin_amdgcn_perm(hi, w0, 0x04030402u),
        __builtin_amdgcn_perm(hi, w1, 0x04010400u),
        __builtin_amdgcn_perm(hi, w1, 0x04030402u));
  }
  static __device__ __forceinline__ float dot_ones(uint32_t pair, float acc) {
    const f16x2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pair), ones, acc, false);
  }
  static __device__ __forceinline__ float widen_scalar(uint32_t h) {
    return static_cast<float>(__builtin_bit_cast(f16_t, static_cast<uint16_t>(h)));
  }
};

// Constants of the 4-bit expansion, hidden from constant folding.  With
// literal operands the compiler emits v_and + v_or (a VOP3 instruction cannot
// carry two literals on gfx9); with the mask in an SGPR and the magic in a
// VGPR it selects a single v_and_or_b32.  The empty asm only launders the
// values; no instruction is emitted, so hazard tracking stays with the compiler.
struct Widen4Consts {
  uint32_t mask;
  uint32_t magic;
};

template <typename T>
__device__ __forceinline__ Widen4Consts make_widen4_consts() {
  Widen4Consts c;
  c.mask = 0x000f000fu;
  c.magic = Mma<T>::kMagic4;
  asm volatile("" : "+s"(c.mask));
  asm volatile("" : "+v"(c.magic));
  return c;
}

// One dword of eight 4-bit codes -> 8 values OFFSET + c.  Register j of the
// result holds codes (j, j + 4), so the matching x order is 0,4,1,5,2,6,3,7.
__device__ __forceinline__ uint4 widen4(uint32_t w, const Widen4Consts& c) {
  return make_uint4(
      (w & c.mask) | c.magic,
      ((w >> 4) & c.mask) | c.magic,
      ((w >> 8) & c.mask) | c.magic,
      ((w >> 12) & c.mask) | c.magic);
}

template <int BITS, int GS>
struct QmvShape {
  static constexpr int kUnit = GS < 64 ? GS : 64;          // codes per unit
  static constexpr int kLaneCodes = kUnit / 4;              // 8 or 16
  static constexpr int kLaneBytes = kLaneCodes * BITS / 8;  // 4, 8 or 16
  static constexpr int kLaneWords = kLaneBytes / 4;
  static constexpr int kMfmaPerUnit = kLaneCodes / 8;       // 1 or 2
  static constexpr int kBlockK = kUnit * kUnitsPerBlock;    // 256 or 512
  static constexpr int kGroupsPerBlock = kBlockK / GS;      // 4 or 8
  static constexpr int kUnitsPerGroup = GS / kUnit;         // 1 or 2
  static constexpr int kSbWords = kGroupsPerBlock / 2;      // dwords of scales per row-block
  static_assert(kLaneWords >= 1 && kGroupsPerBlock >= 2, "shape");
};

template <int WORDS>
__device__ __forceinline__ void load_words(const uint8_t* p, uint32_t (&out)[WORDS]) {
  static_assert(WORDS == 1 || WORDS == 2 || WORDS == 4, "");
  if constexpr (WORDS == 4) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else if constexpr (WORDS == 2) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    out[0] = v.x; out[1] = v.y;
  } else {
    out[0] = *reinterpret_cast<const uint32_t*>(p);
  }
}

// Element g of a row of 16-bit values packed two per dword.
template <typename T, int WORDS>
__device__ __forceinline__ float packed_elem(const uint32_t (&w)[WORDS], int g) {
  const uint32_t d = w[g / 2];
  return Mma<T>::widen_scalar((g & 1) ? (d >> 16) : (d & 0xffffu));
}

// Sum over aligned groups of LANES adjacent lanes, left in every lane of the
// group.  DPP only (no LDS round trips): xor-1 and xor-2 swaps inside a quad,
// then mirrored halves of 8 and of 16 lanes.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(LANES == 4 || LANES == 8 || LANES == 16, "");
  auto dpp_add = [](float x, auto ctrl) {
    constexpr int kCtrl = decltype(ctrl)::value;
    const int moved = __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, x), kCtrl, 0xf, 0xf, true);
    return x + __builtin_bit_cast(float, moved);
  };
  v = dpp_add(v, IntC<0xB1>{}); // quad_perm [1,0,3,2]
  v = dpp_add(v, IntC<0x4E>{}); // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) {
    v = dpp_add(v, IntC<0x141>{}); // row_half_mirror
  }
  if constexpr (LANES >= 16) {
    v = dpp_add(v, IntC<0x140>{}); // row_mirror
  }
  return v;
}

// Everything one wave needs of one K-block, as registers: the packed codes of
// its 8 units for both sub-tiles, the block's scales and biases, and
// (lanes < kXLanes) 8 elements of each row of x.
template <int BITS, int GS, int MAXM>
struct BlockRegs {
  using S = QmvShape<BITS, GS>;
  uint32_t w[kSubTiles][kUnitsPerBlock][S::kLaneWords];
  uint32_t s[kSubTiles][S::kSbWords];
  uint32_t b[kSubTiles][S::kSbWords];
  uint4 x[MAXM];
};

// Uniform (scalar) bases and per-lane 32-bit byte offsets of a wave's loads.
struct QmvAddr {
  const uint8_t* w; // first row of the tile
  const uint8_t* s;
  const uint8_t* b;
  const uint8_t* x;
  uint32_t w_lane[kSubTiles];  // row * row_bytes + kb * lane_bytes
  uint32_t sb_lane[kSubTiles]; // row * groups * 2
  uint32_t x_lane;             // lane * 16
};

template <int BITS, int GS, int MAXM>
__device__ __forceinline__ void load_block(
    BlockRegs<BITS, GS, MAXM>& r,
    const QmvAddr& ad,
    int blk,
    int M,
    int K,
    bool x_lane_live) {
  using S = QmvShape<BITS, GS>;
  constexpr int unit_bytes = S::kUnit * BITS / 8;
  // x first: it must not queue behind the weight stream
  const uint8_t* xp = ad.x + static_cast<size_t>(blk) * (S::kBlockK * 2);
#pragma unroll
  for (int m = 0; m < MAXM; ++m) {
    r.x[m] = make_uint4(0, 0, 0, 0);
    if ((MAXM <= 2 || m < M) && x_lane_live) {
      r.x[m] = *reinterpret_cast<const uint4*>(
          xp + static_cast<size_t>(m) * K * 2 + ad.x_lane);
    }
  }
  const uint8_t* wp = ad.w + static_cast<size_t>(blk) * (kUnitsPerBlock * unit_bytes);
#pragma unroll
  for (int u = 0; u < kUnitsPerBlock; ++u) {
#pragma unroll
    for (int t = 0; t < kSubTiles; ++t) {
      load_words<S::kLaneWords>(wp + ad.w_lane[t] + u * unit_bytes, r.w[t][u]);
    }
  }
  const size_t sb_blk = static_cast<size_t>(blk) * (S::kGroupsPerBlock * 2);
#pragma unroll
  for (int t = 0; t < kSubTiles; ++t) {
    load_words<S::kSbWords>(ad.s + sb_blk + ad.sb_lane[t], r.s[t]);
    load_words<S::kSbWords>(ad.b + sb_blk + ad.sb_lane[t], r.b[t]);
  }
}

// Orders one wavefront's LDS writes before its later LDS reads (the lanes of
// a wavefront run in lockstep; only the memory ordering has to be stated).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// MAXM: the largest M this instantiation accepts (M == MAXM when MAXM <= 2).
// PIPE: register sets per wave (2 = ping-pong for waves with several blocks).
template <typename T, int BITS, int GS, int MAXM, int WAVES, int PIPE>
__global__ __launch_bounds__(WAVES * 64) void qmv_mfma_kernel(const QmmArgs a) {
  using S = QmvShape<BITS, GS>;
  using Regs = BlockRegs<BITS, GS, MAXM>;
  constexpr int kThreads = WAVES * 64;
  constexpr float kOffset = (BITS == 4) ? Mma<T>::kOffset4 : Mma<T>::kOffset8;
  constexpr int kXsStride = S::kBlockK + 8; // elements: 16-byte rows, skewed banks
  constexpr int kXLanes = S::kBlockK / 8;   // lanes that carry 8 elements of x
  constexpr int LPG = GS / 8;               // lanes per group while staging x
  constexpr int MR = MAXM < 4 ? MAXM : 4;   // live accumulator registers
  constexpr int BR = (MAXM + 3) / 4;        // bias rows per lane: m = 4*i + kb

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nl = lane & 15;
  const int kb = lane >> 4;
  const int M = (MAXM <= 2) ? MAXM : a.M;
  const int K = a.K;
  const int N = a.N;
  const int n0 = blockIdx.x * kTileN;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  const int groups = K / GS;
  const int nblk = K / S::kBlockK;
  const uint32_t row_bytes = static_cast<uint32_t>(K / 8) * BITS;

  // ---- addresses: scalar bases, 32-bit lane offsets; loads go out at once ----
  const int rows_here = (N - n0 < kTileN) ? N - n0 : kTileN;
  QmvAddr ad;
  ad.w = p.w + static_cast<size_t>(n0) * row_bytes;
  ad.s = reinterpret_cast<const uint8_t*>(p.scales + static_cast<size_t>(n0) * groups);
  ad.b = reinterpret_cast<const uint8_t*>(p.biases + static_cast<size_t>(n0) * groups);
  ad.x = reinterpret_cast<const uint8_t*>(p.x);
#pragma unroll
  for (int t = 0; t < kSubTiles; ++t) {
    const int want = t * 16 + nl;
    const int row = (want < rows_here) ? want : rows_here - 1; // clamp: stay in bounds
    ad.w_lane[t] = static_cast<uint32_t>(row) * row_bytes + kb * S::kLaneBytes;
    ad.sb_lane[t] = static_cast<uint32_t>(row) * groups * 2;
  }
  ad.x_lane = lane * 16;
  const bool x_lane_live = lane < kXLanes;

  Regs regs[PIPE];
  int blk = wave;
#pragma unroll
  for (int i = 0; i < PIPE; ++i) {
    if (blk + i * WAVES < nblk) {
      load_block<BITS, GS, MAXM>(regs[i], ad, blk + i * WAVES, M, K, x_lane_live);
    }
  }

  // Per-wave LDS: this wave's K-block of x (in operand order) and the sums of
  // x over each group of the block.
  const uint32_t wave_bytes = static_cast<uint32_t>(M) * kXsStride * sizeof(T) +
      static_cast<uint32_t>(M) * S::kGroupsPerBlock * 4;
  T* xs = reinterpret_cast<T*>(smem + wave * wave_bytes);
  float* sx = reinterpret_cast<float*>(
      smem + wave * wave_bytes + static_cast<uint32_t>(M) * kXsStride * sizeof(T));

  const Widen4Consts w4c = make_widen4_consts<T>();

  float total[kSubTiles][MR];
  float bias_acc[kSubTiles][BR];
#pragma unroll
  for (int t = 0; t < kSubTiles; ++t) {
#pragma unroll
    for (int i = 0; i < MR; ++i) {
      total[t][i] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < BR; ++i) {
      bias_acc[t][i] = 0.0f;
    }
  }

  // Rows of A beyond M only feed rows of D that are never read, so those
  // lanes may load any valid row.
  const T* xa = xs + static_cast<uint32_t>(nl < M ? nl : 0) * kXsStride + kb * S::kLaneCodes;

  auto process = [&](const Regs& cur) {
    // ---- stage x in operand order, with its group sums ----
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      if (MAXM <= 2 || m < M) {
        const uint4 v = cur.x[m];
        float part = Mma<T>::dot_ones(v.x, 0.0f);
        part = Mma<T>::dot_ones(v.y, part);
        part = Mma<T>::dot_ones(v.z, part);
        part = Mma<T>::dot_ones(v.w, part);
        part = group_sum<LPG>(part);
        if (x_lane_live) {
          if ((lane % LPG) == 0) {
            sx[m * S::kGroupsPerBlock + lane / LPG] = part;
          }
          uint4 o = v;
          if constexpr (BITS == 4) {
            // element order 0,4,1,5,2,6,3,7 (see widen4)
            o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
            o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
            o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
            o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
          }
          *reinterpret_cast<uint4*>(xs + static_cast<uint32_t>(m) * kXsStride + lane * 8) = o;
        }
      }
    }
    wave_lds_sync();

    // ---- consume ----
#pragma unroll
    for (int u = 0; u < kUnitsPerBlock; ++u) {
      floatx4 acc[kSubTiles] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
      for (int d = 0; d < S::kMfmaPerUnit; ++d) {
        const uint4 av = *reinterpret_cast<const uint4*>(xa + u * S::kUnit + d * 8);
#pragma unroll
        for (int t = 0; t < kSubTiles; ++t) {
          uint4 bv;
          if constexpr (BITS == 4) {
            bv = widen4(cur.w[t][u][d], w4c);
          } else {
            bv = Mma<T>::widen8(cur.w[t][u][2 * d], cur.w[t][u][2 * d + 1]);
          }
          acc[t] = Mma<T>::mfma(av, bv, acc[t]);
        }
      }
#pragma unroll
      for (int t = 0; t < kSubTiles; ++t) {
        const float s = packed_elem<T>(cur.s[t], u / S::kUnitsPerGroup);
#pragma unroll
        for (int i = 0; i < MR; ++i) {
          total[t][i] = fmaf(s, acc[t][i], total[t][i]);
        }
      }
    }
    // bias (and the -OFFSET*scale correction) against the group sums of x
#pragma unroll
    for (int g = 0; g < S::kGroupsPerBlock; ++g) {
      float sxv[BR];
#pragma unroll
      for (int i = 0; i < BR; ++i) {
        const int m = 4 * i + kb;
        sxv[i] = (m < M) ? sx[m * S::kGroupsPerBlock + g] : 0.0f;
      }
#pragma unroll
      for (int t = 0; t < kSubTiles; ++t) {
        const float beff =
            fmaf(-kOffset, packed_elem<T>(cur.s[t], g), packed_elem<T>(cur.b[t], g));
#pragma unroll
        for (int i = 0; i < BR; ++i) {
          bias_acc[t][i] = fmaf(beff, sxv[i], bias_acc[t][i]);
        }
      }
    }
    wave_lds_sync(); // the next block overwrites xs / sx
  };

  if constexpr (PIPE == 1) {
    for (; blk < nblk; blk += WAVES) {
      process(regs[0]);
      if (blk + WAVES < nblk) {
        load_block<BITS, GS, MAXM>(regs[0], ad, blk + WAVES, M, K, x_lane_live);
      }
    }
  } else {
    // Ping-pong: while one block is consumed the loads of the block after next
    // are already in flight.
    while (blk < nblk) {
      process(regs[0]);
      if (blk + 2 * WAVES < nblk) {
        load_block<BITS, GS, MAXM>(regs[0], ad, blk + 2 * WAVES, M, K, x_lane_live);
      }
      blk += WAVES;
      if (blk >= nblk) {
        break;
      }
      process(regs[PIPE - 1]);
      if (blk + 2 * WAVES < nblk) {
        load_block<BITS, GS, MAXM>(regs[PIPE - 1], ad, blk + 2 * WAVES, M, K, x_lane_live);
      }
      blk += WAVES;
    }
  }

  // ---- reduce over waves (and the four kb slices of the bias terms) ----
  __syncthreads(); // every wave is done with its staging area
  const int mp = (M + 3) & ~3;
  float* redm = reinterpret_cast<float*>(smem); // [WAVES][mp][32]  MFMA part
  float* redb = redm + WAVES * mp * kTileN;      // [WAVES][mp][32]  bias part
#pragma unroll
  for (int t = 0; t < kSubTiles; ++t) {
#pragma unroll
    for (int i = 0; i < MR; ++i) {
      // D layout of v_mfma_f32_16x16x32: register i of lane (nl, kb) is row
      // 4*kb + i, column nl.
      const int m = 4 * kb + i;
      if (m < M) {
        redm[(wave * mp + m) * kTileN + t * 16 + nl] = total[t][i];
      }
    }
#pragma unroll
    for (int i = 0; i < BR; ++i) {
      const int m = 4 * i + kb;
      if (m < M) {
        redb[(wave * mp + m) * kTileN + t * 16 + nl] = bias_acc[t][i];
      }
    }
  }
  __syncthreads();
  for (int idx = tid; idx < M * kTileN; idx += kThreads) {
    const int m = idx / kTileN;
    const int n = idx - m * kTileN;
    float y = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      y += redm[(w * mp + m) * kTileN + n] + redb[(w * mp + m) * kTileN + n];
    }
    if (n < rows_here) {
      p.out[static_cast<size_t>(m) * N + n0 + n] = from_f32<T>(p.valid ? y : 0.0f);
    }
  }
}

template <int BITS, int GS>
size_t qmv_mfma_smem_bytes(int M, int waves) {
  using S = QmvShape<BITS, GS>;
  const size_t wave_bytes = static_cast<size_t>(M) * (S::kBlockK + 8) * 2 +
      static_cast<size_t>(M) * S::kGroupsPerBlock * 4;
  const int mp = (M + 3) & ~3;
  const size_t red_bytes = static_cast<size_t>(2) * waves * mp * kTileN * 4;
  const size_t stage = wave_bytes * waves;
  return stage > red_bytes ? stage : red_bytes;
}

} // namespace

bool qmv_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  if (dtype == MLXROCM_FLOAT32 || !(bits == 4 || bits == 8)) {
    return false;
  }
  if (a.M > 8 || a.M < 1) {
    return false;
  }
  const int unit = gs < 64 ? gs : 64;
  if (a.K % (unit * kUnitsPerBlock) != 0) {
    return false;
  }
  // 32-bit lane offsets inside a 32-row tile
  if (static_cast<int64_t>(a.K) * bits / 8 * kTileN >= (int64_t{1} << 31)) {
    return false;
  }
  // vector loads of a block's scales / biases need whole-block alignment
  return a.sb_batch_stride % 8 == 0;
}

int launch_qmv_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const dim3 grid((a.N + kTileN - 1) / kTileN, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] batch=%d exceeds the grid", a.L);
  }
  MLXROCM_REHEARSE("qmv_mfma");
  auto run = [&](auto tval, auto bval, auto gval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    constexpr int W = 8;
    const size_t smem = qmv_mfma_smem_bytes<B, G>(a.M, W);
    const int nblk = a.K / QmvShape<B, G>::kBlockK;
    auto go = [&](auto maxm, auto pipe) -> int {
      constexpr int MAXM = decltype(maxm)::value;
      constexpr int PIPE = decltype(pipe)::value;
      auto kern = qmv_mfma_kernel<T, B, G, MAXM, W, PIPE>;
      if (smem > 48 * 1024) {
        MLXROCM_HIP_TRY(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern),
            hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(smem)));
      }
      kern<<<grid, W * 64, smem, s>>>(a);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    };
    auto by_pipe = [&](auto maxm) -> int {
      // one register set when every wave has at most one K-block
      return nblk <= W ? go(maxm, IntC<1>{}) : go(maxm, IntC<2>{});
    };
    if (a.M == 1) {
      return by_pipe(IntC<1>{});
    } else if (a.M == 2) {
      return by_pipe(IntC<2>{});
    } else if (a.M <= 4) {
      return by_pipe(IntC<4>{});
    }
    return by_pipe(IntC<8>{});
  };
  auto by_group = [&](auto tval, auto bval) -> int {
    switch (gs) {
      case 32:
        return run(tval, bval, IntC<32>{});
      case 64:
        return run(tval, bval, IntC<64>{});
      default:
        return run(tval, bval, IntC<128>{});
    }
  };
  auto by_bits = [&](auto tval) -> int {
    return bits == 4 ? by_group(tval, IntC<4>{}) : by_group(tval, IntC<8>{});
  };
  return dtype == MLXROCM_BFLOAT16 ? by_bits(bf16_t{}) : by_bits(f16_t{});
}

} // namespace mlxrocm
