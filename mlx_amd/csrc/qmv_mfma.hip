// qmv_mfma.hip -- decode GEMV (transpose=true, M <= 16) for 16-bit element
// types and 4/8-bit codes, written for gfx950.
//
// The kernel is an HBM streaming kernel: every packed weight, scale and bias is
// read exactly once, in 16-byte lane loads that are all issued before the first
// one is consumed.  The arithmetic rides on the matrix cores so that the vector
// ALU only has to widen codes:
//
//   * A wavefront owns 32 output rows.  Lane (n = lane % 32, kb = lane / 32)
//     loads the codes of row n; the two kb halves together hold one "unit" of
//     U consecutive codes (one quantization group, or a slice of one).
//   * Codes become MFMA B operands without arithmetic: a 4-bit code c is OR-ed
//     into the mantissa of the constant 128.0 (bf16) / 1024.0 (f16), giving
//     exactly OFFSET + c; 8-bit codes are converted with cvt_f32_ubyte (bf16) or
//     a byte permute into 1024.0 (f16).
//   * x is the MFMA A operand (rows = the M <= 16 rows of x, zero padded to 32),
//     staged once per workgroup in LDS in the k-order the code expansion
//     produces.  v_mfma_f32_32x32x16 then yields, per unit and per lane,
//     P[m][n] = sum_k x[m][k] * (OFFSET + c[n][k]) in fp32.
//   * y[m][n] = sum_g scale[n][g] * P_g[m][n] + (bias[n][g] - OFFSET*scale[n][g])
//     * sum_{k in g} x[m][k]; the group sums of x are computed while staging.
//
// A workgroup of W wavefronts covers all of K for its 32 rows (wave w takes the
// K-blocks w, w+W, ...) and reduces the partial results through LDS.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTileN = 32;       // output rows per workgroup
constexpr int kUnitsPerBlock = 8; // units a wave loads at once

template <typename T>
struct Mma;

template <>
struct Mma<bf16_t> {
  static constexpr uint32_t kMagic4 = 0x43004300u; // 128.0 | 128.0
  static constexpr float kOffset4 = 128.0f;
  static constexpr float kOffset8 = 0.0f;
  static __device__ __forceinline__ floatx16
  mfma(const uint4& a, const uint4& b, const floatx16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
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
};

template <>
struct Mma<f16_t> {
  static constexpr uint32_t kMagic4 = 0x64006400u; // 1024.0 | 1024.0
  static constexpr float kOffset4 = 1024.0f;
  static constexpr float kOffset8 = 1024.0f;
  static __device__ __forceinline__ floatx16
  mfma(const uint4& a, const uint4& b, const floatx16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
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
};

// One dword of eight 4-bit codes -> 8 values OFFSET + c.  Register j of the
// result holds codes (j, j + 4), so the matching x order is 0,4,1,5,2,6,3,7.
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
  // codes held by one lane pair per load
  static constexpr int kUnit = (BITS == 4) ? (GS >= 64 ? 64 : 32) : 32;
  static constexpr int kLaneBytes = kUnit / 2 * BITS / 8; // 16 or 8
  static constexpr int kLaneWords = kLaneBytes / 4;
  static constexpr int kMfmaPerUnit = kUnit / 16;
  static constexpr int kBlockK = kUnit * kUnitsPerBlock;
  static constexpr int kGroupsPerBlock = kBlockK / GS; // 2, 4 or 8
  static constexpr int kUnitsPerGroup = GS / kUnit;    // 1, 2 or 4
  static_assert(kGroupsPerBlock >= 2 && kUnitsPerGroup >= 1, "shape");
};

template <int BITS, int GS>
struct BlockRegs {
  using S = QmvShape<BITS, GS>;
  uint32_t w[kUnitsPerBlock][S::kLaneWords];
  uint16_t s[S::kGroupsPerBlock];
  uint16_t b[S::kGroupsPerBlock];
};

template <int N>
__device__ __forceinline__ void load_u16xN(const void* p, uint16_t (&out)[N]) {
  static_assert(N == 2 || N == 4 || N == 8, "");
  if constexpr (N == 8) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    out[0] = v.x & 0xffff; out[1] = v.x >> 16;
    out[2] = v.y & 0xffff; out[3] = v.y >> 16;
    out[4] = v.z & 0xffff; out[5] = v.z >> 16;
    out[6] = v.w & 0xffff; out[7] = v.w >> 16;
  } else if constexpr (N == 4) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    out[0] = v.x & 0xffff; out[1] = v.x >> 16;
    out[2] = v.y & 0xffff; out[3] = v.y >> 16;
  } else {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(p);
    out[0] = v & 0xffff; out[1] = v >> 16;
  }
}

template <typename T>
__device__ __forceinline__ float half_bits_to_f32(uint16_t h) {
  if constexpr (sizeof(T) == 2 && __is_same(T, bf16_t)) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
  } else {
    return static_cast<float>(__builtin_bit_cast(f16_t, h));
  }
}

template <int BITS, int GS>
__device__ __forceinline__ void load_block(
    BlockRegs<BITS, GS>& r,
    const uint8_t* wrow, // row start + kb * kLaneBytes
    const uint16_t* srow,
    const uint16_t* brow,
    int blk) {
  using S = QmvShape<BITS, GS>;
  constexpr int unit_bytes = S::kUnit * BITS / 8;
  const uint8_t* p = wrow + static_cast<size_t>(blk) * kUnitsPerBlock * unit_bytes;
#pragma unroll
  for (int u = 0; u < kUnitsPerBlock; ++u) {
    if constexpr (S::kLaneWords == 4) {
      const uint4 v = *reinterpret_cast<const uint4*>(p + u * unit_bytes);
      r.w[u][0] = v.x; r.w[u][1] = v.y; r.w[u][2] = v.z; r.w[u][3] = v.w;
    } else {
      const uint2 v = *reinterpret_cast<const uint2*>(p + u * unit_bytes);
      r.w[u][0] = v.x; r.w[u][1] = v.y;
    }
  }
  load_u16xN<S::kGroupsPerBlock>(srow + blk * S::kGroupsPerBlock, r.s);
  load_u16xN<S::kGroupsPerBlock>(brow + blk * S::kGroupsPerBlock, r.b);
}

// Orders one wavefront's LDS writes before its later LDS reads (the lanes of
// a wavefront run in lockstep; only the memory ordering has to be stated).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// MR: accumulator registers that can hold a real row of x (1, 2, 4 or 8);
// MAXM: the largest M this instantiation accepts.
template <typename T, int BITS, int GS, int MR, int MAXM, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void qmv_mfma_kernel(const QmmArgs a) {
  using S = QmvShape<BITS, GS>;
  constexpr int kThreads = WAVES * 64;
  constexpr float kOffset = (BITS == 4) ? Mma<T>::kOffset4 : Mma<T>::kOffset8;
  constexpr int kXsStride = S::kBlockK + 8; // elements: 16-byte rows, skewed banks
  constexpr int kXLanes = S::kBlockK / 8;   // lanes that carry 8 elements of x
  constexpr int LPG = GS / 8;               // lanes per group while staging x
  constexpr int BR = (MAXM + 1) / 2;        // bias rows per lane: m = 2*i + kb

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int nl = lane & 31;
  const int kb = lane >> 5;
  const int M = a.M;
  const int K = a.K;
  const int N = a.N;
  const int n0 = blockIdx.x * kTileN;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  const int groups = K / GS;
  const int nblk = K / S::kBlockK;

  // Per-wave LDS: this wave's K-block of x (in operand order) and the sums of
  // x over each group of the block.
  const size_t wave_bytes =
      static_cast<size_t>(M) * kXsStride * sizeof(T) + static_cast<size_t>(M) * S::kGroupsPerBlock * 4;
  T* xs = reinterpret_cast<T*>(smem + wave * wave_bytes);
  float* sx = reinterpret_cast<float*>(
      smem + wave * wave_bytes + static_cast<size_t>(M) * kXsStride * sizeof(T));

  const int n_row = (n0 + nl < N) ? n0 + nl : N - 1; // clamp: loads stay in bounds
  const uint8_t* wrow =
      p.w + static_cast<size_t>(n_row) * (K / 8) * BITS + kb * S::kLaneBytes;
  const uint16_t* srow =
      reinterpret_cast<const uint16_t*>(p.scales) + static_cast<size_t>(n_row) * groups;
  const uint16_t* brow =
      reinterpret_cast<const uint16_t*>(p.biases) + static_cast<size_t>(n_row) * groups;

  const Widen4Consts w4c = make_widen4_consts<T>();

  float total[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    total[r] = 0.0f;
  }
  float bias_acc[BR];
#pragma unroll
  for (int i = 0; i < BR; ++i) {
    bias_acc[i] = 0.0f;
  }

  // Rows of A beyond M only feed rows of D that are never read, so those
  // lanes may load any valid row.
  const T* xa = xs + static_cast<size_t>(nl < M ? nl : 0) * kXsStride + kb * (S::kUnit / 2);

  for (int blk = wave; blk < nblk; blk += WAVES) {
    const int k_blk = blk * S::kBlockK;
    // ---- x first (it must not queue behind the weight stream) ----
    uint4 xv[MAXM];
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      xv[m] = make_uint4(0, 0, 0, 0);
      if (m < M && lane < kXLanes) {
        xv[m] = *reinterpret_cast<const uint4*>(
            p.x + static_cast<size_t>(m) * K + k_blk + lane * 8);
      }
    }
    // ---- then every weight, scale and bias of the block ----
    BlockRegs<BITS, GS> cur;
    load_block<BITS, GS>(cur, wrow, srow, brow, blk);

    // ---- stage x in operand order, with its group sums ----
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      if (m < M) {
        union {
          uint4 u;
          T e[8];
        } raw;
        raw.u = xv[m];
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          part += to_f32(raw.e[i]);
        }
#pragma unroll
        for (int off = LPG / 2; off > 0; off >>= 1) {
          part += __shfl_xor(part, off, 64);
        }
        if (lane < kXLanes) {
          if ((lane % LPG) == 0) {
            sx[m * S::kGroupsPerBlock + lane / LPG] = part;
          }
          const uint4 v = xv[m];
          uint4 o = v;
          if constexpr (BITS == 4) {
            // element order 0,4,1,5,2,6,3,7 (see widen4)
            o.x = (v.x & 0xffffu) | (v.z << 16);
            o.y = (v.x >> 16) | (v.z & 0xffff0000u);
            o.z = (v.y & 0xffffu) | (v.w << 16);
            o.w = (v.y >> 16) | (v.w & 0xffff0000u);
          }
          *reinterpret_cast<uint4*>(xs + static_cast<size_t>(m) * kXsStride + lane * 8) = o;
        }
      }
    }
    wave_lds_sync();

    // ---- consume ----
    float sc[S::kGroupsPerBlock];
#pragma unroll
    for (int g = 0; g < S::kGroupsPerBlock; ++g) {
      sc[g] = half_bits_to_f32<T>(cur.s[g]);
    }
#pragma unroll
    for (int u = 0; u < kUnitsPerBlock; ++u) {
      floatx16 acc = {0};
#pragma unroll
      for (int d = 0; d < S::kMfmaPerUnit; ++d) {
        const uint4 av = *reinterpret_cast<const uint4*>(xa + u * S::kUnit + d * 8);
        uint4 bv;
        if constexpr (BITS == 4) {
          bv = widen4(cur.w[u][d], w4c);
        } else {
          bv = Mma<T>::widen8(cur.w[u][2 * d], cur.w[u][2 * d + 1]);
        }
        acc = Mma<T>::mfma(av, bv, acc);
      }
      const float s = sc[u / S::kUnitsPerGroup];
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        total[r] = fmaf(s, acc[r], total[r]);
      }
    }
    // bias (and the -OFFSET*scale correction) against the group sums of x
#pragma unroll
    for (int g = 0; g < S::kGroupsPerBlock; ++g) {
      const float beff = fmaf(-kOffset, sc[g], half_bits_to_f32<T>(cur.b[g]));
#pragma unroll
      for (int i = 0; i < BR; ++i) {
        const int m = 2 * i + kb;
        if (m < M) {
          bias_acc[i] = fmaf(beff, sx[m * S::kGroupsPerBlock + g], bias_acc[i]);
        }
      }
    }
    wave_lds_sync(); // the next block overwrites xs / sx
  }

  // ---- reduce over waves (and the two kb halves of the bias terms) ----
  __syncthreads(); // every wave is done with its staging area
  const int mp = (M + 1) & ~1;
  float* redm = reinterpret_cast<float*>(smem); // [WAVES][mp][32]  MFMA part
  float* redb = redm + WAVES * mp * kTileN;      // [WAVES][mp][32]  bias part
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    // D layout of v_mfma_f32_32x32x16: register r of lane (nl, kb) is row
    // 8*(r/4) + 4*kb + r%4, column nl.
    const int m = 8 * (r / 4) + 4 * kb + (r % 4);
    if (m < M) {
      redm[(wave * mp + m) * kTileN + nl] = total[r];
    }
  }
#pragma unroll
  for (int i = 0; i < BR; ++i) {
    const int m = 2 * i + kb;
    if (m < M) {
      redb[(wave * mp + m) * kTileN + nl] = bias_acc[i];
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
    if (n0 + n < N) {
      p.out[static_cast<size_t>(m) * N + n0 + n] = from_f32<T>(p.valid ? y : 0.0f);
    }
  }
}

template <int BITS, int GS>
size_t qmv_mfma_smem_bytes(int M, int waves) {
  using S = QmvShape<BITS, GS>;
  const size_t wave_bytes = static_cast<size_t>(M) * (S::kBlockK + 8) * 2 +
      static_cast<size_t>(M) * S::kGroupsPerBlock * 4;
  const int mp = (M + 1) & ~1;
  const size_t red_bytes = static_cast<size_t>(2) * waves * mp * kTileN * 4;
  const size_t stage = wave_bytes * waves;
  return stage > red_bytes ? stage : red_bytes;
}

} // namespace

bool qmv_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  if (dtype == MLXROCM_FLOAT32 || !(bits == 4 || bits == 8)) {
    return false;
  }
  if (a.M > 16 || a.M < 1) {
    return false;
  }
  const int unit = (bits == 4) ? (gs >= 64 ? 64 : 32) : 32;
  if (a.K % (unit * kUnitsPerBlock) != 0) {
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
  auto run = [&](auto tval, auto bval, auto gval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    constexpr int W = 8;
    const size_t smem = qmv_mfma_smem_bytes<B, G>(a.M, W);
    auto go = [&](auto mr, auto maxm) -> int {
      constexpr int MR = decltype(mr)::value;
      constexpr int MAXM = decltype(maxm)::value;
      auto kern = qmv_mfma_kernel<T, B, G, MR, MAXM, W>;
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
    if (a.M == 1) {
      return go(IntC<1>{}, IntC<1>{});
    } else if (a.M == 2) {
      return go(IntC<2>{}, IntC<2>{});
    } else if (a.M <= 4) {
      return go(IntC<4>{}, IntC<4>{});
    } else if (a.M <= 8) {
      return go(IntC<4>{}, IntC<8>{});
    }
    return go(IntC<8>{}, IntC<16>{});
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
