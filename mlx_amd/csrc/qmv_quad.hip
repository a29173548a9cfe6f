// qmv_quad.hip -- decode GEMV (transpose=true) for 1..8 rows of x, 16-bit element
// types, 4/8-bit codes, on the 4x4x4 matrix instruction of gfx950.
//
// v_mfma_f32_4x4x4_16b computes 16 independent 4x4 products per wavefront: lane
// (blk, i) = (l / 4, l % 4) supplies row i of block blk's A (4 values along k)
// and column i of its B, and receives column i of D (register t = row t, i.e.
// the product of A's row t with this lane's B column -- measured on gfx950).
// Here a block is a slice of k and the instruction is used as 16 small dot
// engines:
//   B  = four consecutive rows of W: lane (blk, i) holds 16 bytes of packed
//        codes of row r0 + i, the 32 (4-bit) or 16 (8-bit) codes at
//        k = slot * S + blk * 32|16.  One load instruction therefore reads 256
//        contiguous bytes from each of four rows: whole lines only.
//   A  = x: lane (blk, j) holds the same k slice of row j of x (rows 4..7 in a
//        second operand set), kept in registers for the whole kernel.
//   D  = lane (blk, i) ends up with the partial dot products of W row r0 + i
//        with up to four rows of x -- in the lane that also fetched that row's
//        scale and bias, so the affine part is applied without any exchange:
//        y += s * D + (b - OFFSET * s) * sum(x), once per 16-byte load (a lane's
//        codes never straddle a quantization group).
// Codes are widened without arithmetic (4-bit: OR-ed into the mantissa of 128.0
// / 1024.0, which pairs codes (j, j + 4): x is held in the matching order
// 0,4,1,5 | 2,6,3,7), so the vector ALU spends ~1 instruction per code
// regardless of the number of rows of x; the multiplies run on the matrix
// pipe.  K is split over KW wavefronts of a workgroup (S slots of 512 | 256
// codes each), rows over the other 8 / KW; the 16 block partials are added with
// lane permutes and the KW partials through LDS.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

template <typename T>
struct Quad;

template <>
struct Quad<bf16_t> {
  static constexpr uint32_t kMagic4 = 0x43004300u; // 128.0 | 128.0
  static constexpr float kOffset4 = 128.0f;
  static constexpr float kOffset8 = 0.0f;
  static constexpr uint32_t kOnes = 0x3f803f80u;
  static __device__ __forceinline__ float4_t mfma(uint2 a, uint2 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
        __builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
  }
  // 4 bytes -> 4 bf16 (0..255 are exact), natural order
  static __device__ __forceinline__ uint2 widen8(uint32_t w) {
    union {
      bf16_t h[4];
      uint2 u;
    } r;
    r.h[0] = static_cast<bf16_t>(static_cast<float>(w & 0xffu));
    r.h[1] = static_cast<bf16_t>(static_cast<float>((w >> 8) & 0xffu));
    r.h[2] = static_cast<bf16_t>(static_cast<float>((w >> 16) & 0xffu));
    r.h[3] = static_cast<bf16_t>(static_cast<float>(w >> 24));
    return r.u;
  }
};

template <>
struct Quad<f16_t> {
  static constexpr uint32_t kMagic4 = 0x64006400u; // 1024.0 | 1024.0
  static constexpr float kOffset4 = 1024.0f;
  static constexpr float kOffset8 = 1024.0f;
  static constexpr uint32_t kOnes = 0x3c003c00u;
  static __device__ __forceinline__ float4_t mfma(uint2 a, uint2 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(
        __builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
  }
  // byte c -> f16 bits 0x64cc = 1024 + c
  static __device__ __forceinline__ uint2 widen8(uint32_t w) {
    constexpr uint32_t hi = 0x64646464u;
    return make_uint2(
        __builtin_amdgcn_perm(hi, w, 0x04010400u), __builtin_amdgcn_perm(hi, w, 0x04030402u));
  }
};

// 16-byte load of data that is read exactly once.
__device__ __forceinline__ uint4 load_once(const uint8_t* p) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// v of lane l + v of lane l ^ mask (mask 16 or 32): through the LDS crossbar.
__device__ __forceinline__ float add_xor_lane(float v, int lane, int mask) {
  const int other = __builtin_amdgcn_ds_bpermute((lane ^ mask) * 4, __builtin_bit_cast(int, v));
  return v + __builtin_bit_cast(float, other);
}

// Sum over the 16 blocks: lanes with the same l % 4.  Valid in every lane.
__device__ __forceinline__ float sum_blocks(float v, int lane) {
  // inside a row of 16 lanes: rotate by 4 and by 8
  int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false);
  v += __builtin_bit_cast(float, t); // row_ror:4
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false);
  v += __builtin_bit_cast(float, t); // row_ror:8
  v = add_xor_lane(v, lane, 16);
  v = add_xor_lane(v, lane, 32);
  return v;
}


// MB: operand sets of x (rows 0..3, 4..7).  S: slots (one 16-byte load per lane
// each) of K per wavefront.  KW: wavefronts that split K.
// XLDS: x reaches the lanes through one coalesced read per workgroup and LDS
// (4 MB K elements of LDS); otherwise every lane fetches its slices itself.
// MC: columns of an operand set that are live (rows of x: M = 1, 2, or more).
// QPW: row quads per wave, whose loads are in flight together.
template <typename T, int BITS, int MB, int S, int KW, int kSbLoads, bool XLDS, int MC, int QPW>
__global__ __launch_bounds__(512) void qmv_quad_kernel(const QmmArgs a, const int gs_shift) {
  constexpr int kQuadsPerWave = QPW;
  constexpr int RW = 8 / KW;
  constexpr int kLaneCodes = 128 / BITS;      // codes in a lane's 16 bytes
  constexpr int kSlotCodes = 16 * kLaneCodes; // 512 or 256 codes of k per load instruction
  constexpr int kSteps = kLaneCodes / 4;      // matrix instructions per load
  constexpr float kOffset = (BITS == 4) ? Quad<T>::kOffset4 : Quad<T>::kOffset8;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kw = wave % KW;
  const int rw = wave / KW;
  const int blk = lane >> 2;
  const int i = lane & 3;
  const int K = a.K;
  const int N = a.N;
  const int M = a.M;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);
  const int groups = K >> gs_shift;
  const uint32_t row_bytes = static_cast<uint32_t>(K / 8) * BITS;
  const int nslots = K / kSlotCodes; // K is a multiple of the slot size

  // ---- x: raw loads first.  XLDS: the workgroup's threads share out the rows
  // of x in 16-byte units; else this lane's own slices of row i (and 4 + i) ----
  constexpr int kXU = kLaneCodes / 8; // 16-byte pieces per slice
  constexpr int kXRaw = XLDS ? 4 * MB : MB * S * kXU;
  uint4 xraw[kXRaw];
  bool xlive[MB][S];
  const int units_per_row = K / 8;
  const int x_units = M * units_per_row;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int c = 0; c < S; ++c) {
      xlive[mb][c] = 4 * mb + i < M && kw * S + c < nslots;
    }
  }
  if constexpr (XLDS) {
#pragma unroll
    for (int n = 0; n < kXRaw; ++n) {
      const int idx = tid + n * 512;
      xraw[n] = make_uint4(0, 0, 0, 0);
      if (idx < x_units) {
        xraw[n] = *reinterpret_cast<const uint4*>(p.x + static_cast<size_t>(idx) * 8);
      }
    }
  } else {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int c = 0; c < S; ++c) {
        const bool live = xlive[mb][c];
        const T* src = p.x + static_cast<size_t>(live ? 4 * mb + i : 0) * K +
            (live ? kw * S + c : 0) * kSlotCodes + blk * kLaneCodes;
#pragma unroll
        for (int u = 0; u < kXU; ++u) {
          xraw[(mb * S + c) * kXU + u] = *reinterpret_cast<const uint4*>(src + 8 * u);
        }
      }
    }
  }
  // ---- rows: kQuadsPerWave quads of four, every load issued right behind the x
  // loads (loads return in order: x first, and its setup overlaps the rest) ----
  const int quad0 = (blockIdx.x * RW + rw) * kQuadsPerWave;
  uint4 wv[kQuadsPerWave][S];
  // Scales and biases: the groups of this wave's k range are fetched as dwords
  // (two 16-bit values each), lane (blk, i) taking word blk % 8 of row i's
  // scales (blk < 8) or biases (blk >= 8), kSbLoads words apart per load; the
  // lane that needs a value picks it from its owner with ds_bpermute.
  uint32_t sbw[kQuadsPerWave][kSbLoads];
  const int g_first = (kw * S * kSlotCodes) >> gs_shift; // first group of this wave
  {
    const int wd = blk & 7;
    const T* sb_base = blk < 8 ? p.scales : p.biases;
#pragma unroll
    for (int q = 0; q < kQuadsPerWave; ++q) {
      const int r = (quad0 + q) * 4 + i;
      const int row = r < N ? r : N - 1; // clamp: stay in bounds
#pragma unroll
      for (int t = 0; t < kSbLoads; ++t) {
        int g = g_first + 2 * (8 * t + wd);
        g = g + 1 < groups ? g : groups - 2; // clamp: a valid word nobody reads
        sbw[q][t] = *reinterpret_cast<const uint32_t*>(
            sb_base + static_cast<size_t>(row) * groups + g);
      }
    }
  }
#pragma unroll
  for (int q = 0; q < kQuadsPerWave; ++q) {
    const int r = (quad0 + q) * 4 + i;
    const int row = r < N ? r : N - 1;
    const uint8_t* wrow = p.w + static_cast<size_t>(row) * row_bytes;
#pragma unroll
    for (int c = 0; c < S; ++c) {
      const int slot = kw * S + c;
      const int sl = slot < nslots ? slot : nslots - 1; // x is zero there
      wv[q][c] = load_once(wrow + static_cast<uint32_t>(sl) * (kSlotCodes / 8 * BITS) + blk * 16);
    }
  }

  // ---- x into the operand order ----
  // LDS image (XLDS): piece u of slice (slot, mb) of lane l at
  // (((slot MB + mb) kXU + u) 64 + l) 16, so that a wave reads whole KiB.
  if constexpr (XLDS) {
    for (int n = 0; n < kXRaw; ++n) {
      const int idx = tid + n * 512;
      if (idx < x_units) {
        const int m = idx / units_per_row;
        const int k = (idx - m * units_per_row) * 8;
        const int slot = k / kSlotCodes;
        const int b = (k % kSlotCodes) / kLaneCodes;
        const int u = (k % kLaneCodes) / 8;
        const uint32_t pos =
            (((slot * MB + (m >> 2)) * kXU + u) * 64 + (b * 4 + (m & 3))) * 16;
        *reinterpret_cast<uint4*>(smem + pos) = xraw[n];
      }
    }
    __syncthreads();
  }
  uint2 xr[MB][S][kSteps];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int c = 0; c < S; ++c) {
#pragma unroll
      for (int u = 0; u < kXU; ++u) {
        uint4 v;
        if constexpr (XLDS) {
          v = make_uint4(0, 0, 0, 0);
          if (xlive[mb][c]) {
            v = *reinterpret_cast<const uint4*>(
                smem + ((((kw * S + c) * MB + mb) * kXU + u) * 64 + lane) * 16);
          }
        } else {
          v = xraw[(mb * S + c) * kXU + u];
          if (!xlive[mb][c]) {
            v = make_uint4(0, 0, 0, 0);
          }
        }
        if constexpr (BITS == 4) {
          // elements 0..7 -> (0,4,1,5) and (2,6,3,7): the pairs the 4-bit
          // expansion produces from one word
          xr[mb][c][2 * u].x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
          xr[mb][c][2 * u].y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
          xr[mb][c][2 * u + 1].x = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
          xr[mb][c][2 * u + 1].y = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
        } else {
          xr[mb][c][2 * u] = make_uint2(v.x, v.y);
          xr[mb][c][2 * u + 1] = make_uint2(v.z, v.w);
        }
      }
    }
  }
  // sum of x over each slice: one pass with B = ones leaves, in every lane of a
  // block, the sums of that block's slice of rows 0..3 of x
  float4_t sx[MB][S];
  {
    const uint2 ones = make_uint2(Quad<T>::kOnes, Quad<T>::kOnes);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int c = 0; c < S; ++c) {
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < kSteps; ++t) {
          acc = Quad<T>::mfma(xr[mb][c][t], ones, acc);
        }
        sx[mb][c] = acc;
      }
    }
  }

  uint32_t mask4 = 0x000f000fu;
  uint32_t magic4 = Quad<T>::kMagic4;
  asm volatile("" : "+s"(mask4));
  asm volatile("" : "+v"(magic4));

  float y[kQuadsPerWave][MB][4];
#pragma unroll
  for (int q = 0; q < kQuadsPerWave; ++q) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int j = 0; j < MC; ++j) {
        y[q][mb][j] = 0.0f;
      }
    }
#pragma unroll
    for (int c = 0; c < S; ++c) {
      const uint32_t w[4] = {wv[q][c].x, wv[q][c].y, wv[q][c].z, wv[q][c].w};
      float4_t d[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        d[mb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        uint2 a0, a1;
        if constexpr (BITS == 4) {
          a0.x = (w[u] & mask4) | magic4;         // codes (0, 4)
          a0.y = ((w[u] >> 4) & mask4) | magic4;  // codes (1, 5)
          a1.x = ((w[u] >> 8) & mask4) | magic4;  // codes (2, 6)
          a1.y = ((w[u] >> 12) & mask4) | magic4; // codes (3, 7)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            d[mb] = Quad<T>::mfma(xr[mb][c][2 * u], a0, d[mb]);
            d[mb] = Quad<T>::mfma(xr[mb][c][2 * u + 1], a1, d[mb]);
          }
        } else {
          a0 = Quad<T>::widen8(w[u]);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            d[mb] = Quad<T>::mfma(xr[mb][c][u], a0, d[mb]);
          }
        }
      }
      // group of this lane's codes, relative to the wave's first group
      const int gl = ((c * kSlotCodes + blk * kLaneCodes) >> gs_shift);
      const int word = gl >> 1;
      const int t_sel = word >> 3; // which of the kSbLoads words
      uint32_t mine = sbw[q][0];
#pragma unroll
      for (int t = 1; t < kSbLoads; ++t) {
        mine = t_sel == t ? sbw[q][t] : mine;
      }
      const int owner = ((word & 7) * 4 + i) * 4; // byte address of lane (word % 8, i)
      const uint32_t s_word =
          static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(owner, static_cast<int>(mine)));
      const uint32_t b_word = static_cast<uint32_t>(
          __builtin_amdgcn_ds_bpermute(owner + 32 * 4, static_cast<int>(mine)));
      const int sh = (gl & 1) * 16;
      const float s = to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(s_word >> sh)));
      const float beff =
          fmaf(-kOffset, s, to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(b_word >> sh))));
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
        for (int j = 0; j < MC; ++j) {
          y[q][mb][j] = fmaf(s, d[mb][j], y[q][mb][j]);
          y[q][mb][j] = fmaf(beff, sx[mb][c][j], y[q][mb][j]);
        }
      }
    }
  }

  // ---- blocks -> rows (every lane), then k-waves -> output ----
#pragma unroll
  for (int q = 0; q < kQuadsPerWave; ++q) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int j = 0; j < MC; ++j) {
        y[q][mb][j] = sum_blocks(y[q][mb][j], lane);
      }
    }
  }
  // partial sums [RW][KW][quads][MB * 4 (m)][4 (row)], behind the x image
  float* red = reinterpret_cast<float*>(
      smem + (XLDS ? static_cast<size_t>(4 * MB) * K * sizeof(T) : 0));
  if (lane < 4) {
#pragma unroll
    for (int q = 0; q < kQuadsPerWave; ++q) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
        for (int j = 0; j < MC; ++j) {
          red[(((rw * KW + kw) * kQuadsPerWave + q) * (MB * 4) + mb * 4 + j) * 4 + lane] =
              y[q][mb][j];
        }
      }
    }
  }
  __syncthreads();
  constexpr int kOutputs = RW * kQuadsPerWave * MB * 4 * 4; // up to 1024
#pragma unroll
  for (int o = tid; o < kOutputs; o += 512) {
    const int ri = o & 3;
    const int m = (o >> 2) % (MB * 4);
    const int q = (o / (4 * MB * 4)) % kQuadsPerWave;
    const int w = o / (4 * MB * 4 * kQuadsPerWave);
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < KW; ++k) {
      total += red[(((w * KW + k) * kQuadsPerWave + q) * (MB * 4) + m) * 4 + ri];
    }
    const int row = ((blockIdx.x * RW + w) * kQuadsPerWave + q) * 4 + ri;
    if (row < N && m < M) {
      p.out[static_cast<size_t>(m) * N + row] = from_f32<T>(p.valid ? total : 0.0f);
    }
  }
}

struct QuadPlan {
  int kw; // 0: not covered
  int s;
};

QuadPlan quad_plan(int K, int bits, int M = 1) {
  const int slot_codes = 16 * (128 / bits);
  QuadPlan pl{0, 0};
  if (K % slot_codes != 0) {
    return pl;
  }
  const int need = K / slot_codes;
  if (M > 4 && need >= 8 && need <= 32) {
    // two operand sets of x: all eight wavefronts split K, so that a wave holds
    // as few slices of x as possible (registers decide the occupancy here)
    const int s8 = (need + 7) / 8;
    pl.kw = 8;
    pl.s = s8 == 3 ? 4 : s8;
    return pl;
  }
  // as many k-waves as keep at most 4 slots per wave; few slots per wave keep x
  // in few registers
  for (int kw = 1; kw <= 8; kw *= 2) {
    const int s = (need + kw - 1) / kw;
    if (s <= 4 && (s <= 2 || kw == 8)) {
      pl.kw = kw;
      pl.s = s == 3 ? 4 : s;
      return pl;
    }
  }
  return pl;
}

} // namespace

bool qmv_quad_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  (void)gs;
  // the kernel is written for 4- and 8-bit codes; only 4-bit is dispatched: at
  // 8 bits the widening of the codes costs what the matrix instruction saves
  if (dtype == MLXROCM_FLOAT32 || bits != 4) {
    return false;
  }
  if (a.M < 1 || a.M > 8) {
    return false;
  }
  // scale / bias words are fetched as aligned dwords
  if ((a.K / gs) % 2 != 0 || a.sb_batch_stride % 2 != 0) {
    return false;
  }
  return quad_plan(a.K, bits).kw != 0;
}

// Workgroups of a launch with 5..8 rows of x (two operand sets: one workgroup
// per compute unit at a time, so the launch runs in rounds of that many).
long qmv_quad_workgroups_two_sets(const QmmArgs& a, int bits) {
  const QuadPlan pl = quad_plan(a.K, bits, 8);
  if (pl.kw == 0) {
    return 0;
  }
  const int rows_per_wg = (8 / pl.kw) * 4 * 4;
  return static_cast<long>((a.N + rows_per_wg - 1) / rows_per_wg) * a.L;
}

int launch_qmv_quad(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  const QuadPlan pl = quad_plan(a.K, bits, a.M);
  if (pl.kw == 0) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] K=%d is not covered by the quad kernel", a.K);
  }
  MLXROCM_REHEARSE("qmv_quad(kw=%d,sets=%d)", pl.kw, a.M <= 4 ? 1 : 2);
  const int gs_shift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  const int rw = 8 / pl.kw;
  const int mb = a.M <= 4 ? 1 : 2;
  const size_t x_bytes = static_cast<size_t>(4 * mb) * a.K * 2;
  // x through LDS while a few workgroups still fit a compute unit
  const bool xlds = x_bytes + 8 * 4 * mb * 16 * sizeof(float) <= 64 * 1024 &&
      static_cast<size_t>(a.M) * (a.K / 8) <= static_cast<size_t>(4 * mb) * 512;
  // Row quads per wave: four keep the most loads in flight, but a small N then
  // leaves compute units without a workgroup.  Measured at K = 4096 (two
  // row-waves): 1024 rows 5.6 -> 3.4 us, 4096 rows 6.2 -> 4.7, 11008 rows
  // 9.3 -> 8.1 with fewer quads; from ~1.5 workgroups per unit on four quads win.
  int qpw = 4;
  if (mb == 1 && xlds && pl.kw <= 4) {
    const long want = compute_units() * 3L / 2;
    while (qpw > 1 && static_cast<long>((a.N + rw * qpw * 4 - 1) / (rw * qpw * 4)) * a.L < want) {
      qpw /= 2;
    }
  }
  const int rows_per_wg = rw * qpw * 4;
  const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, a.L);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] batch=%d exceeds the grid", a.L);
  }
  const size_t red_bytes = static_cast<size_t>(8) * qpw * mb * 16 * sizeof(float);
  const size_t smem = red_bytes + (xlds ? x_bytes : 0);
  // dwords of scales per row and wave, eight per load
  const int sb_words = pl.s * 16 * (128 / bits) / gs / 2;
  const int sb_loads = sb_words <= 8 ? 1 : (sb_words <= 16 ? 2 : 4);
  auto go = [&](auto tval, auto bval, auto mbv, auto sval, auto kwv, auto mcv) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int MB = decltype(mbv)::value;
    constexpr int S = decltype(sval)::value;
    constexpr int KW = decltype(kwv)::value;
    constexpr int MC = decltype(mcv)::value;
    auto launch = [&](auto kern) -> int {
      if (smem > 48 * 1024) {
        MLXROCM_HIP_TRY(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern),
            hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(smem)));
      }
      kern<<<grid, 512, smem, s>>>(a, gs_shift);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    };
    auto by_qpw = [&](auto f) -> int {
      if constexpr (MB == 1 && KW <= 4) {
        if (qpw == 1) {
          return f(IntC<1>{});
        }
        if (qpw == 2) {
          return f(IntC<2>{});
        }
      }
      return f(IntC<4>{});
    };
    if (xlds) {
      // the x image needs whole slots: S * KW covers K exactly or x is zero there
      if (sb_loads == 1) {
        return by_qpw([&](auto qv) { return launch(qmv_quad_kernel<T, B, MB, S, KW, 1, true, MC, decltype(qv)::value>); });
      } else if (sb_loads == 2) {
        return by_qpw([&](auto qv) { return launch(qmv_quad_kernel<T, B, MB, S, KW, 2, true, MC, decltype(qv)::value>); });
      }
      return by_qpw([&](auto qv) { return launch(qmv_quad_kernel<T, B, MB, S, KW, 4, true, MC, decltype(qv)::value>); });
    }
    if (sb_loads == 1) {
      return launch(qmv_quad_kernel<T, B, MB, S, KW, 1, false, MC, 4>);
    } else if (sb_loads == 2) {
      return launch(qmv_quad_kernel<T, B, MB, S, KW, 2, false, MC, 4>);
    }
    return launch(qmv_quad_kernel<T, B, MB, S, KW, 4, false, MC, 4>);
  };
  auto by_mc = [&](auto tval, auto bval, auto mbv, auto sval, auto kwv) -> int {
    if constexpr (decltype(mbv)::value == 1) {
      if (a.M == 1) {
        return go(tval, bval, mbv, sval, kwv, IntC<1>{});
      }
      if (a.M == 2) {
        return go(tval, bval, mbv, sval, kwv, IntC<2>{});
      }
    }
    return go(tval, bval, mbv, sval, kwv, IntC<4>{});
  };
  auto by_kw = [&](auto tval, auto bval, auto mbv, auto sval) -> int {
    switch (pl.kw) {
      case 1:
        return by_mc(tval, bval, mbv, sval, IntC<1>{});
      case 2:
        return by_mc(tval, bval, mbv, sval, IntC<2>{});
      case 4:
        return by_mc(tval, bval, mbv, sval, IntC<4>{});
      default:
        return by_mc(tval, bval, mbv, sval, IntC<8>{});
    }
  };
  auto by_s = [&](auto tval, auto bval, auto mbv) -> int {
    switch (pl.s) {
      case 1:
        return by_kw(tval, bval, mbv, IntC<1>{});
      case 2:
        return by_kw(tval, bval, mbv, IntC<2>{});
      default:
        return by_kw(tval, bval, mbv, IntC<4>{});
    }
  };
  auto by_mb = [&](auto tval, auto bval) -> int {
    return mb == 1 ? by_s(tval, bval, IntC<1>{}) : by_s(tval, bval, IntC<2>{});
  };
  auto by_bits = [&](auto tval) -> int {
    return by_mb(tval, IntC<4>{});
  };
  return dtype == MLXROCM_BFLOAT16 ? by_bits(bf16_t{}) : by_bits(f16_t{});
}

} // namespace mlxrocm
