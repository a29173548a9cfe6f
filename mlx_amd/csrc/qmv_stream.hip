// qmv_stream.hip -- decode GEMV (transpose=true, M <= 2) for 16-bit element
// types and 4/8-bit codes: a pure HBM streaming kernel for gfx950.
//
// Layout.  A packed weight row is read in "chunks" of 1 KiB: one
// global_load_dwordx4 per wavefront, lane l taking bytes [16 l, 16 l + 16) of the
// chunk, so every load instruction covers eight whole 128-byte lines of one row
// and nothing else.  (Measured on MI355X: a row-per-lane layout that touches 16
// or 32 rows per load instruction runs at ~3 TB/s even out of the last-level
// cache; whole-line loads are what the memory pipeline wants.)
//
//   * A wavefront owns kRowsPerWave output rows and a fixed set of CPW chunks
//     of K.  The slices of x that match its lanes' code positions stay in
//     registers for the whole kernel; x reaches them through one coalesced
//     global read per workgroup and an LDS transpose, which also leaves each
//     lane's sum of x in LDS (computed once per workgroup, not once per wave).
//   * Codes are widened without arithmetic (a 4-bit code OR-ed into the
//     mantissa of 128.0 / 1024.0; 8-bit codes by cvt_f32_ubyte or a byte
//     permute) and multiplied with v_dot2_f32_{bf16,f16}, fp32 accumulation;
//     for one row of x and 4-bit codes the 4x4x4 matrix instruction does the
//     dot products instead (a lane's slice of x as its row of A, its codes as
//     its column of B, the diagonal of the result kept), beside the vector ALU.
//   * A lane's 16 bytes lie inside one quantization group, so the affine part
//     is two FMAs per load:  y += s * dot + (b - OFFSET * s) * sum(x_lane).
//   * All loads of a wave's rows are issued before the first is consumed; the
//     row sums are finished with DPP reductions (no LDS), and k-slices held by
//     different waves are added through LDS.
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kChunkBytes = 1024; // 64 lanes x 16 bytes

template <typename T>
struct Dot;

template <>
struct Dot<bf16_t> {
  static constexpr uint32_t kMagic4 = 0x43004300u; // 128.0 | 128.0
  static constexpr float kOffset4 = 128.0f;
  static constexpr float kOffset8 = 0.0f;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(
        __builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  }
  // 16 independent 4x4x4 products: register t of the result in lane (blk, i) is
  // A's row t (the four values lane (blk, t) passes) times this lane's B column
  static __device__ __forceinline__ float4_t mfma444(uint2 a, uint2 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
        __builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen_scalar(uint32_t h) {
    return __uint_as_float(h << 16);
  }
  // the 16-bit value at bit offset `sh` (0 or 16) of a word, widened
  static __device__ __forceinline__ float half_of_word(uint32_t w, int sh) {
    return __uint_as_float((w << (16 - sh)) & 0xffff0000u);
  }
  // 4 bytes -> 2 dwords of bf16 pairs (0..255 are exact in bf16), natural order
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
  static constexpr uint32_t kOnes = 0x3f803f80u;
};

template <>
struct Dot<f16_t> {
  static constexpr uint32_t kMagic4 = 0x64006400u; // 1024.0 | 1024.0
  static constexpr float kOffset4 = 1024.0f;
  static constexpr float kOffset8 = 1024.0f;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(
        __builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  }
  static __device__ __forceinline__ float4_t mfma444(uint2 a, uint2 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(
        __builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen_scalar(uint32_t h) {
    return static_cast<float>(__builtin_bit_cast(f16_t, static_cast<uint16_t>(h)));
  }
  static __device__ __forceinline__ float half_of_word(uint32_t w, int sh) {
    return widen_scalar(w >> sh);
  }
  // byte c -> f16 bits 0x64cc = 1024 + c
  static __device__ __forceinline__ uint2 widen8(uint32_t w) {
    constexpr uint32_t hi = 0x64646464u;
    return make_uint2(
        __builtin_amdgcn_perm(hi, w, 0x04010400u),
        __builtin_amdgcn_perm(hi, w, 0x04030402u));
  }
  static constexpr uint32_t kOnes = 0x3c003c00u;
};

// Constants of the 4-bit expansion kept opaque so that (w & mask) | magic is
// selected as one v_and_or_b32 (mask in an SGPR, magic in a VGPR).
struct Widen4Consts {
  uint32_t mask;
  uint32_t magic;
};

template <typename T>
__device__ __forceinline__ Widen4Consts make_widen4_consts() {
  Widen4Consts c;
  c.mask = 0x000f000fu;
  c.magic = Dot<T>::kMagic4;
  asm volatile("" : "+s"(c.mask));
  asm volatile("" : "+v"(c.magic));
  return c;
}

template <int BITS, int GS>
struct StreamShape {
  static constexpr int kLaneCodes = 128 / BITS;       // codes in 16 bytes
  static constexpr int kChunkCodes = kLaneCodes * 64; // 2048 or 1024
  static constexpr int kXRegs = kLaneCodes / 2;       // x dwords per chunk
  // CPW: chunks of K per wave -- 4 KiB of a row, but at most 64 groups so
  // that a wave's scale words fit half a wavefront
  static constexpr int kMaxChunks = (BITS == 4) ? 2 : 4;
  static constexpr int kGroupChunks = 64 * GS / kChunkCodes;
  static constexpr int kChunksPerWave = kGroupChunks < kMaxChunks ? kGroupChunks : kMaxChunks;
  // rows per wave: 8 KiB of packed weights in flight per wave either way
  static constexpr int kRowsPerWave = 4 / kChunksPerWave;
  static_assert(kChunksPerWave >= 1, "shape");
};

// 16-byte load of data that is read exactly once: nontemporal, so the stream
// does not displace x, scales and biases from the caches.
__device__ __forceinline__ uint4 load_streaming(const uint8_t* p) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// x + the value of the lane that a quad permutation pairs this lane with.
template <int CTRL>
__device__ __forceinline__ float quad_add(float x) {
  const int moved = __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false);
  return x + __builtin_bit_cast(float, moved);
}

// Sum of all 64 lanes, valid in lane 63 (DPP: two quad swaps, two mirrors,
// then row broadcasts across the four rows of 16).
__device__ __forceinline__ float wave_sum_dpp(float v) {
  auto step = [](float x, auto ctrl, auto rmask) {
    constexpr int kCtrl = decltype(ctrl)::value;
    constexpr int kRow = decltype(rmask)::value;
    const int moved = __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, x), kCtrl, kRow, 0xf, false);
    return x + __builtin_bit_cast(float, moved);
  };
  v = step(v, IntC<0xB1>{}, IntC<0xf>{});  // quad_perm [1,0,3,2]
  v = step(v, IntC<0x4E>{}, IntC<0xf>{});  // quad_perm [2,3,0,1]
  v = step(v, IntC<0x141>{}, IntC<0xf>{}); // row_half_mirror
  v = step(v, IntC<0x140>{}, IntC<0xf>{}); // row_mirror: every lane has its row's sum
  v = step(v, IntC<0x142>{}, IntC<0xa>{}); // row_bcast15 into rows 1 and 3
  v = step(v, IntC<0x143>{}, IntC<0xc>{}); // row_bcast31 into rows 2 and 3
  return v;
}

// KW: waves that split K between them; RW: row-waves; the workgroup owns
// RW * kRowsPerWave rows.  M is 1 or 2.  FULL: K is exactly KW * CPW chunks, so
// no lane ever falls outside a row and the loads carry no predicate.
template <typename T, int BITS, int GS, int M, int RW, int KW, bool FULL, int RM = 1, bool MD = false,
          bool GLU = false>
// (At least two waves per SIMD: the kernel needs under 80 registers, and with a
// budget of 256 the compiler keeps the 4x4x4 results in vector registers; with
// the 512 that a workgroup of 256 threads may claim it puts them in accumulation
// registers and reads each one back with v_accvgpr_read.)
__global__ __launch_bounds__(RW * KW * 64) __attribute__((amdgpu_waves_per_eu(2))) void
qmv_stream_kernel(const QmmArgs a) {
  using S = StreamShape<BITS, GS>;
  constexpr int CPW = S::kChunksPerWave;
  constexpr int kRowsPerWave = S::kRowsPerWave * RM;
  constexpr int kThreads = RW * KW * 64;
  constexpr float kOffset = (BITS == 4) ? Dot<T>::kOffset4 : Dot<T>::kOffset8;
  constexpr bool kMatrixDot = BITS == 4 && M == 1 && MD;
  static_assert(GS >= S::kLaneCodes, "a lane's 16 bytes stay inside one group");

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kw = wave % KW;
  const int rw = wave / KW;
  const int K = a.K;
  const int N = a.N;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  const int groups = K / GS;
  const uint32_t row_bytes = static_cast<uint32_t>(K / 8) * BITS;
  // GLU: the wave's two rows are row n of the gate weight (a.w) and row n of the
  // up weight (a.w_alt); it writes y[n] = silu(gate . x) * (up . x).
  static_assert(!GLU || (kRowsPerWave == 2 && M == 1), "gated form: a row pair per wave, one row of x");
  const int row0 = GLU ? (blockIdx.x * RW + rw) : (blockIdx.x * RW + rw) * kRowsPerWave;
  auto row_of = [&](int r) {
    const int row = GLU ? row0 : row0 + r;
    return row < N ? row : N - 1; // clamp: stay in bounds
  };

  // ---- 1. x: one coalesced read per workgroup (issued first) ----
  const int x_units = M * (K / 8); // 16-byte units
  const uint8_t* xbytes = reinterpret_cast<const uint8_t*>(p.x);
  // up to kUpfront units per thread are fetched ahead of the weight stream (a
  // long K split over four or eight k-waves needs up to four per row of x)
  constexpr int kUpfront = KW >= 4 ? 4 : 2;
  uint4 xv[kUpfront];
#pragma unroll
  for (int u = 0; u < kUpfront; ++u) {
    xv[u] = make_uint4(0, 0, 0, 0);
    if (tid + u * kThreads < x_units) {
      xv[u] = *reinterpret_cast<const uint4*>(
          xbytes + static_cast<uint32_t>(tid + u * kThreads) * 16);
    }
  }

  // ---- 2. every weight / scale / bias load of this wave ----
  // Scales and biases: one dword load per row fetches both (lanes 0..31 the
  // wave's scale words, lanes 32..63 its bias words, whole lines each); every
  // lane then picks its group's value from the owning lane with ds_bpermute.
  const int c0 = kw * CPW; // first chunk of this wave
  constexpr int kWaveGroups = CPW * S::kChunkCodes / GS; // groups per row per wave
  constexpr int kSbWordsPerWave = kWaveGroups / 2;
  static_assert(kSbWordsPerWave <= 32, "scale words of a wave fit half a wavefront");
  const int g_base = kw * kWaveGroups;
  uint4 wv[kRowsPerWave][CPW];
  uint32_t sbw[kRowsPerWave];
  const int sb_word = lane & 31;
  // clamp: lanes past the wave's (or the row's) last group reread a valid word
  int sb_group = g_base + 2 * sb_word;
  sb_group = (sb_group + 1 < groups) ? sb_group : groups - 2;
  const uint8_t* sb_lane_base =
      reinterpret_cast<const uint8_t*>(lane < 32 ? p.scales : p.biases) +
      static_cast<size_t>(sb_group) * 2;
  const uint8_t* sb_lane_alt = sb_lane_base;
  const uint8_t* w_alt = p.w;
  if constexpr (GLU) {
    sb_lane_alt =
        reinterpret_cast<const uint8_t*>(lane < 32 ? a.scales_alt : a.biases_alt) +
        static_cast<size_t>(sb_group) * 2;
    w_alt = reinterpret_cast<const uint8_t*>(a.w_alt);
  }
  // The small scale/bias loads go first: loads complete in order, so a scale
  // queued behind the whole weight stream would hold back the first row.
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int row = row_of(r);
    sbw[r] = *reinterpret_cast<const uint32_t*>(
        ((GLU && r == 1) ? sb_lane_alt : sb_lane_base) + static_cast<size_t>(row) * groups * 2);
  }
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int row = row_of(r);
    const uint8_t* wrow = ((GLU && r == 1) ? w_alt : p.w) + static_cast<size_t>(row) * row_bytes;
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const uint32_t byte = static_cast<uint32_t>(c0 + c) * kChunkBytes + lane * 16;
      if constexpr (FULL) {
        wv[r][c] = load_streaming(wrow + byte);
      } else {
        wv[r][c] = make_uint4(0, 0, 0, 0);
        if (byte < row_bytes) {
          wv[r][c] = load_streaming(wrow + byte);
        }
      }
    }
  }
  // Which lane holds this lane's group, per chunk, and which half of the word.
  int sb_src[CPW];  // byte address for ds_bpermute (source lane * 4)
  int sb_odd[CPW];
#pragma unroll
  for (int c = 0; c < CPW; ++c) {
    int g = (c * S::kChunkCodes + lane * S::kLaneCodes) / GS; // group inside the wave
    if constexpr (!FULL) {
      // lanes past the end of the row only need some valid, finite value
      int ga = g_base + g;
      ga = ga < groups ? ga : groups - 1;
      g = ga > g_base ? ga - g_base : 0;
    }
    sb_src[c] = (g / 2) * 4;
    sb_odd[c] = (g & 1) * 16; // bit offset of the group's value in its word
  }

  // ---- 3. x through LDS into the lanes that need it ----
  // LDS layout per x row: for chunk c, piece t (16 bytes = 8 elements) of lane
  // l sits at ((c * P + t) * 64 + l) * 16, P = pieces per lane per chunk, so a
  // wave's reads of piece t are conflict free.
  constexpr int P = S::kLaneCodes / 8;
  const int nchunks = (K + S::kChunkCodes - 1) / S::kChunkCodes;
  const uint32_t xrow_bytes = static_cast<uint32_t>(nchunks) * P * 64 * 16;
  float* sx_lds = reinterpret_cast<float*>(smem + M * xrow_bytes); // [M][nchunks][64]
  auto stage_x = [&](int idx, const uint4& v) {
    // row of x (M <= 2: a compare instead of a division) and the 8-element
    // unit inside it, in unsigned arithmetic (shifts and masks)
    const uint32_t row_units = static_cast<uint32_t>(K) / 8u;
    const uint32_t m = (M > 1 && static_cast<uint32_t>(idx) >= row_units) ? 1u : 0u;
    const uint32_t e = static_cast<uint32_t>(idx) - m * row_units;
    const uint32_t l = (e / P) & 63u;
    const uint32_t t = e % P;
    const uint32_t c = e / (P * 64u);
    uint4 o = v;
    if constexpr (BITS == 4) {
      // element order 0,4,1,5,2,6,3,7: register j pairs codes (j, j+4)
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    }
    *reinterpret_cast<uint4*>(
        smem + m * xrow_bytes + ((static_cast<uint32_t>(c) * P + t) * 64 + l) * 16) = o;
    // sum of the P pieces that one lane of a chunk will hold: the P threads
    // that stage them are neighbours (idx % P == tid % P), so two quad swaps
    // finish it, and every wave reads the sum instead of recomputing it
    float part = Dot<T>::dot2(v.x, Dot<T>::kOnes, 0.0f);
    part = Dot<T>::dot2(v.y, Dot<T>::kOnes, part);
    part = Dot<T>::dot2(v.z, Dot<T>::kOnes, part);
    part = Dot<T>::dot2(v.w, Dot<T>::kOnes, part);
    part = quad_add<0xB1>(part); // quad_perm [1,0,3,2]
    if constexpr (P == 4) {
      part = quad_add<0x4E>(part); // quad_perm [2,3,0,1]
    }
    if (t == 0) {
      sx_lds[(m * nchunks + c) * 64 + l] = part;
    }
  };
#pragma unroll
  for (int u = 0; u < kUpfront; ++u) {
    if (tid + u * kThreads < x_units) {
      stage_x(tid + u * kThreads, xv[u]);
    }
  }
  // longer x: the remaining units follow the weight loads in the queue
  for (int idx = tid + kUpfront * kThreads; idx < x_units; idx += kThreads) {
    stage_x(idx, *reinterpret_cast<const uint4*>(xbytes + static_cast<uint32_t>(idx) * 16));
  }
  __syncthreads();

  uint32_t xr[M][CPW][S::kXRegs];
  float sx[M][CPW];
#pragma unroll
  for (int m = 0; m < M; ++m) {
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const bool live = FULL ||
          (static_cast<uint32_t>(c0 + c) * kChunkBytes + lane * 16) < row_bytes;
#pragma unroll
      for (int t = 0; t < P; ++t) {
        uint4 v;
        if constexpr (FULL) {
          v = *reinterpret_cast<const uint4*>(
              smem + m * xrow_bytes +
              ((static_cast<uint32_t>(c0 + c) * P + t) * 64 + lane) * 16);
        } else {
          v = make_uint4(0, 0, 0, 0);
          if (live) {
            v = *reinterpret_cast<const uint4*>(
                smem + m * xrow_bytes +
                ((static_cast<uint32_t>(c0 + c) * P + t) * 64 + lane) * 16);
          }
        }
        xr[m][c][4 * t + 0] = v.x;
        xr[m][c][4 * t + 1] = v.y;
        xr[m][c][4 * t + 2] = v.z;
        xr[m][c][4 * t + 3] = v.w;
      }
      sx[m][c] = live ? sx_lds[(m * nchunks + c0 + c) * 64 + lane] : 0.0f;
    }
  }

  // ---- 4. consume rows as they arrive ----
  const Widen4Consts w4c = make_widen4_consts<T>();
  float y[kRowsPerWave][M];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      y[r][m] = 0.0f;
    }
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const uint32_t w[4] = {wv[r][c].x, wv[r][c].y, wv[r][c].z, wv[r][c].w};
      float dot[M];
      if constexpr (kMatrixDot) {
        // The 4x4x4 matrix instruction as a four-element dot product per lane:
        // with this lane's x slice as its row of A and its codes as its column
        // of B, register (lane % 4) of the result is the lane's own product and
        // the other three pair it with its neighbours' slices (unused).  One
        // instruction replaces two v_dot2 and runs beside the vector ALU.
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t q0 = (w[d] & w4c.mask) | w4c.magic;
          const uint32_t q1 = ((w[d] >> 4) & w4c.mask) | w4c.magic;
          const uint32_t q2 = ((w[d] >> 8) & w4c.mask) | w4c.magic;
          const uint32_t q3 = ((w[d] >> 12) & w4c.mask) | w4c.magic;
          acc = Dot<T>::mfma444(
              make_uint2(xr[0][c][4 * d + 0], xr[0][c][4 * d + 1]), make_uint2(q0, q1), acc);
          acc = Dot<T>::mfma444(
              make_uint2(xr[0][c][4 * d + 2], xr[0][c][4 * d + 3]), make_uint2(q2, q3), acc);
        }
        const float d01 = (lane & 1) ? acc[1] : acc[0];
        const float d23 = (lane & 1) ? acc[3] : acc[2];
        dot[0] = (lane & 2) ? d23 : d01;
      } else {
      // two accumulator chains: dwords 0, 2 and dwords 1, 3
      float dacc[M][4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
          dacc[m][d] = d < 2 ? 0.0f : dacc[m][d >= 2 ? d - 2 : 0];
        }
        if constexpr (BITS == 4) {
          const uint32_t q0 = (w[d] & w4c.mask) | w4c.magic;
          const uint32_t q1 = ((w[d] >> 4) & w4c.mask) | w4c.magic;
          const uint32_t q2 = ((w[d] >> 8) & w4c.mask) | w4c.magic;
          const uint32_t q3 = ((w[d] >> 12) & w4c.mask) | w4c.magic;
#pragma unroll
          for (int m = 0; m < M; ++m) {
            dacc[m][d] = Dot<T>::dot2(xr[m][c][4 * d + 0], q0, dacc[m][d]);
            dacc[m][d] = Dot<T>::dot2(xr[m][c][4 * d + 1], q1, dacc[m][d]);
            dacc[m][d] = Dot<T>::dot2(xr[m][c][4 * d + 2], q2, dacc[m][d]);
            dacc[m][d] = Dot<T>::dot2(xr[m][c][4 * d + 3], q3, dacc[m][d]);
          }
        } else {
          const uint2 q = Dot<T>::widen8(w[d]);
#pragma unroll
          for (int m = 0; m < M; ++m) {
            dacc[m][d] = Dot<T>::dot2(xr[m][c][2 * d + 0], q.x, dacc[m][d]);
            dacc[m][d] = Dot<T>::dot2(xr[m][c][2 * d + 1], q.y, dacc[m][d]);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
        dot[m] = dacc[m][2] + dacc[m][3];
      }
      }
      const uint32_t s_word = static_cast<uint32_t>(
          __builtin_amdgcn_ds_bpermute(sb_src[c], static_cast<int>(sbw[r])));
      const uint32_t b_word = static_cast<uint32_t>(
          __builtin_amdgcn_ds_bpermute(sb_src[c] + 128, static_cast<int>(sbw[r])));
      const float s = Dot<T>::half_of_word(s_word, sb_odd[c]);
      const float beff = fmaf(-kOffset, s, Dot<T>::half_of_word(b_word, sb_odd[c]));
#pragma unroll
      for (int m = 0; m < M; ++m) {
        y[r][m] = fmaf(s, dot[m], y[r][m]);
        y[r][m] = fmaf(beff, sx[m][c], y[r][m]);
      }
    }
  }

  // ---- 5. lanes -> row sums (lane 63), then k-waves -> output ----
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      y[r][m] = wave_sum_dpp(y[r][m]);
    }
  }
  // the gate with the roundings of the unfused chain: both products, the sigmoid,
  // gate * sigmoid and the final product are each rounded to T
  auto gated = [](float gate, float up) {
    const float g = to_f32(from_f32<T>(gate));
    const float u = to_f32(from_f32<T>(up));
    const float sg = to_f32(from_f32<T>(1.0f / (1.0f + __expf(-g))));
    const float h = to_f32(from_f32<T>(g * sg));
    return from_f32<T>(h * u);
  };
  if constexpr (GLU && KW == 1) {
    if (lane == 63 && row0 < N) {
      p.out[row0] = gated(y[0][0], y[1][0]);
    }
  } else if constexpr (KW == 1) {
    if (lane == 63) {
#pragma unroll
      for (int r = 0; r < kRowsPerWave; ++r) {
        if (row0 + r < N) {
#pragma unroll
          for (int m = 0; m < M; ++m) {
            p.out[static_cast<size_t>(m) * N + row0 + r] =
                from_f32<T>(p.valid ? y[r][m] : 0.0f);
          }
        }
      }
    }
  } else {
    __syncthreads(); // x staging area is reused for the partial sums
    float* red = reinterpret_cast<float*>(smem); // [RW][KW][rows][M]
    if (lane == 63) {
#pragma unroll
      for (int r = 0; r < kRowsPerWave; ++r) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
          red[((rw * KW + kw) * kRowsPerWave + r) * M + m] = y[r][m];
        }
      }
    }
    __syncthreads();
    if constexpr (GLU) {
      if (tid < RW) {
        float gate = 0.0f, up = 0.0f;
#pragma unroll
        for (int k = 0; k < KW; ++k) {
          gate += red[(tid * KW + k) * 2 + 0];
          up += red[(tid * KW + k) * 2 + 1];
        }
        const int n = blockIdx.x * RW + tid;
        if (n < N) {
          p.out[n] = gated(gate, up);
        }
      }
    } else if (tid < RW * kRowsPerWave * M) {
      const int m = tid % M;
      const int r = (tid / M) % kRowsPerWave;
      const int w = tid / (M * kRowsPerWave);
      float total = 0.0f;
#pragma unroll
      for (int k = 0; k < KW; ++k) {
        total += red[((w * KW + k) * kRowsPerWave + r) * M + m];
      }
      const int row = (blockIdx.x * RW + w) * kRowsPerWave + r;
      if (row < N) {
        p.out[static_cast<size_t>(m) * N + row] = from_f32<T>(p.valid ? total : 0.0f);
      }
    }
  }
}

template <int BITS, int GS>
size_t stream_smem_bytes(int M, int K, int rw, int kw, int rm) {
  using S = StreamShape<BITS, GS>;
  const int kRowsPerWave = S::kRowsPerWave * rm;
  const int nchunks = (K + S::kChunkCodes - 1) / S::kChunkCodes;
  // the staged x image, then one partial sum of x per lane and chunk
  const size_t x_bytes = static_cast<size_t>(M) * nchunks * (S::kLaneCodes / 8) * 64 * 16 +
      static_cast<size_t>(M) * nchunks * 64 * 4;
  const size_t red_bytes = static_cast<size_t>(rw) * kw * kRowsPerWave * M * 4;
  return x_bytes > red_bytes ? x_bytes : red_bytes;
}

// Workgroup shape: KW waves cover K (CPW chunks each), RW row-waves fill the
// workgroup up to 8 waves.
struct StreamPlan {
  int kw;
  int rw;
  int rm; // multiple of the shape's rows per wave
};

template <int BITS, int GS>
StreamPlan stream_plan(int K, int N, int M) {
  using S = StreamShape<BITS, GS>;
  const int nchunks = (K + S::kChunkCodes - 1) / S::kChunkCodes;
  const int need = (nchunks + S::kChunksPerWave - 1) / S::kChunksPerWave;
  StreamPlan pl;
  pl.kw = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : (need <= 8 ? 8 : 0)));
  pl.rw = pl.kw == 0 ? 0 : 8 / pl.kw;
  pl.rm = 1;
  // Long K (four or eight k-waves): every workgroup stages the whole of x for
  // the few rows it owns, so give a wave four rows while the grid still covers
  // the compute units 1.5 times (4096 x 14336 8-bit: 17.8 -> 15.9 us, 4096 x 11008
  // 4-bit: 10.7 -> 9.9 us).
  if (pl.kw >= 4) {
    const long want = compute_units() * 3L / 2;
    int rm = 4 / S::kRowsPerWave;
    while (rm > 1 && (N + pl.rw * S::kRowsPerWave * rm - 1) / (pl.rw * S::kRowsPerWave * rm) < want) {
      rm /= 2;
    }
    pl.rm = rm;
  }
  // One k-wave, one row of x, 4-bit: workgroups of seven or four waves when that
  // does not raise the number of rows the busiest compute unit ends up with
  // (14336 rows on 256 units: 4 x 14 or 7 x 8 rows instead of 4 x 16).  Seven
  // waves put exactly seven on every SIMD with a quarter fewer workgroups staging
  // x than four do: 14336 x 4096, 8.04 us with eight or four waves, 7.84 with seven;
  // where the shape does not balance the smaller workgroup is slower (measured for
  // four waves: 3-6 % faster when it lowers the busiest unit's rows, slower when
  // not), and 8-bit codes are slower either way.
  if (pl.kw == 1 && M == 1 && BITS == 4) {
    const long cus = compute_units();
    auto busiest = [&](int rw) {
      const long rows = static_cast<long>(rw) * S::kRowsPerWave * pl.rm;
      const long wgs = (N + rows - 1) / rows;
      return (wgs + cus - 1) / cus * rows;
    };
    if (busiest(7) <= busiest(4) && busiest(7) < busiest(8)) {
      pl.rw = 7;
    } else if (busiest(4) < busiest(8)) {
      pl.rw = 4;
    }
  }
  return pl;
}

} // namespace

bool qmv_stream_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  if (dtype == MLXROCM_FLOAT32 || !(bits == 4 || bits == 8)) {
    return false;
  }
  if (a.M < 1 || a.M > 2) {
    return false;
  }
  // scale / bias words are fetched as aligned dwords
  if ((a.K / gs) % 2 != 0 || a.sb_batch_stride % 2 != 0) {
    return false;
  }
  StreamPlan pl{0, 0, 1};
  size_t smem = 0;
  auto probe = [&](auto bval, auto gval) {
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    pl = stream_plan<B, G>(a.K, a.N, a.M);
    smem = pl.kw == 0 ? 0 : stream_smem_bytes<B, G>(a.M, a.K, pl.rw, pl.kw, pl.rm);
  };
  auto by_group = [&](auto bval) {
    if (gs == 32) {
      probe(bval, IntC<32>{});
    } else if (gs == 64) {
      probe(bval, IntC<64>{});
    } else {
      probe(bval, IntC<128>{});
    }
  };
  if (bits == 4) {
    by_group(IntC<4>{});
  } else {
    by_group(IntC<8>{});
  }
  if (pl.kw == 0) {
    return false; // K beyond 8 k-waves
  }
  return smem <= 72 * 1024; // x image of 64 KiB (M = 2, K = 16384, 4-bit) + its sums
}

// Gated form (y = silu(gate . x) * (up . x), a.w_alt set): one row of x, every K
// the kernel covers.  A wave owns one row pair: shapes whose waves own four rows
// (4-bit, groups of 32) are not covered.
template <int BITS, int GS>
constexpr int glu_row_multiple() {
  // rows per wave must come to two
  return StreamShape<BITS, GS>::kRowsPerWave == 1 ? 2 : (StreamShape<BITS, GS>::kRowsPerWave == 2 ? 1 : 0);
}

bool qmv_stream_glu_supported(const QmmArgs& a, int gs, int bits, int dtype) {
  if (a.w_alt == nullptr || a.M != 1 || a.L != 1 || a.lhs_indices != nullptr) {
    return false;
  }
  if (!qmv_stream_supported(a, gs, bits, dtype)) {
    return false;
  }
  bool ok = false;
  auto probe = [&](auto bval, auto gval) {
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    ok = glu_row_multiple<B, G>() != 0 && stream_plan<B, G>(a.K, 2 * a.N, 1).kw != 0;
  };
  auto by_group = [&](auto bval) {
    if (gs == 32) {
      probe(bval, IntC<32>{});
    } else if (gs == 64) {
      probe(bval, IntC<64>{});
    } else {
      probe(bval, IntC<128>{});
    }
  };
  if (bits == 4) {
    by_group(IntC<4>{});
  } else {
    by_group(IntC<8>{});
  }
  return ok;
}

int launch_qmv_stream_glu(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  if (!qmv_stream_glu_supported(a, gs, bits, dtype)) {
    return fail(MLXROCM_UNSUPPORTED, "[qmv] shape not covered by the gated GEMV");
  }
  MLXROCM_REHEARSE("qmv_stream_glu");
  auto run = [&](auto tval, auto bval, auto gval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    using S = StreamShape<B, G>;
    constexpr int RM = glu_row_multiple<B, G>();
    if constexpr (RM == 0) {
      return fail(MLXROCM_UNSUPPORTED, "[qmv] shape not covered by the gated GEMV");
    } else {
      StreamPlan pl = stream_plan<B, G>(a.K, 2 * a.N, 1);
      if (pl.rw == 7) {
        pl.rw = 8; // the gated form has four- and eight-wave workgroups
      }
      const size_t smem = stream_smem_bytes<B, G>(1, a.K, pl.rw, pl.kw, RM);
      const bool full = a.K == pl.kw * S::kChunksPerWave * S::kChunkCodes;
      const dim3 grid((a.N + pl.rw - 1) / pl.rw, 1);
      constexpr bool MD = B == 4 && G >= 64;
      auto go = [&](auto rwv, auto kwv) -> int {
        constexpr int RW = decltype(rwv)::value;
        constexpr int KW = decltype(kwv)::value;
        auto kern = full ? qmv_stream_kernel<T, B, G, 1, RW, KW, true, RM, MD, true>
                         : qmv_stream_kernel<T, B, G, 1, RW, KW, false, RM, MD, true>;
        if (smem > 48 * 1024) {
          MLXROCM_HIP_TRY(hipFuncSetAttribute(
              reinterpret_cast<const void*>(kern),
              hipFuncAttributeMaxDynamicSharedMemorySize,
              static_cast<int>(smem)));
        }
        kern<<<grid, RW * KW * 64, smem, s>>>(a);
        MLXROCM_HIP_TRY(hipGetLastError());
        return static_cast<int>(MLXROCM_OK);
      };
      switch (pl.kw) {
        case 1:
          return pl.rw == 4 ? go(IntC<4>{}, IntC<1>{}) : go(IntC<8>{}, IntC<1>{});
        case 2:
          return go(IntC<4>{}, IntC<2>{});
        case 4:
          return go(IntC<2>{}, IntC<4>{});
        default:
          return go(IntC<1>{}, IntC<8>{});
      }
    }
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

int launch_qmv_stream(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  auto run = [&](auto tval, auto bval, auto gval) -> int {
    using T = decltype(tval);
    constexpr int B = decltype(bval)::value;
    constexpr int G = decltype(gval)::value;
    using S = StreamShape<B, G>;
    const StreamPlan pl = stream_plan<B, G>(a.K, a.N, a.M);
    const size_t smem = stream_smem_bytes<B, G>(a.M, a.K, pl.rw, pl.kw, pl.rm);
    const int rows_per_wg = pl.rw * S::kRowsPerWave * pl.rm;
    const bool full = a.K == pl.kw * S::kChunksPerWave * S::kChunkCodes;
    const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, a.L);
    if (grid.y > 65535u) {
      return fail(MLXROCM_UNSUPPORTED, "[qmv] batch=%d exceeds the grid", a.L);
    }
    MLXROCM_REHEARSE("qmv_stream(rw=%d,kw=%d,rm=%d)", pl.rw, pl.kw, pl.rm);
    auto go = [&](auto mval, auto rwv, auto kwv, auto rmv) -> int {
      constexpr int M = decltype(mval)::value;
      constexpr int RW = decltype(rwv)::value;
      constexpr int KW = decltype(kwv)::value;
      constexpr int RM = decltype(rmv)::value;
      // one row of x, 4-bit, groups of 64 or 128: the dot products on the matrix
      // instruction (1-5 % faster; with 32-wide groups the v_dot2 form is ahead)
      constexpr bool MD = B == 4 && M == 1 && G >= 64;
      auto kern = full ? qmv_stream_kernel<T, B, G, M, RW, KW, true, RM, MD>
                       : qmv_stream_kernel<T, B, G, M, RW, KW, false, RM, MD>;
      if (smem > 48 * 1024) {
        MLXROCM_HIP_TRY(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern),
            hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(smem)));
      }
      kern<<<grid, RW * KW * 64, smem, s>>>(a);
      MLXROCM_HIP_TRY(hipGetLastError());
      return static_cast<int>(MLXROCM_OK);
    };
    auto by_rm = [&](auto mval, auto rwv, auto kwv) -> int {
      if constexpr (decltype(kwv)::value >= 4) {
        if (pl.rm == 2) {
          return go(mval, rwv, kwv, IntC<2>{});
        }
        if (pl.rm == 4) {
          return go(mval, rwv, kwv, IntC<4>{});
        }
      }
      return go(mval, rwv, kwv, IntC<1>{});
    };
    auto by_plan = [&](auto mval) -> int {
      switch (pl.kw) {
        case 1:
          if (pl.rw == 4) {
            return by_rm(mval, IntC<4>{}, IntC<1>{});
          }
          if constexpr (B == 4 && decltype(mval)::value == 1) {
            if (pl.rw == 7) {
              return by_rm(mval, IntC<7>{}, IntC<1>{});
            }
          }
          return by_rm(mval, IntC<8>{}, IntC<1>{});
        case 2:
          return by_rm(mval, IntC<4>{}, IntC<2>{});
        case 4:
          return by_rm(mval, IntC<2>{}, IntC<4>{});
        default:
          return by_rm(mval, IntC<1>{}, IntC<8>{});
      }
    };
    return a.M == 1 ? by_plan(IntC<1>{}) : by_plan(IntC<2>{});
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
