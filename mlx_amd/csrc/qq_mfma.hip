// qq_mfma.hip -- y = xq . wq^T for two operands that are both quantized in an MX
// mode (mxfp8: e4m3 codes, mxfp4: e2m1 codes; one e8m0 scale per 32 codes along
// K) on gfx950's block-scaled matrix instruction v_mfma_scale_f32_16x16x128_f8f6f4:
// a lane supplies 32 codes of one row and one block's scale byte, the
// instruction forms sum_k (a_k 2^(sa-127)) (b_k 2^(sb-127)) over the step's four
// blocks of 32 consecutive codes in fp32 (4-bit codes: a lane's 32 codes are one
// block; 8-bit codes: two runs of 16 from different blocks, see the fragment
// reads -- found by multiplying one-hot rows, not from a manual).  This is what qqmm computes once x has been quantized
// (mlx/ops.cpp:4926-4990; CPU: QQMatmul::eval_cpu, mlx/backend/cpu/quantized.cpp:
// 1322-1356 -- quantize x, dequantize it, multiply by the dequantized w): the
// codes are multiplied as they are, nothing is dequantized.
//
// Workgroup: 512 threads, tile 256 (m) x 128 (n), K-step 128 codes.  Both code
// tiles and their scale dwords go HBM -> LDS by DMA (global_load_lds) into a
// ring of stages; the only loads of the loop are those, so one vmcnt wait and
// one barrier per step order everything.  16-byte pieces of a row are
// XOR-swizzled so that fragment reads hit every bank once.  Wavefront (wm, wn)
// owns a 64 x 64 block: W fragments are the instruction's A operand, x
// fragments its B operand, so a lane holds four consecutive n of one row m of y.
#include <type_traits>

#include "mfma_loads.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

typedef int qq_i32x8 __attribute__((ext_vector_type(8)));
typedef int qq_i32x4 __attribute__((ext_vector_type(4)));
typedef float qq_f32x4 __attribute__((ext_vector_type(4)));
typedef float qq_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kQqBK = 128; // codes per step

// Shape of a workgroup: WM x WN wavefronts, each with MI x NI tiles of 16 x 16
// (m x n).
//   <8, 4, 4, 4, 2>: 256 x 128, eight wavefronts  (8-bit codes: three stages fit)
//   <4, 4, 8, 4, 2>: 256 x 256, eight wavefronts  (4-bit codes, enough tiles)
//   <4, 4, 4, 4, 2>: 256 x 128                    (4-bit codes, few tiles)
// What the shapes trade is bytes fetched per flop: measured at [8192, 4096] x
// [14336, 4096], 4-bit, the 256 x 256 tile runs at 2.5 PFLOP/s and the 256 x 128
// tile at 2.0 (the matrix pipe alone does 6.9).  Four wavefronts of 128 x 128
// (one per SIMD, 256 accumulators in AGPRs, fewer LDS bytes per flop) fetch the
// same bytes and were slower (2.3).
template <int BITS, int MI, int NI, int WM, int WN>
struct QqShape {
  static constexpr int kThreads = 64 * WM * WN;
  static constexpr int kWaves = WM * WN;
  static constexpr int kBM = 16 * MI * WM;
  static constexpr int kBN = 16 * NI * WN;
  static constexpr int kRowBytes = kQqBK * BITS / 8;          // 128 or 64
  static constexpr int kSlots = kRowBytes / 16;                // 16-byte pieces per row: 8 or 4
  static constexpr int kRowsPerDma = 1024 / kRowBytes;         // rows one wavefront load moves: 8 or 16
  static constexpr int kXTile = kBM * kRowBytes;               // bytes
  static constexpr int kWTile = kBN * kRowBytes;
  // one scale dword per tile row, x rows first, padded to whole wavefront loads
  static constexpr int kSDma = (kBM + kBN + kThreads - 1) / kThreads; // per wavefront and step
  static constexpr int kScaleBytes = kSDma * kThreads * 4;
  static constexpr int kStage = kXTile + kWTile + kScaleBytes;
  static constexpr int kStages = (160 * 1024) / kStage > 6 ? 6 : (160 * 1024) / kStage;
  static constexpr int kXDma = kBM / kRowsPerDma / kWaves;     // per wavefront and step
  static constexpr int kWDma = kBN / kRowsPerDma / kWaves;
  static constexpr int kLoads = kXDma + kWDma + kSDma;
  static_assert(kBM % 64 == 0 && kBN % 64 == 0, "a wavefront's scale load stays on one operand");
  static_assert(kBM % (kRowsPerDma * kWaves) == 0 && kBN % (kRowsPerDma * kWaves) == 0, "DMA split");
  static_assert(kStages >= 3, "the loop needs three stages");
  static_assert(MI % 4 == 0 && NI % 4 == 0, "scale bytes travel four to a register");
};

struct QqArgs {
  const uint8_t* xq;     // [M][K bits / 8]
  const uint8_t* xs;     // [M][K / 32]
  const uint8_t* wq;     // [N][K bits / 8]
  const uint8_t* ws;     // [N][K / 32]
  void* out;             // [M][N]
  int M, N, K;
};

// slot of logical piece `piece` of tile row `row`
template <int BITS>
__device__ __forceinline__ int qq_slot(int row, int piece) {
  if constexpr (BITS == 8) {
    return piece ^ (row & 7);
  } else {
    return piece ^ ((row >> 1) & 3);
  }
}

// BIG (4-bit codes): 32 x 32 x 64 instructions instead of 16 x 16 x 128.  With
// nothing but matrix instructions in a loop this GPU runs e2m1 operands at
// 3.97 PFLOP/s in the 16 x 16 x 128 form -- the rate of e4m3 operands, 3.94 --
// and at 6.9 PFLOP/s in the 32 x 32 x 64 form (e4m3: 3.8): only the larger form
// has the doubled 4-bit rate.
template <typename TO, int BITS, int MI, int NI, int WM, int WN, bool BIG = false>
__global__ __launch_bounds__(64 * WM * WN) void qq_mfma_kernel(const QqArgs a) {
  static_assert(!BIG || BITS == 4, "the 32 x 32 x 64 form pays for 4-bit codes only");
  using S = QqShape<BITS, MI, NI, WM, WN>;
  constexpr int kBM = S::kBM;
  constexpr int kBN = S::kBN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave % WN;
  const int wm = wave / WN;
  const int M = a.M, N = a.N, K = a.K;
  const int n0 = blockIdx.x * kBN;
  const int m0 = blockIdx.y * kBM;
  const int nk = K / kQqBK;
  const uint32_t row_bytes = static_cast<uint32_t>(K) * BITS / 8;
  const uint32_t srow_bytes = static_cast<uint32_t>(K) / 32;

  // ---- loader roles.  A DMA instruction of a wavefront moves kRowsPerDma rows
  // of kRowBytes: lane l lands in slot l % kSlots of row l / kSlots and fetches
  // the logical piece that belongs there.
  const int drow = lane / S::kSlots;
  const int dslot = lane % S::kSlots;
  uint32_t xoff[S::kXDma], woff[S::kWDma], soff[S::kSDma];
#pragma unroll
  for (int j = 0; j < S::kXDma; ++j) {
    const int r = (wave * S::kXDma + j) * S::kRowsPerDma + drow; // tile row
    const int m = m0 + r < M ? m0 + r : M - 1;                   // clamp: stay in bounds
    xoff[j] = static_cast<uint32_t>(m) * row_bytes + qq_slot<BITS>(r, dslot) * 16;
  }
#pragma unroll
  for (int j = 0; j < S::kWDma; ++j) {
    const int r = (wave * S::kWDma + j) * S::kRowsPerDma + drow;
    const int n = n0 + r < N ? n0 + r : N - 1;
    woff[j] = static_cast<uint32_t>(n) * row_bytes + qq_slot<BITS>(r, dslot) * 16;
  }
  // scale dwords: load j of wavefront w fills dwords (j kWaves + w) 64 .. + 63 of
  // the scale area; dword d < kBM is x row d's, d < kBM + kBN w row d - kBM's, the
  // rest repeat the last w row (a place nobody reads).  Which operand a load
  // reads is uniform per wavefront (kBM is a multiple of 64).
  auto scale_dword = [&](int j) { return (j * S::kWaves + wave) * 64 + lane; };
#pragma unroll
  for (int j = 0; j < S::kSDma; ++j) {
    const int d = scale_dword(j);
    if (d < kBM) {
      const int m = m0 + d < M ? m0 + d : M - 1;
      soff[j] = static_cast<uint32_t>(m) * srow_bytes;
    } else {
      const int r = d - kBM < kBN ? d - kBM : kBN - 1;
      const int n = n0 + r < N ? n0 + r : N - 1;
      soff[j] = static_cast<uint32_t>(n) * srow_bytes;
    }
  }

  auto lds_addr = [&](int byte_off) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) char*)(smem + byte_off)));
  };
#define QQ_DMA16(voff, gbase, lds_byte)                                          \
  do {                                                                           \
    const uint32_t m0__ = __builtin_amdgcn_readfirstlane(lds_addr(lds_byte));    \
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"            \
                 :                                                               \
                 : "v"(voff), "s"(gbase), "s"(m0__)                              \
                 : "memory");                                                    \
  } while (0)
#define QQ_DMA4(voff, gbase, lds_byte)                                           \
  do {                                                                           \
    const uint32_t m0__ = __builtin_amdgcn_readfirstlane(lds_addr(lds_byte));    \
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1"              \
                 :                                                               \
                 : "v"(voff), "s"(gbase), "s"(m0__)                              \
                 : "memory");                                                    \
  } while (0)

  // all loads of step t (clamped to the last step: the counts stay the same)
  auto issue = [&](int t) {
    const int tc = t < nk ? t : nk - 1;
    const int stage = (t % S::kStages) * S::kStage;
    const uint8_t* xg = a.xq + static_cast<size_t>(tc) * S::kRowBytes;
    const uint8_t* wg = a.wq + static_cast<size_t>(tc) * S::kRowBytes;
#pragma unroll
    for (int j = 0; j < S::kXDma; ++j) {
      QQ_DMA16(xoff[j], xg, stage + (wave * S::kXDma + j) * 1024);
    }
#pragma unroll
    for (int j = 0; j < S::kWDma; ++j) {
      QQ_DMA16(woff[j], wg, stage + S::kXTile + (wave * S::kWDma + j) * 1024);
    }
#pragma unroll
    for (int j = 0; j < S::kSDma; ++j) {
      const int first = (j * S::kWaves + wave) * 64; // uniform
      const uint8_t* sg = (first < kBM ? a.xs : a.ws) + static_cast<size_t>(tc) * 4;
      QQ_DMA4(soff[j], sg, stage + S::kXTile + S::kWTile + first * 4);
    }
  };

  if constexpr (BIG) {
    // ---- 32 x 32 tiles: MI / 2 x NI / 2 per wavefront, two instructions (the
    // halves of the 128-code step) per tile and step.  Lane l supplies row l % 32
    // and the 32 codes [64 h + 32 (l / 32), + 32) of half h: piece 2 h + l / 32.
    constexpr int MT = MI / 2;
    constexpr int NT = NI / 2;
    static_assert(NT % 2 == 0 && (MT == 1 || MT % 2 == 0), "scale bytes travel packed");
    qq_f32x16 acc[NT][MT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
      for (int j = 0; j < MT; ++j) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[i][j][r] = 0.0f;
        }
      }
    }
    const int fr = lane & 31;
    const int kblk = lane >> 5;
    constexpr int kS = S::kStages;
#pragma unroll
    for (int t = 0; t < kS - 1; ++t) {
      issue(t);
    }
    for (int t = 0; t < nk; ++t) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kS - 2) * S::kLoads) : "memory");
      __syncthreads();
      issue(t + kS - 1);
      const uint8_t* st = smem + (t % kS) * S::kStage;
      const uint32_t* sc = reinterpret_cast<const uint32_t*>(st + S::kXTile + S::kWTile);
      qq_i32x4 af[2][NT], bf[2][MT];
      // scale bytes: register q holds tiles 2 q and 2 q + 1, bytes (tile % 2) 2 + h
      int sa[(NT + 1) / 2], sb[(MT + 1) / 2];
      auto two_bytes = [&](uint32_t d) {
        // the blocks of this lane in the two halves: kblk and 2 + kblk
        return ((d >> (8 * kblk)) & 0xffu) | (((d >> (8 * (2 + kblk))) & 0xffu) << 8);
      };
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        const int xr = wm * 16 * MI + 32 * j + fr;
        const uint8_t* row = st + xr * S::kRowBytes;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint4 v = *reinterpret_cast<const uint4*>(row + qq_slot<4>(xr, 2 * h + kblk) * 16);
          bf[h][j] = qq_i32x4{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
        }
        const uint32_t two = two_bytes(sc[xr]);
        if (j % 2 == 0) {
          sb[j / 2] = static_cast<int>(two);
        } else {
          sb[j / 2] |= static_cast<int>(two << 16);
        }
      }
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int wr = wn * 16 * NI + 32 * i + fr;
        const uint8_t* row = st + S::kXTile + wr * S::kRowBytes;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint4 v = *reinterpret_cast<const uint4*>(row + qq_slot<4>(wr, 2 * h + kblk) * 16);
          af[h][i] = qq_i32x4{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
        }
        const uint32_t two = two_bytes(sc[kBM + wr]);
        if (i % 2 == 0) {
          sa[i / 2] = static_cast<int>(two);
        } else {
          sa[i / 2] |= static_cast<int>(two << 16);
        }
      }
      auto wide = [](const qq_i32x4& f) { return qq_i32x8{f[0], f[1], f[2], f[3], 0, 0, 0, 0}; };
#define QQ_MMA32(i, j, h)                                                        \
  if constexpr ((i) < NT && (j) < MT) {                                          \
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                 \
        wide(af[h][i]), wide(bf[h][j]), acc[i][j], 4, 4, ((i) % 2) * 2 + (h),    \
        sa[(i) / 2], ((j) % 2) * 2 + (h), sb[(j) / 2]);                          \
  }
#define QQ_MMA32_ROW(i, h)                                                       \
  QQ_MMA32(i, 0, h) QQ_MMA32(i, 1, h) QQ_MMA32(i, 2, h) QQ_MMA32(i, 3, h)
      QQ_MMA32_ROW(0, 0) QQ_MMA32_ROW(1, 0) QQ_MMA32_ROW(2, 0) QQ_MMA32_ROW(3, 0)
      QQ_MMA32_ROW(0, 1) QQ_MMA32_ROW(1, 1) QQ_MMA32_ROW(2, 1) QQ_MMA32_ROW(3, 1)
#undef QQ_MMA32_ROW
#undef QQ_MMA32
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // D[n][m] 32 x 32: register i of lane (col, half) holds n = 8 (i / 4) + 4 half
    // + i % 4, m = col
    TO* out = static_cast<TO*>(a.out);
    const int col = lane & 31;
    const int half = lane >> 5;
    const bool vec_ok = (N % 4) == 0;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int m = m0 + wm * 16 * MI + 32 * j + col;
      if (m >= M) {
        continue;
      }
#pragma unroll
      for (int i = 0; i < NT; ++i) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int n = n0 + wn * 16 * NI + 32 * i + 8 * g4 + 4 * half;
          if (n >= N) {
            continue;
          }
          const float v0 = acc[i][j][4 * g4 + 0], v1 = acc[i][j][4 * g4 + 1];
          const float v2 = acc[i][j][4 * g4 + 2], v3 = acc[i][j][4 * g4 + 3];
          TO* dst = out + static_cast<size_t>(m) * N + n;
          if (vec_ok && n + 4 <= N) {
            if constexpr (sizeof(TO) == 4) {
              *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
            } else {
              uint2 v;
              v.x = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(v0))) |
                  (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(v1))) << 16);
              v.y = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(v2))) |
                  (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(v3))) << 16);
              *reinterpret_cast<uint2*>(dst) = v;
            }
          } else {
            const float vals[4] = {v0, v1, v2, v3};
            for (int r = 0; r < 4 && n + r < N; ++r) {
              dst[r] = from_f32<TO>(vals[r]);
            }
          }
        }
      }
    }
    return;
  }

  qq_f32x4 acc[NI][MI]; // [n tile][m tile]
#pragma unroll
  for (int i = 0; i < NI; ++i) {
#pragma unroll
    for (int j = 0; j < MI; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }

  const int fr = lane & 15; // row inside a 16-row fragment
  const int kb = lane >> 4; // which 32 codes of the step

  // A fragment: the 32 codes a lane supplies (eight registers of 8-bit codes,
  // four of 4-bit codes).  Scale bytes travel packed, four rows to a register;
  // the instruction's op_sel picks the row's byte.
  using Frag = std::conditional_t<BITS == 8, qq_i32x8, qq_i32x4>;
  struct Frags {
    Frag af[NI], bf[MI];
    int sa[NI / 4], sb[MI / 4];
  };
  auto fragment = [&](const uint8_t* row_base, int r) -> Frag {
    const uint8_t* row = row_base + r * S::kRowBytes;
    if constexpr (BITS == 8) {
      // 8-bit operands: registers 0..3 of lane block kb hold codes 16 kb .. 16 kb + 15
      // of the step, registers 4..7 codes 64 + 16 kb ..; the scale of the codes
      // [32 b, 32 b + 32) is the one lane block b supplies
      const uint4 v0 = *reinterpret_cast<const uint4*>(row + qq_slot<8>(r, kb) * 16);
      const uint4 v1 = *reinterpret_cast<const uint4*>(row + qq_slot<8>(r, 4 + kb) * 16);
      return qq_i32x8{(int)v0.x, (int)v0.y, (int)v0.z, (int)v0.w, (int)v1.x, (int)v1.y, (int)v1.z, (int)v1.w};
    } else {
      const uint4 v0 = *reinterpret_cast<const uint4*>(row + qq_slot<4>(r, kb) * 16);
      return qq_i32x4{(int)v0.x, (int)v0.y, (int)v0.z, (int)v0.w};
    }
  };
  auto operand = [](const Frag& f) -> qq_i32x8 {
    if constexpr (BITS == 8) {
      return f;
    } else {
      return qq_i32x8{f[0], f[1], f[2], f[3], 0, 0, 0, 0};
    }
  };
  // byte kb of four rows' scale dwords, packed (row j in byte j)
  auto pack_scales = [&](const uint32_t* d) {
    const int sh = 8 * kb;
    return static_cast<int>(
        ((d[0] >> sh) & 0xffu) | (((d[16] >> sh) & 0xffu) << 8) | (((d[32] >> sh) & 0xffu) << 16) |
        ((d[48] >> sh) << 24));
  };
  // the fragments and scale bytes of step t, from its stage
  auto read_step = [&](int t, Frags& f) {
    const uint8_t* st = smem + (t % S::kStages) * S::kStage;
    const uint32_t* sc = reinterpret_cast<const uint32_t*>(st + S::kXTile + S::kWTile);
    const int xr0 = wm * 16 * MI + fr; // x tile rows xr0 + 16 j
#pragma unroll
    for (int j = 0; j < MI; ++j) {
      f.bf[j] = fragment(st, xr0 + 16 * j);
    }
#pragma unroll
    for (int q = 0; q < MI / 4; ++q) {
      f.sb[q] = pack_scales(sc + xr0 + 64 * q);
    }
    const int wr0 = wn * 16 * NI + fr; // W tile rows wr0 + 16 i
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      f.af[i] = fragment(st + S::kXTile, wr0 + 16 * i);
    }
#pragma unroll
    for (int q = 0; q < NI / 4; ++q) {
      f.sa[q] = pack_scales(sc + kBM + wr0 + 64 * q);
    }
  };
  // cbsz / blgp: the operand formats (0 = e4m3, 4 = e2m1); op_sel: which byte of
  // the scale registers
#define QQ_MMA(i, j)                                                             \
  if constexpr ((i) < NI && (j) < MI) {                                          \
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(                \
        operand(f.af[i]), operand(f.bf[j]), acc[i][j], BITS == 8 ? 0 : 4,        \
        BITS == 8 ? 0 : 4, (i) % 4, f.sa[(i) / 4], (j) % 4, f.sb[(j) / 4]);      \
  }
#define QQ_MMA_ROW(i)                                                            \
  QQ_MMA(i, 0) QQ_MMA(i, 1) QQ_MMA(i, 2) QQ_MMA(i, 3)                            \
  QQ_MMA(i, 4) QQ_MMA(i, 5) QQ_MMA(i, 6) QQ_MMA(i, 7)
  auto multiply = [&](const Frags& f) {
    QQ_MMA_ROW(0) QQ_MMA_ROW(1) QQ_MMA_ROW(2) QQ_MMA_ROW(3)
    QQ_MMA_ROW(4) QQ_MMA_ROW(5) QQ_MMA_ROW(6) QQ_MMA_ROW(7)
  };
#undef QQ_MMA_ROW
#undef QQ_MMA

  // Steps 0 .. kStages - 2 are requested up front; iteration t waits for step t,
  // asks for step t + kStages - 1 (into the stage that iteration t - 1 read) and
  // multiplies step t.  (Reading the fragments one iteration ahead of their
  // matrix instructions, from a second register set, changed nothing for the
  // 4-bit kernel and cost the 8-bit one, with its three stages, a step of lead.)
  constexpr int kS = S::kStages;
#pragma unroll
  for (int t = 0; t < kS - 1; ++t) {
    issue(t);
  }
  for (int t = 0; t < nk; ++t) {
    // the loads of steps t + 1 .. t + kStages - 2 may still be in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kS - 2) * S::kLoads) : "memory");
    __syncthreads(); // step t is in LDS for everyone; stage (t - 1) % kStages is free
    issue(t + kS - 1);
    Frags f;
    read_step(t, f);
    multiply(f);
  }
  // the clamped extra loads must have landed before the workgroup's LDS is given up
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#undef QQ_DMA16
#undef QQ_DMA4

  // D[n][m]: register r of lane (col, quad) holds n = 4 quad + r, m = col
  TO* out = static_cast<TO*>(a.out);
  const int col = lane & 15;
  const int quad = lane >> 4;
  const bool vec_ok = (N % 4) == 0;
#pragma unroll
  for (int j = 0; j < MI; ++j) {
    const int m = m0 + wm * 16 * MI + 16 * j + col;
    if (m >= M) {
      continue;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = n0 + wn * 16 * NI + 16 * i + 4 * quad;
      if (n >= N) {
        continue;
      }
      TO* dst = out + static_cast<size_t>(m) * N + n;
      if (vec_ok && n + 4 <= N) {
        if constexpr (sizeof(TO) == 4) {
          *reinterpret_cast<float4*>(dst) =
              make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
        } else {
          uint2 v;
          v.x = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(acc[i][j][0]))) |
              (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(acc[i][j][1]))) << 16);
          v.y = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(acc[i][j][2]))) |
              (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, from_f32<TO>(acc[i][j][3]))) << 16);
          *reinterpret_cast<uint2*>(dst) = v;
        }
      } else {
        for (int r = 0; r < 4 && n + r < N; ++r) {
          dst[r] = from_f32<TO>(acc[i][j][r]);
        }
      }
    }
  }
}

template <typename TO, int BITS, int MI, int NI, int WM, int WN, bool BIG = false>
int launch_qq(const QqArgs& a, hipStream_t s) {
  using S = QqShape<BITS, MI, NI, WM, WN>;
  constexpr size_t smem = static_cast<size_t>(S::kStages) * S::kStage;
  static_assert(smem <= 160 * 1024, "LDS");
  const dim3 grid((a.N + S::kBN - 1) / S::kBN, (a.M + S::kBM - 1) / S::kBM, 1);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qqmm] M=%d exceeds the grid", a.M);
  }
  auto kern = qq_mfma_kernel<TO, BITS, MI, NI, WM, WN, BIG>;
  static bool configured = false; // per instantiation
  if (!configured) {
    MLXROCM_HIP_TRY(hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern),
        hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(smem)));
    configured = true;
  }
  kern<<<grid, S::kThreads, smem, s>>>(a);
  MLXROCM_HIP_TRY(hipGetLastError());
  return static_cast<int>(MLXROCM_OK);
}

} // namespace

// Both operands as MX codes with their e8m0 scale bytes; K % 128 == 0; every
// operand below 4 GiB.  mode: MLXROCM_MXFP8 or MLXROCM_MXFP4.
bool qq_mfma_supported(int M, int N, int K, int mode) {
  const int bits = mode == MLXROCM_MXFP8 ? 8 : 4;
  const uint64_t limit = uint64_t{1} << 32;
  return (mode == MLXROCM_MXFP8 || mode == MLXROCM_MXFP4) && K % kQqBK == 0 && K >= kQqBK &&
      M >= 1 && N >= 1 && static_cast<uint64_t>(M) * K * bits / 8 < limit &&
      static_cast<uint64_t>(N) * K * bits / 8 < limit;
}

int launch_qq_mfma(
    const void* xq,
    const uint8_t* xs,
    const uint32_t* wq,
    const uint8_t* ws,
    void* out,
    int M,
    int N,
    int K,
    int mode,
    int dtype,
    hipStream_t s) {
  QqArgs a;
  a.xq = static_cast<const uint8_t*>(xq);
  a.xs = xs;
  a.wq = reinterpret_cast<const uint8_t*>(wq);
  a.ws = ws;
  a.out = out;
  a.M = M;
  a.N = N;
  a.K = K;
  MLXROCM_REHEARSE("qq_mfma(%s)", mode == MLXROCM_MXFP8 ? "e4m3" : "e2m1");
  return dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    if (mode == MLXROCM_MXFP8) {
      return launch_qq<T, 8, 4, 4, 4, 2>(a, s);
    }
    // the wide tile where it still fills the chip
    const long wide = static_cast<long>((M + 255) / 256) * ((N + 255) / 256);
    if (wide >= compute_units()) {
      return launch_qq<T, 4, 4, 8, 4, 2, true>(a, s);
    }
    return launch_qq<T, 4, 4, 4, 4, 2, true>(a, s);
  });
}

} // namespace mlxrocm
