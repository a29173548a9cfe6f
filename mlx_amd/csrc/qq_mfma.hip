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

constexpr int kQqBM = 256;
constexpr int kQqBK = 128; // codes per step
constexpr int kQqThreads = 512;

// NI: 16-column tiles per wavefront along n (4 or 8): the workgroup's tile is
// 256 x 32 NI.  The wider tile halves the bytes fetched per flop; 8-bit codes
// keep the narrow one, whose three stages are what LDS holds.
template <int BITS, int NI>
struct QqShape {
  static constexpr int kBN = 32 * NI;
  static constexpr int kRowBytes = kQqBK * BITS / 8;          // 128 or 64
  static constexpr int kSlots = kRowBytes / 16;                // 16-byte pieces per row: 8 or 4
  static constexpr int kRowsPerDma = 1024 / kRowBytes;         // rows one wavefront load moves: 8 or 16
  static constexpr int kXTile = kQqBM * kRowBytes;             // bytes
  static constexpr int kWTile = kBN * kRowBytes;
  static constexpr int kStage = kXTile + kWTile + 2048;
  static constexpr int kStages = BITS == 8 ? 3 : (NI == 8 ? 4 : 6);
  static constexpr int kXDma = kQqBM / kRowsPerDma / 8;         // per wavefront and step: 4 or 2
  static constexpr int kWDma = kBN / kRowsPerDma / 8;           // 1, 2 or 4
  static constexpr int kLoads = kXDma + kWDma + 1;              // + the scale dwords
  static_assert(kQqBM + kBN <= 512, "one scale dword per thread");
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

template <typename TO, int BITS, int NI>
__global__ __launch_bounds__(kQqThreads) void qq_mfma_kernel(const QqArgs a) {
  using S = QqShape<BITS, NI>;
  constexpr int kQqBN = S::kBN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1;
  const int wm = wave >> 1;
  const int M = a.M, N = a.N, K = a.K;
  const int n0 = blockIdx.x * kQqBN;
  const int m0 = blockIdx.y * kQqBM;
  const int nk = K / kQqBK;
  const uint32_t row_bytes = static_cast<uint32_t>(K) * BITS / 8;
  const uint32_t srow_bytes = static_cast<uint32_t>(K) / 32;

  // ---- loader roles.  A DMA instruction of a wavefront moves kRowsPerDma rows
  // of kRowBytes: lane l lands in slot l % kSlots of row l / kSlots and fetches
  // the logical piece that belongs there.
  const int drow = lane / S::kSlots;
  const int dslot = lane % S::kSlots;
  uint32_t xoff[S::kXDma], woff[S::kWDma];
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
  // scale dwords: thread t < 256 fetches x row t's, t < 384 w row t - 256's, the
  // rest repeat the last w row (same value, a place nobody reads)
  uint32_t soff;
  const uint8_t* sbase;
  if (tid < kQqBM) {
    const int m = m0 + tid < M ? m0 + tid : M - 1;
    soff = static_cast<uint32_t>(m) * srow_bytes;
  } else {
    const int r = tid - kQqBM < kQqBN ? tid - kQqBM : kQqBN - 1;
    const int n = n0 + r < N ? n0 + r : N - 1;
    soff = static_cast<uint32_t>(n) * srow_bytes;
  }
  // waves 0..3 hold x rows, 4..7 w rows: uniform per wavefront
  sbase = wave < 4 ? a.xs : a.ws;

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
    QQ_DMA4(soff, sbase + static_cast<size_t>(tc) * 4, stage + S::kXTile + S::kWTile + wave * 256);
  };

  qq_f32x4 acc[NI][4]; // [n tile][m tile]
#pragma unroll
  for (int i = 0; i < NI; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
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
    Frag af[NI], bf[4];
    int sa[NI / 4], sb;
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
  auto pack_scales = [&](uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3) {
    const int sh = 8 * kb;
    return static_cast<int>(
        ((d0 >> sh) & 0xffu) | (((d1 >> sh) & 0xffu) << 8) | (((d2 >> sh) & 0xffu) << 16) |
        ((d3 >> sh) << 24));
  };
  // the fragments and scale bytes of step t, from its stage
  auto read_step = [&](int t, Frags& f) {
    const uint8_t* st = smem + (t % S::kStages) * S::kStage;
    const uint32_t* sc = reinterpret_cast<const uint32_t*>(st + S::kXTile + S::kWTile);
    const int xr0 = wm * 64 + fr; // x tile rows xr0 + 16 j
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f.bf[j] = fragment(st, xr0 + 16 * j);
    }
    f.sb = pack_scales(sc[xr0], sc[xr0 + 16], sc[xr0 + 32], sc[xr0 + 48]);
    const int wr0 = wn * 16 * NI + fr; // W tile rows wr0 + 16 i
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      f.af[i] = fragment(st + S::kXTile, wr0 + 16 * i);
    }
#pragma unroll
    for (int q = 0; q < NI / 4; ++q) {
      const uint32_t* sw = sc + kQqBM + wr0 + 64 * q;
      f.sa[q] = pack_scales(sw[0], sw[16], sw[32], sw[48]);
    }
  };
  // cbsz / blgp: the operand formats (0 = e4m3, 4 = e2m1); op_sel: which byte of
  // the scale registers
#define QQ_MMA(i, j)                                                             \
  acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(                  \
      operand(f.af[i]), operand(f.bf[j]), acc[i][j], BITS == 8 ? 0 : 4,          \
      BITS == 8 ? 0 : 4, (i) % 4, f.sa[(i) / 4], (j), f.sb);
#define QQ_MMA_ROW(i)                                                            \
  if constexpr ((i) < NI) {                                                      \
    QQ_MMA(i, 0) QQ_MMA(i, 1) QQ_MMA(i, 2) QQ_MMA(i, 3)                          \
  }
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
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + wm * 64 + 16 * j + col;
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

template <typename TO, int BITS, int NI>
int launch_qq(const QqArgs& a, hipStream_t s) {
  using S = QqShape<BITS, NI>;
  constexpr int kQqBN = S::kBN;
  constexpr size_t smem = static_cast<size_t>(S::kStages) * S::kStage;
  static_assert(smem <= 160 * 1024, "LDS");
  const dim3 grid((a.N + kQqBN - 1) / kQqBN, (a.M + kQqBM - 1) / kQqBM, 1);
  if (grid.y > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qqmm] M=%d exceeds the grid", a.M);
  }
  auto kern = qq_mfma_kernel<TO, BITS, NI>;
  static bool configured = false; // per instantiation
  if (!configured) {
    MLXROCM_HIP_TRY(hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern),
        hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(smem)));
    configured = true;
  }
  kern<<<grid, kQqThreads, smem, s>>>(a);
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
      return launch_qq<T, 8, 4>(a, s);
    }
    // the wide tile where it still fills the chip
    const long wide = static_cast<long>((M + kQqBM - 1) / kQqBM) * ((N + 255) / 256);
    if (wide >= compute_units()) {
      return launch_qq<T, 4, 8>(a, s);
    }
    return launch_qq<T, 4, 4>(a, s);
  });
}

} // namespace mlxrocm
