// qmm_mfma_tile.h -- the tile kernel of the prefill GEMM (transpose=true, large M) for 16-bit element
// types and every code width, on the gfx950 matrix cores.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T
//
// A workgroup of 512 threads (8 wavefronts: 4 along M x 2 along N) owns a
// 256 (M) x BN (N) tile of y, BN = 32 NT with NT in {5, 6, 7} chosen on the host
// so that the tile count fills the compute units evenly, and walks K in steps
// of 64 through two LDS stages.  Per step:
//   * the x tile (256 x 64) and the packed W tile (BN rows x 64 codes) of the
//     step after next are fetched into registers;
//   * W is dequantized exactly once per workgroup -- thread (n, h) expands the
//     32 codes [32h, 32h+32) of row n with one scale/bias pair (a K-step never
//     holds more than one group per 32 codes) as fp32 fma(s, code, b), rounds to
//     T and stores them to the idle LDS stage, so the 256 rows of x reuse every
//     weight;
//   * each wavefront computes a 16 NT (N) x 64 (M) block of y^T with
//     v_mfma_f32_16x16x32: A operand = W rows, B operand = x rows, so that a lane
//     ends up with 4 consecutive n of one m.
// The vector-ALU, LDS and global-memory instructions of a step are placed by
// hand in the slots between the MFMAs (one scheduling barrier per slot), so the
// matrix pipe never waits for a block of dequantization work.
// fp32 operands run on the same bf16 matrix path at three times the K length:
// a pre-pass splits x into a high and a low bf16 part, laid out per 64-wide k
// block as [hi | lo | hi]; the kernel pairs those blocks with the weights'
// [hi | hi | lo] parts (dequantized in fp32, split on the fly), which sums to
// x_hi w_hi + x_lo w_hi + x_hi w_lo with fp32 accumulation -- a relative error
// of about 2^-17 per product, inside the fp32 tolerance of the path.
// The x tile never passes through registers: global_load_lds_dwordx4 moves 16
// bytes per lane straight into LDS (a wavefront's 64 pieces land contiguously,
// eight 128-byte rows), three stages deep, with the pieces of a row XOR-swizzled
// by the row number so that the 16-byte fragment reads of 16 consecutive rows
// spread over the banks (an LDS store from registers costs the matrix pipe
// about 30 clocks of issue on its SIMD; the x tile was half of them).  The W
// tile uses the same unpadded, swizzled rows (measured: fragment reads of
// 144-byte padded rows run 20 % slower than swizzled 128-byte rows).  The finished tile is staged through LDS once more so that y is
// written in full 16-byte, row-contiguous stores.
#pragma once

#include "mfma_dequant.h"
#include "mfma_loads.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kBM = 256;
constexpr int kBK = 64;
constexpr int kThreads = 512;
constexpr int kOutPad = 8; // elements of padding per row of the staged y tile

// ---- placement of the side work in the MFMA slots of one K-step -------------
// NS = 8 NT slots.  Everything that writes LDS has to be issued before the
// barrier in slot NS - 14, so the 16 dequantization pairs are spread over the
// first NS - 16 slots: pair q goes to slot q (NS - 16) / 16, the 16-byte store
// of pairs 4r..4r+3 to the slot after pair 4r+3, the direct-to-LDS load of x
// row block i to slot xdma_slot(i) and the packed-W fetch to slot 0.
constexpr int pair_slot(int q, int ns) {
  return q * (ns - 16) / 16;
}
// The four direct-to-LDS loads of an x tile are spread evenly over the slots
// before the barrier: bunched together they compete with the fragment reads for
// the LDS, and every one of them has to be issued before the barrier's wait
// counts it.
constexpr int xdma_slot(int i, int ns) {
  return 1 + i * (ns - 17) / 3;
}
constexpr int pair_at(int m, int ns) {
  for (int q = 0; q < 16; ++q) {
    if (pair_slot(q, ns) == m) {
      return q;
    }
  }
  return -1;
}
constexpr int wstore_at(int m, int ns) {
  for (int r = 0; r < 4; ++r) {
    if (pair_slot(4 * r + 3, ns) + 1 == m) {
      return r;
    }
  }
  return -1;
}

// GROUPED: blockIdx.y walks the tile list of a gather grouped by expert (M == 1
// per index pair): the tile's rows are the x rows of up to 256 index pairs that
// share one expert, fetched and written back through the permutation.
//
// T is the MFMA operand type (what x and the LDS tiles hold), TS the type of
// scales and biases: the same as T, or float in the split fp32 mode (where a.x
// points at the [hi | lo | hi] bf16 image of x and spans 3 K).  TO is the type
// of y: TS, or float when K is cut into k_splits ranges (blockIdx.z), each of
// which writes its partial tile to plane blockIdx.z of a.out.
//
// WN: the weights are [K, N] with the codes (and the groups) running along n
// (transpose=false).  Only the W loader differs: a thread then owns a 4 (k) x
// 8 (n) block of the step's tile -- one word (4-bit) or two (8-bit) from each of
// four consecutive rows of W, each row with its own scale and bias -- and
// stores it to the same [n][k] LDS tile as eight 8-byte column pieces.
// SBI: a.scales points at the image of (scale, bias) pairs (QmmArgs::sb_transposed
// == 2): one dword load per thread and K-step instead of two 16-bit loads.
// FP != 0: the codes are e2m1 / e4m3 numbers (FpPairDequant's modes) instead of
// affine integers; the pair image then holds, per 32 codes, the scale of the
// first 16 in the low half and of the last 16 in the high half (gs_shift == 5).
// FP == 3 (nvfp4) also honours QmmArgs::out_scale.
template <typename T, typename TS, typename TO, int BITS, int NT, bool GROUPED, bool WN = false,
          bool SBI = false, int FP = 0>
__global__ __launch_bounds__(kThreads) void qmm_t_mfma_kernel(
    const QmmArgs a,
    const int gs_shift,
    const int k_splits) {
  constexpr bool kSplit = !std::is_same<T, TS>::value;
  static_assert(!(kSplit && GROUPED), "the grouped gather runs on 16-bit types only");
  static_assert(!(WN && kSplit), "[K, N] weights: 16-bit problems only");
  static_assert(!WN || BITS == 4 || BITS == 8, "[K, N] weights: 4- and 8-bit codes");
  static_assert(
      !SBI || (!WN && !kSplit && sizeof(TS) == 2 && (!GROUPED || FP != 0)),
      "pair image: plain 16-bit launches, and the grouped gather of the fp modes");
  static_assert(FP == 0 || (SBI && BITS == (FP == 2 ? 8 : 4)), "fp codes: pair image, 4 or 8 bits");
  using DQ = std::conditional_t<FP != 0, FpPairDequant<T, (FP != 0 ? FP : 1)>, PairDequant<T, BITS>>;
  constexpr int kBN = 32 * NT;
  constexpr int kNS = 8 * NT; // MFMAs per wavefront per K-step
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // three unpadded x stages (filled by direct-to-LDS loads), then two W stages
  constexpr int kXTile = kBM * kBK; // elements
  constexpr int kXStages = 3;
  constexpr int kWTile = kBN * kBK; // unpadded rows, pieces XOR-swizzled like x
  constexpr int kWBase = kXStages * kXTile;
  T* lds = reinterpret_cast<T*>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1;  // which 16 NT columns (n) of the tile
  const int wm = wave >> 1; // which 64 rows (m) of the tile
  const int N = a.N;
  const int K = a.K;
  const int n0 = blockIdx.x * kBN;
  int M = a.M;
  int m0 = blockIdx.y * kBM;
  int row0 = 0; // grouped: first sorted position of the tile
  // operands of this workgroup's problem
  struct {
    const T* x;
    const uint8_t* w;
    const TS* scales;
    const TS* biases;
    TO* out;
    bool valid;
  } p;
  if constexpr (GROUPED) {
    const int tile = blockIdx.y;
    if (tile >= *a.group_ntiles) {
      return; // the grid covers the worst-case tile count
    }
    const int e = a.group_tiles[3 * tile];
    row0 = a.group_tiles[3 * tile + 1];
    M = a.group_tiles[3 * tile + 2];
    m0 = 0;
    p.x = static_cast<const T*>(a.x);
    p.w = reinterpret_cast<const uint8_t*>(a.w + static_cast<int64_t>(e) * a.w_batch_stride);
    p.scales = static_cast<const TS*>(a.scales) + static_cast<int64_t>(e) * a.sb_batch_stride;
    p.biases = static_cast<const TS*>(a.biases) + static_cast<int64_t>(e) * a.sb_batch_stride;
    p.out = static_cast<TO*>(a.out);
    p.valid = true;
  } else {
    // same resolution as resolve_problem(), with the two element types; with a
    // split K there is one problem and blockIdx.z is the split
    const int l = k_splits > 1 ? 0 : blockIdx.z;
    int64_t xb = l;
    int64_t wb = l;
    p.valid = true;
    if (a.lhs_indices != nullptr) {
      const uint32_t xi = a.lhs_indices[l];
      const uint32_t wi = a.rhs_indices[l];
      p.valid = xi < static_cast<uint32_t>(a.x_batches) && wi < static_cast<uint32_t>(a.n_experts);
      xb = p.valid ? xi : 0;
      wb = p.valid ? wi : 0;
    }
    p.x = static_cast<const T*>(a.x) + xb * a.x_batch_stride;
    p.w = reinterpret_cast<const uint8_t*>(a.w + wb * a.w_batch_stride);
    p.scales = static_cast<const TS*>(a.scales) + wb * a.sb_batch_stride;
    p.biases = static_cast<const TS*>(a.biases) + wb * a.sb_batch_stride;
    const int64_t plane = k_splits > 1 ? blockIdx.z : l;
    p.out = static_cast<TO*>(a.out) + plane * a.M * static_cast<int64_t>(a.N);
  }
  // x as the kernel sees it: three 64-wide blocks per block of K when split
  const int Kx = kSplit ? 3 * K : K;

  // groups and packed words per row of W (rows run along k, or along n when WN)
  const int groups = (WN ? N : K) >> gs_shift;
  const int row_words = (WN ? N : K) / 32 * BITS;

  // ---- loader roles ----
  // x: wavefront w moves rows 32 w + 8 i .. + 7 of the tile with its i-th load
  // (i < 4); lane l lands in piece l % 8 of row l / 8 and fetches the row's
  // logical piece (l % 8) ^ (l / 8).
  const int xr = wave * 32 + (lane >> 3);
  const int xc = (lane & 7) ^ (lane >> 3);
  // W: thread (wr, wh) covers codes [32 wh, 32 wh + 32) of tile row wr; the
  // threads past the tile's rows repeat its last row (same values, same place).
  const int wr = (tid >> 1) < kBN ? (tid >> 1) : kBN - 1;
  const int wh = tid & 1;
  // WN: thread (kg, ng) covers rows 4 kg .. 4 kg + 3 of the step and columns
  // 8 ng .. 8 ng + 7 of the tile; kg runs fastest, so that the 8-byte LDS
  // stores of 16 neighbouring lanes fill one 128-byte tile row.  Threads past
  // the tile repeat its last block.
  constexpr int kColBlocks = kBN / 8;
  constexpr int kWPR = BITS / 4 > 0 ? BITS / 4 : 1; // words per 8 codes (WN: 1 or 2)
  constexpr int kSB = WN ? 4 : 1;                   // scale / bias pairs per thread
  const int wt = tid < 16 * kColBlocks ? tid : 16 * kColBlocks - 1;
  const int kg = wt & 15;
  const int ng = wt >> 4;
  // Where the dequantized weights go in a W stage (element offsets).  Rows are
  // 64 elements, eight 16-byte pieces; piece c of row r sits at c ^ (r % 8).
  // transpose=true: thread (wr, wh) writes pieces 4 wh + j, j < 4, of row wr.
  int wrow_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wrow_off[j] = wr * kBK + (((4 * wh + j) ^ (wr & 7)) * 8);
  }
  // [K, N] weights: the thread's column i (row 8 ng + i of the tile, so r % 8 == i)
  // takes 8 bytes at k = 4 kg: half (kg % 2) of piece kg / 2
  auto wcol_off = [&](int i) { return (8 * ng + i) * kBK + (((kg >> 1) ^ i) * 8) + (kg & 1) * 4; };

  // Per-lane byte offsets from the operands' uniform base pointers (32 bits:
  // the launcher checks the sizes); the K-step's part of an address is uniform
  // and goes into the scalar base, so the loop computes no addresses per lane.
  uint32_t w_voff, sb_voff;
  if constexpr (WN) {
    const int ncol = (n0 + 8 * ng < N) ? n0 + 8 * ng : N - 8; // clamp: stay in bounds
    w_voff = (static_cast<uint32_t>(4 * kg) * row_words + ncol / 8 * kWPR) * 4u;
    // scales / biases arrive transposed, [group][k] (the launcher's pre-pass): the
    // four rows' values are 8 contiguous bytes
    sb_voff = (static_cast<uint32_t>(ncol >> gs_shift) * K + 4 * kg) * static_cast<uint32_t>(sizeof(TS));
  } else {
    const int w_row = (n0 + wr < N) ? n0 + wr : N - 1; // clamp: loads stay in bounds
    w_voff = (static_cast<uint32_t>(w_row) * row_words + wh * BITS) * 4u;
    // group g of row w_row: [row][g], or [g][row] in the transposed image
    sb_voff = (a.sb_transposed ? static_cast<uint32_t>(w_row)
                               : static_cast<uint32_t>(w_row) * groups) *
        static_cast<uint32_t>(SBI ? 2 * sizeof(TS) : sizeof(TS));
  }
  // elements of TS between two groups of one row (pairs: two elements each)
  const size_t sb_gstride = a.sb_transposed ? static_cast<size_t>(N) * (SBI ? 2 : 1) : 1;
  // thread (wr, wh) needs the group of codes [32 wh, 32 wh + 32) of the step:
  // group (k0 + 32 wh) >> gs_shift, i.e. one further than the step's first group
  // only when groups are 32 wide and wh == 1
  const uint32_t sb_half = (!WN && gs_shift == 5 && wh == 1)
      ? static_cast<uint32_t>(sb_gstride * sizeof(TS)) : 0u;
  // Rows of x past M are never stored, so they may read any valid row: the
  // loads then need no predicate.  32-bit byte offsets from p.x.
  uint32_t xoff0, xoff1, xoff2, xoff3;
  {
    auto row_off = [&](int i) {
      const int m = m0 + xr + 8 * i;
      const int mc = m < M ? m : M - 1;
      if constexpr (GROUPED) {
        const uint32_t pair = static_cast<uint32_t>(a.group_perm[row0 + mc]);
        return (a.lhs_indices[pair] * static_cast<uint32_t>(a.x_batch_stride) + xc * 8) * 2u;
      } else {
        return (static_cast<uint32_t>(mc) * static_cast<uint32_t>(Kx) + xc * 8) * 2u;
      }
    };
    xoff0 = row_off(0);
    xoff1 = row_off(1);
    xoff2 = row_off(2);
    xoff3 = row_off(3);
  }

  // registers of the tiles in flight: the packed W of the next K-step and of
  // the step after that (wnext), fetched a whole step ahead
  uint32_t wreg[BITS];
  RawWords<WN ? 1 : BITS> wnext;                 // transpose=true: BITS consecutive words
  RawWords<(WN ? BITS / 4 : 1)> wnext_row[4];    // WN: the words of each of four rows
  uint32_t sreg, breg, snext, bnext = 0;         // one scale / bias as loaded
  uint2 swn, bwn;                                // WN: four 16-bit values each
  RawTuple<2> swn_next, bwn_next;
  // load instructions one QMM_LOAD_W issues (vmcnt counts instructions)
  constexpr int kWLoads = WN ? 6 : (BITS > 4 ? 2 : 1) + (SBI ? 1 : 2);
  auto wn_value = [](const uint2& v, int j) {
    const uint32_t word = j < 2 ? v.x : v.y;
    return to_f32(__builtin_bit_cast(TS, static_cast<
        std::conditional_t<sizeof(TS) == 2, uint16_t, uint32_t>>(word >> (16 * (j & 1)))));
  };

// x rows 32 w + 8 i .. + 7 of the tile at k0, straight into LDS stage `xs`
// (element offset of the stage); completion is counted by vmcnt.
#define QMM_DMA_X1(xs, k0, i, xoff)                                              \
  do {                                                                           \
    const T* g__ = p.x + (k0); /* uniform */                                     \
    const uint32_t m0__ = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(     \
        (__attribute__((address_space(3))) char*)(lds + (xs) + (wave * 32 + 8 * (i)) * kBK))); \
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"            \
                 :                                                               \
                 : "v"(xoff), "s"(g__), "s"(m0__)                                \
                 : "memory");                                                    \
  } while (0)
#define QMM_DMA_X(xs, k0)                                                        \
  do {                                                                           \
    QMM_DMA_X1(xs, k0, 0, xoff0);                                                \
    QMM_DMA_X1(xs, k0, 1, xoff1);                                                \
    QMM_DMA_X1(xs, k0, 2, xoff2);                                                \
    QMM_DMA_X1(xs, k0, 3, xoff3);                                                \
  } while (0)

#define QMM_LOAD_W(k0)                                                           \
  do {                                                                           \
    if constexpr (WN) {                                                          \
      const uint32_t* wp__ = reinterpret_cast<const uint32_t*>(p.w) +            \
          static_cast<size_t>(k0) * row_words; /* uniform */                     \
      _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                      \
        wnext_row[j__].load(w_voff, wp__ + static_cast<size_t>(j__) * row_words); \
      }                                                                          \
      swn_next.template load<0>(sb_voff, p.scales + (k0));                       \
      bwn_next.template load<0>(sb_voff, p.biases + (k0));                       \
    } else {                                                                     \
      /* split mode: blocks 3t, 3t+1, 3t+2 of x all meet block t of W */         \
      const int kw__ = kSplit ? ((k0) / (3 * kBK)) * kBK : (k0);                 \
      wnext.load(w_voff, reinterpret_cast<const uint32_t*>(p.w) + (kw__ / 32) * BITS); \
      /* a K-step lies inside one group when groups are 64 or 128 wide; with    \
         32-wide groups the two halves of a row differ by one group */          \
      const size_t g0__ = static_cast<size_t>(kw__ >> gs_shift) * sb_gstride;    \
      if constexpr (SBI) {                                                       \
        asm volatile("global_load_dword %0, %1, %2"                              \
                     : "=v"(snext)                                               \
                     : "v"(sb_voff + sb_half), "s"(p.scales + g0__));            \
      } else {                                                                   \
        raw_load_value<TS>(snext, sb_voff + sb_half, p.scales + g0__);           \
        raw_load_value<TS>(bnext, sb_voff + sb_half, p.biases + g0__);           \
      }                                                                          \
    }                                                                            \
  } while (0)

// Behind the wait that covers the loads of QMM_LOAD_W: from here on the loaded
// registers may be read (QMM_ROTATE_W).
#define QMM_PIN_W()                                                              \
  do {                                                                           \
    if constexpr (WN) {                                                          \
      _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                      \
        wnext_row[j__].pin();                                                    \
      }                                                                          \
      swn_next.pin();                                                            \
      bwn_next.pin();                                                            \
    } else {                                                                     \
      wnext.pin();                                                               \
      asm volatile("" : "+v"(snext), "+v"(bnext));                               \
    }                                                                            \
  } while (0)

#define QMM_ROTATE_W()                                                           \
  do {                                                                           \
    if constexpr (WN) {                                                          \
      _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                      \
        _Pragma("unroll") for (int u__ = 0; u__ < kWPR; ++u__) {                 \
          wreg[j__ * kWPR + u__] = wnext_row[j__].get(u__);                      \
        }                                                                        \
      }                                                                          \
      swn = make_uint2(swn_next.get(0), swn_next.get(1));                        \
      bwn = make_uint2(bwn_next.get(0), bwn_next.get(1));                        \
    } else {                                                                     \
      _Pragma("unroll") for (int j__ = 0; j__ < BITS; ++j__) {                   \
        wreg[j__] = wnext.get(j__);                                              \
      }                                                                          \
      sreg = snext;                                                              \
      breg = SBI ? snext >> 16 : bnext;                                          \
    }                                                                            \
  } while (0)

#define QMM_STORE_W(stage)                                                       \
  do {                                                                           \
    T* ws__ = lds + kWBase + (stage) * kWTile;                                   \
    uint32_t dq__[16];                                                           \
    if constexpr (WN) {                                                          \
      float sf__[4], bf__[4];                                                    \
      _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                      \
        sf__[j__] = wn_value(swn, j__);                                          \
        bf__[j__] = wn_value(bwn, j__);                                          \
      }                                                                          \
      dequant_cols<T, BITS>(wreg, sf__, bf__, dq__);                             \
      _Pragma("unroll") for (int i__ = 0; i__ < 8; ++i__) {                      \
        *reinterpret_cast<uint2*>(ws__ + wcol_off(i__)) =                        \
            make_uint2(dq__[2 * i__], dq__[2 * i__ + 1]);                        \
      }                                                                          \
    } else {                                                                     \
      if constexpr (FP != 0) {                                                   \
        dequant32_fp<T, (FP != 0 ? FP : 1)>(                                     \
            wreg, raw_value<TS>(sreg), raw_value<TS>(breg), dq__);               \
      } else {                                                                   \
        dequant32<T, BITS>(wreg, raw_value<TS>(sreg), raw_value<TS>(breg), dq__); \
      }                                                                          \
      _Pragma("unroll") for (int j__ = 0; j__ < 4; ++j__) {                      \
        *reinterpret_cast<uint4*>(ws__ + wrow_off[j__]) = make_uint4(            \
            dq__[4 * j__], dq__[4 * j__ + 1], dq__[4 * j__ + 2], dq__[4 * j__ + 3]); \
      }                                                                          \
    }                                                                            \
  } while (0)

  // ---- accumulators: NT (n) x 4 (m) tiles of 16 x 16 ----
  floatx4 acc[NT][4];
#pragma unroll
  for (int i = 0; i < NT; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }

  const int fi = lane & 15; // fragment row inside a 16-row MFMA tile
  const int fk = lane >> 4; // which 8 of the 32 k of an MFMA step
  // x fragment of k slice s: logical piece 4 s + fk of row fi (+ multiples of
  // 16), which sits at piece (4 s + fk) ^ (fi % 8)
  const int xfrag_off0 = (wm * 64 + fi) * kBK + ((fk) ^ (fi & 7)) * 8;
  const int xfrag_off1 = (wm * 64 + fi) * kBK + ((4 + fk) ^ (fi & 7)) * 8;
  const int wfrag_off0 = kWBase + (wn * 16 * NT + fi) * kBK + ((fk) ^ (fi & 7)) * 8;
  const int wfrag_off1 = kWBase + (wn * 16 * NT + fi) * kBK + ((4 + fk) ^ (fi & 7)) * 8;

  // MFMA operand fragments.  All four x fragments of a 32-wide k slice stay in
  // registers (two sets, one per slice); the W fragments stream through a ring
  // of four, each read three groups of four MFMAs before its first use.  W
  // fragment number g of a step is (slice g / NT, tile g % NT); numbers 2 NT..
  // are the first fragments of the next step.
  uint4 bfr[2][4];
  uint4 afr[4];
  // `xs`: element offset of the x stage
  auto read_b = [&](int xs, int s, int b) {
    bfr[s][b] = *reinterpret_cast<const uint4*>(
        lds + xs + (s == 0 ? xfrag_off0 : xfrag_off1) + b * 16 * kBK);
  };
  auto read_a = [&](int stage, int s, int t, int slot) {
    afr[slot] = *reinterpret_cast<const uint4*>(
        lds + stage * kWTile + (s == 0 ? wfrag_off0 : wfrag_off1) + t * 16 * kBK);
  };

  // ---- software pipeline, one barrier per K-step.  Step t issues 8 NT MFMAs
  // on tile t (LDS stage t%2); the slots between them carry, in a fixed order,
  //   * the fragment reads that the MFMAs three groups later need,
  //   * the dequantization of this thread's 32 codes of W tile t+1 (two codes
  //     per slot) and its four 16-byte stores to the idle stage,
  //   * the stores of x tile t+1, each followed by the fetch of the same rows
  //     of a later x tile into the registers just freed,
  //   * the fetch of the packed W of tile t+2 (one step ahead of its use),
  //   * in slot NS - 14 the barrier: by then this wavefront has issued all its
  //     LDS writes of tile t+1 and all its reads of tile t.  The remaining slots
  //     already read the first fragments of tile t+1, so the next step starts
  //     without waiting for LDS.
  // Every step is the same code, the last one included: its fetches are clamped
  // to the last tile and what it stores is never read.
  // This workgroup's K range, in steps of the x image: everything, or split
  // blockIdx.z of k_splits (whole groups of three steps in the split fp32 mode).
  int step_begin = 0;
  int nk = Kx / kBK;
  if (k_splits > 1) {
    constexpr int kUnit = kSplit ? 3 : 1;
    const int units = nk / kUnit;
    const int z = blockIdx.z;
    step_begin = units * z / k_splits * kUnit;
    nk = units * (z + 1) / k_splits * kUnit - step_begin;
  }
  const int kbeg = step_begin * kBK;
  const int klast = (nk - 1) * kBK;
  // x-image offset of local step t, clamped to the range's last step
  auto kclamp = [&](int t) { return kbeg + (t * kBK < klast ? t * kBK : klast); };
  // x tiles 0 and 1 on their way into stages 0 and 1, W tile 0 dequantized into
  // its stage, the packed W of tile 1 in registers
  QMM_DMA_X(0, kbeg);
  QMM_LOAD_W(kbeg);
  QMM_DMA_X(kXTile, kclamp(1));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  QMM_PIN_W();
  __builtin_amdgcn_sched_barrier(0);
  QMM_ROTATE_W();
  QMM_STORE_W(0);
  QMM_LOAD_W(kclamp(1));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // x tiles 0 and 1 have landed too
  QMM_PIN_W();
  __builtin_amdgcn_sched_barrier(0);
  QMM_ROTATE_W();
  __syncthreads();
  int xs_cur = 0;            // stage of the tile being multiplied
  int xs_nxt = kXTile;       // stage of the next tile
  int xs_new = 2 * kXTile;   // free stage: receives the tile after that
  read_b(xs_cur, 0, 0);
  read_a(0, 0, 0, 0);
  read_b(xs_cur, 0, 1);
  read_b(xs_cur, 0, 2);
  read_b(xs_cur, 0, 3);
  read_a(0, 0, 1, 1);
  read_a(0, 0, 2, 2);
  read_a(0, 0, 3, 3);

  // One slot: MFMA number m of a step of parity P and the side work assigned
  // to it.  `t` is the step, cur/nxt its LDS stages.
// MM: the wavefront's 64 rows of the tile hold rows of x (below M).  A
// wavefront whose rows all lie past M (a tile with fewer than 193 rows) takes
// the slots without their matrix instruction and fragment reads: it still loads,
// dequantizes and stores its share of W and joins the barriers, and leaves its
// SIMD's matrix pipe to the wavefront beside it.
#define QMM_SLOT(m, P, MM)                                                       \
  if constexpr ((m) < kNS) {                                                     \
    constexpr int s__ = (m) / (4 * NT);                                          \
    constexpr int t__ = ((m) % (4 * NT)) / 4;                                    \
    constexpr int b__ = (m) % 4;                                                 \
    constexpr int g__ = s__ * NT + t__;              /* W fragment number */     \
    constexpr int e__ = ((P) * 2 * NT + g__) % 4;    /* its ring entry */        \
    if constexpr (MM) {                                                          \
      acc[t__][b__] = mfma16<T>(afr[e__], bfr[s__][b__], acc[t__][b__]);         \
      if constexpr (b__ == 3) {                                                  \
        /* the ring entry just retired takes fragment g + 4 */                   \
        if constexpr (g__ + 4 < 2 * NT) {                                        \
          read_a(cur, (g__ + 4) / NT, (g__ + 4) % NT, e__);                      \
        } else {                                                                 \
          read_a(nxt, 0, g__ + 4 - 2 * NT, e__);                                 \
        }                                                                        \
      }                                                                          \
      if constexpr (s__ == 0 && t__ >= NT - 4 && b__ == 1) {                     \
        read_b(xs_cur, 1, t__ - (NT - 4));                                       \
      }                                                                          \
      if constexpr ((m) == kNS - 12 || (m) == kNS - 11 || (m) == kNS - 10 ||     \
                    (m) == kNS - 8) {                                            \
        read_b(xs_nxt, 0, (m) == kNS - 8 ? 3 : (m) - (kNS - 12));                \
      }                                                                          \
    }                                                                            \
    if constexpr ((m) == 0) {                                                    \
      QMM_LOAD_W(k2);                                                            \
    }                                                                            \
    if constexpr (pair_at((m), kNS) >= 0) {                                      \
      if constexpr (WN) {                                                        \
        dqv[pair_at((m), kNS)] = cdq.template pair<pair_at((m), kNS)>(wreg, sf, bf); \
      } else {                                                                   \
        dqv[pair_at((m), kNS)] =                                                 \
            dq.template pair<pair_at((m), kNS)>(wreg, sf[0], bf[0], low_part);   \
      }                                                                          \
    }                                                                            \
    if constexpr (wstore_at((m), kNS) >= 0) {                                    \
      constexpr int r__ = wstore_at((m), kNS);                                   \
      if constexpr (WN) {                                                        \
        /* pairs 4r .. 4r+3: columns 2r and 2r+1, four rows (k) each */          \
        *reinterpret_cast<uint2*>(ws + wcol_off(2 * r__)) =                      \
            make_uint2(dqv[4 * r__], dqv[4 * r__ + 1]);                          \
        *reinterpret_cast<uint2*>(ws + wcol_off(2 * r__ + 1)) =                  \
            make_uint2(dqv[4 * r__ + 2], dqv[4 * r__ + 3]);                      \
      } else {                                                                   \
        *reinterpret_cast<uint4*>(ws + wrow_off[r__]) = make_uint4(              \
            dqv[4 * r__], dqv[4 * r__ + 1], dqv[4 * r__ + 2], dqv[4 * r__ + 3]); \
      }                                                                          \
    }                                                                            \
    /* x tile tt + 2 into the stage that the barrier of the previous step freed; \
       these are the last loads issued before this step's barrier */            \
    if constexpr ((m) == xdma_slot(0, kNS)) {                                    \
      QMM_DMA_X1(xs_new, kx, 0, xoff0);                                          \
    }                                                                            \
    if constexpr ((m) == xdma_slot(1, kNS)) {                                    \
      QMM_DMA_X1(xs_new, kx, 1, xoff1);                                          \
    }                                                                            \
    if constexpr ((m) == xdma_slot(2, kNS)) {                                    \
      QMM_DMA_X1(xs_new, kx, 2, xoff2);                                          \
    }                                                                            \
    if constexpr ((m) == xdma_slot(3, kNS)) {                                    \
      QMM_DMA_X1(xs_new, kx, 3, xoff3);                                          \
    }                                                                            \
    if constexpr ((m) == kNS - 14) {                                             \
      /* everything but this step's own loads has completed: x tile tt + 1 is   \
         in LDS */                                                               \
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWLoads + 4) : "memory");         \
      __syncthreads();                                                           \
    }                                                                            \
    __builtin_amdgcn_sched_barrier(0);                                           \
  }

#define QMM_SLOTS8(m0, P, MM)                                                    \
  QMM_SLOT((m0) + 0, P, MM) QMM_SLOT((m0) + 1, P, MM) QMM_SLOT((m0) + 2, P, MM)  \
  QMM_SLOT((m0) + 3, P, MM) QMM_SLOT((m0) + 4, P, MM) QMM_SLOT((m0) + 5, P, MM)  \
  QMM_SLOT((m0) + 6, P, MM) QMM_SLOT((m0) + 7, P, MM)

#define QMM_STEP(tt, P, MM)                                                      \
  {                                                                              \
    const int cur = (P);                                                         \
    const int nxt = (P) ^ 1;                                                     \
    const int k2 = kclamp((tt) + 2);                                             \
    const int kx = k2;                                                           \
    T* ws = lds + kWBase + nxt * kWTile;                                         \
    float sf[kSB], bf[kSB];                                                      \
    _Pragma("unroll") for (int j__ = 0; j__ < kSB; ++j__) {                      \
      sf[j__] = WN ? wn_value(swn, j__)                                          \
                   : raw_value<TS>(sreg) * DQ::kCodeScale;                       \
      bf[j__] = WN ? wn_value(bwn, j__) : raw_value<TS>(breg);                   \
    }                                                                            \
    /* the tile prepared in step tt is tile tt + 1: block (tt + 1) % 3 of its   \
       group of three takes the weights' low parts */                           \
    const bool low_part = kSplit && ((tt) + 1) % 3 == 2;                         \
    DQ dq;                                                                       \
    ColDequant<T, (WN ? BITS : 4)> cdq;                                          \
    uint32_t dqv[16];                                                            \
    __builtin_amdgcn_sched_barrier(0);                                           \
    QMM_SLOTS8(0, P, MM) QMM_SLOTS8(8, P, MM) QMM_SLOTS8(16, P, MM)              \
    QMM_SLOTS8(24, P, MM) QMM_SLOTS8(32, P, MM) QMM_SLOTS8(40, P, MM)            \
    QMM_SLOTS8(48, P, MM) QMM_SLOTS8(56, P, MM)                                  \
    /* the packed W fetched in slot 0 is older than the four x loads: it has    \
       had the whole step to arrive */                                          \
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");                             \
    QMM_PIN_W();                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                           \
    QMM_ROTATE_W();                                                              \
    {                                                                            \
      const int freed = xs_cur;                                                  \
      xs_cur = xs_nxt;                                                           \
      xs_nxt = xs_new;                                                           \
      xs_new = freed;                                                            \
    }                                                                            \
  }

  int t = 0;
  // uniform per wavefront: does any of its 64 rows lie below M
  const bool has_rows = __builtin_amdgcn_readfirstlane(m0 + wm * 64 < M ? 1 : 0) != 0;
  if (has_rows) {
    for (; t + 1 < nk; t += 2) {
      QMM_STEP(t, 0, true)
      QMM_STEP(t + 1, 1, true)
    }
    if (t < nk) {
      QMM_STEP(t, 0, true)
    }
  } else {
    for (; t + 1 < nk; t += 2) {
      QMM_STEP(t, 0, false)
      QMM_STEP(t + 1, 1, false)
    }
    if (t < nk) {
      QMM_STEP(t, 0, false)
    }
  }
#undef QMM_STEP
#undef QMM_SLOTS8
#undef QMM_SLOT

  // ---- epilogue.  D[n][m] tiles: register r of lane (col, quad) holds
  // n = 4 quad + r, m = col.  The tile is rounded to TO and staged in LDS as
  // ys[m][n] (the K loop is done with it), then written out row by row in
  // 16-byte pieces, whole rows of the tile contiguous.  fp32 tiles go in two
  // halves of 128 rows, which is what fits.
  constexpr int kPasses = sizeof(TO) == 4 ? 2 : 1;
  constexpr int kPassRows = kBM / kPasses;
  constexpr int kPiece = 16 / static_cast<int>(sizeof(TO)); // elements per 16 bytes
  constexpr int kOutStride = kBN + kOutPad;
  TO* ys = reinterpret_cast<TO*>(smem);
  // the last steps' (clamped) loads must not land in LDS after it changes hands,
  // nor in registers that have been given to something else: their destinations
  // stay allocated until the wait
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  QMM_PIN_W();
  if constexpr (FP == 3) {
    // nvfp4 weights quantized with a tensor-wide scale: the fp32 sums (of a K
    // range, when K is split: the factor distributes over the ranges) take the
    // factor before they are rounded
    if (a.out_scale != nullptr) {
      const float out_factor = *a.out_scale / (448.0f * 6.0f);
#pragma unroll
      for (int i = 0; i < NT; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            acc[i][j][r] *= out_factor;
          }
        }
      }
    }
  }
#pragma unroll
  for (int pass = 0; pass < kPasses; ++pass) {
    __syncthreads(); // LDS is free: K loop (pass 0) or the previous half is done
    if (wm * 64 / kPassRows == pass) {
      const int col = lane & 15;
      const int quad = lane >> 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        TO* yrow = ys + ((wm * 64) % kPassRows + j * 16 + col) * kOutStride +
            wn * 16 * NT + 4 * quad;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          if constexpr (sizeof(TO) == 4) {
            float4 v = make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
            if (!p.valid) {
              v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
            *reinterpret_cast<float4*>(yrow + 16 * i) = v;
          } else {
            uint2 packed;
            packed.x = pack2<TO>(acc[i][j][0], acc[i][j][1]);
            packed.y = pack2<TO>(acc[i][j][2], acc[i][j][3]);
            if (!p.valid) {
              packed = make_uint2(0u, 0u);
            }
            *reinterpret_cast<uint2*>(yrow + 16 * i) = packed;
          }
        }
      }
    }
    __syncthreads();
    constexpr int kChunks = kBN / kPiece;        // 16-byte pieces per tile row
    constexpr int kLanesPerRow = 256 / kPiece;   // a power of two >= kChunks
    constexpr int kRowsPerIter = kThreads / kLanesPerRow;
    const int c = tid % kLanesPerRow;
    const int r0 = tid / kLanesPerRow;
    const bool vec_ok = (N % kPiece) == 0; // rows of y stay 16-byte aligned
    if (c < kChunks) {
#pragma unroll 4
      for (int r = r0; r < kPassRows; r += kRowsPerIter) {
        const int mr = pass * kPassRows + r; // row inside the tile
        const int m = m0 + mr;
        const int n = n0 + c * kPiece;
        if (mr >= M - m0 || m >= M || n >= N) {
          continue;
        }
        const TO* src = ys + r * kOutStride + c * kPiece;
        const size_t orow =
            GROUPED ? static_cast<size_t>(a.group_perm[row0 + mr]) : static_cast<size_t>(m);
        TO* dst = p.out + orow * N + n;
        if (vec_ok && n + kPiece <= N) {
          *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
        } else {
          for (int e = 0; e < kPiece && n + e < N; ++e) {
            dst[e] = src[e];
          }
        }
      }
    }
  }
}

#undef QMM_DMA_X
#undef QMM_DMA_X1
#undef QMM_LOAD_W
#undef QMM_ROTATE_W
#undef QMM_PIN_W
#undef QMM_STORE_W

template <int NT>
constexpr size_t qmm_smem_bytes() {
  constexpr size_t stages =
      (static_cast<size_t>(3) * kBM * kBK + static_cast<size_t>(2) * 32 * NT * kBK) * 2;
  // staged y tile: all 256 rows of a 16-bit tile or 128 rows of an fp32 tile
  constexpr size_t out = static_cast<size_t>(kBM) * (32 * NT + kOutPad) * 2;
  return stages > out ? stages : out;
}

// Tile width (in units of 32 columns) that finishes first: a workgroup needs
// time ~ NT per tile and the tiles run in ceil(tiles / CUs) rounds.
int choose_nt(int M, int N, int L, int min_nt = 5) {
  const long cus = compute_units();
  const long mt = (M + kBM - 1) / kBM;
  int best = 7;
  long best_cost = -1;
  for (int nt = 7; nt >= min_nt; --nt) {
    const long tiles = mt * ((N + 32 * nt - 1) / (32 * nt)) * L;
    const long rounds = (tiles + cus - 1) / cus;
    const long cost = rounds * (nt * 8 + 3); // + fixed per-tile prologue/epilogue
    if (best_cost < 0 || cost < best_cost) {
      best = nt;
      best_cost = cost;
    }
  }
  return best;
}

template <typename T, typename TS, typename TO, int BITS, int NT, bool GROUPED, bool WN = false,
          bool SBI = false, int FP = 0>
int launch_variant(const QmmArgs& a, int gs_shift, dim3 grid, hipStream_t s, int k_splits = 1) {
  constexpr size_t smem = qmm_smem_bytes<NT>();
  if (grid.y > 65535u || grid.z > 65535u) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] M=%d or batch=%d exceed the grid", a.M, a.L);
  }
  auto kern = qmm_t_mfma_kernel<T, TS, TO, BITS, NT, GROUPED, WN, SBI, FP>;
  static bool configured = false; // per instantiation
  if (!configured) {
    MLXROCM_HIP_TRY(hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern),
        hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(smem)));
    configured = true;
  }
  kern<<<grid, kThreads, smem, s>>>(a, gs_shift, k_splits);
  MLXROCM_HIP_TRY(hipGetLastError());
  return static_cast<int>(MLXROCM_OK);
}

int shift_of(int gs) {
  return gs == 32 ? 5 : (gs == 64 ? 6 : 7);
}

} // namespace

} // namespace mlxrocm
