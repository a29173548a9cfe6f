// qmm_slab.hip -- transpose=true products of 4-bit weights with a few rows of x
// per weight matrix (16-bit element types): 5..32 rows of a plain call and the
// small expert groups of a gather.
//
//   y[M, N] = x[M, K] * dequant(W)[N, K]^T
//
// The weights are read once and the work is bound by that stream.  What the
// kernels here are built around:
//   * packed codes go from HBM to LDS without passing through registers
//     (global_load_lds_dwordx4): a wavefront instruction fetches 8 rows x 128
//     bytes, whole cache lines, into a ring of 256-code steps that is private
//     to the wavefront -- no workgroup barrier in the loop, the only
//     synchronisation is the wavefront's own vmcnt;
//   * x does not move while weights stream.  qmm_slab_kernel: a workgroup of 8
//     wavefronts keeps 16 or 32 rows of one 1024-code K range in LDS and walks
//     slabs of 256 weight rows with it; a launch is a flat list of units (x rows
//     of a problem or expert tile, K range, slab) cut into equal consecutive
//     pieces, one per workgroup, so that x is staged once or twice per
//     workgroup.  qmm_rows8_kernel: up to 16 rows of x whose whole K fits LDS,
//     one launch workgroup per 64 weight rows, no K ranges;
//   * codes are widened without arithmetic (OR into the mantissa of 128.0 /
//     1024.0) and multiplied as they are: per quantization group one chain of
//     v_mfma_f32_16x16x32 starting from zero, then acc += scale * chain (four
//     FMAs per 16 x 16 tile and group).  What the offset and the biases add,
//     sum_g X[m][g] * (bias[n][g] - offset * scale[n][g]) with X the sums of x
//     over a group, is one v_mfma_f32_16x16x4_f32 per tile and four groups on
//     exact fp32 operands;
//   * scales and biases arrive once per unit (whole 32- or 64-byte runs of a
//     row per load), results leave one step after their unit ended (stores
//     count in vmcnt like loads);
//   * the K ranges of a row of y are added up from fp32 planes by a second
//     small kernel (one range: written directly); K is a multiple of 256, the
//     last range of a row may be 512 or 768 codes long (not 256);
//   * a gather of up to 512 index pairs is grouped by expert inside the kernel.
// LDS reads are free of bank conflicts by construction: the 16-byte pieces of a
// weight row are stored at piece ^ (row / 2 % 8), rows of x are 16 bytes longer
// than a power of two.
#include "mfma_dequant.h"
#include "qmm_args.h"

namespace mlxrocm {

namespace {

constexpr int kSlWaves = 8;
constexpr int kSlThreads = 64 * kSlWaves;
constexpr int kSlWaveRows = 32;                      // two 16-row MFMA tiles
constexpr int kSlRows = kSlWaves * kSlWaveRows;      // rows of W per slab
constexpr int kSlStep = 256;                         // codes per row and step
constexpr int kSlKrShift = 10;                       // K range of a unit: 1024 codes
constexpr int kSlKr = 1 << kSlKrShift;
constexpr int kSlSteps = kSlKr / kSlStep;            // steps per unit
constexpr int kSlSlotBytes = kSlWaveRows * kSlStep / 2; // packed codes of a step
constexpr int kSlXStride = 2 * kSlKr + 16;           // bytes per staged row of x

// Gathers of up to kSlPlanPairs index pairs over up to kSlPlanExperts experts
// are grouped by expert inside the kernel: every workgroup builds the same
// tile list and sorted order in LDS (a counting sort on ballots, positions
// ascending by pair index inside an expert, so all workgroups agree), which
// saves the planning launch in front of a kernel that lasts a few tens of
// microseconds.
constexpr int kSlPlanPairs = kSlThreads;  // one pair per thread
constexpr int kSlPlanExperts = 64;
constexpr int kSlPlanTiles = kSlPlanPairs / 16 + kSlPlanExperts; // tiles of 16 rows at worst
constexpr int kSlPlanInts = kSlPlanPairs + kSlWaves * (kSlPlanExperts + 1) +
    3 * (kSlPlanExperts + 1) + 3 * kSlPlanTiles + 4;
constexpr int kSlPlanBytes = (kSlPlanInts * 4 + 255) / 256 * 256;

struct SlabPlan {
  int ranges;          // ceil(K / 1024); the last one may hold 2 or 3 steps instead of 4
  int n_slabs;         // ceil(N / 256)
  int workgroups;      // the launch's grid
  float* planes;       // ranges > 1: fp32 [ranges][rows][N]
  int64_t plane_elems; // rows * N
};

template <int GS>
struct SlabShape {
  static constexpr int kGroupsPerStep = kSlStep / GS;        // 8, 4, 2
  static constexpr int kDwords = GS / 32;                    // per lane and group
  static constexpr int kGroupsPerRange = kSlKr / GS;         // 32, 16, 8
  static constexpr int kRowSbBytes = 2 * kGroupsPerRange;    // a row's scales of a unit: 64, 32, 16
  static constexpr int kLanesPerRow = kRowSbBytes / 16;      // 16-byte pieces: 4, 2, 1
  static constexpr int kSbLoads = kLanesPerRow > 2 ? 2 : 1;  // wavefront loads per array and unit
  static constexpr int kSbArrayBytes = kSlWaveRows * kRowSbBytes;
  static constexpr int kSbBytes = 2 * kSbArrayBytes;         // scales + biases of a unit
};

// Ring slots per wavefront: what 160 KiB of LDS leave beside the rows of x.
template <int GS, int MT>
constexpr int slab_stages() {
  return (MT == 1 && GS >= 64) ? 3 : 2;
}

template <int GS, int MT, int MODE>
constexpr size_t slab_smem_bytes() {
  constexpr size_t xr = 16 * MT;
  return (MODE == 2 ? kSlPlanBytes : 0) + xr * kSlXStride + xr * (SlabShape<GS>::kGroupsPerRange + 1) * 4 + xr * 4 + xr * 8 +
      static_cast<size_t>(kSlWaves) *
      (slab_stages<GS, MT>() * kSlSlotBytes + SlabShape<GS>::kSbBytes);
}

template <typename T>
struct WidenMagic;
template <>
struct WidenMagic<bf16_t> {
  static constexpr uint32_t kBits = 0x43004300u; // 128.0 twice
  static constexpr float kOffset = 128.0f;
};
template <>
struct WidenMagic<f16_t> {
  static constexpr uint32_t kBits = 0x64006400u; // 1024.0 twice
  static constexpr float kOffset = 1024.0f;
};

// Eight 4-bit codes -> eight T holding offset + code, in the order
// 0,4,1,5,2,6,3,7 (x is staged in the same order).
// (mask and magic are passed in registers whose contents the compiler cannot
// see, so that it emits one v_and_or_b32 per pair instead of an AND and an OR
// with literal operands.  The instruction must stay the compiler's own: written
// as inline assembly it feeds the matrix instruction without the wait states
// the hazard recognizer inserts for a vector-ALU result, and the matrix
// instruction then reads the register's old contents.)
__device__ __forceinline__ uint4 widen8(uint32_t w, uint32_t mask, uint32_t magic) {
  uint4 r;
  r.x = (w & mask) | magic;
  r.y = ((w >> 4) & mask) | magic;
  r.z = ((w >> 8) & mask) | magic;
  r.w = ((w >> 12) & mask) | magic;
  return r;
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) const char*)p));
}

// A wave-uniform pointer, in scalar registers whatever the compiler believes
// about its uniformity.
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return reinterpret_cast<const void*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// 16 bytes per lane from base + voff to LDS at m0 + 16 * lane.
__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t m0) {
  base = uniform_ptr(base);
  m0 = __builtin_amdgcn_readfirstlane(m0);
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(base), "s"(m0)
               : "memory");
}

// 16 bytes per lane into registers, completion counted by vmcnt like the DMAs
// (the compiler does not know that the value is still in flight: pin() after
// the wait, and nothing may touch the registers in between).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
struct InFlight4 {
  u32x4 v;
  __device__ __forceinline__ void load(const void* base, uint32_t voff) {
    base = uniform_ptr(base);
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(base) : "memory");
  }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(v)); }
};

template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wait_lds_reads() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// What a unit (x rows of one problem or tile, K range, slab) needs; wave-uniform.
template <typename T>
struct SlabUnit {
  const uint8_t* w;   // first row of the weight matrix
  const T* scales;
  const T* biases;
  int range;
  int slab;
  int owner;          // problem (plain) or tile (grouped)
};

// (two waves per SIMD as the register budget: the matrix instructions then keep
// their results in ordinary registers, where the FMAs read them)
// MODE 0: plain call; 1: gather, grouped by the planning kernel; 2: gather,
// grouped here.
template <typename T, int GS, int MT, int MODE>
__global__ __launch_bounds__(kSlThreads, 2) void qmm_slab_kernel(const QmmArgs a, const SlabPlan pl) {
  constexpr bool GROUPED = MODE != 0;
  constexpr bool PLAN = MODE == 2;
  using Shape = SlabShape<GS>;
  constexpr int GPS = Shape::kGroupsPerStep;
  constexpr int DW = Shape::kDwords;
  constexpr int GPR = Shape::kGroupsPerRange;
  constexpr int RB = Shape::kRowSbBytes;
  constexpr int LPR = Shape::kLanesPerRow;
  constexpr int NL = Shape::kSbLoads;
  constexpr int kSbInstrs = 2 * NL; // register loads per unit
  constexpr int XR = 16 * MT;
  constexpr int kStages = slab_stages<GS, MT>();
  constexpr int kAhead = (kStages - 1) * 4; // DMAs of the steps in flight behind the current one
  constexpr int kXsStride = GPR + 1;        // floats
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int N = a.N;
  const int K = a.K;
  const int R = pl.ranges;
  const int groups = K / GS;   // groups per row of W
  const int row_bytes = K / 2;

  // in-kernel planning tables (MODE 2), in front of everything else
  int32_t* lperm = reinterpret_cast<int32_t*>(smem);         // sorted position -> pair
  int32_t* lwave = lperm + kSlPlanPairs;                       // [wave][expert] counts, then bases
  int32_t* lcnt = lwave + kSlWaves * (kSlPlanExperts + 1);     // pairs per expert
  int32_t* lpos = lcnt + kSlPlanExperts + 1;                   // first sorted position
  int32_t* lfirst = lpos + kSlPlanExperts + 1;                 // first tile
  int32_t* ltiles = lfirst + kSlPlanExperts + 1;               // {expert, first position, rows}
  int32_t* lnum = ltiles + 3 * kSlPlanTiles;                   // {tiles, sorted positions}
  uint8_t* xl = smem + (PLAN ? kSlPlanBytes : 0);
  float* xsum = reinterpret_cast<float*>(xl + XR * kSlXStride);
  int32_t* orow = reinterpret_cast<int32_t*>(xsum + XR * kXsStride);
  int64_t* xoff = reinterpret_cast<int64_t*>(orow + XR); // element offset of a staged row in x
  uint8_t* ring = reinterpret_cast<uint8_t*>(xoff + XR) +
      wave * (kStages * kSlSlotBytes + Shape::kSbBytes);
  uint8_t* sbbuf = ring + kStages * kSlSlotBytes; // scales, then biases, of the current unit
  const uint32_t ring_lds = lds_address(ring);

  // ---- this workgroup's piece of the unit list ----
  if constexpr (PLAN) {
    const int n = a.L;
    const int E = a.n_experts;
    int e = E + 1; // no pair
    if (tid < n) {
      const uint32_t xi = a.lhs_indices[tid];
      const uint32_t wi = a.rhs_indices[tid];
      e = (xi < static_cast<uint32_t>(a.x_batches) && wi < static_cast<uint32_t>(E))
          ? static_cast<int>(wi) : E; // E: a pair with an index out of range
    }
    int rank = 0;
    for (int ee = 0; ee < E; ++ee) {
      const uint64_t mask = __ballot(e == ee);
      if (lane == 0) {
        lwave[wave * (kSlPlanExperts + 1) + ee] = __popcll(mask);
      }
      if (e == ee) {
        rank = __builtin_amdgcn_mbcnt_hi(
            static_cast<uint32_t>(mask >> 32),
            __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0));
      }
    }
    __syncthreads();
    if (tid < E) { // counts per expert; the wavefronts' counts become their bases
      int sum = 0;
      for (int w = 0; w < kSlWaves; ++w) {
        const int c = lwave[w * (kSlPlanExperts + 1) + tid];
        lwave[w * (kSlPlanExperts + 1) + tid] = sum;
        sum += c;
      }
      lcnt[tid] = sum;
    }
    __syncthreads();
    if (tid == 0) {
      int pos = 0;
      int tile = 0;
      for (int ee = 0; ee < E; ++ee) {
        lpos[ee] = pos;
        lfirst[ee] = tile;
        pos += lcnt[ee];
        tile += (lcnt[ee] + XR - 1) / XR;
      }
      lnum[0] = tile;
      lnum[1] = pos;
    }
    __syncthreads();
    if (tid < E) {
      const int c = lcnt[tid];
      int t = lfirst[tid];
      for (int r = 0; r < c; r += XR, ++t) { // tiles of as many rows as x is staged with
        ltiles[3 * t + 0] = tid;
        ltiles[3 * t + 1] = lpos[tid] + r;
        ltiles[3 * t + 2] = c - r < XR ? c - r : XR;
      }
    }
    if (e < E) {
      lperm[lpos[e] + lwave[wave * (kSlPlanExperts + 1) + e] + rank] = tid;
    }
    __syncthreads();
    if (blockIdx.x == 0) {
      // for the kernel that adds up the planes; rows of pairs that name no
      // expert or no x are zero
      int32_t* gperm = const_cast<int32_t*>(a.group_perm);
      int32_t* gnum = const_cast<int32_t*>(a.group_ntiles);
      if (tid < lnum[1]) {
        gperm[tid] = lperm[tid];
      }
      if (tid < 2) {
        gnum[tid] = lnum[tid];
      }
      if (e == E) {
        T* row = static_cast<T*>(a.out) + static_cast<size_t>(tid) * N;
        for (int c = 0; c < N; ++c) {
          row[c] = static_cast<T>(0.0f);
        }
      }
    }
  }
  auto tile_field = [&](int t, int f) {
    const int v = PLAN ? ltiles[3 * t + f] : a.group_tiles[3 * t + f];
    return __builtin_amdgcn_readfirstlane(v);
  };
  auto perm_at = [&](int pos) { return PLAN ? lperm[pos] : a.group_perm[pos]; };
  int owners;
  if constexpr (GROUPED) {
    owners = __builtin_amdgcn_readfirstlane(PLAN ? lnum[0] : *a.group_ntiles);
  } else {
    owners = a.L;
  }
  const long total = static_cast<long>(owners) * R * pl.n_slabs;
  const long u0 = total * blockIdx.x / pl.workgroups;
  const long u1 = total * (blockIdx.x + 1) / pl.workgroups;
  if (u0 >= u1) {
    return;
  }
  const int my_units = static_cast<int>(u1 - u0);
  // steps of a unit: four, fewer in the last K range when K is no multiple of 1024
  const int last_steps = K / kSlStep - (R - 1) * kSlSteps;
  auto unit_steps = [&](int range) { return range == R - 1 ? last_steps : kSlSteps; };
  // the last range reads the last GPR groups of a row (whole 16-byte pieces that
  // end where the row ends): its groups start this far into that window
  const int last_shift = R * GPR - groups;

  auto resolve = [&](SlabUnit<T>& u) {
    int64_t e = u.owner;
    if constexpr (GROUPED) {
      e = tile_field(u.owner, 0);
    }
    u.w = reinterpret_cast<const uint8_t*>(a.w + e * a.w_batch_stride);
    u.scales = static_cast<const T*>(a.scales) + e * a.sb_batch_stride;
    u.biases = static_cast<const T*>(a.biases) + e * a.sb_batch_stride;
  };
  auto first_unit = [&](SlabUnit<T>& u) {
    const long combo = u0 / pl.n_slabs;
    u.slab = static_cast<int>(u0 - combo * pl.n_slabs);
    u.owner = static_cast<int>(combo / R);
    u.range = static_cast<int>(combo - static_cast<long>(u.owner) * R);
    resolve(u);
  };
  auto next_unit = [&](SlabUnit<T>& u) {
    if (++u.slab == pl.n_slabs) {
      u.slab = 0;
      if (++u.range == R) {
        u.range = 0;
        ++u.owner;
        resolve(u);
      }
    }
  };

  // ---- fetch side: per-lane pieces of the addresses ----
  // W, DMA i of a step: tile row 8 (i % 2) + lane / 8 of 16-row tile i / 2,
  // LDS piece lane % 8 of that row <- global piece (lane % 8) ^ (row / 2 % 8).
  // Scales / biases of a unit: lane -> 16-byte piece lane % LPR of row
  // lane / LPR (+ 16 for the second load of 32-wide groups): whole 32- or
  // 64-byte runs of a row per instruction, once per unit.
  const int wrow = lane >> 3;
  uint32_t w_off[4];
  uint32_t sb_off[NL];
  auto fetch_offsets = [&](const SlabUnit<T>& u) {
    const int n0 = u.slab * kSlRows + wave * kSlWaveRows;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 8 * (i & 1) + wrow;
      int n = n0 + 16 * (i >> 1) + r;
      n = n < N ? n : N - 1;
      const int piece = (lane & 7) ^ ((r >> 1) & 7);
      w_off[i] = static_cast<uint32_t>(n) * static_cast<uint32_t>(row_bytes) + piece * 16;
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      int n = n0 + (((lane / LPR) + (64 / LPR) * i) & 31);
      n = n < N ? n : N - 1;
      sb_off[i] = static_cast<uint32_t>(n) * static_cast<uint32_t>(groups) * 2u + (lane % LPR) * 16u;
    }
  };
  auto fetch_w = [&](const SlabUnit<T>& u, int j, int slot) {
    const int k0 = (u.range << kSlKrShift) + j * kSlStep;
    const uint8_t* wb = u.w + (k0 >> 1);
    const uint32_t m0 = ring_lds + slot * kSlSlotBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dma16(wb, w_off[i], m0 + i * 1024);
    }
  };
  InFlight4 sbq[kSbInstrs]; // in flight within one loop iteration only
  auto fetch_sb = [&](const SlabUnit<T>& u) {
    const int g0 = u.range * GPR - (u.range == R - 1 ? last_shift : 0);
    const T* sp = u.scales + g0;
    const T* bp = u.biases + g0;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      sbq[i].load(sp, sb_off[i]);
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      sbq[NL + i].load(bp, sb_off[i]);
    }
  };
  u32x4 sbv[kSbInstrs]; // arrived, waiting for the current unit to end
  auto store_sb = [&]() {
    if (LPR > 1 || lane < 32) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        *reinterpret_cast<u32x4*>(sbbuf + i * 1024 + lane * 16) = sbv[i];
        *reinterpret_cast<u32x4*>(sbbuf + Shape::kSbArrayBytes + i * 1024 + lane * 16) = sbv[NL + i];
      }
    }
  };

  // ---- x of (owner, range) into LDS: rows in the widened order, group sums,
  // and the output row of every x row ----
  int M = a.M;     // rows of the current owner
  int row0 = 0;    // grouped: first sorted position of the tile
  auto stage_x = [&](const SlabUnit<T>& u) {
    if constexpr (GROUPED) {
      row0 = tile_field(u.owner, 1);
      M = tile_field(u.owner, 2);
    }
    if (tid < XR) {
      int row = -1;
      int64_t off = 0;
      if (tid < M) {
        if constexpr (GROUPED) {
          // planes are indexed by sorted position, y by index pair
          const int pair = perm_at(row0 + tid);
          row = R > 1 ? row0 + tid : pair;
          off = static_cast<int64_t>(a.lhs_indices[pair]) * a.x_batch_stride;
        } else {
          row = u.owner * a.M + tid;
          off = u.owner * a.x_batch_stride + static_cast<int64_t>(tid) * K;
        }
      }
      orow[tid] = row;
      xoff[tid] = off;
    }
    __syncthreads();
    constexpr int cshift = kSlKrShift - 3; // 16-byte pieces per row = 1 << cshift
    constexpr int kPasses = (XR << cshift) / kSlThreads;
    const T* xbase = static_cast<const T*>(a.x) + (u.range << kSlKrShift);
    const int valid_k = unit_steps(u.range) * kSlStep; // codes of this range
    // all loads first: one memory latency for the whole tile
    uint4 xv[kPasses];
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int c = tid + i * kSlThreads;
      const int m = c >> cshift;
      const int col = c & ((1 << cshift) - 1);
      xv[i] = make_uint4(0u, 0u, 0u, 0u);
      if (m < M && col * 8 < valid_k) {
        xv[i] = *reinterpret_cast<const uint4*>(xbase + xoff[m] + col * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int c = tid + i * kSlThreads;
      const int m = c >> cshift;
      const int col = c & ((1 << cshift) - 1);
      const uint4 v = xv[i];
      // elements e0..e7 -> e0 e4 e1 e5 e2 e6 e3 e7
      uint4 p;
      p.x = (v.x & 0xffffu) | (v.z << 16);
      p.y = (v.x >> 16) | (v.z & 0xffff0000u);
      p.z = (v.y & 0xffffu) | (v.w << 16);
      p.w = (v.y >> 16) | (v.w & 0xffff0000u);
      *reinterpret_cast<uint4*>(xl + m * kSlXStride + col * 16) = p;
      const uint32_t words[4] = {v.x, v.y, v.z, v.w};
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        s += to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(words[k] & 0xffffu)));
        s += to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(words[k] >> 16)));
      }
#pragma unroll
      for (int d = 1; d < GS / 8; d *= 2) {
        s += __shfl_xor(s, d);
      }
      if ((lane & (GS / 8 - 1)) == 0) {
        xsum[m * kXsStride + col / (GS / 8)] = s;
      }
    }
  };

  // ---- compute side: per-lane LDS offsets ----
  // W piece of lane (row r16, quarter q) for group G of a step: bytes
  // [G GS/2 + q GS/8, + GS/8) of the row's 128, 16-byte pieces swizzled.
  const int lane_byte = q * (GS / 8);
  const uint32_t w_lane = r16 * 128 + ((((lane_byte >> 4) ^ (r16 >> 1)) & 7) << 4) + (lane_byte & 15);
  // x: row r16 (+16), codes GS G + (GS/4) q + 8 d of the step
  const uint32_t x_lane = r16 * kSlXStride + 2 * (GS / 4) * q;

  uint32_t wmask = 0x000f000fu;
  uint32_t wmagic = WidenMagic<T>::kBits;
  asm volatile("" : "+v"(wmask), "+v"(wmagic)); // keep both in vector registers

  int sb_shift = 0; // first group of the compute unit inside its scale window
  floatx4 acc[2][MT];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
  }

  // ---- results of a finished unit, stored one step later ----
  // (stores count in vmcnt like loads: issued at the end of a unit they would
  // make the next step's wait for its weights wait for the stores as well)
  floatx4 done[2][MT];
  uint8_t* done_ptr[MT];   // null: no such row; nt = 1 is 16 columns further
  bool done_cols[2] = {false, false};
  bool have_done = false;
  auto flush_done = [&]() {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if (done_ptr[mt] == nullptr || !done_cols[nt]) {
          continue;
        }
        const floatx4 v = done[nt][mt];
        if (R > 1) {
          *reinterpret_cast<floatx4*>(done_ptr[mt] + nt * 16 * sizeof(float)) = v;
        } else {
          uint2 packed;
          packed.x = pack2<T>(v[0], v[1]);
          packed.y = pack2<T>(v[2], v[3]);
          *reinterpret_cast<uint2*>(done_ptr[mt] + nt * 16 * sizeof(T)) = packed;
        }
      }
    }
    have_done = false;
  };

  // One step of one wavefront: all LDS reads first (x before the wait for the
  // step's DMAs, which it does not depend on), then arithmetic only -- two
  // wavefronts share a SIMD and one computes while the other one loads.
  // MTC: 16-row tiles of x that hold rows (a gather tile of up to 16 rows skips
  // the second one).  ENTERED: this iteration's fetch also issued the register
  // loads of the next unit's scales and biases.
  auto compute = [&](auto mtc, auto entered, int j, int slot) {
    constexpr int MTC = decltype(mtc)::value;
    constexpr int kWait = kAhead + (decltype(entered)::value ? kSbInstrs : 0);
    constexpr int kChunks = GPS * DW; // 32-code pieces of the step per lane quarter
    const uint8_t* sl = ring + slot * kSlSlotBytes;
    const uint8_t* xs = xl + x_lane + j * (2 * kSlStep);
    uint4 xf[kChunks][MTC];
#pragma unroll
    for (int G = 0; G < GPS; ++G) {
#pragma unroll
      for (int d = 0; d < DW; ++d) {
#pragma unroll
        for (int mt = 0; mt < MTC; ++mt) {
          xf[G * DW + d][mt] =
              *reinterpret_cast<const uint4*>(xs + mt * 16 * kSlXStride + 2 * (GS * G + 8 * d));
        }
      }
    }
    // group sums of x for the offset / bias term: lane (row r16, quarter q)
    // supplies group q (and q + 4) of the step
    constexpr int kCorr = (GPS + 3) / 4;
    float xa[kCorr][MTC];
    bool live[kCorr];
    int gcl[kCorr];
#pragma unroll
    for (int h = 0; h < kCorr; ++h) {
      const int g = 4 * h + q;
      live[h] = g < GPS;
      gcl[h] = live[h] ? g : 0;
#pragma unroll
      for (int mt = 0; mt < MTC; ++mt) {
        xa[h][mt] = xsum[(mt * 16 + r16) * kXsStride + j * GPS + gcl[h]];
      }
    }
    // scales of the lane's rows for the step's groups, and the lane's group of
    // the offset / bias term (the unit's buffer: no wait needed either)
    uint32_t raw[2][GPS / 2];
    T cs[kCorr][2], cb[kCorr][2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const uint8_t* sp = sbbuf + (nt * 16 + r16) * RB + (j * GPS + sb_shift) * 2;
      if constexpr (GPS == 8) {
        const uint4 v = *reinterpret_cast<const uint4*>(sp);
        raw[nt][0] = v.x; raw[nt][1] = v.y; raw[nt][2] = v.z; raw[nt][3] = v.w;
      } else if constexpr (GPS == 4) {
        const uint2 v = *reinterpret_cast<const uint2*>(sp);
        raw[nt][0] = v.x; raw[nt][1] = v.y;
      } else {
        raw[nt][0] = *reinterpret_cast<const uint32_t*>(sp);
      }
#pragma unroll
      for (int h = 0; h < kCorr; ++h) {
        cs[h][nt] = *reinterpret_cast<const T*>(sp + 2 * gcl[h]);
        cb[h][nt] = *reinterpret_cast<const T*>(sp + 2 * gcl[h] + Shape::kSbArrayBytes);
      }
    }
    wait_vm<kWait>();
    if (have_done) {
      flush_done();
    }
    uint32_t wq[GPS][2][DW];
#pragma unroll
    for (int G = 0; G < GPS; ++G) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const uint8_t* wp = sl + nt * 2048 + (w_lane ^ (G * (GS / 2)));
        if constexpr (DW == 4) {
          const uint4 v = *reinterpret_cast<const uint4*>(wp);
          wq[G][nt][0] = v.x; wq[G][nt][1] = v.y; wq[G][nt][2] = v.z; wq[G][nt][3] = v.w;
        } else if constexpr (DW == 2) {
          const uint2 v = *reinterpret_cast<const uint2*>(wp);
          wq[G][nt][0] = v.x; wq[G][nt][1] = v.y;
        } else {
          wq[G][nt][0] = *reinterpret_cast<const uint32_t*>(wp);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int G = 0; G < GPS; ++G) {
      floatx4 chain[2][MTC];
#pragma unroll
      for (int d = 0; d < DW; ++d) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const uint4 wf = widen8(wq[G][nt][d], wmask, wmagic);
#pragma unroll
          for (int mt = 0; mt < MTC; ++mt) {
            const floatx4 c0 = d == 0 ? floatx4{0.0f, 0.0f, 0.0f, 0.0f} : chain[nt][mt];
            chain[nt][mt] = mfma16<T>(xf[G * DW + d][mt], wf, c0);
          }
        }
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const float scale = to_f32(__builtin_bit_cast(
            T, static_cast<uint16_t>((raw[nt][G / 2] >> (16 * (G & 1))) & 0xffffu)));
#pragma unroll
        for (int mt = 0; mt < MTC; ++mt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            acc[nt][mt][r] = fmaf(scale, chain[nt][mt][r], acc[nt][mt][r]);
          }
        }
      }
    }
#pragma unroll
    for (int h = 0; h < kCorr; ++h) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        float c = fmaf(-WidenMagic<T>::kOffset, to_f32(cs[h][nt]), to_f32(cb[h][nt]));
        c = live[h] ? c : 0.0f;
#pragma unroll
        for (int mt = 0; mt < MTC; ++mt) {
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[h][mt], c, acc[nt][mt], 0, 0, 0);
        }
      }
    }
  };

  // lane (column r16 = row of W, quarter q) holds y[m = 16 mt + 4 q + r][n] in
  // register r.  A 4 x 4 transpose among the four lanes of a quad leaves lane i
  // of quad c with y[m = 16 mt + 4 q + i][n = 4 c .. 4 c + 3]: one 16-byte store
  // per tile instead of four scattered dwords.
  auto quad_transpose = [&](floatx4 v) {
    const bool odd = (lane & 1) != 0;
    const bool high = (lane & 2) != 0;
    // lanes i and i ^ 1 swap the off-diagonal elements of the 2 x 2 blocks
    float sx = odd ? v[0] : v[1];
    float sy = odd ? v[2] : v[3];
    const float px = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, sx), 0xB1, 0xf, 0xf, true));
    const float py = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, sy), 0xB1, 0xf, 0xf, true));
    if (odd) {
      v[0] = px;
      v[2] = py;
    } else {
      v[1] = px;
      v[3] = py;
    }
    // lanes i and i ^ 2 swap the off-diagonal 2 x 2 blocks
    sx = high ? v[0] : v[2];
    sy = high ? v[1] : v[3];
    const float qx = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, sx), 0x4E, 0xf, 0xf, true));
    const float qy = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, sy), 0x4E, 0xf, 0xf, true));
    if (high) {
      v[0] = qx;
      v[1] = qy;
    } else {
      v[2] = qx;
      v[3] = qy;
    }
    return v;
  };
  // The finished unit's tiles, transposed, and where they go (N % 4 == 0: four
  // columns in range or none).
  auto finish_unit = [&](const SlabUnit<T>& u) {
    const int n = u.slab * kSlRows + wave * kSlWaveRows + (r16 & ~3);
    done_cols[0] = n < N;
    done_cols[1] = n + 16 < N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int row = orow[mt * 16 + 4 * q + (lane & 3)];
      done_ptr[mt] = nullptr;
      if (row >= 0) {
        const int64_t at = static_cast<int64_t>(row) * N + n;
        done_ptr[mt] = R > 1
            ? reinterpret_cast<uint8_t*>(pl.planes + u.range * pl.plane_elems + at)
            : reinterpret_cast<uint8_t*>(static_cast<T*>(a.out) + at);
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        done[nt][mt] = quad_transpose(acc[nt][mt]);
        acc[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
    have_done = true;
  };

  // ---- the pipeline ----
  SlabUnit<T> fu; // fetch cursor
  SlabUnit<T> cu; // compute cursor
  first_unit(fu);
  cu = fu;
  fetch_offsets(fu);
  int fj = 0;          // step of fu to fetch next
  int funit = 0;       // which of this workgroup's units fu is
  bool fdone = false;  // every step has been fetched
  int fslot = 0;
  // Fetches the next step; true when it is the first step of a unit, whose
  // scales and biases were then requested ahead of its weights.  Past the end:
  // the last step again (lands in a free slot, never read), so that the
  // outstanding-load count of every wait is the same.
  auto fetch_next = [&]() {
    const bool enters = fj == 0 && funit != 0 && !fdone;
    if (enters) {
      fetch_sb(fu);
    }
    fetch_w(fu, fj, fslot);
    fslot = fslot + 1 == kStages ? 0 : fslot + 1;
    if (!fdone && ++fj == unit_steps(fu.range)) {
      if (funit + 1 < my_units) {
        fj = 0;
        ++funit;
        next_unit(fu);
        fetch_offsets(fu);
      } else {
        fdone = true;
        --fj;
      }
    }
    return enters;
  };
  fetch_sb(fu);
#pragma unroll
  for (int i = 0; i < kStages - 1; ++i) {
    fetch_next(); // steps 0 .. kStages - 2 of the first unit
  }
  stage_x(cu);
  wait_vm<kAhead>(); // the first unit's scales and biases have arrived
#pragma unroll
  for (int i = 0; i < kSbInstrs; ++i) {
    sbq[i].pin();
    sbv[i] = sbq[i].v;
  }
  store_sb();
  __syncthreads();

  bool have_sb = false;
  int cslot = 0;
  for (int un = 0; un < my_units; ++un) {
    const int usteps = unit_steps(cu.range);
    sb_shift = cu.range == R - 1 ? last_shift : 0;
    for (int j = 0; j < usteps; ++j) {
      const bool entered = fetch_next();
      const bool two = MT == 2 && M > 16;
      if (entered) {
        if (two) {
          compute(IntC<MT>{}, IntC<1>{}, j, cslot);
        } else {
          compute(IntC<1>{}, IntC<1>{}, j, cslot);
        }
        wait_vm<4>(); // only this iteration's weight DMAs may still be out
#pragma unroll
        for (int i = 0; i < kSbInstrs; ++i) {
          sbq[i].pin();
          sbv[i] = sbq[i].v;
        }
        have_sb = true;
      } else {
        if (two) {
          compute(IntC<MT>{}, IntC<0>{}, j, cslot);
        } else {
          compute(IntC<1>{}, IntC<0>{}, j, cslot);
        }
      }
      wait_lds_reads();
      cslot = cslot + 1 == kStages ? 0 : cslot + 1;
    }
    finish_unit(cu);
    if (have_sb) {
      store_sb(); // LDS operations of a wavefront execute in order: behind the unit's last reads
      have_sb = false;
    }
    if (un + 1 < my_units) {
      const int owner = cu.owner;
      const int range = cu.range;
      next_unit(cu);
      if (cu.owner != owner || cu.range != range) {
        __syncthreads(); // everyone has finished with the old x
        stage_x(cu);
        __syncthreads();
      }
    }
  }
  if (have_done) {
    flush_done();
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---------------------------------------------------------------------------
// Up to 16 rows of x with all of K resident: the same arithmetic without ranges,
// planes or a unit list.  A workgroup of 4 wavefronts owns 64 rows of W (one
// 16-row tile per wavefront) and keeps the rows of x for the whole of K in LDS
// (M * K * 2 bytes <= 64 KiB), so every element of y is finished where it is
// computed.  Scales and biases of a wavefront's 16 rows go to LDS by DMA once,
// the packed codes through a ring of four 256-code steps.  Grid: N / 64
// workgroups per problem -- one per compute unit for the shapes it is used for.
constexpr int kR8Tiles = 4;              // 16-row tiles of W per workgroup
constexpr int kR8Rows = 16 * kR8Tiles;
constexpr int kR8SlotBytes = 16 * kSlStep / 2;
constexpr int kR8MaxXBytes = 64 * 1024;

// kw: wavefronts per tile (each takes 1 / kw of the K steps); stages: ring slots
// per wavefront
inline size_t rows8_smem_bytes(int M, int K, int gs, int kw, int stages) {
  const size_t groups = K / gs;
  const size_t sums = (static_cast<size_t>(M) * (groups + 1) * 4 + 15) / 16 * 16;
  return static_cast<size_t>(M) * (2 * K + 16) + sums +
      static_cast<size_t>(kR8Tiles) * kw * stages * kR8SlotBytes +
      static_cast<size_t>(kR8Tiles) * 2 * 16 * groups * 2;
}

__device__ __forceinline__ floatx4 quad_transpose4(floatx4 v, int lane) {
  const bool odd = (lane & 1) != 0;
  const bool high = (lane & 2) != 0;
  float sx = odd ? v[0] : v[1];
  float sy = odd ? v[2] : v[3];
  const float px = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, sx), 0xB1, 0xf, 0xf, true));
  const float py = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, sy), 0xB1, 0xf, 0xf, true));
  if (odd) {
    v[0] = px;
    v[2] = py;
  } else {
    v[1] = px;
    v[3] = py;
  }
  sx = high ? v[0] : v[2];
  sy = high ? v[1] : v[3];
  const float qx = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, sx), 0x4E, 0xf, 0xf, true));
  const float qy = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, sy), 0x4E, 0xf, 0xf, true));
  if (high) {
    v[0] = qx;
    v[1] = qy;
  } else {
    v[2] = qx;
    v[3] = qy;
  }
  return v;
}

template <typename T, int GS, int KW, int kR8Stages>
__global__ __launch_bounds__(64 * kR8Tiles * KW) void qmm_rows8_kernel(const QmmArgs a) {
  constexpr int kR8Threads = 64 * kR8Tiles * KW;
  using Shape = SlabShape<GS>;
  constexpr int GPS = Shape::kGroupsPerStep;
  constexpr int DW = Shape::kDwords;
  constexpr int kChunks = GPS * DW;
  constexpr int kAhead = (kR8Stages - 1) * 2;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int M = a.M;
  const int N = a.N;
  const int K = a.K;
  const int groups = K / GS;
  const int row_bytes = K / 2;
  const int rbk = groups * 2;          // bytes of a row's scales
  const int x_stride = 2 * K + 16;     // bytes
  const int xs_stride = groups + 1;    // floats
  const int nsteps = K / kSlStep / KW;      // steps of this wavefront
  const int tile = wave % kR8Tiles;
  const int kpart = wave / kR8Tiles;
  const int step0 = kpart * nsteps;
  const QmmProblem<T> p = resolve_problem<T>(a, blockIdx.y);

  uint8_t* xl = smem;
  float* xsum = reinterpret_cast<float*>(smem + M * x_stride);
  uint8_t* rings = reinterpret_cast<uint8_t*>(xsum) + (M * xs_stride * 4 + 15) / 16 * 16;
  uint8_t* ring = rings + wave * (kR8Stages * kR8SlotBytes);
  // [16 rows][groups] scales, then biases, of the tile (fetched by its first wavefront)
  uint8_t* sbbuf = rings + kR8Tiles * KW * (kR8Stages * kR8SlotBytes) + tile * (2 * 16 * rbk);
  const uint32_t ring_lds = lds_address(ring);
  const uint32_t sb_lds = lds_address(sbbuf);

  const int n0 = blockIdx.x * kR8Rows + tile * 16;
  // ---- scales and biases of the tile's rows: rbk / 64 DMAs per array,
  // lane -> 16-byte piece (i * 64 + lane) of the [16][rbk] block
  if (kpart == 0) {
    const int per_row = rbk >> 4;
    const int dmas = rbk >> 6;
    for (int i = 0; i < dmas; ++i) {
      const int piece = i * 64 + lane;
      const int r = piece / per_row;
      const int c = piece - r * per_row;
      int n = n0 + r;
      n = n < N ? n : N - 1;
      const uint32_t off = static_cast<uint32_t>(n) * static_cast<uint32_t>(rbk) + c * 16;
      dma16(p.scales, off, sb_lds + i * 1024);
      dma16(p.biases, off, sb_lds + 16 * rbk + i * 1024);
    }
  }
  // ---- W: DMA i of a step fetches tile row 8 i + lane / 8, LDS piece lane % 8
  // <- global piece (lane % 8) ^ (row / 2 % 8)
  uint32_t w_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 8 * i + (lane >> 3);
    int n = n0 + r;
    n = n < N ? n : N - 1;
    const int piece = (lane & 7) ^ ((r >> 1) & 7);
    w_off[i] = static_cast<uint32_t>(n) * static_cast<uint32_t>(row_bytes) + piece * 16;
  }
  auto fetch = [&](int j, int slot) {
    const int jc = step0 + (j < nsteps ? j : nsteps - 1); // past the end: again, into a free slot
    const uint8_t* wb = p.w + jc * (kSlStep / 2);
    const uint32_t m0 = ring_lds + slot * kR8SlotBytes;
    dma16(wb, w_off[0], m0);
    dma16(wb, w_off[1], m0 + 1024);
  };
#pragma unroll
  for (int i = 0; i < kR8Stages - 1; ++i) {
    fetch(i, i);
  }

  // ---- x into LDS: rows in the widened order and their group sums
  {
    const int per_row = K >> 3; // 16-byte pieces per row
    const int pieces = M * per_row;
    for (int c0 = 0; c0 < pieces; c0 += 4 * kR8Threads) {
      uint4 xv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = c0 + i * kR8Threads + tid;
        xv[i] = make_uint4(0u, 0u, 0u, 0u);
        if (c < pieces) {
          xv[i] = *reinterpret_cast<const uint4*>(p.x + static_cast<size_t>(c) * 8);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = c0 + i * kR8Threads + tid;
        const int m = c / per_row;
        const int col = c - m * per_row;
        const uint4 v = xv[i];
        uint4 w;
        w.x = (v.x & 0xffffu) | (v.z << 16);
        w.y = (v.x >> 16) | (v.z & 0xffff0000u);
        w.z = (v.y & 0xffffu) | (v.w << 16);
        w.w = (v.y >> 16) | (v.w & 0xffff0000u);
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          s += to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(words[k] & 0xffffu)));
          s += to_f32(__builtin_bit_cast(T, static_cast<uint16_t>(words[k] >> 16)));
        }
#pragma unroll
        for (int d = 1; d < GS / 8; d *= 2) {
          s += __shfl_xor(s, d);
        }
        if (c < pieces) {
          *reinterpret_cast<uint4*>(xl + m * x_stride + col * 16) = w;
          if ((lane & (GS / 8 - 1)) == 0) {
            xsum[m * xs_stride + col / (GS / 8)] = s;
          }
        }
      }
    }
  }
  wait_vm<kAhead>(); // the tile's scales and biases are in LDS before the barrier
  __syncthreads();

  const int xrow = r16 < M ? r16 : M - 1; // rows past M repeat the last one; their results are dropped
  const int lane_byte = q * (GS / 8);
  const uint32_t w_lane = r16 * 128 + ((((lane_byte >> 4) ^ (r16 >> 1)) & 7) << 4) + (lane_byte & 15);
  const uint8_t* x_lane = xl + xrow * x_stride + 2 * (GS / 4) * q;
  const float* xs_lane = xsum + xrow * xs_stride;
  const uint8_t* sb_lane = sbbuf + r16 * rbk;
  uint32_t wmask = 0x000f000fu;
  uint32_t wmagic = WidenMagic<T>::kBits;
  asm volatile("" : "+v"(wmask), "+v"(wmagic));

  floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  int slot = 0;
  int fslot = kR8Stages - 1;
  for (int j = 0; j < nsteps; ++j) {
    fetch(j + kR8Stages - 1, fslot);
    fslot = fslot + 1 == kR8Stages ? 0 : fslot + 1;
    const uint8_t* xs = x_lane + (step0 + j) * (2 * kSlStep);
    uint4 xf[kChunks];
#pragma unroll
    for (int G = 0; G < GPS; ++G) {
#pragma unroll
      for (int d = 0; d < DW; ++d) {
        xf[G * DW + d] = *reinterpret_cast<const uint4*>(xs + 2 * (GS * G + 8 * d));
      }
    }
    constexpr int kCorr = (GPS + 3) / 4;
    float xa[kCorr];
    bool live[kCorr];
    int gcl[kCorr];
#pragma unroll
    for (int h = 0; h < kCorr; ++h) {
      const int g = 4 * h + q;
      live[h] = g < GPS;
      gcl[h] = live[h] ? g : 0;
      xa[h] = xs_lane[(step0 + j) * GPS + gcl[h]];
    }
    wait_vm<kAhead>(); // this step's codes (and, the first time, scales and biases) have landed
    uint32_t raw[GPS / 2];
    T cs[kCorr], cb[kCorr];
    {
      const uint8_t* sp = sb_lane + (step0 + j) * (2 * GPS);
      if constexpr (GPS == 8) {
        const uint4 v = *reinterpret_cast<const uint4*>(sp);
        raw[0] = v.x; raw[1] = v.y; raw[2] = v.z; raw[3] = v.w;
      } else if constexpr (GPS == 4) {
        const uint2 v = *reinterpret_cast<const uint2*>(sp);
        raw[0] = v.x; raw[1] = v.y;
      } else {
        raw[0] = *reinterpret_cast<const uint32_t*>(sp);
      }
#pragma unroll
      for (int h = 0; h < kCorr; ++h) {
        cs[h] = *reinterpret_cast<const T*>(sp + 2 * gcl[h]);
        cb[h] = *reinterpret_cast<const T*>(sp + 2 * gcl[h] + 16 * rbk);
      }
    }
    const uint8_t* sl = ring + slot * kR8SlotBytes;
    uint32_t wq[GPS][DW];
#pragma unroll
    for (int G = 0; G < GPS; ++G) {
      const uint8_t* wp = sl + (w_lane ^ (G * (GS / 2)));
      if constexpr (DW == 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(wp);
        wq[G][0] = v.x; wq[G][1] = v.y; wq[G][2] = v.z; wq[G][3] = v.w;
      } else if constexpr (DW == 2) {
        const uint2 v = *reinterpret_cast<const uint2*>(wp);
        wq[G][0] = v.x; wq[G][1] = v.y;
      } else {
        wq[G][0] = *reinterpret_cast<const uint32_t*>(wp);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int G = 0; G < GPS; ++G) {
      floatx4 chain;
#pragma unroll
      for (int d = 0; d < DW; ++d) {
        const uint4 wf = widen8(wq[G][d], wmask, wmagic);
        const floatx4 c0 = d == 0 ? floatx4{0.0f, 0.0f, 0.0f, 0.0f} : chain;
        chain = mfma16<T>(xf[G * DW + d], wf, c0);
      }
      const float scale = to_f32(__builtin_bit_cast(
          T, static_cast<uint16_t>((raw[G / 2] >> (16 * (G & 1))) & 0xffffu)));
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc[r] = fmaf(scale, chain[r], acc[r]);
      }
    }
#pragma unroll
    for (int h = 0; h < kCorr; ++h) {
      float c = fmaf(-WidenMagic<T>::kOffset, to_f32(cs[h]), to_f32(cb[h]));
      c = live[h] ? c : 0.0f;
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[h], c, acc, 0, 0, 0);
    }
    wait_lds_reads();
    slot = slot + 1 == kR8Stages ? 0 : slot + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the refetches past the end

  // the K parts of a tile meet in LDS (the ring is free now)
  if constexpr (KW > 1) {
    __syncthreads();
    float* part = reinterpret_cast<float*>(rings) + (wave * 64 + lane) * 4;
    if (kpart != 0) {
      *reinterpret_cast<floatx4*>(part) = acc;
    }
    __syncthreads();
    if (kpart != 0) {
      return;
    }
#pragma unroll
    for (int k = 1; k < KW; ++k) {
      acc += *reinterpret_cast<const floatx4*>(part + k * kR8Tiles * 64 * 4);
    }
  }
  // lane i of quad c: y[m = 4 q + i][n0 + 4 c .. + 3]
  const floatx4 v = quad_transpose4(acc, lane);
  const int m = 4 * q + (lane & 3);
  const int n = n0 + (r16 & ~3);
  if (m < M && n < N) {
    uint2 packed;
    packed.x = p.valid ? pack2<T>(v[0], v[1]) : 0u;
    packed.y = p.valid ? pack2<T>(v[2], v[3]) : 0u;
    *reinterpret_cast<uint2*>(p.out + static_cast<size_t>(m) * N + n) = packed;
  }
}

// y = sum over the K ranges of plane[range] (plain call): one thread per four
// outputs, the planes read as one stream each.
template <typename T>
__global__ __launch_bounds__(256) void slab_reduce_kernel(
    const float* planes, int ranges, int64_t plane_elems, T* out) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i >= plane_elems) {
    return;
  }
  floatx4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int r = 0; r < ranges; ++r) {
    s += *reinterpret_cast<const floatx4*>(planes + r * plane_elems + i);
  }
  uint2 packed;
  packed.x = pack2<T>(s[0], s[1]);
  packed.y = pack2<T>(s[2], s[3]);
  *reinterpret_cast<uint2*>(out + i) = packed;
}

// y[perm[pos]] (grouped) = sum over the K ranges of plane[range][pos]
template <typename T>
__global__ __launch_bounds__(256) void slab_reduce_grouped_kernel(
    const float* planes,
    int ranges,
    int64_t plane_elems,
    const int32_t* perm,
    const int32_t* n_rows,
    T* out,
    int N) {
  const int rows = *n_rows;
  const int quads = N / 4;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t pos = i / quads;
  if (pos >= rows) {
    return;
  }
  const int n = static_cast<int>(i - pos * quads) * 4;
  floatx4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int r = 0; r < ranges; ++r) {
    s += *reinterpret_cast<const floatx4*>(planes + r * plane_elems + pos * N + n);
  }
  uint2 packed;
  packed.x = pack2<T>(s[0], s[1]);
  packed.y = pack2<T>(s[2], s[3]);
  *reinterpret_cast<uint2*>(out + static_cast<int64_t>(perm[pos]) * N + n) = packed;
}

template <typename T, int GS, int MT, int MODE>
int launch_one(const QmmArgs& a, const SlabPlan& pl, hipStream_t s) {
  constexpr size_t smem = slab_smem_bytes<GS, MT, MODE>();
  static_assert(smem <= 160 * 1024, "LDS of a compute unit");
  auto kern = qmm_slab_kernel<T, GS, MT, MODE>;
  static bool configured = false; // per instantiation
  if (!configured) {
    MLXROCM_HIP_TRY(hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern),
        hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(smem)));
    configured = true;
  }
  kern<<<pl.workgroups, kSlThreads, smem, s>>>(a, pl);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// (32-wide groups with two tiles of x would need more LDS than a compute unit
// has: qmm_slab_supported() keeps them out)
template <int MODE>
int launch_any(const QmmArgs& a, const SlabPlan& pl, int gs, int dtype, int mt, hipStream_t s) {
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    if (mt == 1) {
      return gs == 32 ? launch_one<T, 32, 1, MODE>(a, pl, s)
                      : (gs == 64 ? launch_one<T, 64, 1, MODE>(a, pl, s)
                                  : launch_one<T, 128, 1, MODE>(a, pl, s));
    }
    if (gs == 32) {
      return fail(MLXROCM_UNSUPPORTED, "[qmm] slab kernel: 32-wide groups with more than 16 rows");
    }
    return gs == 64 ? launch_one<T, 64, 2, MODE>(a, pl, s)
                    : launch_one<T, 128, 2, MODE>(a, pl, s);
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

SlabPlan make_plan(int N, int K, long owners) {
  SlabPlan pl{};
  pl.n_slabs = (N + kSlRows - 1) / kSlRows;
  pl.ranges = (K + kSlKr - 1) >> kSlKrShift;
  const long units = owners * pl.ranges * pl.n_slabs;
  const long cus = compute_units();
  pl.workgroups = static_cast<int>(units < cus ? (units > 0 ? units : 1) : cus);
  return pl;
}

} // namespace

// `rows`: rows of x per weight matrix (a gather tile has up to 32).
bool qmm_slab_shape_ok(int rows, int N, int K, int gs, int bits) {
  if (bits != 4 || rows < 1 || rows > 32 || (gs == 32 && rows > 16)) {
    return false;
  }
  // whole 256-code steps; a last K range of 2..4 of them (one step would be
  // shorter than the fetch distance of the ring)
  if (K < kSlKr || K % kSlStep != 0 || (K / kSlStep) % kSlSteps == 1 || N < 4 || N % 4 != 0) {
    return false;
  }
  // 32-bit byte offsets of a matrix's rows
  return static_cast<int64_t>(N) * (K / 2) < (int64_t{1} << 32);
}

bool qmm_slab_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  if (!transpose || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  return qmm_slab_shape_ok(a.M, a.N, a.K, gs, bits);
}

long qmm_slab_units(const QmmArgs& a) {
  return static_cast<long>(a.L) * ((a.K + kSlKr - 1) >> kSlKrShift) * ((a.N + kSlRows - 1) / kSlRows);
}

// Plain call (no index arrays).  With more than one K range `planes` must hold
// qmm_slab_plane_bytes() bytes.
size_t qmm_slab_plane_bytes(const QmmArgs& a) {
  const int ranges = (a.K + kSlKr - 1) >> kSlKrShift;
  return ranges <= 1 ? 0 : static_cast<size_t>(ranges) * a.L * a.M * a.N * sizeof(float);
}

int launch_qmm_slab(const QmmArgs& a, int gs, int bits, int dtype, void* planes, hipStream_t s) {
  (void)bits;
  const int mt = a.M <= 16 ? 1 : 2;
  SlabPlan pl = make_plan(a.N, a.K, a.L);
  pl.planes = static_cast<float*>(planes);
  pl.plane_elems = static_cast<int64_t>(a.L) * a.M * a.N;
  MLXROCM_REHEARSE("qmm_slab(tiles=%d,ranges=%d)", mt, pl.ranges);
  int rc = launch_any<0>(a, pl, gs, dtype, mt, s);
  if (rc != MLXROCM_OK || pl.ranges <= 1) {
    return rc;
  }
  if (pl.ranges >= 8 && pl.plane_elems < (int64_t{1} << 20)) {
    // many planes of a small y: the reduction that spreads the planes over threads
    return reduce_planes(
        pl.planes, a.out, static_cast<size_t>(pl.plane_elems), pl.ranges, dtype, s);
  }
  const int64_t quads = pl.plane_elems / 4; // (the caller checks plane_elems % 4 == 0)
  const unsigned blocks = static_cast<unsigned>((quads + 255) / 256);
  if (dtype == MLXROCM_BFLOAT16) {
    slab_reduce_kernel<bf16_t><<<blocks, 256, 0, s>>>(
        pl.planes, pl.ranges, pl.plane_elems, static_cast<bf16_t*>(a.out));
  } else {
    slab_reduce_kernel<f16_t><<<blocks, 256, 0, s>>>(
        pl.planes, pl.ranges, pl.plane_elems, static_cast<f16_t*>(a.out));
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// Gather grouped by expert in tiles of up to 32 rows (`a` carries the tile
// list).  planes: qmm_slab_grouped_plane_bytes() bytes.
size_t qmm_slab_grouped_plane_bytes(int n_indices, int N, int K) {
  const int ranges = (K + kSlKr - 1) >> kSlKrShift;
  return ranges <= 1 ? 0 : static_cast<size_t>(ranges) * n_indices * N * sizeof(float);
}

bool qmm_slab_plans_in_kernel(int n_indices, int n_experts) {
  return n_indices <= kSlPlanPairs && n_experts <= kSlPlanExperts;
}

int launch_qmm_slab_grouped(
    const QmmArgs& a, int gs, int bits, int dtype, void* planes, bool plan_in_kernel,
    hipStream_t s) {
  (void)bits;
  // Few pairs per expert (8 on average at most) and the kernel's own grouping:
  // 16-row tiles, which leave LDS for a third ring slot; an expert that does get
  // more than 16 rows is then read once per tile.  32-wide groups have no
  // two-tile form at all.
  const bool one_tile = plan_in_kernel &&
      (gs == 32 || static_cast<int64_t>(a.L) <= 8 * static_cast<int64_t>(a.n_experts));
  const int tile_rows = one_tile ? 16 : kGroupSmallTile;
  SlabPlan pl = make_plan(a.N, a.K, gather_group_max_tiles(a.L, a.n_experts, tile_rows));
  pl.planes = static_cast<float*>(planes);
  pl.plane_elems = static_cast<int64_t>(a.L) * a.N;
  MLXROCM_REHEARSE(
      "qmm_slab_grouped(%s,tile=%d,ranges=%d)", plan_in_kernel ? "plans" : "planned", tile_rows,
      pl.ranges);
  // (mode 1 never runs with one tile of x: the planning kernel makes 32-row tiles)
  int rc = plan_in_kernel ? launch_any<2>(a, pl, gs, dtype, one_tile ? 1 : 2, s)
                          : launch_any<1>(a, pl, gs, dtype, 2, s);
  if (rc != MLXROCM_OK || pl.ranges <= 1) {
    return rc;
  }
  const int64_t threads = static_cast<int64_t>(a.L) * (a.N / 4);
  const unsigned blocks = static_cast<unsigned>((threads + 255) / 256);
  if (dtype == MLXROCM_BFLOAT16) {
    slab_reduce_grouped_kernel<bf16_t><<<blocks, 256, 0, s>>>(
        pl.planes, pl.ranges, pl.plane_elems, a.group_perm, a.group_ntiles + 1,
        static_cast<bf16_t*>(a.out), a.N);
  } else {
    slab_reduce_grouped_kernel<f16_t><<<blocks, 256, 0, s>>>(
        pl.planes, pl.ranges, pl.plane_elems, a.group_perm, a.group_ntiles + 1,
        static_cast<f16_t*>(a.out), a.N);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

// Wavefronts per tile: as many as K has pairs of steps, at most 4.
int rows8_kw(int K) {
  const int steps = K / kSlStep;
  return steps % 4 == 0 && steps >= 8 ? 4 : (steps % 2 == 0 && steps >= 4 ? 2 : 1);
}

// Ring slots per wavefront: as many as LDS leaves (2..4 with four wavefronts
// per tile, 3 otherwise); 0: does not fit.
int rows8_stages(int M, int K, int gs, int kw) {
  const int steps = K / kSlStep / kw;
  for (int st = kw == 4 ? 4 : 3; st >= (kw == 4 ? 2 : 3); --st) {
    if (st <= steps + 1 && rows8_smem_bytes(M, K, gs, kw, st) <= 160 * 1024) {
      return st;
    }
  }
  return 0;
}

// Up to 16 rows of x whose whole K fits LDS (qmm_rows8_kernel).
bool qmm_rows8_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose) {
  if (!transpose || bits != 4 || dtype == MLXROCM_FLOAT32) {
    return false;
  }
  if (a.M < 1 || a.M > 16 || a.N < 4 || a.N % 4 != 0 || a.L > 65535) {
    return false;
  }
  // whole 64-piece DMAs of a 16-row block of scales; whole steps
  if (a.K < 32 * gs || a.K % (32 * gs) != 0 || a.K % kSlStep != 0) {
    return false;
  }
  if (static_cast<size_t>(a.M) * (2 * a.K + 16) > kR8MaxXBytes + 16 * 16 ||
      rows8_stages(a.M, a.K, gs, rows8_kw(a.K)) == 0) {
    return false;
  }
  return static_cast<int64_t>(a.N) * (a.K / 2) < (int64_t{1} << 32);
}

int launch_qmm_rows8(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s) {
  (void)bits;
  const int kw = rows8_kw(a.K);
  const int stages = rows8_stages(a.M, a.K, gs, kw);
  const size_t smem = rows8_smem_bytes(a.M, a.K, gs, kw, stages);
  MLXROCM_REHEARSE("qmm_rows8(kw=%d,slots=%d)", kw, stages);
  const dim3 grid((a.N + kR8Rows - 1) / kR8Rows, a.L);
  auto go = [&](auto kern) -> int {
    // every instantiation decays to the same pointer type, so this lambda exists
    // once: the attribute is set on each launch (a host-side table lookup), not
    // behind a flag the kernels would share
    MLXROCM_HIP_TRY(hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
        160 * 1024));
    kern<<<grid, 64 * kR8Tiles * kw, smem, s>>>(a);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  };
  auto run = [&](auto tval) -> int {
    using T = decltype(tval);
    auto with = [&](auto kwv, auto stv) -> int {
      constexpr int KW = decltype(kwv)::value;
      constexpr int ST = decltype(stv)::value;
      return gs == 32 ? go(qmm_rows8_kernel<T, 32, KW, ST>)
                      : (gs == 64 ? go(qmm_rows8_kernel<T, 64, KW, ST>)
                                  : go(qmm_rows8_kernel<T, 128, KW, ST>));
    };
    if (kw == 4) {
      return stages == 4 ? with(IntC<4>{}, IntC<4>{})
                         : (stages == 3 ? with(IntC<4>{}, IntC<3>{}) : with(IntC<4>{}, IntC<2>{}));
    }
    return kw == 2 ? with(IntC<2>{}, IntC<3>{}) : with(IntC<1>{}, IntC<3>{});
  };
  return dtype == MLXROCM_BFLOAT16 ? run(bf16_t{}) : run(f16_t{});
}

} // namespace mlxrocm
