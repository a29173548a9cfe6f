// qmm_api.hip -- C entry points of quantized_matmul / gather_qmm: argument
// checks, kernel choice, launch.
#include <mutex>

#include "qmm_args.h"

namespace mlxrocm {

namespace {

enum class Family { Qmv, QmmT, QmmN, QmmNaive };

// M up to which the transpose=true path is a row-streaming GEMV: every packed
// weight row is read once and reused across the few rows of x.
constexpr int kQmvMaxM = 8;

// transpose=false at 2/3/5/6 bits: whether the codes are repacked at 4 or 8 bits
// first (run_widened) so that the fast [K, N] kernels apply.
bool widens_codes(int M, int N, int K, int L, int bits, int dtype, bool transpose) {
  return !transpose && widened_bits(bits) != 0 && N % 32 == 0 &&
      (M <= 4 || (M <= 8 && L == 1) || (dtype != MLXROCM_FLOAT32 && K % 64 == 0 && K >= 64));
}

Family choose_family(int M, int N, int K, int L, int bits, int dtype, bool transpose) {
  if (widens_codes(M, N, K, L, bits, dtype, transpose)) {
    bits = widened_bits(bits);
  }
  if (transpose && M <= kQmvMaxM) {
    return Family::Qmv;
  }
  if (transpose && K % 64 == 0 && K >= 64) {
    return Family::QmmT; // fp32 runs on the same matrix path, operands split in two
  }
  if (!transpose && K % 64 == 0 && K >= 64 && dtype != MLXROCM_FLOAT32 && (bits == 4 || bits == 8)) {
    return Family::QmmN; // w [K, N]: the matrix path with a column loader, any M
  }
  return Family::QmmNaive;
}

const char* family_name(Family f) {
  switch (f) {
    case Family::Qmv:
      return "qmv";
    case Family::QmmT:
      return "qmm_t";
    case Family::QmmN:
      return "qmm_n";
    case Family::QmmNaive:
      return "qmm_generic";
  }
  return nullptr;
}

int check_shape(
    const char* who,
    int M,
    int N,
    int K,
    int L,
    int group_size,
    int bits,
    int dtype,
    int transpose) {
  if (!valid_bits(bits)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the requested number of bits %d is not supported; "
        "supported bits are 2, 3, 4, 5, 6 and 8",
        who,
        bits);
  }
  if (!valid_group(group_size)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the requested group size %d is not supported; "
        "supported group sizes are 32, 64 and 128",
        who,
        group_size);
  }
  if (!valid_dtype(dtype)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] unknown dtype %d", who, dtype);
  }
  if (M < 0 || N < 0 || K < 0 || L < 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[%s] negative dimension", who);
  }
  // The quantized axis (K when transposed, N otherwise) is made of whole groups.
  const int quantized_axis = transpose ? K : N;
  if (quantized_axis % group_size != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[%s] the quantized dimension %d is not a multiple of group_size=%d "
        "(transpose=%d)",
        who,
        quantized_axis,
        group_size,
        transpose);
  }
  return MLXROCM_OK;
}

bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

int check_alignment(const char* who, const QmmArgs& a, int dtype) {
  if (!aligned16(a.x) || !aligned16(a.w) || !aligned16(a.scales) ||
      !aligned16(a.biases) || !aligned16(a.out)) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[%s] operand pointers must be 16-byte aligned",
        who);
  }
  const int64_t x_vec = 16 / static_cast<int64_t>(dtype_size(dtype));
  // one problem without indices never applies a batch stride (transpose=false
  // allows any K, so M * K need not be a multiple of 16 bytes there)
  const bool strided = a.L > 1 || a.lhs_indices != nullptr;
  if (strided && (a.x_batch_stride % x_vec != 0 || a.w_batch_stride % 4 != 0)) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[%s] batch strides must keep 16-byte alignment (x stride %lld, w "
        "stride %lld)",
        who,
        static_cast<long long>(a.x_batch_stride),
        static_cast<long long>(a.w_batch_stride));
  }
  return MLXROCM_OK;
}

// Device scratch of one call: the caller's workspace.  In a dry run nothing is
// launched and `need` receives the bytes the same call would claim, so that
// mlxrocm_qmm_workspace_size walks exactly the code the call itself walks.
struct Scratch {
  char* base = nullptr;
  size_t bytes = 0;
  bool dry = false;
  size_t need = 0;
  // Optional: the caller's transposed image of scales and biases
  // (mlxrocm_qmm_sb_image); the prefill path then skips its pre-pass.
  const void* sb_image = nullptr;
};

constexpr size_t kScratchAlign = 256;

int claim(Scratch& sc, size_t bytes, void** out) {
  *out = nullptr;
  if (sc.dry) {
    sc.need = bytes;
    return MLXROCM_OK;
  }
  if (sc.base == nullptr || sc.bytes < bytes) {
    return fail(
        MLXROCM_INVALID_ARGUMENT,
        "[quantized_matmul] this shape needs a workspace of %zu bytes "
        "(mlxrocm_qmm_workspace_size); got %zu",
        bytes,
        sc.base == nullptr ? size_t(0) : sc.bytes);
  }
  *out = sc.base;
  return MLXROCM_OK;
}

// Launch unless this is a dry run.
#define MLXROCM_LAUNCH(sc, call) ((sc).dry ? static_cast<int>(MLXROCM_OK) : (call))

// Rows of x from which the prefill paths transpose scales and biases first (see
// run_qmm_t_transposed_sb).
constexpr int kTransposeSbMinM = 512;

// fp32 prefill: x is split into bf16 high/low parts in scratch, at most
// kSplitScratchBytes of it at a time (row blocks of one batch entry), and each
// block runs on the bf16 matrix path with fp32 scales, biases and output.
constexpr size_t kSplitScratchBytes = size_t(256) << 20;

int run_split_fp32(const QmmArgs& a, int gs, int bits, Scratch& sc, hipStream_t s) {
  const size_t row_bytes = split_x_bytes(1, a.K);
  int rows_per_block = static_cast<int>(kSplitScratchBytes / row_bytes / 256 * 256);
  if (rows_per_block < 256) {
    rows_per_block = 256;
  }
  if (rows_per_block > a.M) {
    rows_per_block = a.M;
  }
  // the kernel addresses x with 32-bit element offsets
  if (static_cast<uint64_t>(rows_per_block) * 3u * static_cast<uint64_t>(a.K) >= (uint64_t(1) << 32)) {
    return MLXROCM_LAUNCH(sc, launch_qmm_naive(a, gs, bits, MLXROCM_FLOAT32, true, s));
  }
  // few tiles: also cut K (one row block, one batch entry only)
  int k_splits = 1;
  if (rows_per_block == a.M && a.L == 1 && (static_cast<int64_t>(a.M) * a.N) % 4 == 0) {
    k_splits = qmm_mfma_k_splits(a.M, a.N, a.K, 1);
  }
  const size_t x_bytes = (split_x_bytes(rows_per_block, a.K) + 255) / 256 * 256;
  const size_t plane = static_cast<size_t>(a.M) * a.N;
  const size_t partial_raw = k_splits > 1 ? plane * k_splits * sizeof(float) : 0;
  const size_t partial_bytes = (partial_raw + 255) / 256 * 256;
  // scales / biases transposed to [K / group][N], as for the 16-bit prefill
  const int G = a.K / gs;
  const int sb_batches = a.sb_batch_stride == 0 ? 1 : a.L;
  const bool sb_t = a.M >= kTransposeSbMinM;
  const size_t sb_bytes = sb_t ? qmm_n_sb_bytes(a.N, G, sb_batches, MLXROCM_FLOAT32) : 0;
  void* region = nullptr;
  int rc = claim(sc, x_bytes + partial_bytes + sb_bytes, &region);
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  void* partial = static_cast<char*>(region) + x_bytes;
  float* sb_image = reinterpret_cast<float*>(static_cast<char*>(region) + x_bytes + partial_bytes);
  const size_t image = static_cast<size_t>(a.N) * G;
  if (sb_t) {
    rc = transpose_sb_for_qmm_n(
        a.scales, a.biases, sb_image, a.N, G, sb_batches, a.sb_batch_stride, MLXROCM_FLOAT32, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
  }
  for (int l = 0; l < a.L; ++l) {
    for (int m_begin = 0; m_begin < a.M; m_begin += rows_per_block) {
      const int rows = (a.M - m_begin < rows_per_block) ? a.M - m_begin : rows_per_block;
      const float* x = static_cast<const float*>(a.x) + l * a.x_batch_stride +
          static_cast<int64_t>(m_begin) * a.K;
      rc = split_x_for_mfma(x, region, static_cast<size_t>(rows), a.K, s);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      QmmArgs part = a;
      part.x = region;
      part.M = rows;
      part.L = 1;
      part.x_batch_stride = static_cast<int64_t>(rows) * 3 * a.K;
      part.w = a.w + l * a.w_batch_stride;
      if (sb_t) {
        const size_t lb = sb_batches == 1 ? 0 : static_cast<size_t>(l) * 2 * image;
        part.scales = sb_image + lb;
        part.biases = sb_image + lb + image;
        part.sb_transposed = 1;
      } else {
        part.scales = static_cast<const float*>(a.scales) + l * a.sb_batch_stride;
        part.biases = static_cast<const float*>(a.biases) + l * a.sb_batch_stride;
      }
      float* out = static_cast<float*>(a.out) +
          (static_cast<int64_t>(l) * a.M + m_begin) * static_cast<int64_t>(a.N);
      part.out = k_splits > 1 ? partial : out;
      rc = launch_qmm_mfma_split(part, gs, bits, s, k_splits);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      if (k_splits > 1) {
        rc = reduce_k_splits(partial, out, plane, k_splits, MLXROCM_FLOAT32, s);
        if (rc != MLXROCM_OK) {
          return rc;
        }
      }
    }
  }
  return MLXROCM_OK;
}

// 16-bit prefill whose tiles would leave most compute units idle: K is cut into
// ranges, the fp32 partial tiles go to the workspace and are added up.
int run_k_split(const QmmArgs& a, int gs, int bits, int dtype, int k_splits, Scratch& sc, hipStream_t s) {
  const size_t plane = static_cast<size_t>(a.M) * a.N;
  void* region = nullptr;
  int rc = claim(sc, plane * k_splits * sizeof(float), &region);
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  QmmArgs part = a;
  part.out = region;
  rc = launch_qmm_mfma_ksplit(part, gs, bits, dtype, k_splits, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  return reduce_k_splits(region, a.out, plane, k_splits, dtype, s);
}

// Prefill (transpose=true, 16-bit types) from 512 rows of x on: the tile kernel
// reads one scale and one bias per thread and K-step, and with the caller's
// [N][K / group] layout every lane of such a load touches a line of its own
// (measured: 15 % of the kernel's time).  A pre-pass transposes both arrays to
// [K / group][N] in the workspace (a few MB, ~5 us), after which
// a wavefront's 32 rows read 64 contiguous bytes.
int run_qmm_t_transposed_sb(
    const QmmArgs& a, int gs, int bits, int dtype, int k_splits, Scratch& sc, hipStream_t s) {
  const int G = a.K / gs;
  const int batches = a.sb_batch_stride == 0 ? 1 : a.L;
  const bool prepacked = sc.sb_image != nullptr;
  const size_t sb_bytes =
      prepacked ? 0 : (qmm_n_sb_bytes(a.N, G, batches, dtype) + 255) / 256 * 256;
  const size_t plane = static_cast<size_t>(a.M) * a.N;
  const size_t partial_bytes = k_splits > 1 ? plane * k_splits * sizeof(float) : 0;
  void* region = nullptr;
  int rc = MLXROCM_OK;
  if (sb_bytes + partial_bytes != 0) {
    rc = claim(sc, sb_bytes + partial_bytes, &region);
  }
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  const void* sb = sc.sb_image;
  if (!prepacked) {
    // rows of the source are the N rows of W, columns its G groups
    rc = transpose_sb_for_qmm_n(
        a.scales, a.biases, region, a.N, G, batches, a.sb_batch_stride, dtype, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    sb = region;
  }
  const size_t image = static_cast<size_t>(a.N) * G;
  QmmArgs part = a;
  part.scales = sb;
  part.biases = static_cast<const char*>(sb) + image * dtype_size(dtype);
  part.sb_batch_stride = batches == 1 ? 0 : static_cast<int64_t>(2 * image);
  part.sb_transposed = 1;
  if (k_splits <= 1) {
    return launch_qmm_mfma(part, gs, bits, dtype, s);
  }
  void* partial = static_cast<char*>(region) + sb_bytes;
  part.out = partial;
  rc = launch_qmm_mfma_ksplit(part, gs, bits, dtype, k_splits, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  return reduce_k_splits(partial, a.out, plane, k_splits, dtype, s);
}

// transpose=false on the matrix cores.  The column loader wants the four
// scales of four consecutive rows of W side by side, so scales and biases are
// first transposed to [group][k] in the workspace (a few MB, a
// few microseconds); few-row shapes also cut K and keep their fp32 partial
// planes there.
// transpose=false, 1..4 rows of x: the streaming kernel, its K ranges added up
// from fp32 planes in the workspace.
int run_qmv_n(const QmmArgs& a, int gs, int bits, int dtype, Scratch& sc, hipStream_t s) {
  const QmvNPlan pl = qmv_n_plan(a, bits);
  if (pl.splits <= 1) {
    return MLXROCM_LAUNCH(sc, launch_qmv_n(a, gs, bits, dtype, nullptr, s));
  }
  const size_t plane = static_cast<size_t>(a.L) * a.M * a.N;
  void* region = nullptr;
  int rc = claim(sc, plane * pl.splits * sizeof(float), &region);
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  rc = launch_qmv_n(a, gs, bits, dtype, static_cast<float*>(region), s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  return reduce_planes(static_cast<const float*>(region), a.out, plane, pl.splits, dtype, s);
}

int run_qmm_n(const QmmArgs& a, int gs, int bits, int dtype, Scratch& sc, hipStream_t s) {
  const int G = a.N / gs;
  const int batches = a.sb_batch_stride == 0 ? 1 : a.L;
  int k_splits = 1;
  if ((static_cast<int64_t>(a.M) * a.N) % 4 == 0) {
    k_splits = qmm_mfma_k_splits(a.M, a.N, a.K, a.L);
  }
  const size_t sb_bytes = (qmm_n_sb_bytes(a.K, G, batches, dtype) + 255) / 256 * 256;
  const size_t plane = static_cast<size_t>(a.M) * a.N;
  const size_t partial_bytes = k_splits > 1 ? plane * k_splits * sizeof(float) : 0;
  void* region = nullptr;
  int rc = claim(sc, sb_bytes + partial_bytes, &region);
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  rc = transpose_sb_for_qmm_n(
      a.scales, a.biases, region, a.K, G, batches, a.sb_batch_stride, dtype, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  const size_t image = static_cast<size_t>(a.K) * G; // elements of one [G][K] image
  QmmArgs part = a;
  part.scales = region;
  part.biases = static_cast<char*>(region) + image * dtype_size(dtype);
  part.sb_batch_stride = batches == 1 ? 0 : static_cast<int64_t>(2 * image);
  if (k_splits <= 1) {
    return launch_qmm_mfma_n(part, gs, bits, dtype, 1, s);
  }
  void* partial = static_cast<char*>(region) + sb_bytes;
  part.out = partial;
  rc = launch_qmm_mfma_n(part, gs, bits, dtype, k_splits, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  return reduce_k_splits(partial, a.out, plane, k_splits, dtype, s);
}

// Where the slab kernel is worth its launch: its units (K ranges x 256-row
// slabs) fill at least half the compute units -- or, with fewer, the weights
// are large enough that the kernels it replaces take longer than its floor of
// 12 us (9..16 rows) or 15 us (17..32 rows, where they run twice).  Graph
// replays, 24 rows: 6144 x 4096: 15.3 against 21.0 us, 5120 x 5120: 15.5
// against 24.5, 2048 x 8192: 14.3 against 20.4; but 4096 x 4096: 14.7 against
// 13.0, 8192 x 2048: 14.2 against 11.6; 12 rows: 5120 x 5120: 12.5 against 14.0.
bool slab_pays(const QmmArgs& a) {
  if (2 * qmm_slab_units(a) >= compute_units()) {
    return true;
  }
  const int64_t codes = static_cast<int64_t>(a.L) * a.N * a.K;
  if (a.M > 16) {
    return codes >= 25000000 || (a.K >= 8192 && codes >= 16000000);
  }
  return a.M > 8 && codes >= 26000000;
}

int run(const QmmArgs& a, int gs, int bits, int dtype, bool transpose, Scratch& sc, hipStream_t s);

// transpose=false at 2, 3, 5 or 6 bits: the [K, N] kernels read whole words
// per 8 codes, which these widths do not offer, so the codes are first repacked
// at 4 or 8 bits into the workspace (same values, same scales and biases) and
// the call goes on at that width -- 4096 x 4096 at 3 bits, one row: 1.4 ms on
// the scalar kernel, two launches of a few microseconds this way.
int run_widened(const QmmArgs& a, int gs, int bits, int dtype, Scratch& sc, hipStream_t s) {
  const int wide = widened_bits(bits);
  const int batches = a.w_batch_stride == 0 ? 1 : a.L;
  const size_t codes = static_cast<size_t>(a.K) * a.N;
  const size_t words_out = codes / 32 * wide;
  const size_t repack_bytes =
      (batches * words_out * sizeof(uint32_t) + kScratchAlign - 1) / kScratchAlign * kScratchAlign;
  QmmArgs inner = a;
  Scratch probe;
  probe.dry = true;
  int rc = run(inner, gs, wide, dtype, false, probe, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  void* region = nullptr;
  rc = claim(sc, repack_bytes + probe.need, &region);
  if (rc != MLXROCM_OK || sc.dry) {
    return rc;
  }
  uint32_t* packed = static_cast<uint32_t*>(region);
  const int64_t words_in = static_cast<int64_t>(codes / 32) * bits;
  if (batches == 1 || a.w_batch_stride == words_in) {
    rc = launch_widen_codes(a.w, packed, codes * batches, bits, s);
  } else {
    for (int l = 0; l < batches && rc == MLXROCM_OK; ++l) {
      rc = launch_widen_codes(a.w + l * a.w_batch_stride, packed + l * words_out, codes, bits, s);
    }
  }
  if (rc != MLXROCM_OK) {
    return rc;
  }
  inner.w = packed;
  inner.w_batch_stride = batches == 1 ? 0 : static_cast<int64_t>(words_out);
  Scratch rest;
  rest.base = static_cast<char*>(region) + repack_bytes;
  rest.bytes = sc.bytes - repack_bytes;
  return run(inner, gs, wide, dtype, false, rest, s);
}

int run(const QmmArgs& a, int gs, int bits, int dtype, bool transpose, Scratch& sc, hipStream_t s) {
  if (a.lhs_indices == nullptr && a.group_tiles == nullptr &&
      widens_codes(a.M, a.N, a.K, a.L, bits, dtype, transpose)) {
    return run_widened(a, gs, bits, dtype, sc, s);
  }
  // w [K, N] with a few rows of x: the streaming kernel (the tile kernel
  // needs 60-70 us for one row of a 4096 x 14336 weight)
  if (!transpose && qmv_n_supported(a, gs, bits, dtype)) {
    return run_qmv_n(a, gs, bits, dtype, sc, s);
  }
  // ... and 5..8 rows: the same kernel twice, four rows and the rest, over the
  // same planes (graph replays, W [14336, 4096] 4-bit: 41-52 us against 65 for the
  // tile kernel, which costs the same whatever M; W [4096, 4096]: 20-25 against 25)
  if (!transpose && a.M >= 5 && a.M <= 8 && a.L == 1) {
    QmmArgs head = a;
    head.M = 4;
    QmmArgs tail = a;
    tail.M = a.M - 4;
    tail.x = static_cast<const char*>(a.x) + static_cast<size_t>(4) * a.K * dtype_size(dtype);
    tail.out = static_cast<char*>(a.out) + static_cast<size_t>(4) * a.N * dtype_size(dtype);
    if (qmv_n_supported(head, gs, bits, dtype) && qmv_n_supported(tail, gs, bits, dtype)) {
      // (the first pass needs the larger workspace: it is the one a dry run sizes)
      const int rc = run_qmv_n(head, gs, bits, dtype, sc, s);
      if (rc != MLXROCM_OK || sc.dry) {
        return rc;
      }
      return run_qmv_n(tail, gs, bits, dtype, sc, s);
    }
  }
  // A few rows of x, beyond what the row-streaming GEMV keeps in registers.
  // Measured on gate/up and down projection shapes (4- and 8-bit):
  //   3..8 rows   the 32-row MFMA GEMV up to K = 8192, the wide kernel (K split
  //               over the wavefronts of a workgroup) beyond;
  //   9..16 rows  the 64-row LDS-staged kernel when N gives it enough
  //               workgroups, the wide kernel otherwise;
  //   17..32 rows the 64-row LDS-staged kernel;
  //   1..2 rows   of a width the row-streaming GEMV does not cover: the wide
  //               kernel as well.
  // 4-bit decode with a few rows of x: the 4x4x4 matrix-instruction GEMV.
  // Measured against the kernels below on gate/up, down-projection and group-32
  // shapes: it wins for 2..4 rows everywhere; for one row only where the
  // row-streaming GEMV splits a long K over all eight wavefronts (K > 8192).
  // With 5..8 rows (two operand sets, one workgroup per compute unit at a time)
  // it wins by 10-60 % from K = 8192 on, with 32-wide groups, and wherever its
  // workgroups fill their last round of compute units (4096, 11008, 12288 or
  // 28672 rows at K = 4096); at 6144 or 14336 rows the last round is half
  // empty and the 32-row MFMA GEMV is 4-12 % ahead.
  // 5..16 rows of 4-bit codes whose x fits LDS for all of K (8 rows at K = 4096,
  // 16 at K = 2048): no K ranges, no planes (14336 x 4096: 11.7-12.2 us against
  // 15.3-15.7 for the kernels below, 8192 x 2048: 6.8-7.4 against 8.5-10.4,
  // 16384 x 2048, 16 rows: 9.0 against 15.0; with up to 4 rows the 4x4x4 kernel stays
  // ahead, and 4096 x 4096 has too few 64-row workgroups: 9.8 against 7.1 us)
  if (transpose && a.M >= 5 && a.M <= 16 && a.lhs_indices == nullptr && a.w_alt == nullptr &&
      a.group_tiles == nullptr && qmm_rows8_supported(a, gs, bits, dtype, transpose) &&
      2L * ((a.N + 63) / 64) * a.L >= compute_units() &&
      // (every workgroup stages all of x: beyond 1.75 workgroups per compute unit the
      // kernel below, which stages x once per workgroup of a persistent grid, is
      // ahead -- 57344 x 4096, 8 rows: 42.9 against 39.8 us, 128256 x 4096: 88 against 76)
      4L * ((a.N + 63) / 64) * a.L <= 7L * compute_units() &&
      // (32-wide groups: twice the scales in LDS; a second round of workgroups
      // costs more than the kernel below -- 18432..28672 x 4096, 5..7 rows: 25-28
      // against 21 us)
      (gs != 32 || static_cast<long>((a.N + 63) / 64) * a.L <= compute_units())) {
    return MLXROCM_LAUNCH(sc, launch_qmm_rows8(a, gs, bits, dtype, s));
  }
  if (transpose && a.M <= 8 && qmv_quad_supported(a, gs, bits, dtype)) {
    const bool long_k = a.K > 8192;
    bool many_rows = false;
    if (a.M >= 5) {
      const long cus = compute_units();
      const long wgs = qmv_quad_workgroups_two_sets(a, bits);
      const long rounds = (wgs + cus - 1) / cus;
      // a single round, or more than 7/8 of the slots of all rounds in use
      many_rows = a.K >= 8192 || gs == 32 ||
          (wgs > 0 && (rounds <= 1 || wgs * 8 > rounds * cus * 7));
      // (not where the slab kernel below takes the shape, a single K range
      // excepted: 4096 x 14336, 8 rows: 13.5 us there against 16.1 here,
      // 8192 x 8192: 13.9 against 17.3, 5120 x 13824: 20.5 against 29.6,
      // 128256 x 4096: 63 against 104, 151936 x 3584: 73 against 143, 32000 x 4096:
      // 19.9 against 28.1; but 32768 x 1024 with 32-wide groups: 10.4 against 8.9)
      if (a.K >= 2048 && a.lhs_indices == nullptr && a.group_tiles == nullptr &&
          a.w_alt == nullptr && qmm_slab_supported(a, gs, bits, dtype, transpose) &&
          2 * qmm_slab_units(a) >= cus &&
          (qmm_slab_plane_bytes(a) == 0 || (static_cast<int64_t>(a.L) * a.M * a.N) % 4 == 0)) {
        many_rows = false;
      }
    }
    const bool use = (a.M >= 2 && a.M <= 4) ||
        (a.M == 1 && (long_k || !qmv_stream_supported(a, gs, bits, dtype))) || many_rows;
    if (use) {
      return MLXROCM_LAUNCH(sc, launch_qmv_quad(a, gs, bits, dtype, s));
    }
  }
  // 5..32 rows of 4-bit codes: packed rows streamed through LDS, x resident per
  // K range (measured against the kernels below on 4096..28672 x 4096 and
  // 4096 x 14336: 15-34 us against 19-41 us from 9 rows on, level at 5..8 rows).
  // Its units (K ranges x 256-row slabs) must fill at least half the compute
  // units: 4096 x 4096 has 64 of them and stays on the kernels below (12 us
  // against 8 us).
  if (transpose && a.M >= 5 && a.M <= 32 && a.lhs_indices == nullptr &&
      a.group_tiles == nullptr && a.w_alt == nullptr &&
      qmm_slab_supported(a, gs, bits, dtype, transpose) &&
      slab_pays(a)) {
    const size_t plane_bytes = qmm_slab_plane_bytes(a);
    if (plane_bytes == 0 || (static_cast<int64_t>(a.L) * a.M * a.N) % 4 == 0) {
      void* region = nullptr;
      if (plane_bytes != 0) {
        const int rc = claim(sc, plane_bytes, &region);
        if (rc != MLXROCM_OK) {
          return rc;
        }
      }
      return MLXROCM_LAUNCH(sc, launch_qmm_slab(a, gs, bits, dtype, region, s));
    }
  }
  // 33..64 rows: the same kernel twice, 32 rows and the rest; the second
  // pass finds weights in the Infinity Cache where they fit.  The 256-row tile
  // GEMM below costs the same whatever M (graph replays, 64 rows: 14336 x 4096:
  // 37 us, twice the slab kernel: 31; 4096 x 14336: 46.5 against 35; 28672 x 4096:
  // 60 against 50; 128256 x 4096: 270 against 180); from 65 rows on it is ahead.
  if (transpose && a.M > 32 && a.M <= 64 && a.L == 1 && gs != 32 && a.lhs_indices == nullptr &&
      a.group_tiles == nullptr && a.w_alt == nullptr) {
    const int first = 32;
    QmmArgs head = a;
    head.M = first;
    QmmArgs tail = a;
    tail.M = a.M - first;
    tail.x = static_cast<const char*>(a.x) + static_cast<size_t>(first) * a.K * dtype_size(dtype);
    tail.out = static_cast<char*>(a.out) + static_cast<size_t>(first) * a.N * dtype_size(dtype);
    if (qmm_slab_supported(head, gs, bits, dtype, transpose) &&
        qmm_slab_supported(tail, gs, bits, dtype, transpose) &&
        2 * qmm_slab_units(head) >= compute_units()) {
      // both passes use the same planes, one after the other on the stream
      const size_t plane_bytes = qmm_slab_plane_bytes(head);
      void* region = nullptr;
      if (plane_bytes != 0) {
        const int rc = claim(sc, plane_bytes, &region);
        if (rc != MLXROCM_OK) {
          return rc;
        }
      }
      if (sc.dry) {
        return MLXROCM_OK;
      }
      const int rc = launch_qmm_slab(head, gs, bits, dtype, region, s);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      return launch_qmm_slab(tail, gs, bits, dtype, region, s);
    }
  }
  // (two rows of 8-bit codes over a long K: the streaming kernel's dot products
  // are issue-bound there, 28 us against 20 us for the wide kernel at K = 14336)
  const bool few_rows = a.M >= 3 || !qmv_stream_supported(a, gs, bits, dtype) ||
      (a.M == 2 && bits == 8 && a.K > 8192);
  // 17..32 rows over a narrow N (fewer 64-row workgroups than half the compute
  // units): the wide kernel twice, 16 rows each; the second pass finds the
  // weights in the Infinity Cache (4096 x 4096: 24 -> 16 us, 4096 x 14336: 56 -> 45 us)
  if (transpose && a.M > 16 && a.M <= 32 && a.L == 1 && a.lhs_indices == nullptr &&
      a.group_tiles == nullptr && (a.N + 63) / 64 < compute_units() / 2) {
    QmmArgs part = a;
    part.M = 16;
    if (qmv_wide_supported(part, gs, bits, dtype, transpose)) {
      if (sc.dry) {
        return MLXROCM_OK;
      }
      int rc = launch_qmv_wide(part, gs, bits, dtype, s);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      const size_t esize = dtype_size(dtype);
      part.M = a.M - 16;
      part.x = static_cast<const char*>(a.x) + static_cast<size_t>(16) * a.K * esize;
      part.out = static_cast<char*>(a.out) + static_cast<size_t>(16) * a.N * esize;
      return launch_qmv_wide(part, gs, bits, dtype, s);
    }
  }
  // (17..32 rows: the staged kernel walks K serially with N / 64 workgroups, so
  // a narrow N with a long K goes to the tile kernel and its K split instead:
  // 4096 x 14336, 32 rows: 78 us against 57 us)
  const bool narrow_long = a.M > 16 && a.K > 8192 &&
      static_cast<long>((a.N + 63) / 64) * a.L < compute_units() / 2 &&
      a.lhs_indices == nullptr && a.group_tiles == nullptr;
  // (8-bit codes, 3..8 rows over 64 MB of weights or more: the staged kernel is
  // ahead of the MFMA GEMV as it is from 9 rows on -- graph replays, 8 rows:
  // 28672 x 4096: 26 against 37 us, 8192 x 8192: 32 against 45, 49152 x 4096: 38
  // against 55; level at 14336 x 4096 and 128256 x 4096)
  const bool many_bytes = bits == 8 && a.M >= 3 && a.N >= 8192 &&
      static_cast<int64_t>(a.N) * a.K >= (int64_t{64} << 20);
  const bool staged = (a.M > 16 || (a.M > 8 && a.N >= 8192) || many_bytes) && !narrow_long;
  // one row at a width the row-streaming GEMV does not cover (2/3/5/6 bits): the
  // fp32-arithmetic streaming kernel
  if (transpose && a.M == 1 && few_rows && qmv_f32_supported(a, gs, bits, dtype)) {
    return MLXROCM_LAUNCH(sc, launch_qmv_f32(a, gs, bits, dtype, s));
  }
  if (few_rows && !staged && a.M <= 16 && qmv_wide_supported(a, gs, bits, dtype, transpose)) {
    const bool gemv_better = a.M <= 8 && a.K <= 8192 && qmv_mfma_supported(a, gs, bits, dtype);
    if (!gemv_better) {
      return MLXROCM_LAUNCH(sc, launch_qmv_wide(a, gs, bits, dtype, s));
    }
  }
  if (staged && qmm_skinny_supported(a, gs, bits, dtype, transpose)) {
    return MLXROCM_LAUNCH(sc, launch_qmm_skinny(a, gs, bits, dtype, s));
  }
  if (staged && a.M <= 16 && qmv_wide_supported(a, gs, bits, dtype, transpose)) {
    return MLXROCM_LAUNCH(sc, launch_qmv_wide(a, gs, bits, dtype, s));
  }
  // float32 with 9..16 rows: the GEMV kernels twice, eight rows and the rest (the
  // split-bf16 matrix path costs the same whatever M -- graph replays, 14336 x
  // 4096 4-bit: 155 us; eight rows: 66, four: 37)
  if (transpose && dtype == MLXROCM_FLOAT32 && a.M > kQmvMaxM && a.M <= 2 * kQmvMaxM && a.L == 1 &&
      a.lhs_indices == nullptr && a.group_tiles == nullptr) {
    QmmArgs head = a;
    head.M = kQmvMaxM;
    QmmArgs tail = a;
    tail.M = a.M - kQmvMaxM;
    tail.x = static_cast<const char*>(a.x) + static_cast<size_t>(kQmvMaxM) * a.K * sizeof(float);
    tail.out = static_cast<char*>(a.out) + static_cast<size_t>(kQmvMaxM) * a.N * sizeof(float);
    const int rc = run(head, gs, bits, dtype, transpose, sc, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    return run(tail, gs, bits, dtype, transpose, sc, s);
  }
  switch (choose_family(a.M, a.N, a.K, a.L, bits, dtype, transpose)) {
    case Family::QmmT:
      if (qmm_mfma_supported(a, gs, bits, dtype, transpose)) {
        int k_splits = 1;
        if (a.lhs_indices == nullptr && (static_cast<int64_t>(a.M) * a.N) % 4 == 0) {
          k_splits = qmm_mfma_k_splits(a.M, a.N, a.K, a.L);
        }
        if (a.lhs_indices == nullptr && a.M >= kTransposeSbMinM) {
          return run_qmm_t_transposed_sb(a, gs, bits, dtype, k_splits, sc, s);
        }
        if (k_splits > 1) {
          return run_k_split(a, gs, bits, dtype, k_splits, sc, s);
        }
        return MLXROCM_LAUNCH(sc, launch_qmm_mfma(a, gs, bits, dtype, s));
      }
      if (dtype == MLXROCM_FLOAT32 && a.lhs_indices == nullptr) {
        return run_split_fp32(a, gs, bits, sc, s);
      }
      return MLXROCM_LAUNCH(sc, launch_qmm_naive(a, gs, bits, dtype, transpose, s));
    case Family::Qmv:
      if (qmv_stream_supported(a, gs, bits, dtype)) {
        return MLXROCM_LAUNCH(sc, launch_qmv_stream(a, gs, bits, dtype, s));
      }
      if (qmv_mfma_supported(a, gs, bits, dtype)) {
        return MLXROCM_LAUNCH(sc, launch_qmv_mfma(a, gs, bits, dtype, s));
      }
      if (qmv_f32_supported(a, gs, bits, dtype)) {
        return MLXROCM_LAUNCH(sc, launch_qmv_f32(a, gs, bits, dtype, s));
      }
      return MLXROCM_LAUNCH(sc, launch_qmv_generic(a, gs, bits, dtype, s));
    case Family::QmmN:
      if (a.lhs_indices == nullptr && qmm_mfma_supported(a, gs, bits, dtype, transpose)) {
        return run_qmm_n(a, gs, bits, dtype, sc, s);
      }
      return MLXROCM_LAUNCH(sc, launch_qmm_naive(a, gs, bits, dtype, transpose, s));
    case Family::QmmNaive:
      return MLXROCM_LAUNCH(sc, launch_qmm_naive(a, gs, bits, dtype, transpose, s));
  }
  return fail(MLXROCM_UNSUPPORTED, "no kernel");
}

} // namespace

} // namespace mlxrocm

using namespace mlxrocm;

extern "C" const char* mlxrocm_qmm_kernel_name(
    int M,
    int N,
    int K,
    int L,
    int group_size,
    int bits,
    int dtype,
    int transpose) {
  if (check_shape("qmm", M, N, K, L, group_size, bits, dtype, transpose) !=
      MLXROCM_OK) {
    return nullptr;
  }
  return family_name(choose_family(M, N, K, L, bits, dtype, transpose != 0));
}

namespace {

// out[i] = silu(gate[i]) * up[i] with the roundings of the unfused chain
// (sigmoid, gate * sigmoid and the product are each rounded to T, as
// x * sigmoid(x) followed by a multiply is in the element type).
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* gate_up, T* out, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) {
    return;
  }
  const float g = to_f32(gate_up[i]);
  const float u = to_f32(gate_up[n + i]);
  const float sg = to_f32(from_f32<T>(1.0f / (1.0f + __expf(-g))));
  const float h = to_f32(from_f32<T>(g * sg));
  out[i] = from_f32<T>(h * u);
}

} // namespace

extern "C" size_t mlxrocm_qmm_swiglu_workspace_size(int M, int N, int dtype) {
  if (M <= 0 || N <= 0) {
    return 0;
  }
  return static_cast<size_t>(2) * M * N * dtype_size(dtype);
}

extern "C" int mlxrocm_qmm_swiglu(
    const void* x,
    const uint32_t* wq_gate,
    const void* scales_gate,
    const void* biases_gate,
    const uint32_t* wq_up,
    const void* scales_up,
    const void* biases_up,
    void* out,
    void* workspace,
    int M,
    int N,
    int K,
    int group_size,
    int bits,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_qmm_swiglu");
  int rc = check_shape("quantized_swiglu", M, N, K, 1, group_size, bits, dtype, 1);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (M > 8) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[quantized_swiglu] M=%d: the fused gate/up projection covers decode (M <= 8)",
        M);
  }
  if (static_cast<int64_t>(M) * N == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(out, static_cast<size_t>(M) * N * dtype_size(dtype), s);
  }
  if (!x || !wq_gate || !scales_gate || !biases_gate || !wq_up || !scales_up || !biases_up ||
      !out || !workspace) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantized_swiglu] null device pointer");
  }
  if (!aligned16(wq_up) || !aligned16(scales_up) || !aligned16(biases_up) ||
      !aligned16(workspace)) {
    return fail(MLXROCM_UNSUPPORTED, "[quantized_swiglu] operand pointers must be 16-byte aligned");
  }
  QmmArgs a{};
  a.x = x;
  a.w = wq_gate;
  a.scales = scales_gate;
  a.biases = biases_gate;
  a.w_alt = wq_up;
  a.scales_alt = scales_up;
  a.biases_alt = biases_up;
  a.out = workspace; // [2, M, N]: gate, up
  a.M = M;
  a.N = N;
  a.K = K;
  a.L = 2;
  a.x_batches = 2;
  a.n_experts = 2;
  rc = check_alignment("quantized_swiglu", a, dtype);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  // one row of x on the row-streaming GEMV: the gate is applied in the kernel's
  // epilogue and nothing passes through the workspace
  {
    QmmArgs one = a;
    one.L = 1;
    one.out = out;
    if (qmv_stream_glu_supported(one, group_size, bits, dtype)) {
      return launch_qmv_stream_glu(one, group_size, bits, dtype, s);
    }
  }
  Scratch none; // decode shapes with transpose != 0 claim no scratch
  rc = run(a, group_size, bits, dtype, true, none, s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  const size_t n = static_cast<size_t>(M) * N;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  rc = dispatch_dtype(dtype, [&](auto tval) {
    using T = decltype(tval);
    swiglu_kernel<T><<<blocks, 256, 0, s>>>(
        static_cast<const T*>(workspace), static_cast<T*>(out), n);
    MLXROCM_HIP_TRY(hipGetLastError());
    return static_cast<int>(MLXROCM_OK);
  });
  return rc;
}

namespace {

// Body of mlxrocm_qmm and, as a dry run, of mlxrocm_qmm_workspace_size.
int qmm_entry(
    const void* x,
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t sb_batch_stride,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    Scratch& sc,
    hipStream_t s) {
  int rc = check_shape(
      "quantized_matmul", M, N, K, L, group_size, bits, dtype, transpose);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * L == 0) {
    return MLXROCM_OK; // empty output
  }
  if (K == 0) {
    return MLXROCM_LAUNCH(
        sc, launch_zero_fill(out, static_cast<size_t>(M) * N * L * dtype_size(dtype), s));
  }
  if (x_batch_stride < 0 || w_batch_stride < 0 || sb_batch_stride < 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantized_matmul] negative stride");
  }
  QmmArgs a{};
  a.x = x;
  a.w = wq;
  a.scales = scales;
  a.biases = biases;
  a.out = out;
  a.M = M;
  a.N = N;
  a.K = K;
  a.L = L;
  a.x_batch_stride = x_batch_stride;
  a.w_batch_stride = w_batch_stride;
  a.sb_batch_stride = sb_batch_stride;
  a.lhs_indices = nullptr;
  a.rhs_indices = nullptr;
  a.x_batches = L;
  a.n_experts = L;
  if (!sc.dry) {
    if (!x || !wq || !scales || !biases || !out) {
      return fail(
          MLXROCM_INVALID_ARGUMENT, "[quantized_matmul] null device pointer");
    }
    rc = check_alignment("quantized_matmul", a, dtype);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    if (sc.base != nullptr && (reinterpret_cast<uintptr_t>(sc.base) % kScratchAlign) != 0) {
      return fail(
          MLXROCM_INVALID_ARGUMENT,
          "[quantized_matmul] the workspace must be %zu-byte aligned",
          kScratchAlign);
    }
  }
  return run(a, group_size, bits, dtype, transpose != 0, sc, s);
}

} // namespace

extern "C" size_t mlxrocm_qmm_workspace_size(
    int M,
    int N,
    int K,
    int L,
    int batched_weights,
    int group_size,
    int bits,
    int dtype,
    int transpose) {
  Scratch sc;
  sc.dry = true;
  // the strides only say "one weight for every batch entry" or "one each"
  const int64_t w_stride = batched_weights ? 4096 : 0;
  const int64_t x_stride = static_cast<int64_t>(M) * K;
  if (qmm_entry(
          nullptr, nullptr, nullptr, nullptr, nullptr, M, N, K, L, x_stride, w_stride,
          w_stride, group_size, bits, dtype, transpose, sc, nullptr) != MLXROCM_OK) {
    return 0;
  }
  return sc.need;
}

extern "C" int mlxrocm_qmm(
    const void* x,
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t sb_batch_stride,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_qmm");
  Scratch sc;
  sc.base = static_cast<char*>(workspace);
  sc.bytes = workspace != nullptr ? workspace_bytes : 0;
  return qmm_entry(
      x, wq, scales, biases, out, M, N, K, L, x_batch_stride, w_batch_stride,
      sb_batch_stride, group_size, bits, dtype, transpose, sc,
      static_cast<hipStream_t>(stream));
}

extern "C" size_t mlxrocm_qmm_sb_image_size(int N, int K, int batches, int group_size, int dtype) {
  if (N <= 0 || K <= 0 || batches <= 0 || group_size <= 0 || K % group_size != 0) {
    return 0;
  }
  return qmm_n_sb_bytes(N, K / group_size, batches, dtype);
}

extern "C" int mlxrocm_qmm_sb_image(
    const void* scales,
    const void* biases,
    void* image,
    int N,
    int K,
    int batches,
    int64_t sb_batch_stride,
    int group_size,
    int dtype,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_qmm_sb_image");
  if (N <= 0 || K <= 0 || batches <= 0 || (group_size != 32 && group_size != 64 && group_size != 128) ||
      K % group_size != 0 || sb_batch_stride < 0 ||
      (dtype != MLXROCM_FLOAT32 && dtype != MLXROCM_FLOAT16 && dtype != MLXROCM_BFLOAT16)) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qmm_sb_image] invalid shape or dtype");
  }
  if (!scales || !biases || !image) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[qmm_sb_image] null device pointer");
  }
  return transpose_sb_for_qmm_n(
      scales, biases, image, N, K / group_size, batches, sb_batch_stride, dtype,
      static_cast<hipStream_t>(stream));
}

extern "C" int mlxrocm_qmm_prepacked(
    const void* x,
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    const void* sb_image,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t sb_batch_stride,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_qmm_prepacked");
  if (sb_image != nullptr && (reinterpret_cast<uintptr_t>(sb_image) & 15u) != 0) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[quantized_matmul] the image must be 16-byte aligned");
  }
  Scratch sc;
  sc.base = static_cast<char*>(workspace);
  sc.bytes = workspace != nullptr ? workspace_bytes : 0;
  sc.sb_image = transpose != 0 ? sb_image : nullptr;
  return qmm_entry(
      x, wq, scales, biases, out, M, N, K, L, x_batch_stride, w_batch_stride,
      sb_batch_stride, group_size, bits, dtype, transpose, sc,
      static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// The no-allocation variant of mlxrocm_qmm.
//
// Device scratch for callers that cannot allocate: one array in the library's
// device image, so every GPU the library runs on holds its own copy from the
// moment the code object is loaded until the process ends.  In host code the
// name below is only a handle for hipGetSymbolAddress; the address a kernel
// may use is looked up once per device and kept in g_static_scratch.
constexpr size_t kStaticScratchBytes = size_t(64) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_static_mu;
void* g_static_scratch[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (first call on a device
// resolves it; later calls only read the table).
int static_scratch(void** out) {
  int dev = 0;
  MLXROCM_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) {
    return fail(MLXROCM_UNSUPPORTED, "[quantized_matmul_static] device %d out of range", dev);
  }
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (g_static_scratch[dev] == nullptr) {
    void* ptr = nullptr;
    MLXROCM_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) {
      return fail(MLXROCM_HIP_ERROR, "[quantized_matmul_static] no address for the scratch array");
    }
    g_static_scratch[dev] = ptr;
  }
  *out = g_static_scratch[dev];
  return MLXROCM_OK;
}

} // namespace

extern "C" int mlxrocm_qmm_static(
    const void* x,
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t sb_batch_stride,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_qmm_static");
  void* region = nullptr;
  int rc = static_scratch(&region);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  const size_t need = mlxrocm_qmm_workspace_size(
      M, N, K, L, w_batch_stride != 0 || sb_batch_stride != 0, group_size, bits, dtype, transpose);
  if (need > kStaticScratchBytes) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[quantized_matmul_static] this shape needs %zu bytes of scratch, the built-in "
        "buffer holds %zu; use mlxrocm_qmm with a workspace",
        need,
        kStaticScratchBytes);
  }
  // Nothing the kernels keep in scratch has to start at zero: the transposed
  // scale / bias image, the split x and every partial plane are written in
  // full before they are read, so the previous call's contents need no clearing.
  Scratch sc;
  sc.base = static_cast<char*>(region);
  sc.bytes = kStaticScratchBytes;
  return qmm_entry(
      x, wq, scales, biases, out, M, N, K, L, x_batch_stride, w_batch_stride,
      sb_batch_stride, group_size, bits, dtype, transpose, sc,
      static_cast<hipStream_t>(stream));
}

// Small expert groups of 4-bit weights run on the slab kernel, whose K ranges
// meet in fp32 planes behind the grouping tables.
bool group_gather_small(int K, int n_indices, int n_experts) {
  return K % 128 == 0 && static_cast<int64_t>(n_indices) <= 64 * static_cast<int64_t>(n_experts);
}
bool group_gather_slab(int N, int K, int n_indices, int n_experts, int gs, int bits) {
  // (32-wide groups only in the 16-row tiles of the kernel's own grouping)
  const int rows = gs == 32 && qmm_slab_plans_in_kernel(n_indices, n_experts) ? 16 : 32;
  return group_gather_small(K, n_indices, n_experts) && qmm_slab_shape_ok(rows, N, K, gs, bits);
}

// Grouping by expert pays when every expert's weights are shared by several
// index pairs; it needs one row of x per pair, the matrix-core GEMM, 32-bit
// element offsets into x and a workspace for the sorted order.
// (Where the slab kernel groups the pairs itself there is no planning launch
// to pay for, and a pair that shares its expert with no other still costs what
// its own GEMV would: grouping pays from 8 pairs on -- 8 experts of
// [14336, 4096], top-2: 8 tokens 52 us against 98 us one GEMV per pair, 12
// tokens 53 against 155, 4 tokens 46 against 44, 2 tokens 34 against 24.)
bool group_gather(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int x_batches,
    int64_t x_batch_stride,
    int group_size,
    int bits,
    int dtype,
    bool transpose) {
  if (M != 1 || !transpose || dtype == MLXROCM_FLOAT32 || K % 64 != 0 || K < 64) {
    return false;
  }
  // (... for experts of 4 MB and more: one GEMV over a smaller one takes about a
  // microsecond -- 64 experts of [1408, 2048], 12 pairs: 9 us against 19.5)
  const bool few = n_indices >= 8 && qmm_slab_plans_in_kernel(n_indices, n_experts) &&
      static_cast<int64_t>(N) * K >= (int64_t{8} << 20) &&
      group_gather_slab(N, K, n_indices, n_experts, group_size, bits);
  // (from one pair per expert on average: 64 experts of [2048, 1408], top-6, 32
  // tokens: 99 us one GEMV per pair, 47 us grouped; 8-bit, 16 tokens: 88 against 50)
  if (!few &&
      (n_indices < 32 || static_cast<int64_t>(n_indices) < static_cast<int64_t>(n_experts))) {
    return false;
  }
  if (static_cast<int64_t>(x_batches) * x_batch_stride + K >= (int64_t(1) << 32)) {
    return false;
  }
  if (gather_group_max_tiles(n_indices, n_experts, kGroupSmallTile) > 65535) {
    return false;
  }
  return gather_group_workspace_bytes(n_indices, n_experts) > 0;
}

// transpose=false (what the backward pass of an expert layer asks for): the
// pairs are sorted by expert in 256-row tiles for the tile GEMM's column
// loader, which reads scales and biases from [group][k] images -- those of all
// experts are made behind the grouping tables first.
constexpr size_t kGroupTablesAlign = 256;
size_t group_gather_n_tables(int n_indices, int n_experts) {
  return (gather_group_workspace_bytes(n_indices, n_experts) + kGroupTablesAlign - 1) /
      kGroupTablesAlign * kGroupTablesAlign;
}
bool group_gather_n(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int x_batches,
    int64_t x_batch_stride,
    int bits,
    int dtype,
    bool transpose) {
  if (M != 1 || transpose || dtype == MLXROCM_FLOAT32 || K % 64 != 0 || K < 64 || N < 8 ||
      (bits != 4 && bits != 8)) {
    return false;
  }
  // (one product per pair has no fast kernel with [K, N] weights: 8 experts of
  // [14336, 4096], 32 pairs: 5.5 ms against 0.37 ms grouped, which is what a
  // single 256-row tile per expert costs -- grouping pays from a few pairs on)
  if (n_indices < 4) {
    return false;
  }
  if (static_cast<int64_t>(x_batches) * x_batch_stride + K >= (int64_t(1) << 32)) {
    return false;
  }
  if (gather_group_max_tiles(n_indices, n_experts, kGroupLargeTile) > 65535) {
    return false;
  }
  return gather_group_workspace_bytes(n_indices, n_experts) > 0;
}

extern "C" size_t mlxrocm_gather_qmm_workspace_size(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    int /*rhs_sorted*/) {
  // x_batches / stride are unknown here; mlxrocm_gather_qmm checks them and
  // falls back to the ungrouped launch if they rule grouping out.
  if (group_gather_n(M, N, K, n_indices, n_experts, 1, 0, bits, dtype, transpose != 0)) {
    return group_gather_n_tables(n_indices, n_experts) +
        qmm_n_sb_bytes(K, N / group_size, n_experts, dtype);
  }
  if (!group_gather(M, N, K, n_indices, n_experts, 1, 0, group_size, bits, dtype, transpose != 0)) {
    return 0;
  }
  size_t bytes = gather_group_workspace_bytes(n_indices, n_experts);
  if (group_gather_slab(N, K, n_indices, n_experts, group_size, bits)) {
    bytes += qmm_slab_grouped_plane_bytes(n_indices, N, K);
  }
  return bytes;
}

extern "C" int mlxrocm_gather_qmm(
    const void* x,
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    void* out,
    int M,
    int N,
    int K,
    int n_indices,
    int x_batches,
    int n_experts,
    int64_t x_batch_stride,
    int64_t w_expert_stride,
    int64_t sb_expert_stride,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    int /*rhs_sorted*/,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_gather_qmm");
  int rc = check_shape(
      "gather_qmm", M, N, K, n_indices, group_size, bits, dtype, transpose);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * n_indices == 0) {
    return MLXROCM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (K == 0) {
    return launch_zero_fill(
        out, static_cast<size_t>(M) * N * n_indices * dtype_size(dtype), s);
  }
  if (!x || !wq || !scales || !biases || !out || !lhs_indices ||
      !rhs_indices) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qmm] null device pointer");
  }
  if (x_batches <= 0 || n_experts <= 0 || x_batch_stride < 0 ||
      w_expert_stride < 0 || sb_expert_stride < 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT, "[gather_qmm] invalid batch description");
  }
  QmmArgs a{};
  a.x = x;
  a.w = wq;
  a.scales = scales;
  a.biases = biases;
  a.out = out;
  a.M = M;
  a.N = N;
  a.K = K;
  a.L = n_indices;
  a.x_batch_stride = x_batch_stride;
  a.w_batch_stride = w_expert_stride;
  a.sb_batch_stride = sb_expert_stride;
  a.lhs_indices = lhs_indices;
  a.rhs_indices = rhs_indices;
  a.x_batches = x_batches;
  a.n_experts = n_experts;
  rc = check_alignment("gather_qmm", a, dtype);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (workspace != nullptr &&
      group_gather(
          M, N, K, n_indices, n_experts, x_batches, x_batch_stride, group_size, bits, dtype,
          transpose != 0) &&
      workspace_bytes >= gather_group_workspace_bytes(n_indices, n_experts)) {
    if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) {
      return fail(MLXROCM_INVALID_ARGUMENT, "[gather_qmm] workspace must be 4-byte aligned");
    }
    // small groups (at most 64 pairs per expert on average) go to the few-row
    // kernel in 32-row tiles, larger ones to the 256-row tile GEMM
    const bool small = group_gather_small(K, n_indices, n_experts);
    const size_t tables = gather_group_workspace_bytes(n_indices, n_experts);
    const bool slab = group_gather_slab(N, K, n_indices, n_experts, group_size, bits) &&
        (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0 && // 16-byte stores into the planes
        workspace_bytes >= tables + qmm_slab_grouped_plane_bytes(n_indices, N, K);
    if (slab && qmm_slab_plans_in_kernel(n_indices, n_experts)) {
      // few pairs: the kernel groups them itself, one launch less
      bind_gather_group(a, kGroupSmallTile, workspace);
      return launch_qmm_slab_grouped(
          a, group_size, bits, dtype, static_cast<char*>(workspace) + tables, true, s);
    }
    rc = launch_gather_group(a, dtype, small ? kGroupSmallTile : kGroupLargeTile, workspace, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    if (slab) {
      return launch_qmm_slab_grouped(
          a, group_size, bits, dtype, static_cast<char*>(workspace) + tables, false, s);
    }
    return small ? launch_qmm_skinny_grouped(a, group_size, bits, dtype, s)
                 : launch_qmm_mfma_grouped(a, group_size, bits, dtype, s);
  }
  if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0 &&
      group_gather_n(
          M, N, K, n_indices, n_experts, x_batches, x_batch_stride, bits, dtype, transpose != 0)) {
    const int G = N / group_size;
    const int images = sb_expert_stride == 0 ? 1 : n_experts;
    const size_t tables = group_gather_n_tables(n_indices, n_experts);
    if (workspace_bytes >= tables + qmm_n_sb_bytes(K, G, images, dtype)) {
      rc = launch_gather_group(a, dtype, kGroupLargeTile, workspace, s);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      char* image = static_cast<char*>(workspace) + tables;
      rc = transpose_sb_for_qmm_n(scales, biases, image, K, G, images, sb_expert_stride, dtype, s);
      if (rc != MLXROCM_OK) {
        return rc;
      }
      const size_t one = static_cast<size_t>(K) * G; // elements of one [G][K] image
      a.scales = image;
      a.biases = image + one * dtype_size(dtype);
      a.sb_batch_stride = images == 1 ? 0 : static_cast<int64_t>(2 * one);
      return launch_qmm_mfma_grouped_n(a, group_size, bits, dtype, s);
    }
  }
  // One grid z-slot per index pair; large index lists go in slices.
  constexpr int kMaxZ = 65535;
  for (int first = 0; first < n_indices; first += kMaxZ) {
    QmmArgs part = a;
    part.L = (n_indices - first < kMaxZ) ? n_indices - first : kMaxZ;
    part.lhs_indices = lhs_indices + first;
    part.rhs_indices = rhs_indices + first;
    part.out = static_cast<char*>(out) +
        static_cast<size_t>(first) * M * N * dtype_size(dtype);
    Scratch none; // no launch with index arrays claims scratch
    rc = run(part, group_size, bits, dtype, transpose != 0, none, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
  }
  return MLXROCM_OK;
}
