// qmm_api.hip -- C entry points of quantized_matmul / gather_qmm: argument
// checks, kernel choice, launch.
#include <atomic>
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

int check_alignment(
    const char* who, const QmmArgs& a, int dtype, bool transpose = true, int bits = 0) {
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
  // [K, N] weights with a K that is not a multiple of 16 bytes: the rows of x are
  // unaligned anyway, the kernels of that case read x element by element, and a
  // stack of such matrices (x [B, 1, 67]) cannot have an aligned stride
  const bool x_by_elements = !transpose && a.K % x_vec != 0;
  // likewise the packed rows: when a row is not a whole number of 16-byte pieces
  // the kernels of that shape load words, and a stack of such matrices (three of
  // [3, 32] at 6 bits: 18 words each) has no aligned stride either
  const int64_t row_words = static_cast<int64_t>(transpose ? a.K : a.N) / 32 * bits;
  const bool w_by_words = bits != 0 && row_words % 4 != 0;
  if (strided &&
      ((!x_by_elements && a.x_batch_stride % x_vec != 0) ||
       (!w_by_words && a.w_batch_stride % 4 != 0))) {
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
    // a call may claim more than once (two passes over the same region): the
    // workspace has to hold the largest request
    sc.need = bytes > sc.need ? bytes : sc.need;
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
    rc = interleave_sb_for_qmm_t(
        a.scales, a.biases, region, a.N, G, batches, a.sb_batch_stride, s);
    if (rc != MLXROCM_OK) {
      return rc;
    }
    sb = region;
  }
  const size_t image = static_cast<size_t>(a.N) * G; // pairs of one weight matrix
  QmmArgs part = a;
  part.scales = sb;
  part.biases = sb; // (unused: a pair holds both)
  part.sb_batch_stride = batches == 1 ? 0 : static_cast<int64_t>(2 * image);
  part.sb_transposed = 2;
  if (k_splits <= 1) {
    return launch_qmm_mfma_pairs(part, gs, bits, dtype, s);
  }
  void* partial = static_cast<char*>(region) + sb_bytes;
  part.out = partial;
  rc = launch_qmm_mfma_ksplit_pairs(part, gs, bits, dtype, k_splits, s);
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
  if (codes % 32 != 0) {
    return fail(MLXROCM_UNSUPPORTED, "[qmm] K * N = %zu is not a multiple of 32 codes", codes);
  }
  const size_t repack_bytes =
      (static_cast<size_t>(batches) * words_out * sizeof(uint32_t) + kScratchAlign - 1) /
      kScratchAlign * kScratchAlign;
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
  const size_t region_words = repack_bytes / sizeof(uint32_t);
  const int64_t words_in = static_cast<int64_t>(codes / 32) * bits;
  if (batches == 1 || a.w_batch_stride == words_in) {
    rc = launch_widen_codes(a.w, packed, region_words, codes * batches, bits, s);
  } else {
    for (int l = 0; l < batches && rc == MLXROCM_OK; ++l) {
      rc = launch_widen_codes(
          a.w + l * a.w_batch_stride, packed + l * words_out, region_words - l * words_out, codes,
          bits, s);
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

// ---------------------------------------------------------------------------
// Kernel choice.  One call of the dispatcher is a `Call`; the table below is
// walked top to bottom and the first rule whose predicate holds runs.  A
// predicate reads the problem only (never the scratch), so a sizing run, a
// rehearsal and the real call take the same rule.  Every threshold is a
// measurement on the 256-CU part; the rule's `evidence` string carries the
// figures (microseconds per launch unless stated; "A against B" = this rule
// against the rules below it).
struct Call {
  const QmmArgs& a;
  int gs;
  int bits;
  int dtype;
  bool transpose;
  Scratch& sc;
  hipStream_t s;
};

struct Rule {
  const char* name;
  bool (*applies)(const Call&);
  int (*launch)(const Call&);
  const char* evidence;
};

// no index arrays, no grouped tile list
bool plain(const QmmArgs& a) {
  return a.lhs_indices == nullptr && a.group_tiles == nullptr;
}

// x rows [first, first + rows) of a single problem
QmmArgs row_block(const Call& c, int first, int rows) {
  QmmArgs part = c.a;
  const size_t esize = dtype_size(c.dtype);
  part.M = rows;
  part.x = static_cast<const char*>(c.a.x) + static_cast<size_t>(first) * c.a.K * esize;
  part.out = static_cast<char*>(c.a.out) + static_cast<size_t>(first) * c.a.N * esize;
  return part;
}

bool planes_aligned(const QmmArgs& a) {
  return qmm_slab_plane_bytes(a) == 0 || (static_cast<int64_t>(a.L) * a.M * a.N) % 4 == 0;
}

// 5..8 rows on the 4x4x4 kernel run two operand sets, one workgroup per compute
// unit at a time: worth it over a long K, with 32-wide groups, or where the
// workgroups fill their last round of compute units -- unless the slab kernel
// takes the shape.
bool quad_pays_5_to_8(const Call& c) {
  const QmmArgs& a = c.a;
  const long cus = compute_units();
  const long wgs = qmv_quad_workgroups_two_sets(a, c.bits);
  const long rounds = (wgs + cus - 1) / cus;
  const bool fits = a.K >= 8192 || c.gs == 32 ||
      (wgs > 0 && (rounds <= 1 || wgs * 8 > rounds * cus * 7));
  const bool slab_takes_it = a.K >= 2048 && plain(a) && a.w_alt == nullptr &&
      qmm_slab_supported(a, c.gs, c.bits, c.dtype, c.transpose) &&
      2 * qmm_slab_units(a) >= cus && planes_aligned(a);
  return fits && !slab_takes_it;
}

// shapes beyond what the row-streaming GEMV keeps in registers
bool few_rows(const Call& c) {
  return c.a.M >= 3 || !qmv_stream_supported(c.a, c.gs, c.bits, c.dtype) ||
      (c.a.M == 2 && c.bits == 8 && c.a.K > 8192);
}

// where the 64-row LDS-staged kernel is the choice among the few-row kernels
bool staged(const Call& c) {
  const QmmArgs& a = c.a;
  const bool narrow_long = a.M > 16 && a.K > 8192 &&
      static_cast<long>((a.N + 63) / 64) * a.L < compute_units() / 2 && plain(a);
  const bool many_bytes = c.bits == 8 && a.M >= 3 && a.N >= 8192 &&
      static_cast<int64_t>(a.N) * a.K >= (int64_t{64} << 20);
  return (a.M > 16 || (a.M > 8 && a.N >= 8192) || many_bytes) && !narrow_long;
}

Family family_of(const Call& c) {
  return choose_family(c.a.M, c.a.N, c.a.K, c.a.L, c.bits, c.dtype, c.transpose);
}

int tile_k_splits(const Call& c) {
  if (c.a.lhs_indices == nullptr && (static_cast<int64_t>(c.a.M) * c.a.N) % 4 == 0) {
    return qmm_mfma_k_splits(c.a.M, c.a.N, c.a.K, c.a.L);
  }
  return 1;
}

bool tile_t(const Call& c) {
  return family_of(c) == Family::QmmT && qmm_mfma_supported(c.a, c.gs, c.bits, c.dtype, c.transpose);
}

// Two passes over the same scratch, one after the other on the stream.
int two_passes(const Call& c, const QmmArgs& head, const QmmArgs& tail) {
  const int rc = run(head, c.gs, c.bits, c.dtype, c.transpose, c.sc, c.s);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  return run(tail, c.gs, c.bits, c.dtype, c.transpose, c.sc, c.s);
}

int slab_launch(const Call& c, const QmmArgs& a, void* region) {
  return MLXROCM_LAUNCH(c.sc, launch_qmm_slab(a, c.gs, c.bits, c.dtype, region, c.s));
}

const Rule kRules[] = {
    {"widen_codes",
     [](const Call& c) {
       return plain(c.a) &&
           widens_codes(c.a.M, c.a.N, c.a.K, c.a.L, c.bits, c.dtype, c.transpose);
     },
     [](const Call& c) { return run_widened(c.a, c.gs, c.bits, c.dtype, c.sc, c.s); },
     "transpose=false at 2/3/5/6 bits: codes repacked at 4 or 8 bits, then this table again. "
     "4096x4096 3-bit, one row: 1.39 ms on the scalar kernel, 14.2 us this way; 5..128 rows "
     "1.3-1.4 ms -> 32-34 us"},
    {"qmv_n",
     [](const Call& c) { return !c.transpose && qmv_n_supported(c.a, c.gs, c.bits, c.dtype); },
     [](const Call& c) { return run_qmv_n(c.a, c.gs, c.bits, c.dtype, c.sc, c.s); },
     "w [K, N], 1..4 rows: streaming kernel over packed rows + plane reduction. 4096x14336 "
     "4-bit, one row: 15.5 against 67.7 (tile kernel); 14336x4096 8-bit: 18.7 against 59.4"},
    {"qmv_n_twice",
     [](const Call& c) {
       if (c.transpose || c.a.M < 5 || c.a.M > 8 || c.a.L != 1) {
         return false;
       }
       const QmmArgs head = row_block(c, 0, 4);
       const QmmArgs tail = row_block(c, 4, c.a.M - 4);
       return qmv_n_supported(head, c.gs, c.bits, c.dtype) &&
           qmv_n_supported(tail, c.gs, c.bits, c.dtype);
     },
     [](const Call& c) {
       // (both passes use the same planes; the sizing run keeps the larger claim)
       const QmmArgs head = row_block(c, 0, 4);
       const QmmArgs tail = row_block(c, 4, c.a.M - 4);
       const int rc = run_qmv_n(head, c.gs, c.bits, c.dtype, c.sc, c.s);
       if (rc != MLXROCM_OK) {
         return rc;
       }
       return run_qmv_n(tail, c.gs, c.bits, c.dtype, c.sc, c.s);
     },
     "w [K, N], 5..8 rows: the streaming kernel twice (4 rows, the rest). Graph replays, W "
     "[14336,4096] 4-bit: 41-52 against 65 (tile kernel, same cost whatever M); W [4096,4096]: "
     "20-25 against 25"},
    {"qmm_rows8",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       const long wgs = static_cast<long>((a.N + 63) / 64) * a.L;
       return c.transpose && a.M >= 5 && a.M <= 16 && plain(a) && a.w_alt == nullptr &&
           qmm_rows8_supported(a, c.gs, c.bits, c.dtype, c.transpose) &&
           2 * wgs >= compute_units() && 4 * wgs <= 7L * compute_units() &&
           (c.gs != 32 || wgs <= compute_units());
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmm_rows8(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "4-bit, 5..16 rows whose x fits LDS for all of K, 0.5..1.75 workgroups per CU (one round "
     "for 32-wide groups). 14336x4096: 11.7-12.2 against 15.3-15.7; 8192x2048: 6.8-7.4 against "
     "8.5-10.4; 16384x2048, 16 rows: 9.0 against 15.0. Not 4096x4096 (9.8 against 7.1), not "
     "beyond 1.75 WG/CU (57344x4096, 8 rows: 42.9 against 39.8; 128256x4096: 88 against 76), "
     "32-wide groups only one round (18432..28672x4096, 5..7 rows: 25-28 against 21)"},
    {"qmv_quad",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       if (!c.transpose || a.M > 8 || !qmv_quad_supported(a, c.gs, c.bits, c.dtype)) {
         return false;
       }
       if (a.M >= 2 && a.M <= 4) {
         return true;
       }
       if (a.M == 1) {
         return a.K > 8192 || !qmv_stream_supported(a, c.gs, c.bits, c.dtype);
       }
       return quad_pays_5_to_8(c);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_quad(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "4-bit on the 4x4x4 matrix instruction. 14336x4096: 2 rows 9.6 against 12.3, 3 rows 10.7 "
     "against 15.1, 4 rows 10.9 against 14.9; 4096x14336: 1 row 10.8 against 12.4 (K > 8192 "
     "only: at K <= 8192 the streaming GEMV is ahead, 8.1 against 9.4). 5..8 rows, 8 rows "
     "shown: 4096x4096 6.6 against 8.3, 12288x4096 13.7 against 15.4, 4096x8192 9.9 against "
     "25.4; not where the last round is half empty (14336x4096: 16.5 against 16.3) nor where "
     "the slab kernel takes the shape (4096x14336: 16.1 against 13.5, 128256x4096: 104 "
     "against 63)"},
    {"qmm_slab",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       return c.transpose && a.M >= 5 && a.M <= 32 && plain(a) && a.w_alt == nullptr &&
           qmm_slab_supported(a, c.gs, c.bits, c.dtype, c.transpose) && slab_pays(a) &&
           planes_aligned(a);
     },
     [](const Call& c) {
       const size_t plane_bytes = qmm_slab_plane_bytes(c.a);
       void* region = nullptr;
       if (plane_bytes != 0) {
         const int rc = claim(c.sc, plane_bytes, &region);
         if (rc != MLXROCM_OK) {
           return rc;
         }
       }
       return slab_launch(c, c.a, region);
     },
     "4-bit, 5..32 rows: packed rows by DMA through LDS, x resident per K range; units must "
     "fill half the CUs or the weights exceed 25 M codes (16 M at K >= 8192; 26 M for 9..16 "
     "rows). 14336x4096: 9 rows 15.5 against 19.3, 16 rows 16.9 against 19.6, 32 rows 21.5 "
     "against 23.2; 4096x14336: 32 rows 20.3 against 41.3; 24 rows 6144x4096 15.3 against "
     "21.0; not 4096x4096 (14.7 against 13.0) nor 8192x2048 (14.2 against 11.6)"},
    {"qmm_slab_twice",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       if (!c.transpose || a.M <= 32 || a.M > 64 || a.L != 1 || c.gs == 32 || !plain(a) ||
           a.w_alt != nullptr) {
         return false;
       }
       const QmmArgs head = row_block(c, 0, 32);
       const QmmArgs tail = row_block(c, 32, a.M - 32);
       return qmm_slab_supported(head, c.gs, c.bits, c.dtype, c.transpose) &&
           qmm_slab_supported(tail, c.gs, c.bits, c.dtype, c.transpose) &&
           2 * qmm_slab_units(head) >= compute_units();
     },
     [](const Call& c) {
       const QmmArgs head = row_block(c, 0, 32);
       const QmmArgs tail = row_block(c, 32, c.a.M - 32);
       // both passes use the same planes, one after the other on the stream
       const size_t plane_bytes = qmm_slab_plane_bytes(head);
       void* region = nullptr;
       if (plane_bytes != 0) {
         const int rc = claim(c.sc, plane_bytes, &region);
         if (rc != MLXROCM_OK) {
           return rc;
         }
       }
       const int rc = slab_launch(c, head, region);
       if (rc != MLXROCM_OK) {
         return rc;
       }
       return slab_launch(c, tail, region);
     },
     "4-bit, 33..64 rows: the slab kernel twice (32 rows, the rest); the tile GEMM costs the "
     "same whatever M. Graph replays, 64 rows: 14336x4096 34.4 against 37.0, 4096x14336 35.1 "
     "against 46.5, 28672x4096 49.1 against 59.6, 128256x4096 180 against 270; from 65 rows "
     "on the tile GEMM is ahead"},
    {"qmv_wide_twice",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       if (!c.transpose || a.M <= 16 || a.M > 32 || a.L != 1 || !plain(a) ||
           (a.N + 63) / 64 >= compute_units() / 2) {
         return false;
       }
       return qmv_wide_supported(row_block(c, 0, 16), c.gs, c.bits, c.dtype, c.transpose);
     },
     [](const Call& c) {
       const QmmArgs head = row_block(c, 0, 16);
       const QmmArgs tail = row_block(c, 16, c.a.M - 16);
       const int rc = MLXROCM_LAUNCH(c.sc, launch_qmv_wide(head, c.gs, c.bits, c.dtype, c.s));
       if (rc != MLXROCM_OK) {
         return rc;
       }
       return MLXROCM_LAUNCH(c.sc, launch_qmv_wide(tail, c.gs, c.bits, c.dtype, c.s));
     },
     "17..32 rows over a narrow N (fewer 64-row workgroups than half the CUs): the wide kernel "
     "twice, the second pass from the Infinity Cache. 4096x4096: 24 -> 16; 4096x14336: 56 -> 45"},
    {"qmv_f32",
     [](const Call& c) {
       return c.transpose && c.a.M == 1 && few_rows(c) &&
           qmv_f32_supported(c.a, c.gs, c.bits, c.dtype);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_f32(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "one row at a width or type the row-streaming GEMV does not cover (2/3/5/6 bits, "
     "float32): fp32-arithmetic streaming kernel. bf16 11008x4096 g32: 8.6/9.4/11.5/12.4 at "
     "2/3/5/6 bits against 14.4-17.5 (wide kernel); f32 4096x4096 4-bit 7.5 against 10.8"},
    {"qmv_wide",
     [](const Call& c) {
       const QmmArgs& a = c.a;
       if (!few_rows(c) || staged(c) || a.M > 16 ||
           !qmv_wide_supported(a, c.gs, c.bits, c.dtype, c.transpose)) {
         return false;
       }
       const bool gemv_better =
           a.M <= 8 && a.K <= 8192 && qmv_mfma_supported(a, c.gs, c.bits, c.dtype);
       return !gemv_better;
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_wide(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "up to 16 rows, every width, K split over the wavefronts of a workgroup: 3..8 rows over "
     "K > 8192 (4096x14336 4-bit: 17-18 against 39-59 for the MFMA GEMV), 9..16 rows at "
     "N < 8192, two rows at odd widths; 8-bit two rows over K > 8192: 20 against 28 (streaming)"},
    {"qmm_skinny",
     [](const Call& c) {
       return staged(c) && qmm_skinny_supported(c.a, c.gs, c.bits, c.dtype, c.transpose);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmm_skinny(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "17..32 rows (9..16 at N >= 8192): 64 rows of W per workgroup staged through LDS. "
     "14336x4096, 32 rows: 27 against 45 (tile kernel). 8-bit, 3..8 rows over >= 64 MB, 8 "
     "rows: 28672x4096 26 against 37, 8192x8192 32 against 45. Not a narrow N over K > 8192 "
     "(4096x14336, 32 rows: 78 against 57 for the tile kernel with split K)"},
    {"qmv_wide_staged",
     [](const Call& c) {
       return staged(c) && c.a.M <= 16 &&
           qmv_wide_supported(c.a, c.gs, c.bits, c.dtype, c.transpose);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_wide(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "the shapes of the rule above that the staged kernel does not support (K not a multiple "
     "of its step): the wide kernel"},
    {"fp32_rows_twice",
     [](const Call& c) {
       return c.transpose && c.dtype == MLXROCM_FLOAT32 && c.a.M > kQmvMaxM &&
           c.a.M <= 2 * kQmvMaxM && c.a.L == 1 && plain(c.a);
     },
     [](const Call& c) {
       return two_passes(c, row_block(c, 0, kQmvMaxM), row_block(c, kQmvMaxM, c.a.M - kQmvMaxM));
     },
     "float32, 9..16 rows: this table twice (8 rows, the rest); the split-bf16 matrix path "
     "costs the same whatever M. Graph replays, 14336x4096 4-bit: 89 at 9 rows, 132 at 16, "
     "against 155; 4096x14336: 76 / 117 against 171"},
    {"qmm_t_tile_sb_transposed",
     [](const Call& c) {
       return tile_t(c) && c.a.lhs_indices == nullptr && c.a.M >= kTransposeSbMinM;
     },
     [](const Call& c) {
       return run_qmm_t_transposed_sb(c.a, c.gs, c.bits, c.dtype, tile_k_splits(c), c.sc, c.s);
     },
     "prefill from 512 rows: scales and biases transposed to [K/group][N] first (5.2 us at "
     "14336x4096), after which a wavefront's 32 rows read 64 contiguous bytes; with the "
     "caller's layout those loads were 15 % of the tile kernel's time. M=2048, 14336x4096: "
     "199.5 per call, 1206 TFLOP/s"},
    {"qmm_t_tile_k_split",
     [](const Call& c) { return tile_t(c) && tile_k_splits(c) > 1; },
     [](const Call& c) {
       return run_k_split(c.a, c.gs, c.bits, c.dtype, tile_k_splits(c), c.sc, c.s);
     },
     "few tiles: K cut into up to 16 ranges of at least 8 steps, fp32 planes + reduction. "
     "M=512, N=4096: 75 -> 43; K=14336: 249 -> 92; 3584x18944, 128 rows: 45.6 (16 ranges) "
     "against 57.5 (8)"},
    {"qmm_t_tile",
     [](const Call& c) { return tile_t(c); },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmm_mfma(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "256 x (128..224) tiles on v_mfma_f32_16x16x32, every width, 16-bit types, K % 64 == 0"},
    {"qmm_t_split_fp32",
     [](const Call& c) {
       return family_of(c) == Family::QmmT && c.dtype == MLXROCM_FLOAT32 &&
           c.a.lhs_indices == nullptr;
     },
     [](const Call& c) { return run_split_fp32(c.a, c.gs, c.bits, c.sc, c.s); },
     "float32 prefill as three bf16 products per product (x and W split in high and low "
     "parts): x [1024,4096] x W [11008,4096]: 0.39 ms against 280 ms (scalar kernel)"},
    {"qmv_stream",
     [](const Call& c) {
       return family_of(c) == Family::Qmv && qmv_stream_supported(c.a, c.gs, c.bits, c.dtype);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_stream(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "decode GEMV, 1..2 rows, 4/8-bit, 16-bit types: whole-line loads of one row per wavefront "
     "instruction. 14336x4096 4-bit g64, one row: 8.1 (4.1 TB/s)"},
    {"qmv_mfma",
     [](const Call& c) {
       return family_of(c) == Family::Qmv && qmv_mfma_supported(c.a, c.gs, c.bits, c.dtype);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_mfma(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "3..8 rows, 4/8-bit, K <= 8192 on v_mfma_f32_16x16x32 (lanes = rows of W): 15-16 at "
     "14336x4096 4-bit"},
    {"qmv_f32_rows",
     [](const Call& c) {
       return family_of(c) == Family::Qmv && qmv_f32_supported(c.a, c.gs, c.bits, c.dtype);
     },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_f32(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "float32 (and odd widths), 2..4 rows at K <= 8192 with a slice of every x row in "
     "registers: 11008x4096 4-bit, 2 rows 17.3 against 28.0 (generic)"},
    {"qmv_generic",
     [](const Call& c) { return family_of(c) == Family::Qmv; },
     [](const Call& c) {
       return MLXROCM_LAUNCH(c.sc, launch_qmv_generic(c.a, c.gs, c.bits, c.dtype, c.s));
     },
     "functional floor of the GEMV regime: any width, group, type, K"},
    {"qmm_n_tile",
     [](const Call& c) {
       return family_of(c) == Family::QmmN && c.a.lhs_indices == nullptr &&
           qmm_mfma_supported(c.a, c.gs, c.bits, c.dtype, c.transpose);
     },
     [](const Call& c) { return run_qmm_n(c.a, c.gs, c.bits, c.dtype, c.sc, c.s); },
     "w [K, N] on the tile GEMM's column loader (4/8-bit, 16-bit types, K % 64 == 0), scales "
     "and biases transposed to [group][k] first: x [2048,4096] x W [4096,14336] 0.35 ms "
     "against 12.7 ms (scalar kernel)"},
    {"qmm_naive",
     [](const Call&) { return true; },
     [](const Call& c) {
       return MLXROCM_LAUNCH(
           c.sc, launch_qmm_naive(c.a, c.gs, c.bits, c.dtype, c.transpose, c.s));
     },
     "functional floor: one thread per output (or per 8 outputs of a [K, N] weight), any shape"},
};

int run(const QmmArgs& a, int gs, int bits, int dtype, bool transpose, Scratch& sc, hipStream_t s) {
  const Call c{a, gs, bits, dtype, transpose, sc, s};
  for (const Rule& rule : kRules) {
    if (rule.applies(c)) {
      if (rehearsing() && !sc.dry) {
        note_launch("[%s]", rule.name);
      }
      return rule.launch(c);
    }
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
    rc = check_alignment("quantized_matmul", a, dtype, transpose != 0, bits);
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
  if (dtype != MLXROCM_FLOAT32) {
    // what the 16-bit prefill path reads: (scale, bias) pairs, [K / group][N]
    return interleave_sb_for_qmm_t(
        scales, biases, image, N, K / group_size, batches, sb_batch_stride,
        static_cast<hipStream_t>(stream));
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
std::atomic<void*> g_static_scratch[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (first call on a device
// resolves it; later calls only read the table).
int static_scratch(void** out) {
  int dev = 0;
  MLXROCM_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) {
    return fail(MLXROCM_UNSUPPORTED, "[quantized_matmul_static] device %d out of range", dev);
  }
  // the table is written once per device: later calls take no lock
  void* ptr = g_static_scratch[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    std::lock_guard<std::mutex> lock(g_static_mu);
    ptr = g_static_scratch[dev].load(std::memory_order_relaxed);
    if (ptr == nullptr) {
      MLXROCM_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
      if (ptr == nullptr) {
        return fail(MLXROCM_HIP_ERROR, "[quantized_matmul_static] no address for the scratch array");
      }
      g_static_scratch[dev].store(ptr, std::memory_order_release);
    }
  }
  *out = ptr;
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
  // the grouped kernels reach x through 32-bit byte offsets (16-bit elements)
  if ((static_cast<int64_t>(x_batches) * x_batch_stride + K) * 2 >= (int64_t(1) << 32)) {
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
  // the grouped kernels reach x through 32-bit byte offsets (16-bit elements)
  if ((static_cast<int64_t>(x_batches) * x_batch_stride + K) * 2 >= (int64_t(1) << 32)) {
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

namespace {
int gather_entry(
    const void* x, const uint32_t* wq, const void* scales, const void* biases,
    const uint32_t* lhs_indices, const uint32_t* rhs_indices, void* out, int M, int N, int K,
    int n_indices, int x_batches, int n_experts, int64_t x_batch_stride, int64_t w_expert_stride,
    int64_t sb_expert_stride, int group_size, int bits, int dtype, int transpose, void* workspace,
    size_t workspace_bytes, hipStream_t s);
} // namespace

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
  return gather_entry(
      x, wq, scales, biases, lhs_indices, rhs_indices, out, M, N, K, n_indices, x_batches,
      n_experts, x_batch_stride, w_expert_stride, sb_expert_stride, group_size, bits, dtype,
      transpose, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

namespace {

int gather_entry(
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
    void* workspace,
    size_t workspace_bytes,
    hipStream_t s) {
  int rc = check_shape(
      "gather_qmm", M, N, K, n_indices, group_size, bits, dtype, transpose);
  if (rc != MLXROCM_OK) {
    return rc;
  }
  if (static_cast<int64_t>(M) * N * n_indices == 0) {
    return MLXROCM_OK;
  }
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
  rc = check_alignment("gather_qmm", a, dtype, transpose != 0, bits);
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

} // namespace

namespace {

// Stand-ins for device pointers in a rehearsal: aligned, never dereferenced
// (the host path computes addresses from them and every launch is skipped).
void* fake_device_pointer(int which) {
  return reinterpret_cast<void*>(uintptr_t{1} << 40 | static_cast<uintptr_t>(which) << 32);
}

} // namespace

extern "C" int mlxrocm_qmm_plan(
    int M,
    int N,
    int K,
    int L,
    int batched_weights,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes) {
  RehearsalScope rehearsal(plan, plan_bytes);
  Scratch sc;
  sc.base = workspace_bytes != 0 ? static_cast<char*>(fake_device_pointer(5)) : nullptr;
  sc.bytes = workspace_bytes;
  const int64_t w_stride = batched_weights ? int64_t{1} << 28 : 0;
  return qmm_entry(
      fake_device_pointer(0), static_cast<const uint32_t*>(fake_device_pointer(1)),
      fake_device_pointer(2), fake_device_pointer(3), fake_device_pointer(4), M, N, K, L,
      static_cast<int64_t>(M) * K, w_stride, w_stride, group_size, bits, dtype, transpose, sc,
      nullptr);
}

extern "C" int mlxrocm_gather_qmm_plan(
    int M,
    int N,
    int K,
    int n_indices,
    int x_batches,
    int n_experts,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes) {
  RehearsalScope rehearsal(plan, plan_bytes);
  // a dense stack of experts, x rows one after the other
  const int64_t w_stride = transpose
      ? static_cast<int64_t>(N) * (static_cast<int64_t>(K) * bits / 32)
      : static_cast<int64_t>(K) * (static_cast<int64_t>(N) * bits / 32);
  const int64_t sb_stride = transpose ? static_cast<int64_t>(N) * (K / group_size)
                                      : static_cast<int64_t>(K) * (N / group_size);
  return gather_entry(
      fake_device_pointer(0), static_cast<const uint32_t*>(fake_device_pointer(1)),
      fake_device_pointer(2), fake_device_pointer(3),
      static_cast<const uint32_t*>(fake_device_pointer(6)),
      static_cast<const uint32_t*>(fake_device_pointer(7)), fake_device_pointer(4), M, N, K,
      n_indices, x_batches, n_experts, static_cast<int64_t>(M) * K, w_stride, sb_stride,
      group_size, bits, dtype, transpose,
      workspace_bytes != 0 ? fake_device_pointer(5) : nullptr, workspace_bytes, nullptr);
}

extern "C" int mlxrocm_qmm_rule_count(void) {
  return static_cast<int>(sizeof(kRules) / sizeof(kRules[0]));
}

extern "C" const char* mlxrocm_qmm_rule_name(int i) {
  return i >= 0 && i < mlxrocm_qmm_rule_count() ? kRules[i].name : nullptr;
}

extern "C" const char* mlxrocm_qmm_rule_evidence(int i) {
  return i >= 0 && i < mlxrocm_qmm_rule_count() ? kRules[i].evidence : nullptr;
}
