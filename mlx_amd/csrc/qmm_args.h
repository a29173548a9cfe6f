// qmm_args.h -- problem descriptor shared by the quantized-matmul kernels.
#pragma once

#include "common.h"

namespace mlxrocm {

// One launch covers L problems.  Without index arrays problem l reads x batch l
// and weight batch l (stride 0 = one shared weight); with them it reads
// x[lhs[l]] and w[rhs[l]] (GatherQMM).
struct QmmArgs {
  const void* x;
  const uint32_t* w;
  const void* scales;
  const void* biases;
  void* out;
  int M;
  int N;
  int K;
  int L;
  int64_t x_batch_stride;  // elements
  int64_t w_batch_stride;  // uint32 words
  int64_t sb_batch_stride; // elements
  const uint32_t* lhs_indices;
  const uint32_t* rhs_indices;
  int x_batches; // bounds for gathered indices
  int n_experts;
  // Grouped gather (M == 1): the index pairs sorted by expert and cut into tiles
  // of up to group_tile_rows rows.  group_tiles holds {expert, first sorted position, rows}
  // per tile, group_perm maps a sorted position to its index pair, group_ntiles
  // points at the number of tiles followed by the number of sorted positions
  // (both known on the device only).  All null otherwise.
  const int32_t* group_tiles;
  const int32_t* group_perm;
  const int32_t* group_ntiles;
  int group_tile_rows;
  // Prefill tile kernel only: scales / biases point at a transposed image
  // [K / group][N], so that the lanes of a wavefront, which own consecutive rows
  // of W, read consecutive values.  0: the caller's [N][K / group] arrays.
  // 1: two images, scales and biases (transpose_sb_for_qmm_n with the roles of K
  // and N swapped; float32 operands).  2: one image of (scale, bias) pairs, a.scales
  // pointing at it (interleave_sb_for_qmm_t; 16-bit types): one load per thread
  // and K-step fetches both.
  int sb_transposed;
  // Two weight matrices sharing one x (the gate and up projections of a gated
  // MLP): with L == 2 and these set, problem 1 reads them instead of w / scales /
  // biases advanced by a batch stride.  Null otherwise.  Honoured by the kernels
  // that resolve their operands with resolve_problem (every decode kernel).
  const uint32_t* w_alt;
  const void* scales_alt;
  const void* biases_alt;
  // nvfp4 weights quantized with a tensor-wide scale (one float on the device):
  // the fp32 sums are multiplied by *out_scale / (448 * 6) before they are
  // rounded (mlx/backend/cuda/quantized/qmm/qmv.cu:163-165).  Null otherwise;
  // read only by the kernels of the floating-point modes with groups of 16.
  const float* out_scale;
};

// Resolved operand pointers of problem l.  `valid` is false when a gathered
// index is out of range; the problem's output is then zero-filled.
template <typename T>
struct QmmProblem {
  const T* x;
  const uint8_t* w;
  const T* scales;
  const T* biases;
  T* out;
  bool valid;
};

template <typename T>
__device__ __forceinline__ QmmProblem<T> resolve_problem(
    const QmmArgs& a,
    int l) {
  QmmProblem<T> p;
  int64_t xb = l;
  int64_t wb = l;
  p.valid = true;
  if (a.lhs_indices != nullptr) {
    const uint32_t xi = a.lhs_indices[l];
    const uint32_t wi = a.rhs_indices[l];
    p.valid = xi < static_cast<uint32_t>(a.x_batches) &&
        wi < static_cast<uint32_t>(a.n_experts);
    xb = p.valid ? xi : 0;
    wb = p.valid ? wi : 0;
  }
  p.x = static_cast<const T*>(a.x) + xb * a.x_batch_stride;
  p.w = reinterpret_cast<const uint8_t*>(a.w + wb * a.w_batch_stride);
  p.scales = static_cast<const T*>(a.scales) + wb * a.sb_batch_stride;
  p.biases = static_cast<const T*>(a.biases) + wb * a.sb_batch_stride;
  if (a.w_alt != nullptr && l == 1) {
    p.w = reinterpret_cast<const uint8_t*>(a.w_alt);
    p.scales = static_cast<const T*>(a.scales_alt);
    p.biases = static_cast<const T*>(a.biases_alt);
  }
  p.out = static_cast<T*>(a.out) +
      static_cast<int64_t>(l) * a.M * static_cast<int64_t>(a.N);
  return p;
}

// Launchers implemented per kernel family; each returns an mlxrocm_status.
int launch_qmv_generic(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
int launch_qmm_naive(
    const QmmArgs& a,
    int gs,
    int bits,
    int dtype,
    bool transpose,
    hipStream_t s);

bool qmv_stream_supported(const QmmArgs& a, int gs, int bits, int dtype);
int launch_qmv_stream(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
bool qmv_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype);
int launch_qmv_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
bool qmm_mfma_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose);
int launch_qmm_mfma(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
// The same reading the (scale, bias) pair image (a.sb_transposed == 2, a.scales
// pointing at it; interleave_sb_for_qmm_t), whole K and split K.
int launch_qmm_mfma_pairs(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
int launch_qmm_mfma_ksplit_pairs(
    const QmmArgs& a, int gs, int bits, int dtype, int k_splits, hipStream_t s);

// The tile kernel for the floating-point modes (qmm_mfma_fp.hip): `mode` is a
// mlxrocm_fp_mode, a.scales the scale image that fp_scale_image_for_qmm_t builds
// from the caller's byte scales (batches * (K / 32) * N dwords), K % 64 == 0,
// 16-bit dtype.
int fp_scale_image_for_qmm_t(
    const uint8_t* scales,
    void* out,
    int N,
    int K,
    int batches,
    int64_t src_stride,
    int mode,
    int dtype,
    hipStream_t s);
int launch_qmm_mfma_fp(const QmmArgs& a, int mode, int dtype, int k_splits, hipStream_t s);
// The same kernel on a gather grouped by expert (launch_gather_group's tables in
// `a`, one scale image per expert).
int launch_qmm_mfma_fp_grouped(const QmmArgs& a, int mode, int dtype, hipStream_t s);

// qqmm in the MX modes on the block-scaled matrix instruction (qq_mfma.hip):
// x as codes and scale bytes (fp_quantize_activations, fp_quantize.hip) times
// the quantized w, both [rows][K]; K % 128 == 0.
bool qq_mfma_supported(int M, int N, int K, int mode);
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
    hipStream_t s);
int fp_quantize_activations(
    const void* x, void* codes, uint8_t* scales, size_t n_elems, int mode, int dtype, hipStream_t s);

bool qmv_wide_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose);
int launch_qmv_wide(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
bool qmm_skinny_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose);
int launch_qmm_skinny(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
int launch_zero_fill(void* p, size_t bytes, hipStream_t s);

// Grouping of gathered index pairs by expert (gather_group.hip) and the grouped
// launch of the matrix-core GEMM over its tiles (qmm_mfma.hip).
constexpr int kGroupLargeTile = 256; // rows per tile of the tile GEMM
constexpr int kGroupSmallTile = 32;  // rows per tile of the few-row kernel
size_t gather_group_workspace_bytes(int n_indices, int n_experts);
int gather_group_max_tiles(int n_indices, int n_experts, int tile_rows);
int launch_gather_group(QmmArgs& a, int dtype, int tile_rows, void* workspace, hipStream_t s);
// Only points the grouped-mode fields of `a` into the workspace (no launch).
void bind_gather_group(QmmArgs& a, int tile_rows, void* workspace);
int launch_qmm_skinny_grouped(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
// Up to 32 rows of x per weight matrix, 4-bit codes, 16-bit types, K % 1024 == 0:
// packed rows streamed through LDS, x resident per K range.  With more than one
// K range the partial sums go through fp32 planes (`planes`, *_plane_bytes()).
bool qmm_slab_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose);
bool qmm_slab_shape_ok(int rows, int N, int K, int gs, int bits);
// Up to 16 rows of x with M * K * 2 bytes <= 64 KiB of LDS: all of K resident, no planes.
// widen_codes.hip: 2/3-bit codes repacked as 4-bit, 5/6-bit as 8-bit (values kept)
int widened_bits(int bits);
int launch_widen_codes(
    const uint32_t* src, uint32_t* dst, size_t dst_words, size_t codes, int bits, hipStream_t s);
bool qmm_rows8_supported(const QmmArgs& a, int gs, int bits, int dtype, bool transpose);
int launch_qmm_rows8(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
long qmm_slab_units(const QmmArgs& a); // work items of a plain call
size_t qmm_slab_plane_bytes(const QmmArgs& a);
int launch_qmm_slab(const QmmArgs& a, int gs, int bits, int dtype, void* planes, hipStream_t s);
size_t qmm_slab_grouped_plane_bytes(int n_indices, int N, int K);
// plan_in_kernel: the kernel groups the pairs itself (`a` carries the index
// arrays and, from bind_gather_group, where the sorted order goes for the plane
// reduction); otherwise launch_gather_group must have run.
bool qmm_slab_plans_in_kernel(int n_indices, int n_experts);
int launch_qmm_slab_grouped(
    const QmmArgs& a, int gs, int bits, int dtype, void* planes, bool plan_in_kernel,
    hipStream_t s);
// fp32 operands on the bf16 matrix path: x is first split into bf16 high and
// low parts (split_x_for_mfma into a buffer of split_x_bytes), then
// launch_qmm_mfma_split runs with a.x pointing at that buffer.
size_t split_x_bytes(size_t rows, int K);
int split_x_for_mfma(const void* x, void* xs, size_t rows, int K, hipStream_t s);
int launch_qmm_mfma_split(const QmmArgs& a, int gs, int bits, hipStream_t s, int k_splits);
// Few tiles: K is cut into qmm_mfma_k_splits() ranges whose fp32 partial tiles
// (k_splits planes of M x N behind a.out) reduce_k_splits() adds up.
int qmm_mfma_k_splits(int M, int N, int K, int L);
// transpose=false (w [K, N*bits/32]), 4/8-bit, 16-bit types, K % 64 == 0; with
// k_splits > 1 `a.out` points at k_splits fp32 planes as for the k-split launch.
// `a.scales` / `a.biases` must point at [group][k] images (transpose_sb_for_qmm_n).
int launch_qmm_mfma_n(const QmmArgs& a, int gs, int bits, int dtype, int k_splits, hipStream_t s);
size_t qmm_n_sb_bytes(int K, int G, int batches, int dtype);
// scales / biases [N][G] (16-bit types) -> per batch entry [G][N] pairs
// (scale in the low half of a dword, bias in the high half); same size as the
// two separate images.
int interleave_sb_for_qmm_t(
    const void* scales,
    const void* biases,
    void* out,
    int N,
    int G,
    int batches,
    int64_t src_stride,
    hipStream_t s);
int transpose_sb_for_qmm_n(
    const void* scales,
    const void* biases,
    void* out,
    int K,
    int G,
    int batches,
    int64_t src_stride,
    int dtype,
    hipStream_t s);
// transpose=false with 1..4 rows of x, 4/8-bit, every element type: a streaming
// kernel over the packed rows of W.  K is cut into `splits` ranges of `range`
// rows; with more than one range `partial` receives `splits` fp32 planes of
// [L, M, N] for reduce_planes.
struct QmvNPlan {
  int range;
  int splits;
};
bool qmv_n_supported(const QmmArgs& a, int gs, int bits, int dtype);
QmvNPlan qmv_n_plan(const QmmArgs& a, int bits);
int launch_qmv_n(const QmmArgs& a, int gs, int bits, int dtype, float* partial, hipStream_t s);
// y (n elements, n % 4 == 0) = sum of `splits` fp32 planes; built for many planes.
int reduce_planes(const float* partial, void* out, size_t n, int splits, int dtype, hipStream_t s);
// gated decode GEMV: y = silu(w . x) * (w_alt . x) in one launch (one row of x)
bool qmv_stream_glu_supported(const QmmArgs& a, int gs, int bits, int dtype);
int launch_qmv_stream_glu(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
// decode GEMV in fp32 arithmetic (transpose=true): every width and element type,
// one row of x at K <= 16384, two to four rows at K <= 8192.
bool qmv_f32_supported(const QmmArgs& a, int gs, int bits, int dtype);
int launch_qmv_f32(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
// 1..8 rows of x on the 4x4x4 matrix instruction: transpose=true, 16-bit types,
// 4-bit, K a multiple of 512 codes and at most 16384, an even number of groups.
bool qmv_quad_supported(const QmmArgs& a, int gs, int bits, int dtype);
int launch_qmv_quad(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
long qmv_quad_workgroups_two_sets(const QmmArgs& a, int bits);
int launch_qmm_mfma_ksplit(const QmmArgs& a, int gs, int bits, int dtype, int k_splits, hipStream_t s);
int reduce_k_splits(const void* partial, void* out, size_t n, int k_splits, int dtype, hipStream_t s);
int launch_qmm_mfma_grouped(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);
// transpose=false form: scales / biases are the [group][k] images of all experts
int launch_qmm_mfma_grouped_n(const QmmArgs& a, int gs, int bits, int dtype, hipStream_t s);

// Compute units of the current device (read once).
inline int compute_units() {
  static int cus = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      return 256;
    }
    return prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }();
  return cus;
}

} // namespace mlxrocm
