/*
 * mlx_rocm_qmm.h -- C ABI of the MI355X (gfx950) implementation of MLX's affine
 * group-wise quantized matmul path.
 *
 * This is the thin layer the C++ `eval_gpu` bodies of a `mlx/backend/rocm` tree
 * call: plain pointers and sizes, a HIP stream handle, an int status.  Nothing
 * here allocates or frees device memory except the mlxrocm_malloc family:
 * entry points that need device scratch take it from a workspace the caller
 * provides (its size comes from the matching *_workspace_size function).
 *
 * Conventions
 *   - All data pointers are DEVICE pointers (or host-visible pinned memory).
 *   - `dtype` is the element type shared by x, scales, biases and out
 *     (MLX promotes them to one type before the primitive, mlx/ops.cpp:4816-4818).
 *   - Packed weights are uint32 words; code e of a row occupies bits
 *     [e*bits, (e+1)*bits) of the row's little-endian bit stream.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Every
 *     compute entry point only enqueues work and returns.
 *   - Return value: MLXROCM_OK, or a negative mlxrocm_status; the message of the
 *     last failure on the calling thread is returned by mlxrocm_last_error().
 *     No exception crosses this boundary.
 */
#ifndef MLX_ROCM_QMM_H
#define MLX_ROCM_QMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLXROCM_ABI_VERSION 4

typedef enum {
  MLXROCM_OK = 0,
  MLXROCM_INVALID_ARGUMENT = -1, /* std::invalid_argument on the C++ side */
  MLXROCM_UNSUPPORTED = -2,      /* "no ROCm implementation" runtime_error */
  MLXROCM_HIP_ERROR = -3,        /* a HIP runtime call failed */
  MLXROCM_OUT_OF_MEMORY = -4
} mlxrocm_status;

typedef enum {
  MLXROCM_FLOAT32 = 0,
  MLXROCM_FLOAT16 = 1,
  MLXROCM_BFLOAT16 = 2,
  /* The quantization entry points take the three types above; the element
   * copies also take the rest of mlx::core::Dtype (mlx/dtype.h:15-30). */
  MLXROCM_BOOL = 3,
  MLXROCM_UINT8 = 4,
  MLXROCM_UINT16 = 5,
  MLXROCM_UINT32 = 6,
  MLXROCM_UINT64 = 7,
  MLXROCM_INT8 = 8,
  MLXROCM_INT16 = 9,
  MLXROCM_INT32 = 10,
  MLXROCM_INT64 = 11,
  MLXROCM_FLOAT64 = 12,
  MLXROCM_COMPLEX64 = 13
} mlxrocm_dtype;

typedef void* mlxrocm_stream_t; /* hipStream_t */
typedef void* mlxrocm_event_t;  /* hipEvent_t  */

int mlxrocm_abi_version(void);
const char* mlxrocm_last_error(void);

/* ------------------------------------------------------------------------ */
/* Quantize / dequantize                                                     */
/* ------------------------------------------------------------------------ */

/*
 * Replaces fast::Quantize::eval_gpu with dequantize_ == false
 * (mlx/fast_primitives.h:355-356; CPU body mlx/backend/cpu/quantized.cpp:1229-1280,
 * algorithm quantize<T,U> :1148-1211).  w holds n_elems = rows*K elements,
 * row-contiguous, K % group_size == 0.  Outputs: wq n_elems*bits/32 words,
 * scales and biases n_elems/group_size elements of `dtype`.  Results are
 * bit-identical to the CPU backend's.
 */
int mlxrocm_affine_quantize(
    const void* w,
    uint32_t* wq,
    void* scales,
    void* biases,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype,
    mlxrocm_stream_t stream);

/*
 * Replaces fast::Quantize::eval_gpu with dequantize_ == true
 * (created by affine_dequantize for Device::gpu, mlx/ops.cpp:5327-5338).
 * out[e] = T(T(code_e) * scale) + bias, two roundings as in the op graph the
 * CPU runs (mlx/ops.cpp:5320-5324).  out holds n_elems elements.
 */
int mlxrocm_affine_dequantize(
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype,
    mlxrocm_stream_t stream);

/*
 * The floating-point quantization modes (mlx/primitives.h QuantizationMode,
 * mlx/ops.cpp:4675-4707 for the group size and bits each mode fixes):
 *   mxfp4: e2m1 codes, groups of 32, one e8m0 scale byte per group
 *   mxfp8: e4m3 codes, groups of 32, one e8m0 scale byte per group
 *   nvfp4: e2m1 codes, groups of 16, one e4m3 scale byte per group
 * No biases.  Codes are packed little-end first into uint32 words exactly as
 * the affine codes are (eight 4-bit or four 8-bit codes per word).
 */
typedef enum {
  MLXROCM_MXFP4 = 0,
  MLXROCM_MXFP8 = 1,
  MLXROCM_NVFP4 = 2
} mlxrocm_fp_mode;

/*
 * Replaces fp_quantize (mlx/ops.cpp:5101-5205, the CPU op graph it builds when
 * the stream is not on a GPU) and the GPU primitive behind it
 * (mlx/backend/cuda/quantized/fp_quantize.cu).  w: n_elems elements of dtype,
 * n_elems a multiple of the mode's group size; wq: n_elems * bits / 32 words;
 * scales: n_elems / group_size bytes.  Scale of a group: mxfp*: e8m0 of
 * round(log2(amax / max_code_value)) evaluated in double; nvfp4: e4m3 of
 * amax / 6.  Elements are divided by the decoded scale in dtype and rounded to
 * the nearest code (e2m1: first nearest of the value table, as argmin does;
 * e4m3: round to nearest even with saturation at 448).
 */
int mlxrocm_fp_quantize(
    const void* w,
    uint32_t* wq,
    uint8_t* scales,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream);

/* Replaces fp_dequantize (mlx/ops.cpp:5342-5440; CPU kernel
 * mlx/backend/cpu/quantized.cpp:49-62 dequantize_scale, :1322-1356):
 * out[i] = dtype(value(code i) * scale(group of i)). */
int mlxrocm_fp_dequantize(
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream);

/* Quantize and dequantize in one pass without materialising the codes: what
 * qqmm applies to its activation operand (mlx/ops.cpp:4926-4990; CPU:
 * fp_quantize_dequantize, mlx/backend/cpu/quantized.cpp:1049-1128, called from
 * QQMatmul::eval_cpu :1322-1356).  It follows that function's fp32 rules -- the
 * scale from float log2 rounded half away from zero, e2m1 codes by its
 * threshold table (ties to the even code) -- which are not the rules of
 * mlxrocm_fp_quantize on ties, as in the reference. */
int mlxrocm_fp_quantize_dequantize(
    const void* x,
    void* out,
    size_t n_elems,
    int mode,
    int dtype,
    mlxrocm_stream_t stream);

/*
 * quantized_matmul for the floating-point modes (mlx/ops.cpp:4784-4834 with
 * mode != "affine"; CPU kernels mlx/backend/cpu/quantized.cpp:449-698
 * fp_qmm / fp_qmm_t and their dispatch).  Shapes as mlxrocm_qmm: x [L, M, K],
 * transpose: w [L, N, K bits / 32], scales [L, N, K / group_size] bytes;
 * otherwise w [L, K, N bits / 32], scales [L, K, N / group_size]; out
 * [L, M, N].  Batch strides in elements (x), words (w) and bytes (scales); a
 * stride of 0 broadcasts.  Products and sums are evaluated in fp32 and rounded
 * once to dtype.  workspace: mlxrocm_fp_qmm_workspace_size bytes of device
 * scratch, 16-byte aligned, used only during the call (prefill shapes decode
 * the scales into an image first; 0 bytes for decode shapes, float32 and
 * transpose == 0, and then it may be NULL).
 */
size_t mlxrocm_fp_qmm_workspace_size(
    int M,
    int N,
    int K,
    int L,
    int batched_weights, /* scales_batch_stride != 0 */
    int mode,
    int dtype,
    int transpose);
int mlxrocm_fp_qmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    int M,
    int N,
    int K,
    int L,
    int64_t x_batch_stride,
    int64_t w_batch_stride,
    int64_t scales_batch_stride,
    int mode,
    int dtype,
    int transpose,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

/*
 * qqmm with a quantized second operand (mlx/ops.cpp:4926-4990; CPU:
 * QQMatmul::eval_cpu, mlx/backend/cpu/quantized.cpp:1322-1360, which takes one
 * row of x): y = quantize_dequantize(x) . dequantize(w)^T.  x [M, K] and out
 * [M, N] in dtype, w [N, K bits / 32], scales [N, K / group_size] bytes.  In the
 * MX modes (mxfp4; mxfp8 for the 16-bit dtypes) with K a multiple of 128 and 16
 * rows of x or more, x is quantized to codes by the rules of
 * mlxrocm_fp_quantize_dequantize and both operands' codes are multiplied on the
 * block-scaled matrix instruction (v_mfma_scale_f32_16x16x128_f8f6f4) -- the
 * same real products, summed exactly for e2m1 codes and with about 17 bits
 * below the largest product of a 128-code step for e4m3 codes; otherwise x is
 * quantized and dequantized in dtype and takes the kernels of mlxrocm_fp_qmm.  workspace: mlxrocm_fp_qqmm_workspace_size bytes,
 * 256-byte aligned, used only during the call.
 */
size_t mlxrocm_fp_qqmm_workspace_size(int M, int N, int K, int mode, int dtype);
int mlxrocm_fp_qqmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    void* out,
    int M,
    int N,
    int K,
    int mode,
    int dtype,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

/* mlxrocm_qmm_plan for the two entry points above: what a call with these
 * shape arguments and this much workspace would launch, written into `plan`
 * as "a+b+c" without touching a device, or the error it would return. */
int mlxrocm_fp_qmm_plan(
    int M,
    int N,
    int K,
    int L,
    int batched_weights,
    int mode,
    int dtype,
    int transpose,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes);
int mlxrocm_fp_qqmm_plan(
    int M,
    int N,
    int K,
    int mode,
    int dtype,
    size_t workspace_bytes,
    char* plan,
    size_t plan_bytes);

/* gather_qmm for the floating-point modes (mlx/ops.cpp:5553-5629 with
 * mode != "affine"; CPU: mlx/backend/cpu/quantized.cpp:806-900 fp_bs_qmm_dispatch_mode).
 * Arguments as mlxrocm_gather_qmm without biases; pair i multiplies
 * x[lhs_indices[i]] by w[rhs_indices[i]]; a pair with an index out of range
 * writes zeros.  workspace (optional, 256-byte aligned,
 * mlxrocm_fp_gather_qmm_workspace_size bytes; batched_scales = scales_expert_stride
 * != 0): with it, a call with one row of x per pair, a 16-bit dtype, transpose = 1
 * and at least 32 pairs and four per expert sorts the pairs by expert and
 * multiplies every expert's weights once for all its rows on the matrix cores;
 * without it, or for other shapes, one streaming product per pair. */
size_t mlxrocm_fp_gather_qmm_workspace_size(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int batched_scales,
    int mode,
    int dtype,
    int transpose);
int mlxrocm_fp_gather_qmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
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
    int64_t scales_expert_stride,
    int mode,
    int dtype,
    int transpose,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

/*
 * mx.to_fp8 / mx.from_fp8 (mlx/ops.cpp:5519-5552; fast::ConvertFP8,
 * mlx/backend/cpu/quantized.cpp:1282-1320 with detail::ToFP8 / FromFP8,
 * mlx/backend/cpu/unary_ops.h:120-174): elementwise float <-> e4m3 bytes, round
 * to nearest even, saturating at 448 (0x7E) with the sign carried over; the
 * decoder has no NaN or infinity codes (0x7F is 480).  x / out in dtype, 16-byte
 * aligned; the byte array 8-byte aligned; any n_elems.
 */
int mlxrocm_to_fp8(
    const void* x, uint8_t* out, size_t n_elems, int dtype, mlxrocm_stream_t stream);
int mlxrocm_from_fp8(
    const uint8_t* x, void* out, size_t n_elems, int dtype, mlxrocm_stream_t stream);

/*
 * gather_qqmm (mlx/ops.cpp:5631-5681; GPU only in the reference:
 * GatherQQMM::eval_gpu, mlx/backend/cuda/quantized/qqmm.cpp:210-281 -- the CPU
 * backend throws "NYI", mlx/backend/cpu/quantized.cpp:1362-1364): every matrix
 * of x is quantized and dequantized in its own type, then pair i multiplies
 * x_hat[lhs_indices[i]] by the transposed w[rhs_indices[i]].  Arguments as
 * mlxrocm_fp_gather_qmm with transpose = 1; x_batch_stride >= M * K.
 * global_scale_x / global_scale_w: both null, or (nvfp4) both one float32 on
 * the device, as in mlxrocm_nvfp4_qqmm_global.  workspace:
 * mlxrocm_fp_gather_qqmm_workspace_size bytes (x_hat, then what
 * mlxrocm_fp_gather_qmm asks for), 256-byte aligned, used only during the call.
 */
size_t mlxrocm_fp_gather_qqmm_workspace_size(
    int M,
    int N,
    int K,
    int n_indices,
    int x_batches,
    int n_experts,
    int batched_scales,
    int mode,
    int dtype);
int mlxrocm_fp_gather_qqmm(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    const float* global_scale_x,
    const float* global_scale_w,
    void* out,
    int M,
    int N,
    int K,
    int n_indices,
    int x_batches,
    int n_experts,
    int64_t x_batch_stride,
    int64_t w_expert_stride,
    int64_t scales_expert_stride,
    int mode,
    int dtype,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

/*
 * nvfp4 with a tensor-wide scale (`global_scale` of mx.quantize / mx.dequantize
 * / mx.qqmm, mlx/ops.cpp:4756-4782, 5101-5131, 5342-5398; one float32 on the
 * device, usually max |w|).  The reference implements it on the GPU only
 * (mlx/ops.cpp:4760-4766); these entry points follow the CUDA kernels' fp32
 * arithmetic (mlx/backend/cuda/quantized/fp_quantize.cuh:73-215, 548-592):
 *   scale_enc = 448 * 6 / global_scale
 *   scale byte = e4m3(max |group| / 6 * scale_enc)
 *   code = e2m1, nearest with ties to even, of w * (scale_enc / value(scale byte))
 *   dequantize: code value * (value(scale byte) * (global_scale / (448 * 6)))
 * Layouts as in mlxrocm_fp_quantize / mlxrocm_fp_dequantize with mode nvfp4.
 */
int mlxrocm_nvfp4_quantize_global(
    const void* w,
    const float* global_scale,
    uint32_t* wq,
    uint8_t* scales,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream);
int mlxrocm_nvfp4_dequantize_global(
    const uint32_t* wq,
    const uint8_t* scales,
    const float* global_scale,
    void* out,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream);
/* fp_quantize_dequantize with a tensor-wide scale
 * (mlx/backend/cuda/quantized/fp_quantize.cuh:73-145): what qqmm applies to x. */
int mlxrocm_nvfp4_quantize_dequantize_global(
    const void* x,
    const float* global_scale,
    void* out,
    size_t n_elems,
    int dtype,
    mlxrocm_stream_t stream);
/* qqmm in nvfp4 with both tensor-wide scales (QQMatmul::eval_gpu,
 * mlx/backend/cuda/quantized/qqmm.cpp:100-208, the route it takes without a
 * block-scaled GEMM library): x_hat = quantize_dequantize(x, global_scale_x) in
 * dtype; y = (x_hat . codes-times-block-scales^T) * (global_scale_w / (448 * 6)),
 * the factor applied to the fp32 sums (mlx/backend/cuda/quantized/qmm/qmv.cu:163-165).
 * workspace: mlxrocm_fp_qqmm_workspace_size(M, N, K, MLXROCM_NVFP4, dtype) bytes. */
int mlxrocm_nvfp4_qqmm_global(
    const void* x,
    const uint32_t* wq,
    const uint8_t* scales,
    const float* global_scale_x,
    const float* global_scale_w,
    void* out,
    int M,
    int N,
    int K,
    int dtype,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

/*
 * GGML tensor types the GGUF loader keeps quantized (ids as in the GGUF file
 * format; every other quantized type is dequantized to fp16 by MLX's loader,
 * mlx/io/gguf.cpp, and is not handled here).
 */
typedef enum {
  MLXROCM_GGML_Q4_0 = 2,
  MLXROCM_GGML_Q4_1 = 3,
  MLXROCM_GGML_Q8_0 = 8
} mlxrocm_ggml_type_t;

/*
 * Replaces the load-time conversion gguf_load_quantized (mlx/io/gguf_quants.cpp:
 * 102-166; block decoders extract_q4_0_data :33-52, extract_q4_1_data :54-74,
 * extract_q8_0_data :76-100, nibble order unpack_32_4 :13-31) for tensor data
 * already resident in device memory.  blocks holds n_blocks GGML blocks of 32
 * weights (18, 20 or 34 bytes each, back to back); outputs are the affine
 * triplet with group size 32: wq n_blocks*4 words (Q4_*, bits = 4) or
 * n_blocks*8 words (Q8_0, bits = 8), scales and biases n_blocks fp16 values
 * (Q4_0: bias = -8 d, Q8_0: bias = -128 d and codes = int8 + 128).  blocks and
 * wq must be 16-byte aligned.
 */
int mlxrocm_gguf_repack(
    const void* blocks,
    uint32_t* wq,
    void* scales,
    void* biases,
    size_t n_blocks,
    int ggml_type,
    mlxrocm_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Quantized matmul                                                          */
/* ------------------------------------------------------------------------ */

/*
 * Replaces QuantizedMatmul::eval_gpu (mlx/primitives.h:1631; CPU body
 * mlx/backend/cpu/quantized.cpp:924-964, batch loop :383-419).
 *
 *   transpose != 0: out[l] = x[l] @ dequant(w[l]).T   w [N, K*bits/32]
 *   transpose == 0: out[l] = x[l] @ dequant(w[l])     w [K, N*bits/32]
 *
 * x is [L, M, K] with batch stride x_batch_stride (elements); out is a dense
 * [L, M, N].  w_batch_stride (uint32 words) and sb_batch_stride (elements) are
 * 0 when one weight matrix is shared by every batch (w.ndim() == 2 in MLX).
 * The kernel is picked from M, N, K, bits, group_size and dtype.
 *
 * `workspace` is device memory of at least mlxrocm_qmm_workspace_size(...)
 * bytes, 256-byte aligned, owned by the caller (an eval_gpu body allocates it
 * like any other temporary and keeps it until the stream has passed the call);
 * it may be NULL when that size is 0.  Shapes that use it: float32 operands
 * with M > 16 (M > 8 in a batch of problems) and transpose != 0 (x split into two bfloat16 parts for the
 * matrix cores); 16-bit calls whose tile grid would leave compute units idle (K
 * is split; fp32 partial results); 16-bit prefill calls with M >= 512 and every
 * transpose == 0 call on the matrix cores (a transposed copy of scales and
 * biases, 4 * N * K / group_size bytes); transpose == 0 calls with 1..8 rows of
 * x and K > 64 (one fp32 plane of the output per 64 rows of K); transpose == 0
 * calls at 2, 3, 5 or 6 bits (the codes repacked at 4 or 8 bits: K * N / 2 or
 * K * N bytes per weight matrix, plus what the call needs at that width); 5..64 rows of
 * x over 4-bit weights with transpose != 0 and K a multiple of 256 beyond
 * 1024 (one fp32 plane of the output per started 1024 codes of K; 33..64
 * rows take the same path 32 rows at a time and need what 32 rows need).  Calls with one to
 * four rows of x and transpose != 0 never use one.  The call only enqueues work: it allocates
 * nothing, takes no lock and does not synchronize, so it can be captured in a
 * HIP graph.  A workspace that is too small is MLXROCM_INVALID_ARGUMENT.
 */
size_t mlxrocm_qmm_workspace_size(
    int M,
    int N,
    int K,
    int L,
    int batched_weights, /* != 0: one weight matrix per batch entry */
    int group_size,
    int bits,
    int dtype,
    int transpose);
int mlxrocm_qmm(
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
    mlxrocm_stream_t stream);

/*
 * Prefill calls (16-bit types, transpose != 0, M >= 512) first transpose scales
 * and biases to [K / group_size][N] (scale, bias) pairs so that consecutive rows
 * of W read consecutive values, both with one load (a few MB, about 5 us per
 * call).  Weights do not change
 * between calls: a caller that keeps that image beside a weight skips the
 * pre-pass.  The reference has no such cache -- its GPU backends read scales in
 * the caller's layout (mlx/backend/cuda/quantized/qmm/qmm.cu:143-146,
 * mlx/backend/metal/quantized.cpp:1799-1801); an eval_gpu body would hang the
 * image on the weight array's sibling list or key it by the scales' buffer.
 *
 * mlxrocm_qmm_sb_image_size: bytes of the image of `batches` weight matrices.
 * mlxrocm_qmm_sb_image: builds it (scales / biases [batches][N][K / group_size],
 * sb_batch_stride elements apart; image 16-byte aligned device memory).
 * mlxrocm_qmm_prepacked: mlxrocm_qmm with the image as an extra argument (NULL:
 * exactly mlxrocm_qmm).  Shapes that do not read an image ignore it; results
 * are those of mlxrocm_qmm bit for bit.  The workspace may then be smaller than
 * mlxrocm_qmm_workspace_size by mlxrocm_qmm_sb_image_size rounded up to 256.
 */
size_t mlxrocm_qmm_sb_image_size(int N, int K, int batches, int group_size, int dtype);
int mlxrocm_qmm_sb_image(
    const void* scales,
    const void* biases,
    void* image,
    int N,
    int K,
    int batches,
    int64_t sb_batch_stride,
    int group_size,
    int dtype,
    mlxrocm_stream_t stream);
int mlxrocm_qmm_prepacked(
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
    mlxrocm_stream_t stream);

/*
 * mlxrocm_qmm without the workspace argument, for callers that cannot
 * allocate device memory at all (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  The scratch the shapes listed above need comes from a 64 MiB
 * array inside the library's device image (one copy per GPU, held until the
 * process ends); a shape that needs more is refused with MLXROCM_UNSUPPORTED.
 * The first call on a device looks the array's address up (no allocation; do
 * it once outside a graph capture -- an empty call, M == 0, is enough).  All
 * calls on one GPU share the array: calls that may overlap in time (different
 * streams or host threads without an ordering between them) race on it.
 * Results are those of mlxrocm_qmm bit for bit.
 */
int mlxrocm_qmm_static(
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
    mlxrocm_stream_t stream);

/*
 * Gated-MLP decode: out = silu(x @ dequant(w_gate).T) * (x @ dequant(w_up).T),
 * both projections in one launch over the shared x, then one elementwise pass.
 * No single primitive of the reference corresponds to it: it fuses the two
 * QuantizedMatmul calls and the `nn.silu(gate(x)) * up(x)` arithmetic that
 * callers of nn.QuantizedLinear (python/mlx/nn/layers/quantized.py:205-307)
 * issue per MLP block; intermediate results are rounded to the element type
 * where that chain rounds them.  x [M, K] (M <= 8), both weights [N, K*bits/32]
 * with scales / biases [N, K/group_size], out [M, N].  `workspace` is device
 * memory of mlxrocm_qmm_swiglu_workspace_size(M, N, dtype) bytes, 16-byte
 * aligned, owned by the caller (the two projections before the gate is
 * applied; shapes whose gate is applied inside the GEMV leave it untouched);
 * the call allocates nothing.
 */
size_t mlxrocm_qmm_swiglu_workspace_size(int M, int N, int dtype);
int mlxrocm_qmm_swiglu(
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
    mlxrocm_stream_t stream);

/*
 * Replaces GatherQMM::eval_gpu (mlx/primitives.h:1698; CPU body
 * mlx/backend/cpu/quantized.cpp:966-1047, loop :700-747):
 *
 *   out[i] = qmm(x[lhs_indices[i]], w[rhs_indices[i]])   for i < n_indices
 *
 * Indices are flat batch indices (uint32, dense vectors of length n_indices).
 * x has x_batches matrices [M, K] x_batch_stride elements apart; the weights are
 * n_experts matrices w_expert_stride words (sb_expert_stride elements) apart, so
 * a sliced expert stack needs no copy.  out is a dense [n_indices, M, N].
 * rhs_sorted != 0 promises rhs_indices is non-decreasing (right_sorted_).
 * workspace (4-byte aligned device memory) must hold
 * mlxrocm_gather_qmm_workspace_size(...) bytes and may be NULL when that is 0:
 * with many index pairs per expert (M == 1, 16-bit types) the pairs are sorted
 * by expert into it and every expert's weights are read once for all its rows
 * (small expert groups of 4-bit weights also keep ceil(K / 1024) fp32 planes of
 * [n_indices, N] there; the pointer must then be 16-byte aligned; with
 * transpose == 0, 4- or 8-bit codes and at least four pairs the [group][k]
 * images of every expert's scales and biases follow the tables, 16-byte
 * aligned as well);
 * without a workspace the call falls back to one product per pair.  Index
 * values are range-checked on the device; an out-of-range pair produces zeros
 * instead of a wild access.
 */
int mlxrocm_gather_qmm(
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
    int rhs_sorted,
    void* workspace,
    size_t workspace_bytes,
    mlxrocm_stream_t stream);

size_t mlxrocm_gather_qmm_workspace_size(
    int M,
    int N,
    int K,
    int n_indices,
    int n_experts,
    int group_size,
    int bits,
    int dtype,
    int transpose,
    int rhs_sorted);

/* Name of the kernel family the dispatcher would pick (for logs and tests):
 * "qmv", "qmm_t", "qmm_n", "qmm_generic".  Returns NULL for invalid arguments. */
const char* mlxrocm_qmm_kernel_name(
    int M,
    int N,
    int K,
    int L,
    int group_size,
    int bits,
    int dtype,
    int transpose);

/*
 * What mlxrocm_qmm would do for a shape, without touching a device: the call
 * is rehearsed -- same argument checks, same kernel choice, the same workspace
 * claims against `workspace_bytes` -- and every launch is recorded instead of
 * issued.  `plan` receives the record as text, "[rule]+kernel(params)+kernel..."
 * ("[rule]" = the entry of the dispatch table that took the shape; a call that
 * re-enters the table, e.g. after repacking odd code widths, shows every
 * entry), truncated to plan_bytes - 1 characters.  Returns what the call would
 * return: MLXROCM_INVALID_ARGUMENT when workspace_bytes is too small.  No
 * counterpart in the reference (its CUDA backend picks kernels in
 * mlx/backend/cuda/quantized/quantized.cpp:95-136 and qmm/qmm.cu:64-100 without
 * an introspection hook); it exists so that the kernel choice and the
 * workspace sizes can be tested on a machine without a GPU.
 */
int mlxrocm_qmm_plan(
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
    size_t plan_bytes);

/* The same for mlxrocm_gather_qmm. */
int mlxrocm_gather_qmm_plan(
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
    size_t plan_bytes);

/* The dispatch table of mlxrocm_qmm, first match wins: number of entries, and
 * entry i's name and the measurements its thresholds rest on (static strings;
 * NULL beyond the table). */
int mlxrocm_qmm_rule_count(void);
const char* mlxrocm_qmm_rule_name(int i);
const char* mlxrocm_qmm_rule_evidence(int i);

/* ------------------------------------------------------------------------ */
/* Element copies with dtype conversion                                      */
/* ------------------------------------------------------------------------ */

/*
 * The data movement eval_gpu bodies do around the matmul kernels: making an
 * operand row-contiguous, converting scales/biases to the activation type,
 * astype of a result, filling with a scalar.  Replaces copy_gpu_inplace and
 * fill_gpu (mlx/backend/gpu/copy.h:14-51; CUDA kernels
 * mlx/backend/cuda/copy/copy_contiguous.cu, copy_general.cu,
 * copy_general_input.cu).  All pointers are device memory; offsets are applied
 * by the caller (pointer + offset * item size).  Conversions follow static_cast:
 * round-to-nearest-even into float types (16-bit floats through fp32),
 * truncation toward zero into integers, != 0 into bool; complex64 -> real drops
 * the imaginary part, real -> complex64 sets it to zero.
 */
size_t mlxrocm_dtype_size(int dtype); /* bytes per element, 0 if unknown */

/* dst[i] = (dst_dtype) src[i] for i < n, or src[0] for every i when
 * broadcast_scalar is non-zero (CopyType::Vector / CopyType::Scalar). */
int mlxrocm_copy_contiguous(
    const void* src,
    int src_dtype,
    void* dst,
    int dst_dtype,
    size_t n,
    int broadcast_scalar,
    mlxrocm_stream_t stream);

/* dst[sum_d i_d * dst_strides[d]] = (dst_dtype) src[sum_d i_d * src_strides[d]]
 * over the index space `shape` (CopyType::General / GeneralGeneral).  Strides
 * are in elements and may be zero or negative; dst_strides == NULL means a
 * row-contiguous destination.  Extent-1 and jointly contiguous dimensions are
 * merged first; more than 8 remaining dimensions are MLXROCM_UNSUPPORTED. */
int mlxrocm_copy_strided(
    const void* src,
    int src_dtype,
    const int64_t* src_strides,
    void* dst,
    int dst_dtype,
    const int64_t* dst_strides,
    int ndim,
    const int64_t* shape,
    mlxrocm_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Device memory with explicit residency, streams, events                    */
/* ------------------------------------------------------------------------ */

/*
 * The allocator behind allocator::malloc / free and the memory counters of
 * mlx/allocator.h:52-75 and mlx/memory.h for a ROCm build (model:
 * mlx/backend/cuda/allocator.cpp:142-399).  Buffers are device-resident
 * (hipMalloc) and recycled through a size-bucketed cache; nothing is
 * host-visible unless copied explicitly with the memcpy calls below.
 */
int mlxrocm_malloc(void** ptr, size_t size);
int mlxrocm_free(void* ptr);
size_t mlxrocm_buffer_size(const void* ptr); /* allocated size, 0 if unknown */
size_t mlxrocm_get_active_memory(void);
size_t mlxrocm_get_peak_memory(void);
void mlxrocm_reset_peak_memory(void);
size_t mlxrocm_get_cache_memory(void);
size_t mlxrocm_set_cache_limit(size_t limit); /* returns the previous limit */
size_t mlxrocm_set_memory_limit(size_t limit);
size_t mlxrocm_get_memory_limit(void);
void mlxrocm_clear_cache(void);

/* Pinned host staging memory (what Buffer::raw_ptr() hands to CPU readers). */
int mlxrocm_host_malloc(void** ptr, size_t size);
int mlxrocm_host_free(void* ptr);

int mlxrocm_memcpy_h2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s);
int mlxrocm_memcpy_d2h(void* dst, const void* src, size_t n, mlxrocm_stream_t s);
int mlxrocm_memcpy_d2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s);

/* Stream plumbing behind mlx::core::Stream (gpu::new_stream / synchronize,
 * mlx/backend/gpu/eval.h:11-18).  Streams are created at default priority. */
int mlxrocm_stream_create(mlxrocm_stream_t* stream);
int mlxrocm_stream_destroy(mlxrocm_stream_t stream);
int mlxrocm_stream_synchronize(mlxrocm_stream_t stream);

/* Event plumbing behind mlx::core::Event (mlx/event.h; model
 * mlx/backend/cuda/event.cu:330-420). */
int mlxrocm_event_create(mlxrocm_event_t* event);
/* An event without timing whose synchronize sleeps instead of spinning: for a
 * host thread that waits on GPU completion (mlx/backend/cuda/worker.cpp:8-10). */
int mlxrocm_event_create_blocking(mlxrocm_event_t* event);
int mlxrocm_event_destroy(mlxrocm_event_t event);
int mlxrocm_event_record(mlxrocm_event_t event, mlxrocm_stream_t stream);
int mlxrocm_event_wait(mlxrocm_event_t event, mlxrocm_stream_t stream);
int mlxrocm_event_synchronize(mlxrocm_event_t event);
int mlxrocm_event_query(mlxrocm_event_t event); /* 1 done, 0 pending, <0 error */
int mlxrocm_event_elapsed_ms(float* ms, mlxrocm_event_t start, mlxrocm_event_t stop);

int mlxrocm_device_count(void);
/* name: >= 256 bytes.  Any out pointer may be NULL. */
int mlxrocm_device_info(
    int device,
    char* name,
    int* compute_units,
    size_t* total_memory,
    int* clock_khz);

#ifdef __cplusplus
}
#endif
#endif /* MLX_ROCM_QMM_H */
