// quantized.cpp -- eval_gpu of the quantization primitives for the ROCm
// backend: QuantizedMatmul, QQMatmul, GatherQMM, GatherQQMM, fast::Quantize and
// fast::ConvertFP8
// (mlx/primitives.h:1616-1717, mlx/fast_primitives.h:337-371), in the affine
// mode and the floating-point modes mxfp4 / mxfp8 / nvfp4.
//
// Each body does what the CUDA backend's does around its kernels
// (mlx/backend/cuda/quantized/quantized.cpp:15-324): make operands dense where
// the kernels need it, allocate the output, translate `array`s into the plain
// pointers / sizes / strides of the C ABI, enqueue on the stream's encoder and
// retain what the kernels read.  Every arithmetic decision (kernel choice,
// tiling) lives behind mlxrocm_qmm / mlxrocm_gather_qmm.
#include <sstream>
#include <limits>
#include <stdexcept>

#include "mlx/allocator.h"
#include "mlx/backend/gpu/copy.h"
#include "mlx/fast_primitives.h"
#include "mlx/primitives.h"
#include "mlx/utils.h"

#include "allocator.h"
#include "device.h"

namespace mlx::core {

namespace {

int dtype_code(Dtype t, const char* who) {
  switch (t) {
    case float32:
      return MLXROCM_FLOAT32;
    case float16:
      return MLXROCM_FLOAT16;
    case bfloat16:
      return MLXROCM_BFLOAT16;
    default: {
      std::ostringstream msg;
      msg << "[" << who << "] Only float32, float16 and bfloat16 are supported "
          << "by the ROCm backend but got " << t << ".";
      throw std::runtime_error(msg.str());
    }
  }
}

int fp_mode_code(QuantizationMode mode) {
  switch (mode) {
    case QuantizationMode::Mxfp4:
      return MLXROCM_MXFP4;
    case QuantizationMode::Mxfp8:
      return MLXROCM_MXFP8;
    default:
      return MLXROCM_NVFP4;
  }
}

// nvfp4 takes an optional tensor-wide scale as a trailing input
// (mlx/ops.cpp:5124-5128, 5393-5397, 4966-4969): one float32 on the device.
const float* global_scale_ptr(const array& g, rocm::CommandEncoder& enc) {
  return rocm::gpu_ptr<float>(g, enc.stream());
}

array ensure_row_contiguous(
    const array& x,
    rocm::CommandEncoder& enc,
    const Stream& s) {
  // The kernels use 16-byte vector loads: a view that starts off that grid is
  // copied like a strided one.
  if (x.flags().row_contiguous && x.offset() % 16 == 0) {
    return x;
  }
  array copy = contiguous_copy_gpu(x, s);
  enc.add_temporary(copy);
  return copy;
}

// Only the trailing matrix has to be dense (mlx/backend/cpu/quantized.cpp:974-990);
// leading dims keep their strides.
array ensure_dense_matrices(
    const array& x,
    rocm::CommandEncoder& enc,
    const Stream& s) {
  if (x.ndim() >= 2 && x.strides()[x.ndim() - 1] == 1 &&
      x.strides()[x.ndim() - 2] == x.shape(-1) && x.offset() % 16 == 0) {
    return x;
  }
  array copy = contiguous_copy_gpu(x, s);
  enc.add_temporary(copy);
  return copy;
}

// Stride between consecutive matrices of a stack whose leading dims are
// either absent, a single dim, or row-contiguous.
int64_t matrix_stride(const array& a) {
  if (a.ndim() <= 2) {
    return 0;
  }
  return a.strides()[a.ndim() - 3];
}

// A temporary of at least `bytes` bytes.  Shapes are 32-bit, so the array is
// [rows, 1 MiB] of uint8: workspaces beyond 2 GiB keep an exact row count.
array workspace_array(size_t bytes) {
  constexpr size_t kRow = size_t(1) << 20;
  const size_t rows = (bytes + kRow - 1) / kRow;
  if (rows > static_cast<size_t>(std::numeric_limits<int>::max())) {
    throw std::runtime_error("[quantized_matmul] workspace beyond 2^51 bytes");
  }
  array ws({static_cast<int>(rows), static_cast<int>(kRow)}, uint8, nullptr, {});
  ws.set_data(allocator::malloc(rows * kRow));
  return ws;
}

bool single_batch_stride(const array& a) {
  // true when element i of the flattened leading dims sits at i * stride
  int64_t expect = matrix_stride(a);
  for (int d = a.ndim() - 3; d >= 0; --d) {
    if (a.shape(d) != 1 && a.strides()[d] != expect) {
      return false;
    }
    expect *= a.shape(d);
  }
  return true;
}

} // namespace

void QuantizedMatmul::eval_gpu(const std::vector<array>& inputs, array& out) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);
  const bool affine = mode_ == QuantizationMode::Affine;

  array x = ensure_row_contiguous(inputs[0], enc, s);
  array w = ensure_row_contiguous(inputs[1], enc, s);
  array scales = ensure_row_contiguous(inputs[2], enc, s);

  out.set_data(allocator::malloc(out.nbytes()));

  const int K = x.shape(-1);
  int M = x.ndim() > 1 ? x.shape(-2) : 1;
  const int N = out.shape(-1);
  int L = (M == 0 || K == 0) ? 0 : static_cast<int>(x.size() / (size_t(K) * M));
  // w.ndim() == 2: one weight for every batch (mlx/backend/cpu/quantized.cpp:396-397)
  const int64_t w_stride = w.ndim() > 2 ? int64_t(w.shape(-1)) * w.shape(-2) : 0;
  const int64_t sb_stride =
      w.ndim() > 2 ? int64_t(scales.shape(-1)) * scales.shape(-2) : 0;
  if (w.ndim() == 2 && L > 1) {
    // x is row-contiguous here, so the batch folds into its rows and the weight
    // is read once for all of them (mlx/backend/metal/quantized.cpp:1799-1801)
    const int64_t rows = int64_t(M) * L;
    if (rows > std::numeric_limits<int>::max()) {
      throw std::runtime_error("[quantized_matmul] more than 2^31 - 1 rows of x");
    }
    M = static_cast<int>(rows);
    L = 1;
  }
  const int dt = dtype_code(x.dtype(), "quantized_matmul");

  if (!affine) {
    // inputs are {x, w, scales}: no biases (mlx/ops.cpp:4816-4821)
    const int mode = fp_mode_code(mode_);
    const size_t ws_bytes = mlxrocm_fp_qmm_workspace_size(
        M, N, K, L, w.ndim() > 2, mode, dt, transpose_ ? 1 : 0);
    void* ws_ptr = nullptr;
    if (ws_bytes > 0) {
      array ws = workspace_array(ws_bytes);
      enc.add_temporary(ws);
      ws_ptr = rocm::gpu_ptr<void>(ws, enc.stream());
    }
    rocm::check(mlxrocm_fp_qmm(
        rocm::gpu_ptr<void>(x, enc.stream()),
        rocm::gpu_ptr<uint32_t>(w, enc.stream()),
        rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
        rocm::gpu_ptr<void>(out, enc.stream()),
        M,
        N,
        K,
        L,
        int64_t(M) * K,
        w_stride,
        sb_stride,
        mode,
        dt,
        transpose_ ? 1 : 0,
        ws_ptr,
        ws_bytes,
        enc.stream()));
    return;
  }
  array biases = ensure_row_contiguous(inputs[3], enc, s);

  // device scratch of the call: a temporary like any other
  const size_t ws_bytes = mlxrocm_qmm_workspace_size(
      M, N, K, L, w.ndim() > 2, group_size_, bits_, dt, transpose_ ? 1 : 0);
  void* ws_ptr = nullptr;
  if (ws_bytes > 0) {
    array ws = workspace_array(ws_bytes);
    enc.add_temporary(ws);
    ws_ptr = rocm::gpu_ptr<void>(ws, enc.stream());
  }

  rocm::check(mlxrocm_qmm(
      rocm::gpu_ptr<void>(x, enc.stream()),
      rocm::gpu_ptr<uint32_t>(w, enc.stream()),
      rocm::gpu_ptr<void>(scales, enc.stream()),
      rocm::gpu_ptr<void>(biases, enc.stream()),
      rocm::gpu_ptr<void>(out, enc.stream()),
      M,
      N,
      K,
      L,
      int64_t(M) * K,
      w_stride,
      sb_stride,
      group_size_,
      bits_,
      dt,
      transpose_ ? 1 : 0,
      ws_ptr,
      ws_bytes,
      enc.stream()));
}

namespace {

// mx.quantize of a floating-point second operand inside qqmm / gather_qqmm,
// with the tensor-wide scale when there is one (quantize_input,
// mlx/backend/cuda/quantized/qqmm.cpp:17-54).
void quantize_weights(
    const array& w,
    array& wq,
    array& scales,
    const float* global_scale,
    int mode,
    int dt,
    rocm::CommandEncoder& enc) {
  if (global_scale != nullptr) {
    rocm::check(mlxrocm_nvfp4_quantize_global(
        rocm::gpu_ptr<void>(w, enc.stream()),
        global_scale,
        rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
        rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
        w.size(),
        dt,
        enc.stream()));
    return;
  }
  rocm::check(mlxrocm_fp_quantize(
      rocm::gpu_ptr<void>(w, enc.stream()),
      rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
      rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
      w.size(),
      mode,
      dt,
      enc.stream()));
}

} // namespace

// x is quantized and dequantized on the fly in its own type, then multiplied by
// the transposed quantized w: what QQMatmul::eval_cpu does for one row of x
// (mlx/backend/cpu/quantized.cpp:1322-1360), here for any number of rows.  A
// floating-point w (inputs {x, w}) is quantized into temporaries first, as the
// CUDA backend does (mlx/backend/cuda/quantized/qqmm.cpp).
void QQMatmul::eval_gpu(const std::vector<array>& inputs, array& out) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);
  if (mode_ == QuantizationMode::Affine) {
    throw std::runtime_error("[qqmm] Affine quantization is not supported.");
  }
  const bool w_quantized = inputs[1].dtype() == uint32;
  // nvfp4: {..., global_scale_x, global_scale_w} may follow (mlx/ops.cpp:4966-4969)
  const size_t base_size = w_quantized ? 3u : 2u;
  const bool has_global_scales =
      mode_ == QuantizationMode::Nvfp4 && inputs.size() == base_size + 2;
  const float* gx = has_global_scales ? global_scale_ptr(inputs[base_size], enc) : nullptr;
  const float* gw = has_global_scales ? global_scale_ptr(inputs[base_size + 1], enc) : nullptr;
  const int mode = fp_mode_code(mode_);

  array x = ensure_row_contiguous(inputs[0], enc, s);
  array w = ensure_row_contiguous(inputs[1], enc, s);
  const int K = x.shape(-1);
  const int N = out.shape(-1);
  const int64_t rows = K == 0 ? 0 : static_cast<int64_t>(x.size() / size_t(K));
  if (rows > std::numeric_limits<int>::max()) {
    throw std::runtime_error("[qqmm] more than 2^31 - 1 rows of x");
  }
  const int dt = dtype_code(x.dtype(), "qqmm");

  array scales = w_quantized ? ensure_row_contiguous(inputs[2], enc, s)
                             : array({N, K / group_size_}, uint8, nullptr, {});
  if (!w_quantized) {
    if (w.dtype() != x.dtype()) {
      throw std::runtime_error("[qqmm] x and a floating-point w must share one type");
    }
    array wq({N, K * bits_ / 32}, uint32, nullptr, {});
    wq.set_data(allocator::malloc(wq.nbytes()));
    scales.set_data(allocator::malloc(scales.nbytes()));
    enc.add_temporary(wq);
    enc.add_temporary(scales);
    quantize_weights(w, wq, scales, gw, mode, dt, enc);
    w = wq;
  }

  out.set_data(allocator::malloc(out.nbytes()));
  // x is quantized inside the call: to codes for the block-scaled matrix
  // instruction (MX modes, 16 rows or more), else to x_hat in its own type
  const size_t ws_bytes =
      mlxrocm_fp_qqmm_workspace_size(static_cast<int>(rows), N, K, mode, dt);
  void* ws_ptr = nullptr;
  if (ws_bytes > 0) {
    array ws = workspace_array(ws_bytes);
    enc.add_temporary(ws);
    ws_ptr = rocm::gpu_ptr<void>(ws, enc.stream());
  }
  if (has_global_scales) {
    rocm::check(mlxrocm_nvfp4_qqmm_global(
        rocm::gpu_ptr<void>(x, enc.stream()),
        rocm::gpu_ptr<uint32_t>(w, enc.stream()),
        rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
        gx,
        gw,
        rocm::gpu_ptr<void>(out, enc.stream()),
        static_cast<int>(rows),
        N,
        K,
        dt,
        ws_ptr,
        ws_bytes,
        enc.stream()));
    return;
  }
  rocm::check(mlxrocm_fp_qqmm(
      rocm::gpu_ptr<void>(x, enc.stream()),
      rocm::gpu_ptr<uint32_t>(w, enc.stream()),
      rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
      rocm::gpu_ptr<void>(out, enc.stream()),
      static_cast<int>(rows),
      N,
      K,
      mode,
      dt,
      ws_ptr,
      ws_bytes,
      enc.stream()));
}

// gather_qqmm (mlx/ops.cpp:5631-5681): inputs {x, w, lhs, rhs [, scales_w]
// [, global_scale_x, global_scale_w]}.  Every matrix of x is quantized and
// dequantized in its own type inside the call, then gathered pairs are
// multiplied, as GatherQQMM::eval_gpu of the CUDA backend does
// (mlx/backend/cuda/quantized/qqmm.cpp:210-281).
void GatherQQMM::eval_gpu(const std::vector<array>& inputs, array& out) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);
  if (mode_ == QuantizationMode::Affine) {
    throw std::runtime_error("[gather_qqmm] Affine quantization is not supported.");
  }
  const bool w_quantized = inputs[1].dtype() == uint32;
  const size_t base_size = w_quantized ? 5u : 4u;
  const bool has_global_scales =
      mode_ == QuantizationMode::Nvfp4 && inputs.size() == base_size + 2;
  const float* gx = has_global_scales ? global_scale_ptr(inputs[base_size], enc) : nullptr;
  const float* gw = has_global_scales ? global_scale_ptr(inputs[base_size + 1], enc) : nullptr;
  const int mode = fp_mode_code(mode_);

  array x = ensure_row_contiguous(inputs[0], enc, s);
  array w = ensure_row_contiguous(inputs[1], enc, s);
  array lhs = ensure_row_contiguous(inputs[2], enc, s);
  array rhs = ensure_row_contiguous(inputs[3], enc, s);
  const int K = x.shape(-1);
  const int M = x.shape(-2);
  const int N = out.shape(-1);
  const int dt = dtype_code(x.dtype(), "gather_qqmm");

  array scales = w_quantized ? ensure_row_contiguous(inputs[4], enc, s) : w;
  if (!w_quantized) {
    if (w.dtype() != x.dtype()) {
      throw std::runtime_error("[gather_qqmm] x and a floating-point w must share one type");
    }
    auto q_shape = w.shape();
    q_shape.back() = K * bits_ / 32;
    auto s_shape = w.shape();
    s_shape.back() = K / group_size_;
    array wq(q_shape, uint32, nullptr, {});
    scales = array(s_shape, uint8, nullptr, {});
    wq.set_data(allocator::malloc(wq.nbytes()));
    scales.set_data(allocator::malloc(scales.nbytes()));
    enc.add_temporary(wq);
    enc.add_temporary(scales);
    quantize_weights(w, wq, scales, gw, mode, dt, enc);
    w = wq;
  }

  out.set_data(allocator::malloc(out.nbytes()));
  const int n_idx = static_cast<int>(lhs.size());
  const int x_batches = (M == 0 || K == 0) ? 0 : static_cast<int>(x.size() / (size_t(K) * M));
  const int n_experts = (N == 0 || w.shape(-1) == 0)
      ? 0
      : static_cast<int>(w.size() / (size_t(w.shape(-1)) * w.shape(-2)));
  const size_t ws_bytes = mlxrocm_fp_gather_qqmm_workspace_size(
      M, N, K, n_idx, x_batches, n_experts, 1, mode, dt);
  void* ws_ptr = nullptr;
  if (ws_bytes > 0) {
    array ws = workspace_array(ws_bytes);
    enc.add_temporary(ws);
    ws_ptr = rocm::gpu_ptr<void>(ws, enc.stream());
  }
  rocm::check(mlxrocm_fp_gather_qqmm(
      rocm::gpu_ptr<void>(x, enc.stream()),
      rocm::gpu_ptr<uint32_t>(w, enc.stream()),
      rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
      rocm::gpu_ptr<uint32_t>(lhs, enc.stream()),
      rocm::gpu_ptr<uint32_t>(rhs, enc.stream()),
      gx,
      gw,
      rocm::gpu_ptr<void>(out, enc.stream()),
      M,
      N,
      K,
      n_idx,
      x_batches,
      n_experts,
      int64_t(M) * K,
      int64_t(N) * w.shape(-1),
      int64_t(N) * scales.shape(-1),
      mode,
      dt,
      ws_ptr,
      ws_bytes,
      enc.stream()));
}

void GatherQMM::eval_gpu(const std::vector<array>& inputs, array& out) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);
  const bool affine = mode_ == QuantizationMode::Affine;
  // inputs: {x, w, scales, biases, lhs, rhs}; without biases in the
  // floating-point modes (mlx/ops.cpp:5601-5618)
  const int first_index = affine ? 4 : 3;

  array x = ensure_row_contiguous(inputs[0], enc, s);
  array w = ensure_dense_matrices(inputs[1], enc, s);
  array scales = ensure_dense_matrices(inputs[2], enc, s);
  array biases = affine ? ensure_dense_matrices(inputs[3], enc, s) : scales;
  // A stack the kernels can address as base + e * stride keeps its layout
  // (sliced expert stacks); anything more exotic is made dense.
  if (!single_batch_stride(w) || !single_batch_stride(scales) ||
      !single_batch_stride(biases) ||
      matrix_stride(scales) != matrix_stride(biases)) {
    w = ensure_row_contiguous(w, enc, s);
    scales = ensure_row_contiguous(scales, enc, s);
    biases = affine ? ensure_row_contiguous(biases, enc, s) : scales;
  }
  array lhs = ensure_row_contiguous(inputs[first_index], enc, s);
  array rhs = ensure_row_contiguous(inputs[first_index + 1], enc, s);

  out.set_data(allocator::malloc(out.nbytes()));

  const int K = x.shape(-1);
  const int M = x.shape(-2);
  const int N = out.shape(-1);
  const int n_idx = static_cast<int>(lhs.size());
  const int x_batches = (M == 0 || K == 0) ? 0 : static_cast<int>(x.size() / (size_t(K) * M));
  const int n_experts =
      static_cast<int>(w.size() / (size_t(w.shape(-1)) * w.shape(-2)));
  const int dt = dtype_code(x.dtype(), "gather_qmm");

  if (!affine) {
    const int64_t scales_stride = scales.ndim() > 2 ? matrix_stride(scales) : 0;
    const size_t fp_ws_bytes = mlxrocm_fp_gather_qmm_workspace_size(
        M, N, K, n_idx, n_experts, scales_stride != 0, fp_mode_code(mode_), dt, transpose_ ? 1 : 0);
    void* fp_ws = nullptr;
    if (fp_ws_bytes > 0) {
      array ws = workspace_array(fp_ws_bytes);
      enc.add_temporary(ws);
      fp_ws = rocm::gpu_ptr<void>(ws, enc.stream());
    }
    rocm::check(mlxrocm_fp_gather_qmm(
        rocm::gpu_ptr<void>(x, enc.stream()),
        rocm::gpu_ptr<uint32_t>(w, enc.stream()),
        rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
        rocm::gpu_ptr<uint32_t>(lhs, enc.stream()),
        rocm::gpu_ptr<uint32_t>(rhs, enc.stream()),
        rocm::gpu_ptr<void>(out, enc.stream()),
        M,
        N,
        K,
        n_idx,
        x_batches,
        n_experts,
        int64_t(M) * K,
        w.ndim() > 2 ? matrix_stride(w) : 0,
        scales_stride,
        fp_mode_code(mode_),
        dt,
        transpose_ ? 1 : 0,
        fp_ws,
        fp_ws_bytes,
        enc.stream()));
    return;
  }

  const size_t ws_bytes = mlxrocm_gather_qmm_workspace_size(
      M, N, K, n_idx, n_experts, group_size_, bits_, dt, transpose_, right_sorted_);
  void* ws_ptr = nullptr;
  if (ws_bytes > 0) {
    array ws = workspace_array(ws_bytes);
    enc.add_temporary(ws);
    ws_ptr = rocm::gpu_ptr<void>(ws, enc.stream());
  }

  rocm::check(mlxrocm_gather_qmm(
      rocm::gpu_ptr<void>(x, enc.stream()),
      rocm::gpu_ptr<uint32_t>(w, enc.stream()),
      rocm::gpu_ptr<void>(scales, enc.stream()),
      rocm::gpu_ptr<void>(biases, enc.stream()),
      rocm::gpu_ptr<uint32_t>(lhs, enc.stream()),
      rocm::gpu_ptr<uint32_t>(rhs, enc.stream()),
      rocm::gpu_ptr<void>(out, enc.stream()),
      M,
      N,
      K,
      n_idx,
      x_batches,
      n_experts,
      int64_t(M) * K,
      w.ndim() > 2 ? matrix_stride(w) : 0,
      scales.ndim() > 2 ? matrix_stride(scales) : 0,
      group_size_,
      bits_,
      dt,
      transpose_ ? 1 : 0,
      right_sorted_ ? 1 : 0,
      ws_ptr,
      ws_bytes,
      enc.stream()));
}

// mx.to_fp8 / mx.from_fp8 (mlx/ops.cpp:5519-5552): elementwise, any shape.
void fast::ConvertFP8::eval_gpu(
    const std::vector<array>& inputs,
    std::vector<array>& outputs) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);
  array in = ensure_row_contiguous(inputs[0], enc, s);
  array& out = outputs[0];
  out.set_data(allocator::malloc(out.nbytes()));
  if (to_fp8_) {
    rocm::check(mlxrocm_to_fp8(
        rocm::gpu_ptr<void>(in, enc.stream()),
        rocm::gpu_ptr<uint8_t>(out, enc.stream()),
        in.size(),
        dtype_code(in.dtype(), "to_fp8"),
        enc.stream()));
  } else {
    rocm::check(mlxrocm_from_fp8(
        rocm::gpu_ptr<uint8_t>(in, enc.stream()),
        rocm::gpu_ptr<void>(out, enc.stream()),
        in.size(),
        dtype_code(out.dtype(), "from_fp8"),
        enc.stream()));
  }
}

void fast::Quantize::eval_gpu(
    const std::vector<array>& inputs,
    std::vector<array>& outputs) {
  auto& s = stream();
  auto& enc = rocm::get_command_encoder(s);

  if (mode_ != QuantizationMode::Affine) {
    // fp_quantize: {w [, global_scale]} -> {wq, scales}; fp_dequantize:
    // {wq, scales [, global_scale]} -> {w} (mlx/ops.cpp:5124-5128, 5393-5397)
    const int mode = fp_mode_code(mode_);
    if (dequantize_) {
      array wq = ensure_row_contiguous(inputs[0], enc, s);
      array scales = ensure_row_contiguous(inputs[1], enc, s);
      array& w = outputs[0];
      w.set_data(allocator::malloc(w.nbytes()));
      if (inputs.size() > 2) {
        rocm::check(mlxrocm_nvfp4_dequantize_global(
            rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
            rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
            global_scale_ptr(inputs[2], enc),
            rocm::gpu_ptr<void>(w, enc.stream()),
            w.size(),
            dtype_code(w.dtype(), "dequantize"),
            enc.stream()));
        return;
      }
      rocm::check(mlxrocm_fp_dequantize(
          rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
          rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
          rocm::gpu_ptr<void>(w, enc.stream()),
          w.size(),
          mode,
          dtype_code(w.dtype(), "dequantize"),
          enc.stream()));
    } else {
      array w = ensure_row_contiguous(inputs[0], enc, s);
      array& wq = outputs[0];
      array& scales = outputs[1];
      wq.set_data(allocator::malloc(wq.nbytes()));
      scales.set_data(allocator::malloc(scales.nbytes()));
      if (inputs.size() > 1) {
        rocm::check(mlxrocm_nvfp4_quantize_global(
            rocm::gpu_ptr<void>(w, enc.stream()),
            global_scale_ptr(inputs[1], enc),
            rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
            rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
            w.size(),
            dtype_code(w.dtype(), "quantize"),
            enc.stream()));
        return;
      }
      rocm::check(mlxrocm_fp_quantize(
          rocm::gpu_ptr<void>(w, enc.stream()),
          rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
          rocm::gpu_ptr<uint8_t>(scales, enc.stream()),
          w.size(),
          mode,
          dtype_code(w.dtype(), "quantize"),
          enc.stream()));
    }
    return;
  }

  if (dequantize_) {
    array wq = ensure_row_contiguous(inputs[0], enc, s);
    array scales = ensure_row_contiguous(inputs[1], enc, s);
    array biases = ensure_row_contiguous(inputs[2], enc, s);
    array& w = outputs[0];
    w.set_data(allocator::malloc(w.nbytes()));
    rocm::check(mlxrocm_affine_dequantize(
        rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
        rocm::gpu_ptr<void>(scales, enc.stream()),
        rocm::gpu_ptr<void>(biases, enc.stream()),
        rocm::gpu_ptr<void>(w, enc.stream()),
        w.size(),
        group_size_,
        bits_,
        dtype_code(w.dtype(), "dequantize"),
        enc.stream()));
  } else {
    array w = ensure_row_contiguous(inputs[0], enc, s);
    array& wq = outputs[0];
    array& scales = outputs[1];
    array& biases = outputs[2];
    wq.set_data(allocator::malloc(wq.nbytes()));
    scales.set_data(allocator::malloc(scales.nbytes()));
    biases.set_data(allocator::malloc(biases.nbytes()));
    rocm::check(mlxrocm_affine_quantize(
        rocm::gpu_ptr<void>(w, enc.stream()),
        rocm::gpu_ptr<uint32_t>(wq, enc.stream()),
        rocm::gpu_ptr<void>(scales, enc.stream()),
        rocm::gpu_ptr<void>(biases, enc.stream()),
        w.size(),
        group_size_,
        bits_,
        dtype_code(w.dtype(), "quantize"),
        enc.stream()));
  }
}

} // namespace mlx::core
