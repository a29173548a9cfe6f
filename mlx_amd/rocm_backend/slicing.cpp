// slicing.cpp -- concatenate_gpu and compute_dynamic_offset, the two functions
// of mlx/backend/gpu/slicing.h:9-38 each GPU backend supplies itself (CUDA:
// mlx/backend/cuda/slicing.cpp:14-108).  slice_gpu and pad_gpu are shared code
// over copy_gpu_inplace.
#include <stdexcept>

#include "mlx/backend/gpu/copy.h"
#include "mlx/backend/gpu/slicing.h"

namespace mlx::core {

void concatenate_gpu(
    const std::vector<array>& inputs,
    array& out,
    int axis,
    const Stream& s) {
  out.set_data(allocator::malloc(out.nbytes()));
  // Each input lands in its own window of the output: same strides as `out`,
  // shifted along `axis` by the extents before it.
  auto window_flags = out.flags();
  window_flags.contiguous = false;
  window_flags.row_contiguous = false;
  window_flags.col_contiguous = false;
  int64_t start = 0;
  for (const array& in : inputs) {
    array window(in.shape(), out.dtype(), nullptr, {});
    window.copy_shared_buffer(
        out, out.strides(), window_flags, window.size(), out.strides()[axis] * start);
    const bool whole_rows = axis == 0 && in.flags().row_contiguous;
    copy_gpu_inplace(
        in, window, whole_rows ? CopyType::Vector : CopyType::GeneralGeneral, s);
    start += in.shape(axis);
  }
}

array compute_dynamic_offset(
    const array&,
    const Strides&,
    const std::vector<int>&,
    const Stream&) {
  throw std::runtime_error(
      "[compute_dynamic_offset] slicing at offsets read from device arrays has no ROCm implementation.");
}

} // namespace mlx::core
