// copy.cpp -- copy_gpu / copy_gpu_inplace / fill_gpu / reshape_gpu of the ROCm
// backend (interface: mlx/backend/gpu/copy.h:14-51; CUDA counterpart:
// mlx/backend/cuda/copy.cu:8-131).  The shared helpers built on these
// (contiguous_copy_gpu, reshape_in_eval ..., mlx/backend/gpu/copy.cpp) and the
// data-movement primitives of mlx/backend/gpu/primitives.cpp come with them.
//
// The kernels sit behind two entry points of the C ABI: a contiguous one
// (CopyType::Scalar and Vector) and a strided one that takes MLX's shape and
// element strides as they are -- merging of dimensions happens on the other
// side of the ABI, so nothing is collapsed here.
#include <stdexcept>
#include <vector>

#include "mlx/backend/common/utils.h"
#include "mlx/backend/gpu/copy.h"

#include "allocator.h"
#include "device.h"

namespace mlx::core {

namespace {

int copy_dtype(Dtype dt) {
  switch (dt) {
    case float32:
      return MLXROCM_FLOAT32;
    case float16:
      return MLXROCM_FLOAT16;
    case bfloat16:
      return MLXROCM_BFLOAT16;
    case bool_:
      return MLXROCM_BOOL;
    case uint8:
      return MLXROCM_UINT8;
    case uint16:
      return MLXROCM_UINT16;
    case uint32:
      return MLXROCM_UINT32;
    case uint64:
      return MLXROCM_UINT64;
    case int8:
      return MLXROCM_INT8;
    case int16:
      return MLXROCM_INT16;
    case int32:
      return MLXROCM_INT32;
    case int64:
      return MLXROCM_INT64;
    case float64:
      return MLXROCM_FLOAT64;
    case complex64:
      return MLXROCM_COMPLEX64;
  }
  throw std::invalid_argument("[copy_gpu] unknown dtype");
}

} // namespace

void copy_gpu(const array& in, array& out, CopyType ctype, const Stream& s) {
  // A donated input of the same type already is the output.
  bool donated = set_copy_output_data(in, out, ctype);
  if (donated && in.dtype() == out.dtype()) {
    return;
  }
  // The output was just made dense: its strides need not be walked.
  copy_gpu_inplace(
      in, out, ctype == CopyType::GeneralGeneral ? CopyType::General : ctype, s);
}

void copy_gpu_inplace(
    const array& in,
    array& out,
    const Shape& shape,
    const Strides& i_strides,
    const Strides& o_strides,
    int64_t i_offset,
    int64_t o_offset,
    CopyType ctype,
    const Stream& s,
    std::optional<array> dynamic_i_offset,
    std::optional<array> dynamic_o_offset) {
  if (out.size() == 0) {
    return;
  }
  if (dynamic_i_offset || dynamic_o_offset) {
    throw std::runtime_error(
        "[copy_gpu_inplace] offsets read from device arrays have no ROCm implementation.");
  }
  auto& enc = rocm::get_command_encoder(s);
  const int src_dt = copy_dtype(in.dtype());
  const int dst_dt = copy_dtype(out.dtype());
  const char* src = static_cast<const char*>(rocm::gpu_ptr<void>(in, enc.stream())) +
      i_offset * static_cast<int64_t>(in.itemsize());
  char* dst = rocm::gpu_ptr<char>(out, enc.stream()) +
      o_offset * static_cast<int64_t>(out.itemsize());

  switch (ctype) {
    case CopyType::Scalar:
      rocm::check(mlxrocm_copy_contiguous(
          src, src_dt, dst, dst_dt, out.data_size(), /* broadcast_scalar */ 1, enc.stream()));
      break;
    case CopyType::Vector:
      rocm::check(mlxrocm_copy_contiguous(
          src, src_dt, dst, dst_dt, in.data_size(), 0, enc.stream()));
      break;
    case CopyType::General:
    case CopyType::GeneralGeneral: {
      std::vector<int64_t> dims(shape.begin(), shape.end());
      std::vector<int64_t> si(i_strides.begin(), i_strides.end());
      std::vector<int64_t> so(o_strides.begin(), o_strides.end());
      rocm::check(mlxrocm_copy_strided(
          src,
          src_dt,
          si.data(),
          dst,
          dst_dt,
          ctype == CopyType::General ? nullptr : so.data(),
          static_cast<int>(dims.size()),
          dims.data(),
          enc.stream()));
      break;
    }
  }
}

void fill_gpu(const array& val, array& out, const Stream& s) {
  if (out.size() == 0) {
    return;
  }
  out.set_data(allocator::malloc(out.nbytes()));
  auto& enc = rocm::get_command_encoder(s);
  rocm::check(mlxrocm_copy_contiguous(
      rocm::gpu_ptr<void>(val, enc.stream()),
      copy_dtype(val.dtype()),
      rocm::gpu_ptr<void>(out, enc.stream()),
      copy_dtype(out.dtype()),
      out.data_size(),
      /* broadcast_scalar */ 1,
      enc.stream()));
}

void reshape_gpu(const array& in, array& out, Stream s) {
  auto [needs_copy, out_strides] = prepare_reshape(in, out);
  if (!needs_copy) {
    shared_buffer_reshape(in, out_strides, out);
    return;
  }
  // Rows of `in` in order are rows of `out` in order: gather into a dense buffer.
  out.set_data(allocator::malloc(out.nbytes()));
  copy_gpu_inplace(
      in,
      out,
      in.shape(),
      in.strides(),
      make_contiguous_strides(in.shape()),
      0,
      0,
      CopyType::General,
      s);
}

} // namespace mlx::core
