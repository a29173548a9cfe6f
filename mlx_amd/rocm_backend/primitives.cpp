// primitives.cpp -- eval_gpu of every primitive the ROCm backend does not
// compute: each throws, naming itself, the way the CUDA backend answers for the
// ones it lacks (mlx/backend/cuda/primitives.cpp:10-38).  The fused fast::
// primitives that have a composed fallback say so through use_fallback(), so
// MLX builds them from basic primitives instead.
//
// What the backend does compute is elsewhere: QuantizedMatmul, GatherQMM and
// fast::Quantize in quantized.cpp; the data-movement primitives (AsType,
// Broadcast, Concatenate, Contiguous, Copy, Full, Pad, Reshape, Slice, Split,
// Transpose, ...) are MLX's shared mlx/backend/gpu/primitives.cpp over this
// backend's copy.cpp and slicing.cpp.
#include <stdexcept>

#include "mlx/distributed/primitives.h"
#include "mlx/fast_primitives.h"
#include "mlx/primitives.h"

namespace mlx::core {

#define ROCM_NO_UNARY(cls)                                              \
  void cls::eval_gpu(const std::vector<array>&, array&) {               \
    throw std::runtime_error(#cls " has no ROCm implementation.");      \
  }

#define ROCM_NO_MULTI(cls)                                                  \
  void cls::eval_gpu(const std::vector<array>&, std::vector<array>&) {      \
    throw std::runtime_error(#cls " has no ROCm implementation.");          \
  }

ROCM_NO_UNARY(Abs)
ROCM_NO_UNARY(Add)
ROCM_NO_UNARY(AddMM)
ROCM_NO_UNARY(Arange)
ROCM_NO_UNARY(ArcCos)
ROCM_NO_UNARY(ArcCosh)
ROCM_NO_UNARY(ArcSin)
ROCM_NO_UNARY(ArcSinh)
ROCM_NO_UNARY(ArcTan)
ROCM_NO_UNARY(ArcTan2)
ROCM_NO_UNARY(ArcTanh)
ROCM_NO_UNARY(ArgPartition)
ROCM_NO_UNARY(ArgReduce)
ROCM_NO_UNARY(ArgSort)
ROCM_NO_UNARY(BitwiseBinary)
ROCM_NO_UNARY(BitwiseInvert)
ROCM_NO_UNARY(BlockMaskedMM)
ROCM_NO_UNARY(GatherMM)
ROCM_NO_UNARY(SegmentedMM)
ROCM_NO_UNARY(Ceil)
ROCM_NO_UNARY(Conjugate)
ROCM_NO_UNARY(Convolution)
ROCM_NO_UNARY(Cos)
ROCM_NO_UNARY(Cosh)
ROCM_NO_UNARY(Divide)
ROCM_NO_UNARY(Select)
ROCM_NO_UNARY(Remainder)
ROCM_NO_UNARY(Equal)
ROCM_NO_UNARY(Erf)
ROCM_NO_UNARY(ErfInv)
ROCM_NO_UNARY(Exp)
ROCM_NO_UNARY(Expm1)
ROCM_NO_UNARY(FFT)
ROCM_NO_UNARY(Floor)
ROCM_NO_UNARY(Gather)
ROCM_NO_UNARY(GatherAxis)
ROCM_NO_UNARY(Greater)
ROCM_NO_UNARY(GreaterEqual)
ROCM_NO_UNARY(Hadamard)
ROCM_NO_UNARY(Imag)
ROCM_NO_UNARY(Less)
ROCM_NO_UNARY(LessEqual)
ROCM_NO_UNARY(Load)
ROCM_NO_UNARY(Log)
ROCM_NO_UNARY(Log1p)
ROCM_NO_UNARY(LogicalNot)
ROCM_NO_UNARY(LogicalAnd)
ROCM_NO_UNARY(LogicalOr)
ROCM_NO_UNARY(LogAddExp)
ROCM_NO_UNARY(LogSumExp)
ROCM_NO_UNARY(Matmul)
ROCM_NO_UNARY(Maximum)
ROCM_NO_UNARY(Minimum)
ROCM_NO_UNARY(Multiply)
ROCM_NO_UNARY(Negative)
ROCM_NO_UNARY(NotEqual)
ROCM_NO_UNARY(Partition)
ROCM_NO_UNARY(Power)
ROCM_NO_UNARY(RandomBits)
ROCM_NO_UNARY(Real)
ROCM_NO_UNARY(Reduce)
ROCM_NO_UNARY(Round)
ROCM_NO_UNARY(Scan)
ROCM_NO_UNARY(Scatter)
ROCM_NO_UNARY(ScatterAxis)
ROCM_NO_UNARY(MaskedScatter)
ROCM_NO_UNARY(Sigmoid)
ROCM_NO_UNARY(Sign)
ROCM_NO_UNARY(Sin)
ROCM_NO_UNARY(Sinh)
ROCM_NO_UNARY(SliceUpdate)
ROCM_NO_UNARY(Softmax)
ROCM_NO_UNARY(SearchSorted)
ROCM_NO_UNARY(Sort)
ROCM_NO_UNARY(Square)
ROCM_NO_UNARY(Sqrt)
ROCM_NO_UNARY(Subtract)
ROCM_NO_UNARY(Tan)
ROCM_NO_UNARY(Tanh)
ROCM_NO_UNARY(Inverse)
ROCM_NO_UNARY(Cholesky)

ROCM_NO_MULTI(Compiled)
ROCM_NO_MULTI(DivMod)
ROCM_NO_MULTI(QRF)
ROCM_NO_MULTI(SVD)
ROCM_NO_MULTI(Eig)
ROCM_NO_MULTI(Eigh)
ROCM_NO_MULTI(LUF)

namespace fast {

ROCM_NO_MULTI(RMSNormVJP)
ROCM_NO_MULTI(LayerNormVJP)
ROCM_NO_MULTI(ScaledDotProductAttentionVJP)
ROCM_NO_MULTI(CustomKernel)
ROCM_NO_MULTI(RMSNorm)
ROCM_NO_MULTI(LayerNorm)
ROCM_NO_MULTI(RoPE)
ROCM_NO_MULTI(ScaledDotProductAttention)

bool RMSNorm::use_fallback(Stream) {
  return true;
}
bool LayerNorm::use_fallback(Stream) {
  return true;
}
bool RoPE::use_fallback(Stream) {
  return true;
}
bool ScaledDotProductAttention::use_fallback(
    const array&,
    const array&,
    const array&,
    bool,
    bool,
    bool,
    bool,
    bool,
    bool,
    Stream) {
  return true;
}
bool ScaledDotProductAttention::supports_bool_mask() {
  return false;
}
bool ScaledDotProductAttentionVJP::use_fallback(const array&, Stream) {
  return true;
}

} // namespace fast

namespace distributed {

ROCM_NO_MULTI(AllReduce)
ROCM_NO_MULTI(AllGather)
ROCM_NO_MULTI(Send)
ROCM_NO_MULTI(Recv)
ROCM_NO_MULTI(ReduceScatter)

} // namespace distributed

} // namespace mlx::core
