// gguf_repack.hip -- GGML block formats Q4_0 / Q4_1 / Q8_0 -> the affine
// triplet (packed codes, fp16 scales, fp16 biases) with group size 32 that the
// quantized-matmul kernels read.  Same results as the load-time conversion in
// mlx/io/gguf_quants.cpp:13-100 (unpack_32_4, extract_q4_0_data,
// extract_q4_1_data, extract_q8_0_data).
//
// A block holds 32 weights: | fp16 d | [fp16 m] | quants |, 18 / 20 / 34 bytes,
// so blocks are only 2-byte aligned.  A workgroup copies its 256 blocks into
// LDS with 16-byte loads (256 blocks are a multiple of 16 bytes in all three
// formats), then every thread converts one block from LDS and writes its codes
// as whole 16-byte pieces.  HBM-bound: 18 + 20 (Q4_0), 20 + 20 (Q4_1) or
// 34 + 36 (Q8_0) bytes per block.
#include "common.h"

namespace mlxrocm {

namespace {

constexpr int kRepackBlock = 256;

enum : int { kQ4_0 = 0, kQ4_1 = 1, kQ8_0 = 2 };

template <int FMT>
struct BlockLayout;
template <>
struct BlockLayout<kQ4_0> {
  static constexpr int bytes = 18, header = 2, words = 4;
};
template <>
struct BlockLayout<kQ4_1> {
  static constexpr int bytes = 20, header = 4, words = 4;
};
template <>
struct BlockLayout<kQ8_0> {
  static constexpr int bytes = 34, header = 2, words = 8;
};

template <int FMT>
__global__ __launch_bounds__(kRepackBlock) void gguf_repack_kernel(
    const uint8_t* __restrict__ blocks,
    uint32_t* __restrict__ wq,
    f16_t* __restrict__ scales,
    f16_t* __restrict__ biases,
    size_t n_blocks) {
  using L = BlockLayout<FMT>;
  __shared__ __attribute__((aligned(16))) uint8_t sm[kRepackBlock * L::bytes];
  const int tid = threadIdx.x;
  const size_t b0 = static_cast<size_t>(blockIdx.x) * kRepackBlock;
  const size_t left = n_blocks - b0;
  const int nb = left < kRepackBlock ? static_cast<int>(left) : kRepackBlock;
  const uint8_t* src = blocks + b0 * L::bytes;
  if (nb == kRepackBlock) {
    constexpr int kPieces = kRepackBlock * L::bytes / 16;
    static_assert(kRepackBlock * L::bytes % 16 == 0, "chunk is whole 16-byte pieces");
    for (int i = tid; i < kPieces; i += kRepackBlock) {
      reinterpret_cast<uint4*>(sm)[i] = reinterpret_cast<const uint4*>(src)[i];
    }
  } else {
    // the last, partial chunk: 2-byte loads stay inside the tensor
    const int halves = nb * L::bytes / 2;
    for (int i = tid; i < halves; i += kRepackBlock) {
      reinterpret_cast<uint16_t*>(sm)[i] = reinterpret_cast<const uint16_t*>(src)[i];
    }
  }
  __syncthreads();
  if (tid >= nb) {
    return;
  }
  const uint8_t* p = sm + tid * L::bytes;
  const f16_t d = *reinterpret_cast<const f16_t*>(p);
  f16_t bias;
  if constexpr (FMT == kQ4_0) {
    bias = static_cast<f16_t>(-8.0f * static_cast<float>(d));
  } else if constexpr (FMT == kQ4_1) {
    bias = *reinterpret_cast<const f16_t*>(p + 2);
  } else {
    bias = static_cast<f16_t>(-128.0f * static_cast<float>(d));
  }
  const uint8_t* q = p + L::header;
  uint32_t out[L::words];
  if constexpr (FMT == kQ8_0) {
    // int8 -> code + 128: flip the sign bit of every byte
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t lo = *reinterpret_cast<const uint16_t*>(q + 4 * i);
      const uint32_t hi = *reinterpret_cast<const uint16_t*>(q + 4 * i + 2);
      out[i] = (lo | (hi << 16)) ^ 0x80808080u;
    }
  } else {
    // byte j holds element j (low nibble) and element j + 16 (high nibble);
    // the packed stream wants element e at bit 4 e.  The quants start 2 bytes
    // into an 18-byte block (Q4_0), so they are read as halfwords; byte reads
    // (what the compiler makes of an indexed byte loop) ran this format at a
    // quarter of the rate of the other two.
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = *reinterpret_cast<const uint16_t*>(q + 4 * i);
      const uint32_t hi = *reinterpret_cast<const uint16_t*>(q + 4 * i + 2);
      w[i] = lo | (hi << 16);
    }
    // the four low nibbles of a word's bytes, packed into 16 bits
    auto squeeze = [](uint32_t v) {
      v &= 0x0f0f0f0fu;
      v = (v | (v >> 4)) & 0x00ff00ffu;
      return (v | (v >> 8)) & 0xffffu;
    };
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      out[i] = squeeze(w[2 * i]) | (squeeze(w[2 * i + 1]) << 16);
      out[2 + i] = squeeze(w[2 * i] >> 4) | (squeeze(w[2 * i + 1] >> 4) << 16);
    }
  }
  const size_t b = b0 + tid;
  uint4* dst = reinterpret_cast<uint4*>(wq + b * L::words);
  dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
  if constexpr (L::words == 8) {
    dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
  }
  scales[b] = d;
  biases[b] = bias;
}

template <int FMT>
int launch_repack(
    const void* blocks,
    uint32_t* wq,
    void* scales,
    void* biases,
    size_t n_blocks,
    hipStream_t s) {
  const size_t grid = (n_blocks + kRepackBlock - 1) / kRepackBlock;
  if (grid > 0x7fffffffu) {
    return fail(MLXROCM_UNSUPPORTED, "[gguf_repack] %zu blocks exceed the grid", n_blocks);
  }
  gguf_repack_kernel<FMT><<<static_cast<unsigned>(grid), kRepackBlock, 0, s>>>(
      static_cast<const uint8_t*>(blocks),
      wq,
      static_cast<f16_t*>(scales),
      static_cast<f16_t*>(biases),
      n_blocks);
  MLXROCM_HIP_TRY(hipGetLastError());
  return static_cast<int>(MLXROCM_OK);
}

} // namespace

} // namespace mlxrocm

extern "C" int mlxrocm_gguf_repack(
    const void* blocks,
    uint32_t* wq,
    void* scales,
    void* biases,
    size_t n_blocks,
    int ggml_type,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_gguf_repack");
  using namespace mlxrocm;
  if (ggml_type != MLXROCM_GGML_Q4_0 && ggml_type != MLXROCM_GGML_Q4_1 &&
      ggml_type != MLXROCM_GGML_Q8_0) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[gguf_repack] GGML type %d is not one of Q4_0 (2), Q4_1 (3), Q8_0 (8)",
        ggml_type);
  }
  if (n_blocks == 0) {
    return static_cast<int>(MLXROCM_OK);
  }
  if (blocks == nullptr || wq == nullptr || scales == nullptr || biases == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[gguf_repack] null pointer");
  }
  if ((reinterpret_cast<uintptr_t>(blocks) | reinterpret_cast<uintptr_t>(wq)) % 16 != 0) {
    return fail(
        MLXROCM_INVALID_ARGUMENT, "[gguf_repack] blocks and wq must be 16-byte aligned");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (ggml_type) {
    case MLXROCM_GGML_Q4_0:
      return launch_repack<kQ4_0>(blocks, wq, scales, biases, n_blocks, s);
    case MLXROCM_GGML_Q4_1:
      return launch_repack<kQ4_1>(blocks, wq, scales, biases, n_blocks, s);
    default:
      return launch_repack<kQ8_0>(blocks, wq, scales, biases, n_blocks, s);
  }
}
