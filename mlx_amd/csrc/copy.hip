// copy.hip -- element copies with dtype conversion and scalar fill: the data
// movement every eval_gpu body needs around the matmul kernels (making an input
// row-contiguous, converting scales/biases to the activation type, astype of
// the result).  Counterpart of copy_gpu_inplace / fill_gpu
// (mlx/backend/gpu/copy.h:14-51; the CUDA kernels are
// mlx/backend/cuda/copy/copy_contiguous.cu and copy_general*.cu).
//
// Both kernels are plain HBM streams: one 16-byte vector per lane on the
// narrower side when source and destination are contiguous and aligned, one
// element per lane with a div/mod walk over at most kMaxDims collapsed
// dimensions otherwise.  Conversions follow static_cast (round-to-nearest-even
// into the float types, truncation toward zero into the integer types, != 0
// into bool); complex64 converts to a real type by dropping the imaginary part
// and from one with a zero imaginary part.
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace mlxrocm {
namespace {

struct complex64 {
  float re;
  float im;
};
// Sixteen opaque bytes: the element of a same-type copy whose innermost runs
// are contiguous and aligned on both sides.
struct alignas(16) bytes16 {
  uint32_t w[4];
};

template <int DT> struct TypeOf;
template <> struct TypeOf<MLXROCM_FLOAT32> { using type = float; };
template <> struct TypeOf<MLXROCM_FLOAT16> { using type = f16_t; };
template <> struct TypeOf<MLXROCM_BFLOAT16> { using type = bf16_t; };
template <> struct TypeOf<MLXROCM_BOOL> { using type = bool; };
template <> struct TypeOf<MLXROCM_UINT8> { using type = uint8_t; };
template <> struct TypeOf<MLXROCM_UINT16> { using type = uint16_t; };
template <> struct TypeOf<MLXROCM_UINT32> { using type = uint32_t; };
template <> struct TypeOf<MLXROCM_UINT64> { using type = uint64_t; };
template <> struct TypeOf<MLXROCM_INT8> { using type = int8_t; };
template <> struct TypeOf<MLXROCM_INT16> { using type = int16_t; };
template <> struct TypeOf<MLXROCM_INT32> { using type = int32_t; };
template <> struct TypeOf<MLXROCM_INT64> { using type = int64_t; };
template <> struct TypeOf<MLXROCM_FLOAT64> { using type = double; };
template <> struct TypeOf<MLXROCM_COMPLEX64> { using type = complex64; };

constexpr int kNumDtypes = 14;
constexpr size_t kItemSize[kNumDtypes] = {4, 2, 2, 1, 1, 2, 4, 8, 1, 2, 4, 8, 8, 8};

template <typename T>
constexpr bool is_half_v = std::is_same_v<T, f16_t> || std::is_same_v<T, bf16_t>;

template <typename S, typename D>
__device__ __forceinline__ D convert(S v) {
  if constexpr (std::is_same_v<S, D>) {
    return v;
  } else if constexpr (std::is_same_v<S, complex64>) {
    if constexpr (std::is_same_v<D, bool>) {
      return v.re != 0.0f || v.im != 0.0f;
    } else {
      return convert<float, D>(v.re);
    }
  } else if constexpr (std::is_same_v<D, complex64>) {
    return complex64{convert<S, float>(v), 0.0f};
  } else if constexpr (std::is_same_v<D, bool>) {
    if constexpr (is_half_v<S>) {
      return static_cast<float>(v) != 0.0f;
    } else {
      return v != S(0);
    }
  } else if constexpr (is_half_v<S> && !std::is_floating_point_v<D>) {
    // 16-bit floats reach the integer types (and each other) through fp32,
    // which holds every one of their values.
    return convert<float, D>(static_cast<float>(v));
  } else if constexpr (is_half_v<D>) {
    // Every source reaches a 16-bit float through fp32.
    return static_cast<D>(static_cast<float>(v));
  } else {
    return static_cast<D>(v);
  }
}

template <typename T, int E>
struct alignas(sizeof(T) * E) Vec {
  T v[E];
};

template <typename S, typename D>
constexpr int vec_elems() {
  constexpr size_t narrow = sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D);
  constexpr int e = static_cast<int>(16 / narrow);
  return e > 8 ? 8 : e;
}

constexpr int kCopyThreads = 256;

// dst[i] = convert(src[i]) (or src[0] when SCALAR) for i < n; E elements per lane.
template <typename S, typename D, int E, bool SCALAR>
__global__ __launch_bounds__(kCopyThreads) void copy_contiguous_kernel(
    const S* __restrict__ src,
    D* __restrict__ dst,
    size_t n) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * kCopyThreads + threadIdx.x) * E;
  if (i >= n) {
    return;
  }
  if constexpr (SCALAR) {
    const D value = convert<S, D>(src[0]);
    if (E > 1 && i + E <= n) {
      Vec<D, E> out;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        out.v[e] = value;
      }
      *reinterpret_cast<Vec<D, E>*>(dst + i) = out;
    } else {
      for (size_t e = i; e < n && e < i + E; ++e) {
        dst[e] = value;
      }
    }
  } else {
    if (E > 1 && i + E <= n) {
      const Vec<S, E> in = *reinterpret_cast<const Vec<S, E>*>(src + i);
      Vec<D, E> out;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        out.v[e] = convert<S, D>(in.v[e]);
      }
      *reinterpret_cast<Vec<D, E>*>(dst + i) = out;
    } else {
      for (size_t e = i; e < n && e < i + E; ++e) {
        dst[e] = convert<S, D>(src[e]);
      }
    }
  }
}

constexpr int kMaxDims = 8;

struct StridedShape {
  int ndim;
  int64_t shape[kMaxDims];
  int64_t src_stride[kMaxDims];
  int64_t dst_stride[kMaxDims];
};

// One element per lane; IDX is uint32_t when every index fits.
template <typename S, typename D, typename IDX>
__global__ __launch_bounds__(kCopyThreads) void copy_strided_kernel(
    const S* __restrict__ src,
    D* __restrict__ dst,
    StridedShape a,
    size_t n) {
  const size_t linear = static_cast<size_t>(blockIdx.x) * kCopyThreads + threadIdx.x;
  if (linear >= n) {
    return;
  }
  IDX rest = static_cast<IDX>(linear);
  int64_t so = 0;
  int64_t dof = 0;
  for (int d = a.ndim - 1; d > 0; --d) {
    const IDX extent = static_cast<IDX>(a.shape[d]);
    const IDX q = rest / extent;
    const IDX c = rest - q * extent;
    so += static_cast<int64_t>(c) * a.src_stride[d];
    dof += static_cast<int64_t>(c) * a.dst_stride[d];
    rest = q;
  }
  so += static_cast<int64_t>(rest) * a.src_stride[0];
  dof += static_cast<int64_t>(rest) * a.dst_stride[0];
  dst[dof] = convert<S, D>(src[so]);
}

// A same-type copy whose source runs along another dimension than the last
// (a transpose): square tiles through LDS, read along the source's unit-stride
// dimension `jd`, written along the destination's (the last one).  A tile row is
// at least one 128-byte line (32 x 32 elements of four or eight bytes, 64 x 64 of
// two, 128 x 128 of one); rows are padded by one dword against bank conflicts.
// The other dimensions are a batch walked with div/mod per workgroup.
template <typename E>
constexpr int tile_width() {
  return sizeof(E) >= 4 ? 32 : static_cast<int>(128 / sizeof(E));
}

struct TransposeShape {
  int ndim;        // of the batch part
  int64_t extent_i;
  int64_t extent_j;
  int64_t src_stride_i; // elements; the source's stride along j is 1
  int64_t dst_stride_j; // elements; the destination's stride along i is 1
  int64_t batch_shape[kMaxDims];
  int64_t batch_src_stride[kMaxDims];
  int64_t batch_dst_stride[kMaxDims];
  int64_t tiles_i;
  int64_t tiles_j;
};

template <typename E>
__global__ __launch_bounds__(256) void transpose_tile_kernel(
    const E* __restrict__ src,
    E* __restrict__ dst,
    TransposeShape t) {
  constexpr int kTile = tile_width<E>();
  constexpr int kPad = sizeof(E) >= 4 ? 1 : static_cast<int>(4 / sizeof(E));
  constexpr int kRowsPerPass = 256 / kTile;
  __shared__ E tile[kTile][kTile + kPad];
  int64_t block = blockIdx.x;
  const int64_t tj = block % t.tiles_j;
  block /= t.tiles_j;
  const int64_t ti = block % t.tiles_i;
  int64_t rest = block / t.tiles_i;
  int64_t so = 0;
  int64_t dof = 0;
  for (int d = t.ndim - 1; d >= 0; --d) {
    const int64_t c = rest % t.batch_shape[d];
    rest /= t.batch_shape[d];
    so += c * t.batch_src_stride[d];
    dof += c * t.batch_dst_stride[d];
  }
  const int tx = threadIdx.x % kTile;
  const int ty = threadIdx.x / kTile;
  const int64_t i0 = ti * kTile;
  const int64_t j0 = tj * kTile;
#pragma unroll
  for (int r = 0; r < kTile; r += kRowsPerPass) {
    const int64_t i = i0 + ty + r;
    const int64_t j = j0 + tx;
    if (i < t.extent_i && j < t.extent_j) {
      tile[ty + r][tx] = src[so + i * t.src_stride_i + j];
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kTile; r += kRowsPerPass) {
    const int64_t j = j0 + ty + r;
    const int64_t i = i0 + tx;
    if (i < t.extent_i && j < t.extent_j) {
      dst[dof + j * t.dst_stride_j + i] = tile[tx][ty + r];
    }
  }
}

template <typename E>
int launch_transpose(const void* src, void* dst, const TransposeShape& t, size_t batch, hipStream_t stream) {
  const size_t blocks = static_cast<size_t>(t.tiles_i) * t.tiles_j * batch;
  if (blocks > 0x7fffffffull) {
    return fail(MLXROCM_UNSUPPORTED, "[copy] too many tiles for one launch");
  }
  transpose_tile_kernel<E><<<dim3(static_cast<unsigned>(blocks)), 256, 0, stream>>>(
      static_cast<const E*>(src), static_cast<E*>(dst), t);
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

bool valid_copy_dtype(int dt) {
  return dt >= 0 && dt < kNumDtypes;
}

// Calls f(TypeOf<dt>::type{}) for a runtime dtype code.
template <typename F>
int with_type(int dt, F&& f) {
  switch (dt) {
#define MLXROCM_CASE(code) \
  case code:               \
    return f(typename TypeOf<code>::type{});
    MLXROCM_CASE(MLXROCM_FLOAT32)
    MLXROCM_CASE(MLXROCM_FLOAT16)
    MLXROCM_CASE(MLXROCM_BFLOAT16)
    MLXROCM_CASE(MLXROCM_BOOL)
    MLXROCM_CASE(MLXROCM_UINT8)
    MLXROCM_CASE(MLXROCM_UINT16)
    MLXROCM_CASE(MLXROCM_UINT32)
    MLXROCM_CASE(MLXROCM_UINT64)
    MLXROCM_CASE(MLXROCM_INT8)
    MLXROCM_CASE(MLXROCM_INT16)
    MLXROCM_CASE(MLXROCM_INT32)
    MLXROCM_CASE(MLXROCM_INT64)
    MLXROCM_CASE(MLXROCM_FLOAT64)
    MLXROCM_CASE(MLXROCM_COMPLEX64)
#undef MLXROCM_CASE
    default:
      return fail(MLXROCM_INVALID_ARGUMENT, "[copy] unknown dtype %d", dt);
  }
}

constexpr size_t kMaxBlocks = 0x7fffffffull;

template <typename S, typename D>
int launch_contiguous(
    const void* src, void* dst, size_t n, bool scalar, hipStream_t stream) {
  constexpr int E = vec_elems<S, D>();
  const bool aligned =
      (scalar || reinterpret_cast<uintptr_t>(src) % (sizeof(S) * E) == 0) &&
      reinterpret_cast<uintptr_t>(dst) % (sizeof(D) * E) == 0;
  const S* s = static_cast<const S*>(src);
  D* d = static_cast<D*>(dst);
  const size_t per_block = static_cast<size_t>(kCopyThreads) * (aligned ? E : 1);
  const size_t blocks = (n + per_block - 1) / per_block;
  if (blocks > kMaxBlocks) {
    return fail(MLXROCM_UNSUPPORTED, "[copy] %zu elements exceed one launch", n);
  }
  const dim3 grid(static_cast<unsigned>(blocks));
  if (aligned && scalar) {
    copy_contiguous_kernel<S, D, E, true><<<grid, kCopyThreads, 0, stream>>>(s, d, n);
  } else if (aligned) {
    copy_contiguous_kernel<S, D, E, false><<<grid, kCopyThreads, 0, stream>>>(s, d, n);
  } else if (scalar) {
    copy_contiguous_kernel<S, D, 1, true><<<grid, kCopyThreads, 0, stream>>>(s, d, n);
  } else {
    copy_contiguous_kernel<S, D, 1, false><<<grid, kCopyThreads, 0, stream>>>(s, d, n);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

template <typename S, typename D>
int launch_strided(
    const void* src, void* dst, const StridedShape& a, size_t n, bool wide, hipStream_t stream) {
  const size_t blocks = (n + kCopyThreads - 1) / kCopyThreads;
  if (blocks > kMaxBlocks) {
    return fail(MLXROCM_UNSUPPORTED, "[copy] %zu elements exceed one launch", n);
  }
  const dim3 grid(static_cast<unsigned>(blocks));
  const S* s = static_cast<const S*>(src);
  D* d = static_cast<D*>(dst);
  if (wide) {
    copy_strided_kernel<S, D, uint64_t><<<grid, kCopyThreads, 0, stream>>>(s, d, a, n);
  } else {
    copy_strided_kernel<S, D, uint32_t><<<grid, kCopyThreads, 0, stream>>>(s, d, a, n);
  }
  MLXROCM_HIP_TRY(hipGetLastError());
  return MLXROCM_OK;
}

} // namespace
} // namespace mlxrocm

using namespace mlxrocm;

extern "C" size_t mlxrocm_dtype_size(int dtype) {
  return valid_copy_dtype(dtype) ? kItemSize[dtype] : 0;
}

extern "C" int mlxrocm_copy_contiguous(
    const void* src,
    int src_dtype,
    void* dst,
    int dst_dtype,
    size_t n,
    int broadcast_scalar,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_copy_contiguous");
  if (!valid_copy_dtype(src_dtype) || !valid_copy_dtype(dst_dtype)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT, "[copy] unknown dtype %d -> %d", src_dtype, dst_dtype);
  }
  if (n == 0) {
    return MLXROCM_OK;
  }
  if (src == nullptr || dst == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[copy] null pointer");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (src_dtype == dst_dtype && !broadcast_scalar) {
    // Same type, same layout: the copy engine's path.
    MLXROCM_HIP_TRY(hipMemcpyAsync(
        dst, src, n * kItemSize[src_dtype], hipMemcpyDeviceToDevice, s));
    return MLXROCM_OK;
  }
  return with_type(src_dtype, [&](auto st) {
    using S = decltype(st);
    return with_type(dst_dtype, [&](auto dt) {
      using D = decltype(dt);
      return launch_contiguous<S, D>(src, dst, n, broadcast_scalar != 0, s);
    });
  });
}

extern "C" int mlxrocm_copy_strided(
    const void* src,
    int src_dtype,
    const int64_t* src_strides,
    void* dst,
    int dst_dtype,
    const int64_t* dst_strides,
    int ndim,
    const int64_t* shape,
    mlxrocm_stream_t stream) {
  mlxrocm::ApiRange api_range("mlxrocm_copy_strided");
  if (!valid_copy_dtype(src_dtype) || !valid_copy_dtype(dst_dtype)) {
    return fail(
        MLXROCM_INVALID_ARGUMENT, "[copy] unknown dtype %d -> %d", src_dtype, dst_dtype);
  }
  if (ndim < 0 || (ndim > 0 && (shape == nullptr || src_strides == nullptr))) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[copy] shape and source strides are required");
  }
  size_t n = 1;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] < 0) {
      return fail(MLXROCM_INVALID_ARGUMENT, "[copy] negative extent");
    }
    n *= static_cast<size_t>(shape[d]);
  }
  if (n == 0) {
    return MLXROCM_OK;
  }
  if (src == nullptr || dst == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[copy] null pointer");
  }

  // Row-contiguous destination strides when none are given.
  int64_t dense[64];
  if (ndim > 64) {
    return fail(MLXROCM_UNSUPPORTED, "[copy] %d dimensions", ndim);
  }
  if (dst_strides == nullptr) {
    int64_t run = 1;
    for (int d = ndim - 1; d >= 0; --d) {
      dense[d] = run;
      run *= shape[d];
    }
    dst_strides = dense;
  }

  // Drop extent-1 dimensions and merge neighbours that both sides walk as one
  // run (outer stride == inner stride * inner extent).
  StridedShape a;
  a.ndim = 0;
  int64_t cs[64], css[64], cds[64];
  int nd = 0;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] == 1) {
      continue;
    }
    if (nd > 0 && css[nd - 1] == src_strides[d] * shape[d] &&
        cds[nd - 1] == dst_strides[d] * shape[d]) {
      cs[nd - 1] *= shape[d];
      css[nd - 1] = src_strides[d];
      cds[nd - 1] = dst_strides[d];
    } else {
      cs[nd] = shape[d];
      css[nd] = src_strides[d];
      cds[nd] = dst_strides[d];
      ++nd;
    }
  }
  if (nd == 0) { // a single element
    cs[0] = 1;
    css[0] = 0;
    cds[0] = 0;
    nd = 1;
  }
  if (nd > kMaxDims) {
    return fail(
        MLXROCM_UNSUPPORTED,
        "[copy] %d dimensions remain after merging; at most %d are supported",
        nd,
        kMaxDims);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (nd == 1 && css[0] == 1 && cds[0] == 1) {
    return mlxrocm_copy_contiguous(src, src_dtype, dst, dst_dtype, n, 0, stream);
  }
  if (nd == 1 && css[0] == 0 && cds[0] == 1) {
    return mlxrocm_copy_contiguous(src, src_dtype, dst, dst_dtype, n, 1, stream);
  }
  // A same-type copy that the destination walks along its last dimension while
  // the source runs along another one: tiled transpose.
  if (src_dtype == dst_dtype && nd >= 2 && cds[nd - 1] == 1 && css[nd - 1] != 1 &&
      cs[nd - 1] >= 8) {
    int jd = -1;
    for (int d = nd - 2; d >= 0; --d) {
      if (css[d] == 1 && cs[d] >= 8) {
        jd = d;
        break;
      }
    }
    bool positive = true;
    for (int d = 0; d < nd; ++d) {
      positive = positive && css[d] >= 0 && cds[d] >= 0;
    }
    if (jd >= 0 && positive) {
      TransposeShape t;
      t.extent_i = cs[nd - 1];
      t.extent_j = cs[jd];
      t.src_stride_i = css[nd - 1];
      t.dst_stride_j = cds[jd];
      const int64_t tile = kItemSize[src_dtype] >= 4 ? 32 : 128 / static_cast<int64_t>(kItemSize[src_dtype]);
      t.tiles_i = (t.extent_i + tile - 1) / tile;
      t.tiles_j = (t.extent_j + tile - 1) / tile;
      t.ndim = 0;
      size_t batch = 1;
      for (int d = 0; d < nd - 1; ++d) {
        if (d == jd) {
          continue;
        }
        t.batch_shape[t.ndim] = cs[d];
        t.batch_src_stride[t.ndim] = css[d];
        t.batch_dst_stride[t.ndim] = cds[d];
        batch *= static_cast<size_t>(cs[d]);
        ++t.ndim;
      }
      for (int d = t.ndim; d < kMaxDims; ++d) {
        t.batch_shape[d] = 1;
        t.batch_src_stride[d] = 0;
        t.batch_dst_stride[d] = 0;
      }
      switch (kItemSize[src_dtype]) {
        case 1:
          return launch_transpose<uint8_t>(src, dst, t, batch, s);
        case 2:
          return launch_transpose<uint16_t>(src, dst, t, batch, s);
        case 4:
          return launch_transpose<uint32_t>(src, dst, t, batch, s);
        default:
          return launch_transpose<uint64_t>(src, dst, t, batch, s);
      }
    }
  }
  // A same-type copy moves bytes: when both sides walk the innermost dimension
  // contiguously, widen the element to 16, 8 or 4 bytes (fewer, wider accesses)
  // as far as extents, strides and base addresses allow.
  size_t item = kItemSize[src_dtype];
  int wide_code = -1; // 16 bytes when -2
  if (src_dtype == dst_dtype && css[nd - 1] == 1 && cds[nd - 1] == 1) {
    for (size_t bytes : {size_t(16), size_t(8), size_t(4)}) {
      if (bytes <= item) {
        break;
      }
      const int64_t v = static_cast<int64_t>(bytes / item);
      bool ok = cs[nd - 1] % v == 0 && reinterpret_cast<uintptr_t>(src) % bytes == 0 &&
          reinterpret_cast<uintptr_t>(dst) % bytes == 0;
      for (int d = 0; ok && d < nd - 1; ++d) {
        ok = css[d] % v == 0 && cds[d] % v == 0;
      }
      if (ok) {
        cs[nd - 1] /= v;
        for (int d = 0; d < nd - 1; ++d) {
          css[d] /= v;
          cds[d] /= v;
        }
        n /= static_cast<size_t>(v);
        wide_code = bytes == 16 ? -2 : (bytes == 8 ? MLXROCM_UINT64 : MLXROCM_UINT32);
        break;
      }
    }
  }
  a.ndim = nd;
  for (int d = 0; d < kMaxDims; ++d) {
    a.shape[d] = d < nd ? cs[d] : 1;
    a.src_stride[d] = d < nd ? css[d] : 0;
    a.dst_stride[d] = d < nd ? cds[d] : 0;
  }
  const bool wide = n > 0xffffffffull;
  if (wide_code == -2) {
    return launch_strided<bytes16, bytes16>(src, dst, a, n, wide, s);
  }
  if (wide_code >= 0) {
    src_dtype = dst_dtype = wide_code;
  }
  return with_type(src_dtype, [&](auto st) {
    using S = decltype(st);
    return with_type(dst_dtype, [&](auto dt) {
      using D = decltype(dt);
      return launch_strided<S, D>(src, dst, a, n, wide, s);
    });
  });
}
