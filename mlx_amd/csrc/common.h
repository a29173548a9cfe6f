// common.h -- shared definitions of the gfx950 affine-quantization kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mlx_rocm_qmm.h"

namespace mlxrocm {

using f16_t = _Float16;
using bf16_t = __bf16;

constexpr int kWaveSize = 64;

// Thread-local error slot behind mlxrocm_last_error().
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t err, const char* what);

// A roctx range around one entry point of the C ABI, so that a profiler's
// marker trace shows which operator call a kernel belongs to.  The marker
// library is looked up at the first call; without it the range is a no-op.
class ApiRange {
 public:
  explicit ApiRange(const char* name);
  ~ApiRange();
  ApiRange(const ApiRange&) = delete;
  ApiRange& operator=(const ApiRange&) = delete;

 private:
  bool open_;
};

// Rehearsal of a call: the entry point walks its whole host path -- argument
// checks, kernel choice, workspace claims against the size it was given -- but
// every launcher records its name (and the parameters that shape its launch)
// instead of launching.  Nothing touches the device, so the choice of kernels
// can be listed and tested without a GPU (mlxrocm_qmm_plan).  Thread-local.
class RehearsalScope {
 public:
  RehearsalScope(char* buf, size_t cap);
  ~RehearsalScope();
  RehearsalScope(const RehearsalScope&) = delete;
  RehearsalScope& operator=(const RehearsalScope&) = delete;
};
bool rehearsing();
// Appends "name" to the rehearsal's record ("a+b+c"); returns MLXROCM_OK.
int note_launch(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
// At the top of a launcher: in a rehearsal, record and return.
#define MLXROCM_REHEARSE(...)                    \
  do {                                           \
    if (::mlxrocm::rehearsing()) {               \
      return ::mlxrocm::note_launch(__VA_ARGS__); \
    }                                            \
  } while (0)

#define MLXROCM_HIP_TRY(expr)                    \
  do {                                           \
    hipError_t err__ = (expr);                   \
    if (err__ != hipSuccess) {                   \
      return ::mlxrocm::hip_fail(err__, #expr);  \
    }                                            \
  } while (0)

inline bool valid_bits(int bits) {
  return bits == 2 || bits == 3 || bits == 4 || bits == 5 || bits == 6 ||
      bits == 8;
}
inline bool valid_group(int gs) {
  return gs == 32 || gs == 64 || gs == 128;
}
inline bool valid_dtype(int dt) {
  return dt == MLXROCM_FLOAT32 || dt == MLXROCM_FLOAT16 ||
      dt == MLXROCM_BFLOAT16;
}
inline size_t dtype_size(int dt) {
  return dt == MLXROCM_FLOAT32 ? 4 : 2;
}

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);
}

// Value of one arithmetic result rounded to T and widened again.
template <typename T>
__device__ __forceinline__ float round_to(float v) {
  return static_cast<float>(static_cast<T>(v));
}
template <>
__device__ __forceinline__ float round_to<float>(float v) {
  return v;
}

// 8 consecutive elements of T as floats (16-byte or 2x16-byte vector loads).
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
  if constexpr (sizeof(T) == 4) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    union {
      uint4 u;
      T e[8];
    } raw;
    raw.u = *reinterpret_cast<const uint4*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = to_f32(raw.e[i]);
    }
  }
}

template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&v)[8]) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
    union {
      uint4 u;
      T e[8];
    } raw;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      raw.e[i] = from_f32<T>(v[i]);
    }
    *reinterpret_cast<uint4*>(p) = raw.u;
  }
}

// The 8*BITS bits that hold codes [8u, 8u+8) of a packed stream, as one
// 64-bit little-endian value.  `p` is the byte address of unit 0; unit u
// starts at byte u*BITS, which is only guaranteed 1-byte aligned for
// 3/5/6-bit codes.
template <int BITS>
__device__ __forceinline__ uint64_t load_unit(const uint8_t* p, size_t u) {
  const uint8_t* q = p + u * BITS;
  if constexpr (BITS == 2) {
    return *reinterpret_cast<const uint16_t*>(q);
  } else if constexpr (BITS == 4) {
    return *reinterpret_cast<const uint32_t*>(q);
  } else if constexpr (BITS == 8) {
    const uint2 v = *reinterpret_cast<const uint2*>(q);
    return static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32);
  } else if constexpr (BITS == 6) {
    // 6 bytes, always 2-byte aligned
    const uint16_t* h = reinterpret_cast<const uint16_t*>(q);
    return static_cast<uint64_t>(h[0]) | (static_cast<uint64_t>(h[1]) << 16) |
        (static_cast<uint64_t>(h[2]) << 32);
  } else {
    uint64_t v = 0;
#pragma unroll
    for (int i = 0; i < BITS; ++i) {
      v |= static_cast<uint64_t>(q[i]) << (8 * i);
    }
    return v;
  }
}

template <int BITS>
__device__ __forceinline__ uint32_t unit_code(uint64_t unit, int i) {
  return static_cast<uint32_t>(unit >> (i * BITS)) & ((1u << BITS) - 1u);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    v += __shfl_xor(v, off, 64);
  }
  return v;
}

// Dispatch helpers: run `fn` with compile-time element type / bits / group.
template <typename F>
inline int dispatch_dtype(int dtype, F&& fn) {
  switch (dtype) {
    case MLXROCM_FLOAT32:
      return fn(float{});
    case MLXROCM_FLOAT16:
      return fn(f16_t{});
    case MLXROCM_BFLOAT16:
      return fn(bf16_t{});
    default:
      return fail(MLXROCM_INVALID_ARGUMENT, "unknown dtype %d", dtype);
  }
}

template <int V>
struct IntC {
  static constexpr int value = V;
};

template <typename F>
inline int dispatch_bits(int bits, F&& fn) {
  switch (bits) {
    case 2:
      return fn(IntC<2>{});
    case 3:
      return fn(IntC<3>{});
    case 4:
      return fn(IntC<4>{});
    case 5:
      return fn(IntC<5>{});
    case 6:
      return fn(IntC<6>{});
    case 8:
      return fn(IntC<8>{});
    default:
      return fail(
          MLXROCM_INVALID_ARGUMENT,
          "quantization bits must be 2, 3, 4, 5, 6 or 8 (got %d)",
          bits);
  }
}

template <typename F>
inline int dispatch_group(int gs, F&& fn) {
  switch (gs) {
    case 32:
      return fn(IntC<32>{});
    case 64:
      return fn(IntC<64>{});
    case 128:
      return fn(IntC<128>{});
    default:
      return fail(
          MLXROCM_INVALID_ARGUMENT,
          "quantization group size must be 32, 64 or 128 (got %d)",
          gs);
  }
}

} // namespace mlxrocm
