// mfma_loads.h -- global loads issued behind the compiler's back, shared by the
// prefill tile kernels.
#pragma once

#include "common.h"

namespace mlxrocm {

namespace {

// ---- global loads issued behind the compiler's back --------------------------
// The K loop keeps loads of three kinds in flight at once: the direct-to-LDS
// loads of x (needed two barriers later), and the packed W words with their
// scale and bias (needed after the next barrier).  The compiler would wait for
// every outstanding direct-to-LDS load before each LDS read (it cannot tell
// which LDS bytes they write), and any wait it inserted for the W words would
// also wait for the younger x loads (vmcnt completes in order).  So all loads
// of the loop are inline assembly, whose results the compiler believes ready at
// once, and the loop waits for them itself, twice per step.  Right before the
// barrier, a wait that leaves only the step's own loads in flight (the W words
// fetched in slot 0 and the four x loads): the x loads of the step before have
// then landed.  At the end of the step `s_waitcnt vmcnt(4)`: the W words are
// older than the four x loads, so they have arrived -- a whole step after they
// were asked for -- and the x loads stay in flight.  Nothing may read a
// RawWords / raw value between its load and that second wait; every slot of
// the loop ends in a scheduling barrier, so no use moves up.
typedef uint32_t raw_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t raw_u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t raw_u32x4 __attribute__((ext_vector_type(4)));


// K dwords (K = 1..4) exactly as one load instruction fills them: the inline
// assembly writes the tuple itself, so no copy of a half-arrived value exists.
template <int K>
struct RawTuple;
template <>
struct RawTuple<1> {
  uint32_t v;
  template <int OFF>
  __device__ __forceinline__ void load(uint32_t voff, const void* sbase) {
    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF));
  }
  __device__ __forceinline__ uint32_t get(int) const { return v; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(v)); }
};
template <>
struct RawTuple<2> {
  raw_u32x2 v;
  template <int OFF>
  __device__ __forceinline__ void load(uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF));
  }
  __device__ __forceinline__ uint32_t get(int j) const { return v[j]; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(v)); }
};
template <>
struct RawTuple<3> {
  raw_u32x3 v;
  template <int OFF>
  __device__ __forceinline__ void load(uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx3 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF));
  }
  __device__ __forceinline__ uint32_t get(int j) const { return v[j]; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(v)); }
};
template <>
struct RawTuple<4> {
  raw_u32x4 v;
  template <int OFF>
  __device__ __forceinline__ void load(uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF));
  }
  __device__ __forceinline__ uint32_t get(int j) const { return v[j]; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(v)); }
};
template <>
struct RawTuple<0> {
  template <int OFF>
  __device__ __forceinline__ void load(uint32_t, const void*) {}
  __device__ __forceinline__ uint32_t get(int) const { return 0; }
  __device__ __forceinline__ void pin() {}
};

// N consecutive dwords (N = 1..8) as the one or two register tuples the loads
// fill.  pin() marks the place from which the values may be read: it goes right
// behind the wait that covers the loads, and the compiler treats it as the
// definition of the registers.
template <int N>
struct RawWords {
  static constexpr int kA = N >= 4 ? 4 : N; // dwords of the first load
  static constexpr int kB = N - kA;         // of the second (0..4)
  RawTuple<kA> a;
  RawTuple<kB> b;
  // dwords at sbase + voff (a uniform 64-bit base plus a per-lane byte offset)
  __device__ __forceinline__ void load(uint32_t voff, const void* sbase) {
    a.template load<0>(voff, sbase);
    b.template load<16>(voff, sbase);
  }
  __device__ __forceinline__ uint32_t get(int j) const {
    return j < 4 ? a.get(j) : b.get(j - 4);
  }
  __device__ __forceinline__ void pin() {
    a.pin();
    b.pin();
  }
};

// One scale or bias value as loaded: 16 bits in the low half, or a float.
template <typename TS>
__device__ __forceinline__ void raw_load_value(uint32_t& v, uint32_t voff, const void* sbase) {
  if constexpr (sizeof(TS) == 2) {
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase));
  } else {
    asm volatile("global_load_dword %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase));
  }
}
template <typename TS>
__device__ __forceinline__ float raw_value(uint32_t v) {
  if constexpr (sizeof(TS) == 2) {
    return to_f32(__builtin_bit_cast(TS, static_cast<uint16_t>(v)));
  } else {
    return __uint_as_float(v);
  }
}

} // namespace

} // namespace mlxrocm
