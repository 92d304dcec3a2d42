// Device-side scalar/vector types and conversions for gfx950.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipattn {

typedef _Float16 half_t;
typedef __bf16 bf16_t;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

template <typename T>
struct Vec8;
template <>
struct Vec8<half_t> {
  typedef half8_t type;
};
template <>
struct Vec8<bf16_t> {
  typedef bf16x8_t type;
};

template <typename T>
__device__ __forceinline__ float to_float(T x) {
  return (float)x;
}

// Round-to-nearest-even conversions; for bf16 this is gfx950's hardware
// conversion, for fp16 v_cvt_f16_f32.
template <typename T>
__device__ __forceinline__ T from_float(float x) {
  return (T)x;
}

// Arithmetic in T with every result rounded to T, the way the reference's per-operator half / bfloat16
// arithmetic (and torch's CPU ops) round: no contraction into FMAs.
template <typename T>
__device__ __forceinline__ T mul_t(T a, T b) {
#pragma clang fp contract(off)
  return from_float<T>(to_float(a) * to_float(b));
}
template <typename T>
__device__ __forceinline__ T add_t(T a, T b) {
#pragma clang fp contract(off)
  return from_float<T>(to_float(a) + to_float(b));
}
template <typename T>
__device__ __forceinline__ T sub_t(T a, T b) {
#pragma clang fp contract(off)
  return from_float<T>(to_float(a) - to_float(b));
}

// A 16-byte load of data that a kernel reads once: with the non-temporal hint the line is not kept in the
// caches at the expense of data that is used again (or, in a purely streaming kernel, of the lines still on
// their way).  HA_NT_STREAM = 0 builds the plain load, for comparison.
#ifndef HA_NT_STREAM
#define HA_NT_STREAM 1
#endif
__device__ __forceinline__ uint4 load16_once(const void *p) {
#if HA_NT_STREAM
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  const v4u v = __builtin_nontemporal_load(static_cast<const v4u *>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
#else
  return *static_cast<const uint4 *>(p);
#endif
}

// The 16-byte store to match: data that nothing reads again soon.
__device__ __forceinline__ void store16_once(void *p, uint4 v) {
#if HA_NT_STREAM
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  v4u w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, static_cast<v4u *>(p));
#else
  *static_cast<uint4 *>(p) = v;
#endif
}

// Bit-pattern helpers for building MFMA operands out of 32-bit registers.
template <typename V, typename U>
__device__ __forceinline__ V bit_cast(const U &u) {
  static_assert(sizeof(V) == sizeof(U), "bit_cast size mismatch");
  V v;
  __builtin_memcpy(&v, &u, sizeof(V));
  return v;
}

// Sums over a wavefront and over the workgroup (every thread receives the result); the order of the additions
// is fixed by the thread numbers alone, so two kernels that hand these the same per-thread values get the same
// bits.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float block_sum(float v, float *smem /* >= 17 floats */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nwaves ? smem[lane] : 0.f;
    t = wave_sum(t);
    if (lane == 0) smem[16] = t;
  }
  __syncthreads();
  return smem[16];
}

}  // namespace hipattn
