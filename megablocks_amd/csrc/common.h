// Shared helpers for the libmbx kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mbx.h"

namespace mbx {

constexpr int kWave = 64;

#define MBX_HIP_CHECK(expr)                  \
  do {                                       \
    hipError_t e_ = (expr);                  \
    if (e_ != hipSuccess) return (int)e_;    \
  } while (0)

// Returns the launch status of the kernel(s) just enqueued.
static inline int launch_status() { return (int)hipGetLastError(); }

static inline hipStream_t as_stream(mbx_stream_t s) { return (hipStream_t)s; }

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- storage <-> fp32 conversions (round-to-nearest-even, like torch) ----
typedef uint16_t bf16_t;  // raw bits
typedef _Float16 f16_t;

__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);   // v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN
}

template <int DT> struct Elem;
template <> struct Elem<MBX_BF16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float to_f32(type v) { return bf16_to_f32(v); }
  static __device__ __forceinline__ type from_f32(float f) { return f32_to_bf16(f); }
};
template <> struct Elem<MBX_F16> {
  typedef _Float16 type;
  static __device__ __forceinline__ float to_f32(type v) { return (float)v; }
  static __device__ __forceinline__ type from_f32(float f) { return (_Float16)f; }
};
template <> struct Elem<MBX_F32> {
  typedef float type;
  static __device__ __forceinline__ float to_f32(type v) { return v; }
  static __device__ __forceinline__ type from_f32(float f) { return f; }
};

static inline int dtype_bytes(int dtype) { return dtype == MBX_F32 ? 4 : 2; }
static inline int itype_bytes(int itype) { return itype == MBX_I16 ? 2 : (itype == MBX_I32 ? 4 : 8); }

// Reads element i of an array of runtime dtype as fp32 (used for the per-row router weight).
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dtype) {
  if (dtype == MBX_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
  if (dtype == MBX_F16) return (float)((const _Float16*)p)[i];
  return ((const float*)p)[i];
}

// ---- wave64 primitives ----
__device__ __forceinline__ int lane_id() { return __lane_id(); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Inclusive prefix sum across the 64 lanes of a wave.
template <typename T>
__device__ __forceinline__ T wave_inclusive_scan(T v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    T o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  return v;
}

// First e in [0, n) with bins[e] > r (bins inclusive cumsum, non-decreasing); n if none.
__device__ __forceinline__ int upper_bound_i32(const int32_t* __restrict__ bins, int n, int r) {
  int lo = 0, hi = n;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (bins[mid] > r) hi = mid; else lo = mid + 1;
  }
  return lo;
}

}  // namespace mbx
