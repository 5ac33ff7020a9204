// Measurement aids for bench.py (libmbx_probe.so): an MFMA-only loop that shows what the matrix cores sustain on
// given operand values.  Not linked into libmbx.so.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mbx_probe.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// 4 x 4 accumulator tiles of 32 x 32 per wave (256 accumulator registers per lane, as in the grouped GEMM's main loop)
__global__ void __launch_bounds__(256) mfma_loop_32x32x16(const u32x4* __restrict__ in, int64_t n, int iters,
                                                          float* __restrict__ sink, int64_t* __restrict__ clocks) {
  u32x4 a[4], b[4];
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = in[(t * 8 + i) % n];
    b[i] = in[(t * 8 + 4 + i) % n];
  }
  f32x16 c[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][j][r] = 0.f;
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        c[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]), __builtin_bit_cast(bf16x8_t, b[j]),
                                                          c[i][j], 0, 0, 0);
  }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += c[i][j][0] + c[i][j][7];
  sink[t] = s;
  if (t == 0) {
    clocks[0] = t1 - t0;
    clocks[1] = w1 - w0;
  }
}

// the same amount of work per iteration from 16 x 16 x 32 instructions: 64 accumulator tiles of 16 x 16 (8 x 8), i.e.
// the same 256 accumulator registers, with 8 + 8 operand fragments
__global__ void __launch_bounds__(256) mfma_loop_16x16x32(const u32x4* __restrict__ in, int64_t n, int iters,
                                                          float* __restrict__ sink, int64_t* __restrict__ clocks) {
  u32x4 a[8], b[8];
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = in[(t * 16 + i) % n];
    b[i] = in[(t * 16 + 8 + i) % n];
  }
  f32x4 c[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) c[i][j][r] = 0.f;
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[i]), __builtin_bit_cast(bf16x8_t, b[j]),
                                                          c[i][j], 0, 0, 0);
  }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) s += c[i][j][0] + c[i][j][3];
  sink[t] = s;
  if (t == 0) {
    clocks[0] = t1 - t0;
    clocks[1] = w1 - w0;
  }
}

}  // namespace

extern "C" int mbx_probe_mfma(const void* operands, int64_t n_vec16, int kind, int blocks, int iters, float* sink,
                              int64_t* clocks, void* stream) {
  if (!operands || n_vec16 <= 0 || blocks <= 0 || iters < 0 || !sink || !clocks || (kind != 0 && kind != 1)) return -1;
  hipStream_t s = (hipStream_t)stream;
  if (kind == 0) mfma_loop_32x32x16<<<(unsigned)blocks, 256, 0, s>>>((const u32x4*)operands, n_vec16, iters, sink, clocks);
  else mfma_loop_16x16x32<<<(unsigned)blocks, 256, 0, s>>>((const u32x4*)operands, n_vec16, iters, sink, clocks);
  return (int)hipGetLastError();
}
