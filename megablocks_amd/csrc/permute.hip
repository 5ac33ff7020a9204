// Token permutation kernels: gather into expert-major order, fused weighted top-k combine
// back to token order, router-weight gradient, and the capacity-binned variants.
// HBM-bound row copies: one wave per row, 128-bit loads and stores when the row is a
// multiple of 16 bytes and the buffers are 16-byte aligned.
#include "common.h"

#include <mutex>

namespace mbx {
namespace {

constexpr int kRowThreads = 256;
constexpr int kRowWaves = kRowThreads / kWave;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int DT> struct Vec16 {  // 16 bytes of storage <-> fp32 lanes
  static constexpr int kElems = 16 / (int)sizeof(typename Elem<DT>::type);
  static __device__ __forceinline__ void unpack(const u32x4& v, float* f) {
    if (DT == MBX_F32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint16_t lo = (uint16_t)(v[i] & 0xffffu), hi = (uint16_t)(v[i] >> 16);
        if (DT == MBX_BF16) { f[2 * i] = bf16_to_f32(lo); f[2 * i + 1] = bf16_to_f32(hi); }
        else { f[2 * i] = (float)__builtin_bit_cast(_Float16, lo); f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, hi); }
      }
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 v;
    if (DT == MBX_F32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint16_t lo, hi;
        if (DT == MBX_BF16) { lo = f32_to_bf16(f[2 * i]); hi = f32_to_bf16(f[2 * i + 1]); }
        else { lo = __builtin_bit_cast(uint16_t, (_Float16)f[2 * i]); hi = __builtin_bit_cast(uint16_t, (_Float16)f[2 * i + 1]); }
        v[i] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
    }
    return v;
  }
};

// dst[0:hidden] = round(src * scale) (or a plain copy), by one wave.
template <int DT, bool VEC>
__device__ __forceinline__ void wave_copy_row(const typename Elem<DT>::type* __restrict__ src,
                                              typename Elem<DT>::type* __restrict__ dst, int hidden,
                                              bool scaled, float scale) {
  const int lane = lane_id();
  if (VEC) {
    constexpr int E = Vec16<DT>::kElems;
    const int nvec = hidden / E;
    const u32x4* s = (const u32x4*)src;
    u32x4* d = (u32x4*)dst;
    if (!scaled) {
      int c = lane;
      for (; c + 3 * kWave < nvec; c += 4 * kWave) {
        const u32x4 v0 = s[c], v1 = s[c + kWave], v2 = s[c + 2 * kWave], v3 = s[c + 3 * kWave];
        d[c] = v0; d[c + kWave] = v1; d[c + 2 * kWave] = v2; d[c + 3 * kWave] = v3;
      }
      for (; c < nvec; c += kWave) d[c] = s[c];
    } else {
      auto scaled_vec = [&](const u32x4& v) {
        float f[E];
        Vec16<DT>::unpack(v, f);
#pragma unroll
        for (int i = 0; i < E; ++i) f[i] *= scale;
        return Vec16<DT>::pack(f);
      };
      int c = lane;
      for (; c + 3 * kWave < nvec; c += 4 * kWave) {
        const u32x4 v0 = s[c], v1 = s[c + kWave], v2 = s[c + 2 * kWave], v3 = s[c + 3 * kWave];
        d[c] = scaled_vec(v0); d[c + kWave] = scaled_vec(v1); d[c + 2 * kWave] = scaled_vec(v2); d[c + 3 * kWave] = scaled_vec(v3);
      }
      for (; c < nvec; c += kWave) d[c] = scaled_vec(s[c]);
    }
  } else {
    for (int c = lane; c < hidden; c += kWave)
      dst[c] = scaled ? Elem<DT>::from_f32(Elem<DT>::to_f32(src[c]) * scale) : src[c];
  }
}

template <int DT, bool VEC>
__device__ __forceinline__ void wave_zero_row(typename Elem<DT>::type* __restrict__ dst, int hidden) {
  const int lane = lane_id();
  if (VEC) {
    const int nvec = hidden / Vec16<DT>::kElems;
    u32x4* d = (u32x4*)dst;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int c = lane; c < nvec; c += kWave) d[c] = z;
  } else {
    for (int c = lane; c < hidden; c += kWave) dst[c] = Elem<DT>::from_f32(0.f);
  }
}

template <int DT, bool VEC>
__device__ __forceinline__ float wave_dot_row(const typename Elem<DT>::type* __restrict__ a,
                                              const typename Elem<DT>::type* __restrict__ b, int hidden) {
  const int lane = lane_id();
  float acc = 0.f;
  if (VEC) {
    constexpr int E = Vec16<DT>::kElems;
    const int nvec = hidden / E;
    const u32x4* av = (const u32x4*)a;
    const u32x4* bv = (const u32x4*)b;
    auto dot_vec = [&](const u32x4& va, const u32x4& vb) {
      float fa[E], fb[E];
      Vec16<DT>::unpack(va, fa);
      Vec16<DT>::unpack(vb, fb);
#pragma unroll
      for (int i = 0; i < E; ++i) acc += fa[i] * fb[i];
    };
    int c = lane;
    for (; c + 3 * kWave < nvec; c += 4 * kWave) {   // a: rows read once (non-temporal); b: rows other slots read again
      const u32x4 a0 = __builtin_nontemporal_load(av + c), a1 = __builtin_nontemporal_load(av + c + kWave);
      const u32x4 a2 = __builtin_nontemporal_load(av + c + 2 * kWave), a3 = __builtin_nontemporal_load(av + c + 3 * kWave);
      const u32x4 b0 = bv[c], b1 = bv[c + kWave], b2 = bv[c + 2 * kWave], b3 = bv[c + 3 * kWave];
      dot_vec(a0, b0); dot_vec(a1, b1); dot_vec(a2, b2); dot_vec(a3, b3);
    }
    for (; c < nvec; c += kWave) dot_vec(__builtin_nontemporal_load(av + c), bv[c]);
  } else {
    for (int c = lane; c < hidden; c += kWave) acc += Elem<DT>::to_f32(a[c]) * Elem<DT>::to_f32(b[c]);
  }
  return wave_sum(acc);
}

// Sorted slot feeding output row `row` of the expert-major buffer, or -1 for a padding row.
__device__ __forceinline__ int slot_of_row(int row, const int32_t* __restrict__ bins,
                                           const int32_t* __restrict__ padded_bins, int num_bins, int n_slots) {
  if (padded_bins == nullptr) return row < n_slots ? row : -1;
  const int e = upper_bound_i32(padded_bins, num_bins, row);
  if (e >= num_bins) return -1;
  const int pstart = e > 0 ? padded_bins[e - 1] : 0;
  const int start = e > 0 ? bins[e - 1] : 0;
  const int pos = start + (row - pstart);
  return (pos < bins[e] && pos < n_slots) ? pos : -1;
}

// ------------------------------------------------------------------ gather
template <int DT, bool VEC>
__global__ void __launch_bounds__(kRowThreads)
gather_kernel(const void* __restrict__ x_, int64_t tokens, int hidden, int top_k, const int32_t* __restrict__ indices,
              const int32_t* __restrict__ bins, const int32_t* __restrict__ padded_bins, int num_bins,
              const void* __restrict__ weights, int w_dtype, void* __restrict__ out_, int64_t out_rows) {
  typedef typename Elem<DT>::type E;
  const E* x = (const E*)x_;
  E* out = (E*)out_;
  const int n_slots = (int)(tokens * top_k);
  const int wave = threadIdx.x / kWave;
  for (int64_t row = (int64_t)blockIdx.x * kRowWaves + wave; row < out_rows; row += (int64_t)gridDim.x * kRowWaves) {
    E* dst = out + row * hidden;
    const int pos = slot_of_row((int)row, bins, padded_bins, num_bins, n_slots);
    int s = pos >= 0 ? indices[pos] : -1;
    if (s < 0 || s >= n_slots) { wave_zero_row<DT, VEC>(dst, hidden); continue; }
    const float scale = weights ? load_as_f32(weights, s, w_dtype) : 1.f;
    wave_copy_row<DT, VEC>(x + (int64_t)(s / top_k) * hidden, dst, hidden, weights != nullptr, scale);
  }
}

// ------------------------------------------------------------------ slot -> row maps
__global__ void inverse_map_kernel(const int32_t* __restrict__ indices, const int32_t* __restrict__ bin_ids,
                                   const int32_t* __restrict__ bins, const int32_t* __restrict__ padded_bins,
                                   int num_bins, int n_slots, int32_t* __restrict__ inv) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_slots) return;
  const int s = indices[i];
  if (s < 0 || s >= n_slots) return;
  int row = i;
  if (padded_bins != nullptr) {
    const int e = bin_ids ? bin_ids[i] : upper_bound_i32(bins, num_bins, i);   // sorted position i lies in bins[e-1] .. bins[e]
    if (e < 0 || e >= num_bins) return;
    if (e > 0) row = i - bins[e - 1] + padded_bins[e - 1];
  }
  inv[s] = row;
}

__global__ void binned_inverse_map_kernel(const int32_t* __restrict__ indices, const int32_t* __restrict__ bins,
                                          int capacity, int n_slots, int32_t* __restrict__ inv) {
  const int e = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  const int start = e > 0 ? bins[e - 1] : 0;
  int count = bins[e] - start;
  if (count > capacity) count = capacity;
  if (j >= count || start + j >= n_slots) return;
  const int s = indices[start + j];
  if (s < 0 || s >= n_slots) return;
  inv[s] = e * capacity + j;
}

__global__ void fill_kernel(int32_t* __restrict__ p, int64_t n, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

// Zero-fill the rows of an expert-major buffer that no slot owns (padding; a sorted position whose index is not a
// slot), for the kernels that write such a buffer slot by slot.  Lane l of a wave looks at row base + l, and the
// wave clears the rows its ballot names; wave `wave_id` of `waves` takes every waves-th group of 64 rows.
template <int DT>
__device__ __forceinline__ void zero_unowned_rows(typename Elem<DT>::type* __restrict__ out, int64_t out_rows, int hidden,
                                                  const int32_t* __restrict__ indices, const int32_t* __restrict__ bins,
                                                  const int32_t* __restrict__ padded_bins, int num_bins, int n_slots,
                                                  int64_t wave_id, int64_t waves) {
  const int lane = lane_id();
  for (int64_t base = wave_id * kWave; base < out_rows; base += waves * kWave) {
    const int64_t row = base + lane;
    bool empty = false;
    if (row < out_rows) {
      const int pos = slot_of_row((int)row, bins, padded_bins, num_bins, n_slots);
      const int sl = pos >= 0 ? indices[pos] : -1;
      empty = sl < 0 || sl >= n_slots;
    }
    uint64_t todo = __ballot(empty);
    while (todo) {
      const int l = (int)__builtin_ctzll(todo);
      todo &= todo - 1;
      wave_zero_row<DT, true>(out + (base + l) * hidden, hidden);
    }
  }
}

// ------------------------------------------------------------------ gather, one wave per token
// The token's row is read once (the row-major kernel reads it once per slot, from wherever in the expert-major
// order that slot landed) and written to the rows of its top_k slots, inv[t * top_k + j] (-1: none).  Then
// the rows that no slot owns are zero-filled.  The stores are non-temporal (the expert-major copy is top_k times the
// tokens and is not read by this kernel: keeping it out of the caches is worth a fifth of the kernel's time); the loads
// are not: the tokens are a matrix that fits the last-level cache and that a kernel before or after this one touches as
// well (the producer of the tokens, the router; in the backward pass the router-weight gradient reads the same rows of
// the output gradient right afterwards), and a non-temporal load does not find them there (32768 rows of 4 KiB into
// 6 x as many: 153 us from a hot source with plain loads, 187 us with non-temporal ones).
template <int DT>
__global__ void __launch_bounds__(kRowThreads)
gather_tokens_kernel(const void* __restrict__ x_, int64_t tokens, int hidden, int top_k, const int32_t* __restrict__ indices,
                     const int32_t* __restrict__ inv, const int32_t* __restrict__ bins,
                     const int32_t* __restrict__ padded_bins, int num_bins, const void* __restrict__ weights, int w_dtype,
                     void* __restrict__ out_, int64_t out_rows) {
  typedef typename Elem<DT>::type E;
  constexpr int EV = Vec16<DT>::kElems;
  const E* x = (const E*)x_;
  E* out = (E*)out_;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int nvec = hidden / EV;
  const int64_t wave_id = (int64_t)blockIdx.x * kRowWaves + wave, waves = (int64_t)gridDim.x * kRowWaves;
  // a work item: 4 x 64 16-byte columns of one token's row (long rows are shared out over several waves)
  const int chunks = (nvec + 4 * kWave - 1) / (4 * kWave);
  for (int64_t item = wave_id; item < tokens * chunks; item += waves) {
    const int64_t t = item / chunks;
    const int c0 = (int)(item % chunks) * 4 * kWave;
    const u32x4* src = (const u32x4*)(x + t * hidden);
    const int64_t s0 = t * top_k;
    int my_row = lane < top_k ? inv[s0 + lane] : -1;
    my_row = my_row < out_rows ? my_row : -1;             // a map of another routing cannot take a store out of range
    const float my_scale = (weights && lane < top_k) ? load_as_f32(weights, s0 + lane, w_dtype) : 1.f;
    {
      u32x4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = c0 + i * kWave + lane;
        if (c < nvec) v[i] = src[c];
      }
      for (int j = 0; j < top_k; ++j) {
        const int row = __shfl(my_row, j, kWave);
        if (row < 0) continue;
        const float scale = __shfl(my_scale, j, kWave);
        u32x4* dst = (u32x4*)(out + (int64_t)row * hidden);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = c0 + i * kWave + lane;
          if (c >= nvec) continue;
          u32x4 w = v[i];
          if (weights) {
            float f[EV];
            Vec16<DT>::unpack(w, f);
#pragma unroll
            for (int q = 0; q < EV; ++q) f[q] *= scale;
            w = Vec16<DT>::pack(f);
          }
          __builtin_nontemporal_store(w, dst + c);
        }
      }
    }
  }
  zero_unowned_rows<DT>(out, out_rows, hidden, indices, bins, padded_bins, num_bins, (int)(tokens * top_k), wave_id, waves);
}

// A slot -> row map read with a bound: a row at or past `limit` reads as "no row" (-1).
struct BoundedRows {
  const int32_t* __restrict__ map;
  int limit;
  __device__ __forceinline__ int operator[](int64_t s) const {
    const int r = map[s];
    return r < limit ? r : -1;
  }
};

// ------------------------------------------------------------------ combine (scatter)
// out[t] = sum_j round(x[inv[t*k+j]] * w[t*k+j]); one wave per token.  Each product is
// rounded to the storage type before the fp32 sum, as the reference's scaled copy into a
// [tokens, top_k, hidden] buffer followed by sum(dim=1) does.
// BATCH: how many of a token's expert rows are kept in flight together (2, 4 or 8: a larger batch costs
// registers, i.e. resident waves, which the short top_k <= 2 cases need more); top_k > BATCH takes the
// one-row-at-a-time loop.
template <int DT, bool VEC, int BATCH>
__global__ void __launch_bounds__(kRowThreads)
combine_kernel(const void* __restrict__ x_, int64_t tokens, int hidden, int top_k, const int32_t* __restrict__ inv_,
               const void* __restrict__ weights, int w_dtype, void* __restrict__ out_,
               const int32_t* __restrict__ row_limit_ptr, int row_limit_value) {
  typedef typename Elem<DT>::type E;
  const E* x = (const E*)x_;
  E* out = (E*)out_;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  // Rows of x the map may name: below the last padded bin bound (read here) or a bound the host knows.  A map that does
  // not belong to this routing (kept from another one) can then make the result wrong, never a read out of range.
  const BoundedRows inv{inv_, row_limit_ptr ? *row_limit_ptr : row_limit_value};
  for (int64_t t = (int64_t)blockIdx.x * kRowWaves + wave; t < tokens; t += (int64_t)gridDim.x * kRowWaves) {
    E* dst = out + t * hidden;
    const int64_t s0 = t * top_k;
    if (top_k == 1) {
      const int row = inv[s0];
      if (row < 0) { wave_zero_row<DT, VEC>(dst, hidden); continue; }
      const float scale = weights ? load_as_f32(weights, s0, w_dtype) : 1.f;
      wave_copy_row<DT, VEC>(x + (int64_t)row * hidden, dst, hidden, weights != nullptr, scale);
      continue;
    }
    if (VEC && top_k <= BATCH) {
      // Lane j resolves expert j of the token (row in x, router weight); the wave then has the loads of all
      // top_k rows in flight for every 16-byte column instead of one after the other.
      constexpr int EV = Vec16<DT>::kElems;
      const int nvec = hidden / EV;
      const int my_row = lane < top_k ? inv[s0 + lane] : -1;
      const float my_scale = (weights && lane < top_k) ? load_as_f32(weights, s0 + lane, w_dtype) : 1.f;
      const u32x4* src[BATCH];
      float scale[BATCH];
      bool live[BATCH];
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        const int row = __shfl(my_row, j, kWave);
        live[j] = row >= 0;
        src[j] = (const u32x4*)(x + (int64_t)(live[j] ? row : 0) * hidden);
        scale[j] = __shfl(my_scale, j, kWave);
      }
      // eight 16-byte loads per lane in flight whatever top_k is: with two experts per token four columns of the
      // row are worked on together (two loads at a time leave a wave waiting on memory latency most of the time)
      constexpr int COLS = BATCH == 1 ? 1 : 8 / BATCH;   // BATCH 1: the instantiation for top_k = 1, which never gets here
      for (int c0 = lane; c0 < nvec; c0 += kWave * COLS) {
        u32x4 v[COLS][BATCH];
#pragma unroll
        for (int u = 0; u < COLS; ++u) {
          const int c = c0 + u * kWave;
          if (c >= nvec) continue;
#pragma unroll
          for (int j = 0; j < BATCH; ++j)
            if (live[j]) v[u][j] = __builtin_nontemporal_load(src[j] + c);   // expert-major rows are read once
        }
#pragma unroll
        for (int u = 0; u < COLS; ++u) {
          const int c = c0 + u * kWave;
          if (c >= nvec) continue;
          float acc[EV];
#pragma unroll
          for (int i = 0; i < EV; ++i) acc[i] = 0.f;
#pragma unroll
          for (int j = 0; j < BATCH; ++j) {
            if (!live[j]) continue;
            float f[EV];
            Vec16<DT>::unpack(v[u][j], f);
#pragma unroll
            for (int i = 0; i < EV; ++i)
              acc[i] += weights ? Elem<DT>::to_f32(Elem<DT>::from_f32(f[i] * scale[j])) : f[i];
          }
          ((u32x4*)dst)[c] = Vec16<DT>::pack(acc);
        }
      }
    } else if (VEC) {
      constexpr int EV = Vec16<DT>::kElems;
      const int nvec = hidden / EV;
      for (int c = lane; c < nvec; c += kWave) {
        float acc[EV];
#pragma unroll
        for (int i = 0; i < EV; ++i) acc[i] = 0.f;
        for (int j = 0; j < top_k; ++j) {
          const int row = inv[s0 + j];
          if (row < 0) continue;
          const float scale = weights ? load_as_f32(weights, s0 + j, w_dtype) : 1.f;
          float f[EV];
          Vec16<DT>::unpack(__builtin_nontemporal_load((const u32x4*)(x + (int64_t)row * hidden) + c), f);
#pragma unroll
          for (int i = 0; i < EV; ++i)
            acc[i] += weights ? Elem<DT>::to_f32(Elem<DT>::from_f32(f[i] * scale)) : f[i];
        }
        ((u32x4*)dst)[c] = Vec16<DT>::pack(acc);
      }
    } else {
      for (int c = lane; c < hidden; c += kWave) {
        float acc = 0.f;
        for (int j = 0; j < top_k; ++j) {
          const int row = inv[s0 + j];
          if (row < 0) continue;
          const float v = Elem<DT>::to_f32(x[(int64_t)row * hidden + c]);
          acc += weights ? Elem<DT>::to_f32(Elem<DT>::from_f32(v * load_as_f32(weights, s0 + j, w_dtype))) : v;
        }
        dst[c] = Elem<DT>::from_f32(acc);
      }
    }
  }
}

// ------------------------------------------------------------------ wgrad
template <int DT, bool VEC>
__global__ void __launch_bounds__(kRowThreads)
wgrad_kernel(const void* __restrict__ x_, const void* __restrict__ grad_, int64_t tokens, int hidden, int top_k,
             const int32_t* __restrict__ indices, const int32_t* __restrict__ bin_ids, const int32_t* __restrict__ bins,
             const int32_t* __restrict__ padded_bins, int num_bins, void* __restrict__ wgrad_) {
  typedef typename Elem<DT>::type E;
  const E* x = (const E*)x_;
  const E* grad = (const E*)grad_;
  E* wgrad = (E*)wgrad_;
  const int n_slots = (int)(tokens * top_k);
  const int wave = threadIdx.x / kWave;
  for (int i = blockIdx.x * kRowWaves + wave; i < n_slots; i += gridDim.x * kRowWaves) {
    const int s = indices[i];
    if (s < 0 || s >= n_slots) continue;
    int row = i;
    if (padded_bins != nullptr) {
      const int e = bin_ids[i];
      if (e < 0 || e >= num_bins) continue;
      if (e > 0) row = i - bins[e - 1] + padded_bins[e - 1];
    }
    const float d = wave_dot_row<DT, VEC>(x + (int64_t)row * hidden, grad + (int64_t)(s / top_k) * hidden, hidden);
    if (lane_id() == 0) wgrad[s] = Elem<DT>::from_f32(d);
  }
}

// ------------------------------------------------------------------ backward of the weighted scatter, one pass
// Both gradients of out[t] = sum_j w[s] x[row(s)] (s = t top_k + j) read the token's row of `grad`:
//   dx[row(s)] = round(grad[t] * w[s])          (the weighted gather)
//   dw[s]      = <x[row(s)], grad[t]>           (the router-weight gradient)
// One wave per token reads grad[t] once, and for each of its slots reads x[row], accumulates the dot product
// in the order wgrad_kernel does and writes the dx row: N h e bytes of reads through L2 and one launch less
// than the two kernels.  Then the rows of dx that no slot owns are zero-filled, as in gather_tokens_kernel.
// WRITE = false: only dw (a read-only pass; dx is left to gather_tokens_kernel).
template <int DT, int BATCH, bool WRITE>
__global__ void __launch_bounds__(kRowThreads)
scatter_backward_kernel(const void* __restrict__ grad_, const void* __restrict__ x_, int64_t tokens, int hidden, int top_k,
                        const int32_t* __restrict__ indices, const int32_t* __restrict__ inv,
                        const int32_t* __restrict__ bins, const int32_t* __restrict__ padded_bins, int num_bins,
                        const void* __restrict__ weights, int w_dtype, void* __restrict__ dx_, int64_t out_rows,
                        void* __restrict__ wgrad_) {
  typedef typename Elem<DT>::type E;
  constexpr int EV = Vec16<DT>::kElems;
  const E* grad = (const E*)grad_;
  const E* x = (const E*)x_;
  E* dx = (E*)dx_;
  E* wgrad = (E*)wgrad_;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int nvec = hidden / EV;
  const int64_t wave_id = (int64_t)blockIdx.x * kRowWaves + wave, waves = (int64_t)gridDim.x * kRowWaves;
  for (int64_t t = wave_id; t < tokens; t += waves) {
    const u32x4* g = (const u32x4*)(grad + t * hidden);
    const int64_t s0 = t * top_k;
    int my_row = lane < top_k ? inv[s0 + lane] : -1;
    my_row = my_row < out_rows ? my_row : -1;             // x and dx have out_rows rows
    const float my_scale = lane < top_k ? load_as_f32(weights, s0 + lane, w_dtype) : 0.f;
    int row[BATCH];
    float scale[BATCH], acc[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      row[j] = __shfl(my_row, j, kWave);
      scale[j] = __shfl(my_scale, j, kWave);
      acc[j] = 0.f;
    }
    for (int c0 = 0; c0 < nvec; c0 += 4 * kWave) {
      u32x4 gv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = c0 + i * kWave + lane;
        if (c < nvec) gv[i] = __builtin_nontemporal_load(g + c);
      }
      // the loads of slot j + 1 are issued before slot j is worked on
      u32x4 xv[2][4];
      auto fetch = [&](int j, u32x4 (&v)[4]) {
        if (row[j] < 0) return;
        const u32x4* xr = (const u32x4*)(x + (int64_t)row[j] * hidden);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = c0 + i * kWave + lane;
          if (c < nvec) v[i] = __builtin_nontemporal_load(xr + c);
        }
      };
      fetch(0, xv[0]);
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        if (j + 1 < BATCH) fetch(j + 1, xv[(j + 1) & 1]);
        if (row[j] < 0) continue;
        u32x4* dr = (u32x4*)(dx + (int64_t)row[j] * hidden);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = c0 + i * kWave + lane;
          if (c >= nvec) continue;
          float fx[EV], fg[EV];
          Vec16<DT>::unpack(xv[j & 1][i], fx);
          Vec16<DT>::unpack(gv[i], fg);
#pragma unroll
          for (int q = 0; q < EV; ++q) {
            acc[j] += fx[q] * fg[q];
            fg[q] *= scale[j];
          }
          if (WRITE) __builtin_nontemporal_store(Vec16<DT>::pack(fg), dr + c);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const float d = wave_sum(acc[j]);
      if (lane == 0 && row[j] >= 0) wgrad[s0 + j] = Elem<DT>::from_f32(d);
    }
  }
  if (WRITE) zero_unowned_rows<DT>(dx, out_rows, hidden, indices, bins, padded_bins, num_bins, (int)(tokens * top_k), wave_id, waves);
}

// ------------------------------------------------------------------ binned variants
template <int DT, bool VEC>
__global__ void __launch_bounds__(kRowThreads)
binned_gather_kernel(const void* __restrict__ x_, int64_t tokens, int hidden, int top_k, const int32_t* __restrict__ indices,
                     const int32_t* __restrict__ bins, int num_bins, int capacity, const void* __restrict__ weights,
                     int w_dtype, void* __restrict__ out_) {
  typedef typename Elem<DT>::type E;
  const E* x = (const E*)x_;
  E* out = (E*)out_;
  const int n_slots = (int)(tokens * top_k);
  const int wave = threadIdx.x / kWave;
  const int64_t total = (int64_t)num_bins * capacity;
  for (int64_t r = (int64_t)blockIdx.x * kRowWaves + wave; r < total; r += (int64_t)gridDim.x * kRowWaves) {
    const int e = (int)(r / capacity), j = (int)(r % capacity);
    const int start = e > 0 ? bins[e - 1] : 0;
    E* dst = out + r * hidden;
    int s = -1;
    if (start + j < bins[e] && start + j < n_slots) s = indices[start + j];
    if (s < 0 || s >= n_slots) { wave_zero_row<DT, VEC>(dst, hidden); continue; }
    const float scale = weights ? load_as_f32(weights, s, w_dtype) : 1.f;
    wave_copy_row<DT, VEC>(x + (int64_t)(s / top_k) * hidden, dst, hidden, weights != nullptr, scale);
  }
}

template <int DT, bool VEC>
__global__ void __launch_bounds__(kRowThreads)
binned_wgrad_kernel(const void* __restrict__ x_, const void* __restrict__ grad_, int64_t tokens, int hidden, int top_k,
                    const int32_t* __restrict__ indices, const int32_t* __restrict__ bins, int num_bins, int capacity,
                    void* __restrict__ wgrad_) {
  typedef typename Elem<DT>::type E;
  const E* x = (const E*)x_;
  const E* grad = (const E*)grad_;
  E* wgrad = (E*)wgrad_;
  const int n_slots = (int)(tokens * top_k);
  const int wave = threadIdx.x / kWave;
  const int64_t total = (int64_t)num_bins * capacity;
  for (int64_t r = (int64_t)blockIdx.x * kRowWaves + wave; r < total; r += (int64_t)gridDim.x * kRowWaves) {
    const int e = (int)(r / capacity), j = (int)(r % capacity);
    const int start = e > 0 ? bins[e - 1] : 0;
    if (start + j >= bins[e] || start + j >= n_slots) continue;
    const int s = indices[start + j];
    if (s < 0 || s >= n_slots) continue;
    const float d = wave_dot_row<DT, VEC>(x + r * hidden, grad + (int64_t)(s / top_k) * hidden, hidden);
    if (lane_id() == 0) wgrad[s] = Elem<DT>::from_f32(d);
  }
}

template <typename T>
__global__ void zero_kernel(T* __restrict__ p, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = (T)0;
}

// ------------------------------------------------------------------ host helpers
static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

static inline bool can_vec(int dtype, int hidden, const void* a, const void* b, const void* c = nullptr) {
  return ((int64_t)hidden * dtype_bytes(dtype)) % 16 == 0 && aligned16(a) && aligned16(b) && (c == nullptr || aligned16(c));
}

static inline unsigned row_grid(int64_t rows) {
  int64_t blocks = ceil_div(rows, kRowWaves);
  const int64_t cap = 256 * 16;  // 16 resident blocks of 4 waves per CU
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

#define MBX_DISPATCH_DT_VEC(dtype, vec, CALL)                    \
  switch (dtype) {                                               \
    case MBX_BF16: if (vec) { CALL(MBX_BF16, true); } else { CALL(MBX_BF16, false); } break; \
    case MBX_F16: if (vec) { CALL(MBX_F16, true); } else { CALL(MBX_F16, false); } break;    \
    case MBX_F32: if (vec) { CALL(MBX_F32, true); } else { CALL(MBX_F32, false); } break;    \
    default: return MBX_EINVAL;                                  \
  }

static inline bool bad_dtype(int d) { return d != MBX_BF16 && d != MBX_F16 && d != MBX_F32; }

}  // namespace
}  // namespace mbx

using namespace mbx;

extern "C" {

int mbx_gather(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* indices,
               const int32_t* bins, const int32_t* padded_bins, int num_bins, const void* weights, int w_dtype,
               void* out, int64_t out_rows, const int32_t* slot_rows, mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || out_rows < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (weights && bad_dtype(w_dtype)) return MBX_EINVAL;
  if (out_rows == 0 || hidden == 0) return 0;
  if (!out || (tokens > 0 && (!x || !indices)) || (padded_bins && !bins)) return MBX_EINVAL;
  if (tokens * top_k > 0x7fffffff || out_rows > 0x7fffffff) return MBX_ERANGE;
  const bool vec = can_vec(dtype, hidden, x ? x : out, out);
  hipStream_t s = as_stream(stream);
  if (vec && tokens > 0 && top_k <= kWave && slot_rows) {
    // one wave per token, through the slot -> row map
    const int32_t* inv = slot_rows;
    const int64_t items = tokens * ceil_div((int64_t)hidden * dtype_bytes(dtype) / 16, 4 * kWave);
    const unsigned grid = row_grid(items > out_rows / kWave ? items : out_rows / kWave);
    switch (dtype) {
      case MBX_BF16: gather_tokens_kernel<MBX_BF16><<<grid, kRowThreads, 0, s>>>(x, tokens, hidden, top_k, indices, inv, bins, padded_bins, num_bins, weights, w_dtype, out, out_rows); break;
      case MBX_F16: gather_tokens_kernel<MBX_F16><<<grid, kRowThreads, 0, s>>>(x, tokens, hidden, top_k, indices, inv, bins, padded_bins, num_bins, weights, w_dtype, out, out_rows); break;
      default: gather_tokens_kernel<MBX_F32><<<grid, kRowThreads, 0, s>>>(x, tokens, hidden, top_k, indices, inv, bins, padded_bins, num_bins, weights, w_dtype, out, out_rows); break;
    }
    return launch_status();
  }
#define CALL(DT, V) gather_kernel<DT, V><<<row_grid(out_rows), kRowThreads, 0, s>>>(x, tokens, hidden, top_k, indices, bins, padded_bins, num_bins, weights, w_dtype, out, out_rows)
  MBX_DISPATCH_DT_VEC(dtype, vec, CALL)
#undef CALL
  return launch_status();
}

// The slot -> row map of mbx_scatter_static: device memory that is part of the loaded code object, so that the
// entry point never allocates.  Every GPU the library runs on holds its own copy (4 MiB) at its own address until
// the process ends; in host code the array's name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) int32_t g_static_slot_rows[MBX_STATIC_SCATTER_MAX_SLOTS];

// Device address of g_static_slot_rows on the current device, looked up once per device (mbx_init(), or the first
// call of mbx_scatter_static on the device).  The lookup is a runtime call that may not be made while `capturing`
// (a stream, or null) records a graph: then MBX_ECAPTURE, and nothing has been enqueued.
static int static_slot_rows(int32_t** out, hipStream_t capturing = nullptr, bool check_capture = false) {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static int32_t* address[kMaxDevices];
  int dev = 0;
  MBX_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return MBX_EINVAL;
  std::lock_guard<std::mutex> guard(lock);
  if (!address[dev]) {
    if (check_capture) {
      hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
      MBX_HIP_CHECK(hipStreamIsCapturing(capturing, &status));
      if (status != hipStreamCaptureStatusNone) return MBX_ECAPTURE;
    }
    void* p = nullptr;
    MBX_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_slot_rows)));
    if (!p) return MBX_EINVAL;
    address[dev] = (int32_t*)p;
  }
  *out = address[dev];
  return 0;
}

static void build_slot_rows(const int32_t* indices, const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins,
                            int num_bins, int64_t n_slots, int32_t* inv, hipStream_t s) {
  const unsigned fb = (unsigned)(ceil_div(n_slots, 256) < 2048 ? ceil_div(n_slots, 256) : 2048);
  fill_kernel<<<fb, 256, 0, s>>>(inv, n_slots, -1);
  inverse_map_kernel<<<(unsigned)ceil_div(n_slots, 256), 256, 0, s>>>(indices, bin_ids, bins, padded_bins, num_bins, (int)n_slots, inv);
}

int mbx_slot_rows(const int32_t* indices, const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins,
                  int num_bins, int64_t n_slots, int32_t* slot_rows, mbx_stream_t stream) {
  if (n_slots < 0 || num_bins < 0) return MBX_EINVAL;
  if (n_slots == 0) return 0;
  if (!indices || !slot_rows || (padded_bins && !bins)) return MBX_EINVAL;
  if (n_slots > 0x7fffffff) return MBX_ERANGE;
  build_slot_rows(indices, bin_ids, bins, padded_bins, num_bins, n_slots, slot_rows, as_stream(stream));
  return launch_status();
}

// The combine launch of mbx_scatter / mbx_scatter_static: `inv` is the slot -> row map.
// x has *limit_ptr rows (a bound on the device: the last padded bin bound), or limit_value rows if limit_ptr is null.
static int launch_combine(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* inv,
                          const void* weights, int w_dtype, void* out, const int32_t* limit_ptr, int limit_value,
                          hipStream_t s) {
  const bool vec = can_vec(dtype, hidden, x, out);
#define CALL_B(DT, V, B) combine_kernel<DT, V, B><<<row_grid(tokens), kRowThreads, 0, s>>>(x, tokens, hidden, top_k, inv, weights, w_dtype, out, limit_ptr, limit_value)
#define CALL(DT, V)                            \
  do {                                         \
    if (top_k == 1) CALL_B(DT, V, 1);          \
    else if (top_k <= 2) CALL_B(DT, V, 2);     \
    else if (top_k <= 4) CALL_B(DT, V, 4);     \
    else CALL_B(DT, V, 8);                     \
  } while (0)
  MBX_DISPATCH_DT_VEC(dtype, vec, CALL)
#undef CALL
#undef CALL_B
  return launch_status();
}

int mbx_scatter(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* indices,
                const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins, int num_bins,
                const void* weights, int w_dtype, void* out, const int32_t* slot_rows, void* scratch, size_t scratch_bytes,
                mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (weights && bad_dtype(w_dtype)) return MBX_EINVAL;
  if (tokens == 0 || hidden == 0) return 0;
  if (!x || !out || (!slot_rows && (!indices || (padded_bins && !bins)))) return MBX_EINVAL;
  const int64_t n_slots = tokens * top_k;
  if (n_slots > 0x7fffffff) return MBX_ERANGE;
  hipStream_t s = as_stream(stream);
  const int32_t* inv = slot_rows;
  if (!inv) {
    if (!scratch || scratch_bytes < (size_t)n_slots * sizeof(int32_t)) return MBX_ESCRATCH;
    build_slot_rows(indices, bin_ids, bins, padded_bins, num_bins, n_slots, (int32_t*)scratch, s);
    inv = (const int32_t*)scratch;
  }
  return launch_combine(x, dtype, tokens, hidden, top_k, inv, weights, w_dtype, out,
                        padded_bins && num_bins > 0 ? padded_bins + (num_bins - 1) : nullptr, (int)n_slots, s);
}

int mbx_init(void) {
  int32_t* map = nullptr;
  return static_slot_rows(&map);
}

int mbx_scatter_static(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* indices,
                       const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins, int num_bins,
                       const void* weights, int w_dtype, void* out, mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (weights && bad_dtype(w_dtype)) return MBX_EINVAL;
  if (tokens == 0 || hidden == 0) return 0;
  if (!x || !out || !indices || (padded_bins && !bins)) return MBX_EINVAL;
  const int64_t n_slots = tokens * top_k;
  if (n_slots > MBX_STATIC_SCATTER_MAX_SLOTS) return MBX_ERANGE;   // more slots than the static map holds
  int32_t* map = nullptr;
  hipStream_t s = as_stream(stream);
  const int rc = static_slot_rows(&map, s, true);
  if (rc) return rc;
  // every entry the combine reads is rewritten here (fill, then the inverse map): nothing of the previous call is used
  build_slot_rows(indices, bin_ids, bins, padded_bins, num_bins, n_slots, map, s);
  return launch_combine(x, dtype, tokens, hidden, top_k, map, weights, w_dtype, out,
                        padded_bins && num_bins > 0 ? padded_bins + (num_bins - 1) : nullptr, (int)n_slots, s);
}

int mbx_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int hidden, int top_k,
                      const int32_t* indices, const int32_t* bin_ids, const int32_t* bins, const int32_t* padded_bins,
                      int num_bins, void* wgrad, mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (tokens == 0) return 0;
  if (!wgrad || !indices || (hidden > 0 && (!x || !grad)) || (padded_bins && (!bins || !bin_ids))) return MBX_EINVAL;
  const int64_t n_slots = tokens * top_k;
  if (n_slots > 0x7fffffff) return MBX_ERANGE;
  const bool vec = can_vec(dtype, hidden, x, grad);
  hipStream_t s = as_stream(stream);
#define CALL(DT, V) wgrad_kernel<DT, V><<<row_grid(n_slots), kRowThreads, 0, s>>>(x, grad, tokens, hidden, top_k, indices, bin_ids, bins, padded_bins, num_bins, wgrad)
  MBX_DISPATCH_DT_VEC(dtype, vec, CALL)
#undef CALL
  return launch_status();
}

int mbx_scatter_backward(const void* grad, const void* x, int dtype, int64_t tokens, int hidden, int top_k,
                         const int32_t* indices, const int32_t* bins, const int32_t* padded_bins, int num_bins,
                         const void* weights, int w_dtype, const int32_t* slot_rows, void* grad_x, int64_t out_rows,
                         void* wgrad, mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || out_rows < 0 || bad_dtype(dtype) || bad_dtype(w_dtype)) return MBX_EINVAL;
  if (tokens * top_k > 0x7fffffff || out_rows > 0x7fffffff) return MBX_ERANGE;
  // Needs the slot -> row map and whole 16-byte columns.  One pass for one expert per token.  With more, a
  // token's wave would alternate between reading and writing several scattered rows, and the pass takes longer
  // than a write-mostly and a read-only kernel (4 experts: 247 against 212 us, 6 experts: 480 against 375): then
  // the gather by token writes grad_x and the same kernel, without its stores, computes wgrad.
  if (!slot_rows || top_k > 8 || hidden == 0 || !can_vec(dtype, hidden, grad, x, grad_x)) return MBX_EUNSUPPORTED;
  if (tokens == 0) return 0;
  if (!grad || !x || !indices || !weights || !grad_x || !wgrad || (padded_bins && !bins)) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  const unsigned grid = row_grid(tokens > out_rows / kWave ? tokens : out_rows / kWave);
#define CALL(DT, B, W) scatter_backward_kernel<DT, B, W><<<grid, kRowThreads, 0, s>>>(grad, x, tokens, hidden, top_k, indices, slot_rows, bins, padded_bins, num_bins, weights, w_dtype, grad_x, out_rows, wgrad)
#define CALL_DT(DT)                        \
  do {                                     \
    if (top_k == 1) CALL(DT, 1, true);     \
    else {                                 \
      const int64_t items = tokens * ceil_div((int64_t)hidden * dtype_bytes(dtype) / 16, 4 * kWave);                       \
      const unsigned ggrid = row_grid(items > out_rows / kWave ? items : out_rows / kWave);                               \
      gather_tokens_kernel<DT><<<ggrid, kRowThreads, 0, s>>>(grad, tokens, hidden, top_k, indices, slot_rows, bins, padded_bins, num_bins, weights, w_dtype, grad_x, out_rows); \
      if (top_k == 2) CALL(DT, 2, false);  \
      else if (top_k <= 4) CALL(DT, 4, false); \
      else CALL(DT, 8, false);             \
    }                                      \
  } while (0)
  switch (dtype) {
    case MBX_BF16: CALL_DT(MBX_BF16); break;
    case MBX_F16: CALL_DT(MBX_F16); break;
    default: CALL_DT(MBX_F32); break;
  }
#undef CALL_DT
#undef CALL
  return launch_status();
}

int mbx_binned_gather(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* indices,
                      const int32_t* bins, int num_bins, int capacity, const void* weights, int w_dtype, void* out,
                      mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || capacity < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (weights && bad_dtype(w_dtype)) return MBX_EINVAL;
  const int64_t total = (int64_t)num_bins * capacity;
  if (total == 0 || hidden == 0) return 0;
  if (!out || !bins || (tokens > 0 && (!x || !indices))) return MBX_EINVAL;
  if (tokens * top_k > 0x7fffffff || total > 0x7fffffff) return MBX_ERANGE;
  const bool vec = can_vec(dtype, hidden, x ? x : out, out);
  hipStream_t s = as_stream(stream);
#define CALL(DT, V) binned_gather_kernel<DT, V><<<row_grid(total), kRowThreads, 0, s>>>(x, tokens, hidden, top_k, indices, bins, num_bins, capacity, weights, w_dtype, out)
  MBX_DISPATCH_DT_VEC(dtype, vec, CALL)
#undef CALL
  return launch_status();
}

static int binned_inverse(const int32_t* indices, const int32_t* bins, int num_bins, int capacity, int64_t n_slots,
                          int32_t* inv, hipStream_t s) {
  const unsigned fb = (unsigned)(ceil_div(n_slots, 256) < 2048 ? ceil_div(n_slots, 256) : 2048);
  fill_kernel<<<fb, 256, 0, s>>>(inv, n_slots, -1);
  if (num_bins > 0 && capacity > 0) {
    if (num_bins > 65535) return MBX_ERANGE;
    dim3 grid((unsigned)ceil_div(capacity, 256), (unsigned)num_bins);
    binned_inverse_map_kernel<<<grid, 256, 0, s>>>(indices, bins, capacity, (int)n_slots, inv);
  }
  return 0;
}

int mbx_binned_scatter(const void* x, int dtype, int64_t tokens, int hidden, int top_k, const int32_t* indices,
                       const int32_t* bins, int num_bins, int capacity, const void* weights, int w_dtype, void* out,
                       void* scratch, size_t scratch_bytes, mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || capacity < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (weights && bad_dtype(w_dtype)) return MBX_EINVAL;
  if (tokens == 0 || hidden == 0) return 0;
  if (!out || !indices || (num_bins > 0 && !bins) || ((int64_t)num_bins * capacity > 0 && !x)) return MBX_EINVAL;
  const int64_t n_slots = tokens * top_k;
  if (n_slots > 0x7fffffff || (int64_t)num_bins * capacity > 0x7fffffff) return MBX_ERANGE;
  if (!scratch || scratch_bytes < (size_t)n_slots * sizeof(int32_t)) return MBX_ESCRATCH;
  int32_t* inv = (int32_t*)scratch;
  hipStream_t s = as_stream(stream);
  const int rc = binned_inverse(indices, bins, num_bins, capacity, n_slots, inv, s);
  if (rc) return rc;
  return launch_combine(x ? x : out, dtype, tokens, hidden, top_k, inv, weights, w_dtype, out, nullptr, (int)((int64_t)num_bins * capacity), s);
}

int mbx_binned_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int hidden, int top_k,
                             const int32_t* indices, const int32_t* bins, int num_bins, int capacity, void* wgrad,
                             mbx_stream_t stream) {
  if (tokens < 0 || hidden < 0 || top_k <= 0 || num_bins < 0 || capacity < 0 || bad_dtype(dtype)) return MBX_EINVAL;
  if (tokens == 0) return 0;
  const int64_t n_slots = tokens * top_k;
  const int64_t total = (int64_t)num_bins * capacity;
  if (!wgrad || !indices || (num_bins > 0 && !bins) || (total > 0 && hidden > 0 && (!x || !grad))) return MBX_EINVAL;
  if (n_slots > 0x7fffffff || total > 0x7fffffff) return MBX_ERANGE;
  hipStream_t s = as_stream(stream);
  const unsigned fb = (unsigned)(ceil_div(n_slots, 256) < 2048 ? ceil_div(n_slots, 256) : 2048);
  if (dtype_bytes(dtype) == 2) zero_kernel<uint16_t><<<fb, 256, 0, s>>>((uint16_t*)wgrad, n_slots);
  else zero_kernel<uint32_t><<<fb, 256, 0, s>>>((uint32_t*)wgrad, n_slots);
  if (total > 0) {
    const bool vec = can_vec(dtype, hidden, x, grad);
#define CALL(DT, V) binned_wgrad_kernel<DT, V><<<row_grid(total), kRowThreads, 0, s>>>(x, grad, tokens, hidden, top_k, indices, bins, num_bins, capacity, wgrad)
    MBX_DISPATCH_DT_VEC(dtype, vec, CALL)
#undef CALL
  }
  return launch_status();
}

}  // extern "C"
