// Routing / bookkeeping kernels: histogram of expert ids, stable LSD radix sort with an
// end bit, row-wise cumulative sums, block-diagonal topology indices, replicate.
// All integer work; wave64 ballot aggregation and LDS-staged counters.
#include "common.h"

namespace mbx {
namespace {

// ------------------------------------------------------------------ small fills
__global__ void fill_i32_kernel(int32_t* __restrict__ p, int64_t n, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

// Mask of the lanes of this wave whose (valid) value has the same low `nbits` bits.
__device__ __forceinline__ uint64_t match_peers(uint32_t v, bool valid, int nbits) {
  uint64_t peers = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (v >> b) & 1u;
    const uint64_t m = __ballot(valid && bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

__device__ __forceinline__ uint64_t lanemask_lt() { return (1ull << lane_id()) - 1ull; }

// ------------------------------------------------------------------ histogram
constexpr int kHistThreads = 1024;
constexpr int kHistLdsBins = 8192;

// One block per (chunk, row).  Counts land in LDS; lanes holding the same id are merged
// with ballots first when the id space is small, so an LDS atomic is issued once per
// distinct id per wave instead of once per lane.
template <typename T, bool DIRECT>
__global__ void __launch_bounds__(kHistThreads)
histogram_kernel(const T* __restrict__ x, int64_t n, int num_bins, int nbits, int64_t chunk,
                 int32_t* __restrict__ out) {
  extern __shared__ int32_t hist[];
  const int64_t row = blockIdx.y;
  const T* xr = x + row * n;
  int32_t* outr = out + row * (int64_t)num_bins;
  for (int b = threadIdx.x; b < num_bins; b += kHistThreads) hist[b] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * chunk;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  // every lane of a wave runs the same number of rounds so the ballots see whole waves
  for (int64_t base = begin; base < end; base += kHistThreads) {
    const int64_t i = base + threadIdx.x;
    bool valid = i < end;
    int64_t v = valid ? (int64_t)xr[i] : 0;
    valid = valid && v >= 0 && v < num_bins;
    if (nbits > 0) {
      const uint64_t peers = match_peers((uint32_t)v, valid, nbits);
      if (valid && (peers & lanemask_lt()) == 0) atomicAdd(&hist[v], (int32_t)__popcll(peers));
    } else if (valid) {
      atomicAdd(&hist[v], 1);
    }
  }
  __syncthreads();
  for (int b = threadIdx.x; b < num_bins; b += kHistThreads) {
    if (DIRECT) outr[b] = hist[b];
    else if (hist[b]) atomicAdd(&outr[b], hist[b]);
  }
}

// Fallback for id spaces that do not fit LDS: global atomics into a zeroed output.
template <typename T>
__global__ void histogram_global_kernel(const T* __restrict__ x, int64_t n, int num_bins,
                                        int32_t* __restrict__ out) {
  const int64_t row = blockIdx.y;
  const T* xr = x + row * n;
  int32_t* outr = out + row * (int64_t)num_bins;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const int64_t v = (int64_t)xr[i];
    if (v >= 0 && v < num_bins) atomicAdd(&outr[v], 1);
  }
}

template <typename T>
int histogram_impl(const T* x, int64_t rows, int64_t n, int num_bins, int32_t* out, hipStream_t s) {
  if (rows == 0 || num_bins == 0) return 0;
  if (rows > 65535) return MBX_ERANGE;
  int nbits = 0;
  if (num_bins <= 256) { while ((1 << nbits) < num_bins) ++nbits; if (nbits == 0) nbits = 1; }
  const int64_t total = rows * (int64_t)num_bins;
  if (num_bins <= kHistLdsBins) {
    const size_t lds = (size_t)num_bins * sizeof(int32_t);
    if (n <= (int64_t)kHistThreads * 8) {  // one block per row writes its counts directly
      histogram_kernel<T, true><<<dim3(1, (unsigned)rows), kHistThreads, lds, s>>>(x, n, num_bins, nbits, n > 0 ? n : 1, out);
      return launch_status();
    }
    fill_i32_kernel<<<(unsigned)(ceil_div(total, 256) < 1024 ? ceil_div(total, 256) : 1024), 256, 0, s>>>(out, total, 0);
    const int64_t chunk = (int64_t)kHistThreads * 8;
    const int64_t blocks = ceil_div(n, chunk);
    if (blocks > 0x7fffffff) return MBX_ERANGE;
    histogram_kernel<T, false><<<dim3((unsigned)blocks, (unsigned)rows), kHistThreads, lds, s>>>(x, n, num_bins, nbits, chunk, out);
    return launch_status();
  }
  fill_i32_kernel<<<(unsigned)(ceil_div(total, 256) < 1024 ? ceil_div(total, 256) : 1024), 256, 0, s>>>(out, total, 0);
  if (n > 0) {
    int64_t blocks = ceil_div(n, 256 * 8);
    if (blocks > 4096) blocks = 4096;
    histogram_global_kernel<T><<<dim3((unsigned)blocks, (unsigned)rows), 256, 0, s>>>(x, n, num_bins, out);
  }
  return launch_status();
}

// ------------------------------------------------------------------ radix sort
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortItems = 8;                                  // rounds of 64 keys per wave
constexpr int kSortTile = kSortThreads * kSortItems;           // keys per block

template <typename T> struct UnsignedOf;
template <> struct UnsignedOf<int16_t> { typedef uint16_t type; };
template <> struct UnsignedOf<int32_t> { typedef uint32_t type; };
template <> struct UnsignedOf<int64_t> { typedef uint64_t type; };

// Digit of a key for the pass that starts at `shift`: the sign bit is inverted so that a
// full-width sort yields the signed order; `mask` keeps only bits below the end bit.
template <typename T>
__device__ __forceinline__ uint32_t digit_of(T key, int shift, uint32_t mask) {
  typedef typename UnsignedOf<T>::type U;
  U u = (U)key ^ (U)((U)1 << (sizeof(T) * 8 - 1));
  return (uint32_t)(u >> shift) & mask;
}

// Pass step 1: digit counts of every tile, stored digit-major: counts[d * nblocks + block].
template <typename T>
__global__ void __launch_bounds__(kSortThreads)
radix_count_kernel(const T* __restrict__ keys, int64_t n, int shift, uint32_t mask, int nbits,
                   int32_t* __restrict__ counts, int nblocks) {
  __shared__ int32_t hist[kRadix];
  hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const int64_t i = base + it * kSortThreads + threadIdx.x;
    const bool valid = i < n;
    const uint32_t d = valid ? digit_of<T>(keys[i], shift, mask) : 0u;
    const uint64_t peers = match_peers(d, valid, nbits);
    if (valid && (peers & lanemask_lt()) == 0) atomicAdd(&hist[d], (int32_t)__popcll(peers));
  }
  __syncthreads();
  counts[(int64_t)threadIdx.x * nblocks + blockIdx.x] = hist[threadIdx.x];
}

// Pass step 2: exclusive scan, in place, of the digit-major count table (one block of 1024 threads).
__device__ __forceinline__ void block_exclusive_scan_i32(int32_t* __restrict__ data, int64_t n) {
  __shared__ int32_t wave_tot[16];
  __shared__ int32_t carry_s;
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t base = 0; base < n; base += 1024) {
    const int64_t i = base + threadIdx.x;
    const int32_t v = i < n ? data[i] : 0;
    int32_t inc = wave_inclusive_scan(v);
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    int32_t wave_off = 0;
    for (int w = 0; w < wave; ++w) wave_off += wave_tot[w];
    const int32_t carry = carry_s;
    if (i < n) data[i] = carry + wave_off + inc - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry_s = carry + wave_off + inc;
    __syncthreads();
  }
}
__global__ void __launch_bounds__(1024) exclusive_scan_i32_kernel(int32_t* __restrict__ data, int64_t n) {
  block_exclusive_scan_i32(data, n);
}

// The same scan for the one-pass sort of expert ids, which then also knows what histogram and the cumsums of the
// routing step would compute (megablocks/layers/moe.py:167-176, dmoe.py:137-153): after the scan, entry [d][0] of the
// table is the number of ids with a digit below d, so
//   tokens_per_expert[e] = table[e + 1][0] - table[e][0],   bins[e] = table[e + 1][0]        (table[ndigits][0] := n)
// for ids inside [0, num_experts), and padded_bins = cumsum(round_up(tokens_per_expert, pad)) when pad > 0.
__global__ void __launch_bounds__(1024)
route_scan_kernel(int32_t* __restrict__ table, int ndigits, int nblocks, int32_t n, int num_experts, int pad,
                  int32_t* __restrict__ tokens_per_expert, int32_t* __restrict__ bins, int32_t* __restrict__ padded_bins) {
  __shared__ int32_t padded[1024];
  block_exclusive_scan_i32(table, (int64_t)ndigits * nblocks);
  __syncthreads();
  const int e = threadIdx.x;
  int32_t count = 0;
  if (e < num_experts) {
    const int32_t start = e < ndigits ? table[(int64_t)e * nblocks] : n;
    const int32_t next = e + 1 < ndigits ? table[(int64_t)(e + 1) * nblocks] : n;
    count = next - start;
    tokens_per_expert[e] = count;
    bins[e] = next;
  }
  if (pad > 0 && padded_bins != nullptr) {
    padded[e] = e < num_experts ? (count + pad - 1) / pad * pad : 0;
    __syncthreads();
    if (e < num_experts) {
      int32_t run = 0;
      for (int j = 0; j <= e; ++j) run += padded[j];
      padded_bins[e] = run;
    }
  }
}

// Pass step 3: stable scatter.  Wave w of a block owns kSortItems consecutive rounds of 64
// consecutive keys, so "earlier key" means earlier wave, then earlier round, then lower lane.
// slot_rows (with IOTA, i.e. on the first pass, whose values are the key's positions in the input; NULL: not wanted):
// also writes, for the key at input position i that lands at sorted position p, the row of the expert-major buffer
// that holds it: p itself, or with padded_bins the row p - bins[e - 1] + padded_bins[e - 1] of expert e's padded
// block (-1 for a key whose digit is at or past num_bins) -- the map inverse_map_kernel of the permutation kernels
// builds.
template <typename T, bool IOTA>
__global__ void __launch_bounds__(kSortThreads)
radix_scatter_kernel(const T* __restrict__ keys_in, const T* __restrict__ vals_in, int64_t n,
                     int shift, uint32_t mask, int nbits, const int32_t* __restrict__ offsets,
                     int nblocks, T* __restrict__ keys_out, T* __restrict__ vals_out,
                     int32_t* __restrict__ slot_rows = nullptr, const int32_t* __restrict__ bins = nullptr,
                     const int32_t* __restrict__ padded_bins = nullptr, int num_bins = 0) {
  __shared__ int32_t wave_hist[kSortWaves][kRadix];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int w = 0; w < kSortWaves; ++w) wave_hist[w][threadIdx.x] = 0;
  __syncthreads();

  const int64_t wave_base = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * (kWave * kSortItems);
  T key[kSortItems];
  uint32_t dig[kSortItems];
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const int64_t i = wave_base + it * kWave + lane;
    const bool valid = i < n;
    key[it] = valid ? keys_in[i] : (T)0;
    dig[it] = valid ? digit_of<T>(key[it], shift, mask) : 0u;
    const uint64_t peers = match_peers(dig[it], valid, nbits);
    if (valid && (peers & lanemask_lt()) == 0) atomicAdd(&wave_hist[wave][dig[it]], (int32_t)__popcll(peers));
  }
  __syncthreads();
  {  // thread d turns the per-wave counts of digit d into starting positions
    const int d = threadIdx.x;
    int32_t run = offsets[(int64_t)d * nblocks + blockIdx.x];
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const int32_t c = wave_hist[w][d];
      wave_hist[w][d] = run;
      run += c;
    }
  }
  __syncthreads();
  volatile int32_t* cursor = wave_hist[wave];
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const int64_t i = wave_base + it * kWave + lane;
    const bool valid = i < n;
    const uint64_t peers = match_peers(dig[it], valid, nbits);
    int32_t pos = 0;
    if (valid) pos = cursor[dig[it]] + (int32_t)__popcll(peers & lanemask_lt());
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lanemask_lt()) == 0) cursor[dig[it]] += (int32_t)__popcll(peers);
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      keys_out[pos] = key[it];
      vals_out[pos] = IOTA ? (T)i : vals_in[i];
      if (IOTA && slot_rows != nullptr) {
        int32_t row = pos;
        if (padded_bins != nullptr) {
          // The expert of a key is its digit here, as it is for the counts the bins were made of (route_scan_kernel):
          // an id outside [0, num_bins) is then either one more row of the expert its low bits name, counted in that
          // expert's bins, or (digit at or past num_bins) sorted behind the last bin and in nobody's rows.  Every row
          // of the padded buffer inside a bin so has exactly one slot or is padding.
          const int e = (int)dig[it];
          if (e >= num_bins) row = -1;
          else if (e > 0) row = pos - bins[e - 1] + padded_bins[e - 1];
        }
        slot_rows[i] = row;
      }
    }
  }
}

template <typename T>
__global__ void copy_iota_kernel(const T* __restrict__ x, int64_t n, T* __restrict__ keys_out, T* __restrict__ vals_out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) { keys_out[i] = x[i]; vals_out[i] = (T)i; }
}

static inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static inline int sort_passes(int end_bit) { return (end_bit + kRadixBits - 1) / kRadixBits; }

template <typename T>
int sort_impl(const T* x, int64_t n, int end_bit, T* keys_out, T* perm_out, void* scratch,
              size_t scratch_bytes, hipStream_t s) {
  if (n == 0) return 0;
  if (n > 0x7fffffff - kSortTile) return MBX_ERANGE;
  const int bits = (int)sizeof(T) * 8;
  if (end_bit > bits) end_bit = bits;
  const int passes = sort_passes(end_bit);
  if (passes == 0) {
    copy_iota_kernel<T><<<(unsigned)(ceil_div(n, 256) < 2048 ? ceil_div(n, 256) : 2048), 256, 0, s>>>(x, n, keys_out, perm_out);
    return launch_status();
  }
  const int nblocks = (int)ceil_div(n, kSortTile);
  const size_t counts_bytes = align256((size_t)kRadix * nblocks * sizeof(int32_t));
  const size_t buf_bytes = align256((size_t)n * sizeof(T));
  const size_t need = counts_bytes + (passes > 1 ? 2 * buf_bytes : 0);
  if (scratch_bytes < need || scratch == nullptr) return MBX_ESCRATCH;
  int32_t* counts = (int32_t*)scratch;
  T* tmp_keys = (T*)((char*)scratch + counts_bytes);
  T* tmp_vals = (T*)((char*)scratch + counts_bytes + buf_bytes);

  const T* kin = x;
  const T* vin = nullptr;
  for (int p = 0; p < passes; ++p) {
    const int shift = p * kRadixBits;
    const int pass_bits = (end_bit - shift) < kRadixBits ? (end_bit - shift) : kRadixBits;
    const uint32_t mask = (1u << pass_bits) - 1u;
    const bool to_final = ((passes - 1 - p) % 2) == 0;
    T* kout = to_final ? keys_out : tmp_keys;
    T* vout = to_final ? perm_out : tmp_vals;
    radix_count_kernel<T><<<nblocks, kSortThreads, 0, s>>>(kin, n, shift, mask, pass_bits, counts, nblocks);
    exclusive_scan_i32_kernel<<<1, 1024, 0, s>>>(counts, ((int64_t)1 << pass_bits) * nblocks);   // digit-major: digits the pass cannot produce come last
    if (p == 0)
      radix_scatter_kernel<T, true><<<nblocks, kSortThreads, 0, s>>>(kin, nullptr, n, shift, mask, pass_bits, counts, nblocks, kout, vout);
    else
      radix_scatter_kernel<T, false><<<nblocks, kSortThreads, 0, s>>>(kin, vin, n, shift, mask, pass_bits, counts, nblocks, kout, vout);
    kin = kout;
    vin = vout;
  }
  return launch_status();
}

// ------------------------------------------------------------------ cumsum
template <typename T>
__global__ void __launch_bounds__(256) cumsum_kernel(const T* __restrict__ x, int64_t n, int exclusive, T* __restrict__ out) {
  __shared__ T wave_tot[4];
  __shared__ T carry_s;
  const int64_t row = blockIdx.x;
  const T* xr = x + row * n;
  T* outr = out + row * n;
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t base = 0; base < n; base += 256) {
    const int64_t i = base + threadIdx.x;
    const T v = i < n ? xr[i] : (T)0;
    T inc = wave_inclusive_scan<T>(v);
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    T wave_off = 0;
    for (int w = 0; w < wave; ++w) wave_off += wave_tot[w];
    const T carry = carry_s;
    const T incl = (T)(carry + wave_off + inc);
    if (i < n) outr[i] = exclusive ? (T)(incl - v) : incl;
    __syncthreads();
    if (threadIdx.x == 255) carry_s = incl;
    __syncthreads();
  }
}

// ------------------------------------------------------------------ topology
__global__ void topology_kernel(const int32_t* __restrict__ padded_bins, int num_bins, int block_size,
                                int block_rows, int block_cols, int16_t* __restrict__ out) {
  const int64_t total = (int64_t)block_rows * block_cols;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const int row = (int)(i / block_cols), col = (int)(i % block_cols);
    // expert of this block-row: first e with padded_bins[e] / block_size > row
    int lo = 0, hi = num_bins;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (padded_bins[mid] / block_size > row) hi = mid; else lo = mid + 1;
    }
    out[i] = lo < num_bins ? (int16_t)(col + lo * block_cols) : (int16_t)0;
  }
}

// ------------------------------------------------------------------ replicate
template <typename T>
__global__ void replicate_forward_kernel(const T* __restrict__ x, int num_bins, const int32_t* __restrict__ bins,
                                         T* __restrict__ out, int64_t columns) {
  const int e = blockIdx.x;
  const int64_t b = blockIdx.y;
  int64_t start = e > 0 ? bins[e - 1] : 0;
  int64_t end = bins[e];
  if (end > columns) end = columns;
  const T v = x[b * num_bins + e];
  T* o = out + b * columns;
  for (int64_t j = start + threadIdx.x; j < end; j += blockDim.x) o[j] = v;
  if (e == num_bins - 1)
    for (int64_t j = (end > 0 ? end : 0) + threadIdx.x; j < columns; j += blockDim.x) o[j] = (T)0;
}

template <int DT>
__global__ void __launch_bounds__(256) replicate_backward_kernel(const void* __restrict__ grad_, int64_t columns,
                                                                 const int32_t* __restrict__ bins, int num_bins,
                                                                 void* __restrict__ out_) {
  typedef typename Elem<DT>::type E;
  __shared__ float part[4];
  const E* grad = (const E*)grad_;
  E* out = (E*)out_;
  const int e = blockIdx.x;
  const int64_t b = blockIdx.y;
  int64_t start = e > 0 ? bins[e - 1] : 0;
  int64_t end = bins[e];
  if (end > columns) end = columns;
  float acc = 0.f;
  for (int64_t j = start + threadIdx.x; j < end; j += 256) acc += Elem<DT>::to_f32(grad[b * columns + j]);
  acc = wave_sum(acc);
  if (lane_id() == 0) part[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) out[b * num_bins + e] = Elem<DT>::from_f32(part[0] + part[1] + part[2] + part[3]);
}

}  // namespace
}  // namespace mbx

using namespace mbx;

extern "C" {

int mbx_version(void) { return 1; }

const char* mbx_error_string(int code) {
  if (code == 0) return "success";
  if (code == MBX_EINVAL) return "mbx: invalid argument";
  if (code == MBX_ESCRATCH) return "mbx: scratch buffer missing or too small";
  if (code == MBX_ERANGE) return "mbx: size out of the supported range";
  if (code == MBX_EUNSUPPORTED) return "mbx: shape or type not handled by this entry point";
  if (code == MBX_ECAPTURE) return "mbx: first call on this device under stream capture; call mbx_init() beforehand";
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "mbx: unknown error";
}

int mbx_histogram(const void* x, int itype, int64_t rows, int64_t n, int num_bins, int32_t* out, mbx_stream_t stream) {
  if (rows < 0 || n < 0 || num_bins < 0) return MBX_EINVAL;
  if (rows * (int64_t)num_bins == 0) return 0;
  if (!out || (!x && n > 0)) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  switch (itype) {
    case MBX_I16: return histogram_impl<int16_t>((const int16_t*)x, rows, n, num_bins, out, s);
    case MBX_I32: return histogram_impl<int32_t>((const int32_t*)x, rows, n, num_bins, out, s);
    case MBX_I64: return histogram_impl<int64_t>((const int64_t*)x, rows, n, num_bins, out, s);
  }
  return MBX_EINVAL;
}

size_t mbx_sort_scratch_bytes(int64_t n, int itype, int end_bit) {
  if (n <= 0) return 0;
  const int bits = itype_bytes(itype) * 8;
  if (end_bit > bits) end_bit = bits;
  const int passes = sort_passes(end_bit);
  if (passes == 0) return 0;
  const size_t nblocks = (size_t)ceil_div(n, kSortTile);
  size_t need = align256((size_t)kRadix * nblocks * sizeof(int32_t));
  if (passes > 1) need += 2 * align256((size_t)n * itype_bytes(itype));
  return need;
}

int mbx_sort(const void* x, int itype, int64_t n, int end_bit, void* keys_out, void* perm_out, void* scratch,
             size_t scratch_bytes, mbx_stream_t stream) {
  if (n < 0 || end_bit < 0) return MBX_EINVAL;
  if (n == 0) return 0;
  if (!x || !keys_out || !perm_out) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  switch (itype) {
    case MBX_I16: return sort_impl<int16_t>((const int16_t*)x, n, end_bit, (int16_t*)keys_out, (int16_t*)perm_out, scratch, scratch_bytes, s);
    case MBX_I32: return sort_impl<int32_t>((const int32_t*)x, n, end_bit, (int32_t*)keys_out, (int32_t*)perm_out, scratch, scratch_bytes, s);
    case MBX_I64: return sort_impl<int64_t>((const int64_t*)x, n, end_bit, (int64_t*)keys_out, (int64_t*)perm_out, scratch, scratch_bytes, s);
  }
  return MBX_EINVAL;
}

int mbx_route(const int32_t* expert_ids, int64_t n, int num_experts, int end_bit, int pad, int32_t* indices,
              int32_t* bin_ids, int32_t* tokens_per_expert, int32_t* bins, int32_t* padded_bins, int32_t* slot_rows,
              void* scratch, size_t scratch_bytes, mbx_stream_t stream) {
  if (n < 0 || num_experts <= 0 || end_bit <= 0 || pad < 0) return MBX_EINVAL;
  // one 8-bit pass whose digits are the expert ids themselves
  if (end_bit > kRadixBits || num_experts > (1 << end_bit)) return MBX_EUNSUPPORTED;
  if (!tokens_per_expert || !bins || (pad > 0 && !padded_bins)) return MBX_EINVAL;
  if (n > 0 && (!expert_ids || !indices || !bin_ids)) return MBX_EINVAL;
  if (n > 0x7fffffff - kSortTile) return MBX_ERANGE;
  hipStream_t s = as_stream(stream);
  const int nblocks = n > 0 ? (int)ceil_div(n, kSortTile) : 1;
  if (scratch_bytes < (size_t)kRadix * nblocks * sizeof(int32_t) || scratch == nullptr) return MBX_ESCRATCH;
  int32_t* counts = (int32_t*)scratch;
  const uint32_t mask = (1u << end_bit) - 1u;
  const int ndigits = 1 << end_bit;
  // (n = 0: a table of zeros makes every count and bound zero)
  radix_count_kernel<int32_t><<<nblocks, kSortThreads, 0, s>>>(expert_ids, n, 0, mask, end_bit, counts, nblocks);
  route_scan_kernel<<<1, 1024, 0, s>>>(counts, ndigits, nblocks, (int32_t)n, num_experts, pad, tokens_per_expert, bins,
                                       pad > 0 ? padded_bins : nullptr);
  if (n > 0)
    radix_scatter_kernel<int32_t, true><<<nblocks, kSortThreads, 0, s>>>(expert_ids, nullptr, n, 0, mask, end_bit, counts, nblocks,
                                                                        bin_ids, indices, slot_rows, bins,
                                                                        pad > 0 ? padded_bins : nullptr, num_experts);
  return launch_status();
}

int mbx_cumsum(const void* x, int itype, int64_t rows, int64_t n, int exclusive, void* out, mbx_stream_t stream) {
  if (rows < 0 || n < 0) return MBX_EINVAL;
  if (rows == 0 || n == 0) return 0;
  if (!x || !out) return MBX_EINVAL;
  if (rows > 0x7fffffff) return MBX_ERANGE;
  hipStream_t s = as_stream(stream);
  switch (itype) {
    case MBX_I16: cumsum_kernel<int16_t><<<(unsigned)rows, 256, 0, s>>>((const int16_t*)x, n, exclusive, (int16_t*)out); break;
    case MBX_I32: cumsum_kernel<int32_t><<<(unsigned)rows, 256, 0, s>>>((const int32_t*)x, n, exclusive, (int32_t*)out); break;
    case MBX_I64: cumsum_kernel<int64_t><<<(unsigned)rows, 256, 0, s>>>((const int64_t*)x, n, exclusive, (int64_t*)out); break;
    default: return MBX_EINVAL;
  }
  return launch_status();
}

int mbx_topology(const int32_t* padded_bins, int num_bins, int block_size, int block_rows, int block_cols, int16_t* out,
                 mbx_stream_t stream) {
  if (num_bins < 0 || block_size <= 0 || block_rows < 0 || block_cols < 0) return MBX_EINVAL;
  const int64_t total = (int64_t)block_rows * block_cols;
  if (total == 0) return 0;
  if (!out || (!padded_bins && num_bins > 0)) return MBX_EINVAL;
  int64_t blocks = ceil_div(total, 256);
  if (blocks > 4096) blocks = 4096;
  topology_kernel<<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(padded_bins, num_bins, block_size, block_rows, block_cols, out);
  return launch_status();
}

int mbx_replicate_forward(const void* x, int elem_bytes, int64_t batch, int num_bins, const int32_t* bins, void* out,
                          int64_t columns, mbx_stream_t stream) {
  if (batch < 0 || num_bins < 0 || columns < 0) return MBX_EINVAL;
  if (batch == 0 || num_bins == 0 || columns == 0) return 0;
  if (!x || !bins || !out) return MBX_EINVAL;
  if (batch > 65535) return MBX_ERANGE;
  dim3 grid((unsigned)num_bins, (unsigned)batch);
  hipStream_t s = as_stream(stream);
  if (elem_bytes == 2) replicate_forward_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)x, num_bins, bins, (uint16_t*)out, columns);
  else if (elem_bytes == 4) replicate_forward_kernel<uint32_t><<<grid, 256, 0, s>>>((const uint32_t*)x, num_bins, bins, (uint32_t*)out, columns);
  else return MBX_EINVAL;
  return launch_status();
}

int mbx_replicate_backward(const void* grad, int dtype, int64_t batch, int64_t columns, const int32_t* bins, int num_bins,
                           void* out, mbx_stream_t stream) {
  if (batch < 0 || num_bins < 0 || columns < 0) return MBX_EINVAL;
  if (batch == 0 || num_bins == 0) return 0;
  if (!bins || !out || (!grad && columns > 0)) return MBX_EINVAL;
  if (batch > 65535) return MBX_ERANGE;
  dim3 grid((unsigned)num_bins, (unsigned)batch);
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case MBX_BF16: replicate_backward_kernel<MBX_BF16><<<grid, 256, 0, s>>>(grad, columns, bins, num_bins, out); break;
    case MBX_F16: replicate_backward_kernel<MBX_F16><<<grid, 256, 0, s>>>(grad, columns, bins, num_bins, out); break;
    case MBX_F32: replicate_backward_kernel<MBX_F32><<<grid, 256, 0, s>>>(grad, columns, bins, num_bins, out); break;
    default: return MBX_EINVAL;
  }
  return launch_status();
}

}  // extern "C"
