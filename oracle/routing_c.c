/*
 * CPU oracle, plain C: the integer routing ops of databricks/megablocks' dMoE path.
 *
 * TEST INFRASTRUCTURE ONLY: a second, independent restatement beside oracle/routing.py, written as the
 * textbook algorithms rather than library calls.  tests/ compares the two with each other and with the
 * GPU library; nothing in megablocks_amd links or loads it.  Keys and counts travel as int64.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* csrc/histogram.h:20-81 (cub::DeviceHistogram::HistogramEven over [0, num_bins), row by row):
 * out[r, b] = #{c : x[r, c] == b}; values outside the range are counted nowhere. */
void mbxo_histogram(const int64_t* x, int64_t rows, int64_t n, int64_t num_bins, int32_t* out) {
  for (int64_t r = 0; r < rows; ++r) {
    int32_t* o = out + r * num_bins;
    for (int64_t b = 0; b < num_bins; ++b) o[b] = 0;
    for (int64_t c = 0; c < n; ++c) {
      const int64_t v = x[r * n + c];
      if (v >= 0 && v < num_bins) ++o[v];
    }
  }
}

/* megablocks/ops/sort.py:26-38 + csrc/sort.h:20-86 (cub::DeviceRadixSort::SortPairs with an iota payload):
 * stable least-significant-digit radix sort, one bit per pass, on bits [0, end_bit) of keys that are
 * `width` bits wide; in the pass over the sign bit (end_bit == width) the two buckets swap, which gives
 * the signed order.  keys_out[i] = x[perm_out[i]].  Returns 0, or -1 if out of memory. */
int mbxo_sort(const int64_t* x, int64_t n, int end_bit, int width, int64_t* keys_out, int64_t* perm_out) {
  int64_t* tmp = (int64_t*)malloc((size_t)(n > 0 ? n : 1) * sizeof(int64_t));
  if (!tmp) return -1;
  for (int64_t i = 0; i < n; ++i) perm_out[i] = i;
  for (int bit = 0; bit < end_bit && bit < width; ++bit) {
    const int sign_pass = bit == width - 1;
    int64_t zeros = 0;
    for (int64_t i = 0; i < n; ++i) zeros += !(((uint64_t)x[perm_out[i]] >> bit) & 1u);
    /* first bucket: bit clear (bit set in the sign pass: negative keys sort first) */
    int64_t lo = 0, hi = sign_pass ? n - zeros : zeros;
    for (int64_t i = 0; i < n; ++i) {
      const int set = (int)(((uint64_t)x[perm_out[i]] >> bit) & 1u);
      if (set == sign_pass) tmp[lo++] = perm_out[i];
      else tmp[hi++] = perm_out[i];
    }
    memcpy(perm_out, tmp, (size_t)n * sizeof(int64_t));
  }
  for (int64_t i = 0; i < n; ++i) keys_out[i] = x[perm_out[i]];
  free(tmp);
  return 0;
}

/* csrc/cumsum.h:66-156: inclusive / exclusive scan of every row, wrapping in the element width. */
void mbxo_cumsum(const int64_t* x, int64_t rows, int64_t n, int exclusive, int width, int64_t* out) {
  for (int64_t r = 0; r < rows; ++r) {
    uint64_t acc = 0;
    for (int64_t c = 0; c < n; ++c) {
      const uint64_t v = (uint64_t)x[r * n + c];
      const uint64_t res = exclusive ? acc : acc + v;
      acc += v;
      int64_t s = (int64_t)res;
      if (width == 16) s = (int16_t)res;
      if (width == 32) s = (int32_t)res;
      out[r * n + c] = s;
    }
  }
}

/* csrc/indices.h:21-49 (ConstructIndicesKernel): column indices of the block-diagonal topology; the
 * block-rows of expert e list columns e*block_cols .. e*block_cols + block_cols - 1; block-rows past the
 * last bin are zero. */
void mbxo_topology(const int32_t* padded_bins, int64_t num_bins, int64_t block_size, int64_t block_rows,
                   int64_t block_cols, int16_t* out) {
  for (int64_t i = 0; i < block_rows * block_cols; ++i) out[i] = 0;
  int64_t start = 0;
  for (int64_t e = 0; e < num_bins; ++e) {
    const int64_t end = padded_bins[e] / block_size;
    for (int64_t br = start; br < end && br < block_rows; ++br)
      for (int64_t bc = 0; bc < block_cols; ++bc) out[br * block_cols + bc] = (int16_t)(e * block_cols + bc);
    start = end;
  }
}

/* csrc/replicate.h:21-61: out[b, bins[i-1]:bins[i]] = x[b, i] (int64 payload); columns at or past
 * bins[-1] are zero. */
void mbxo_replicate(const int64_t* x, int64_t batch, int64_t num_bins, const int32_t* bins, int64_t columns,
                    int64_t* out) {
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t c = 0; c < columns; ++c) out[b * columns + c] = 0;
    int64_t start = 0;
    for (int64_t i = 0; i < num_bins; ++i) {
      for (int64_t c = start; c < bins[i] && c < columns; ++c) out[b * columns + c] = x[b * num_bins + i];
      start = bins[i];
    }
  }
}

/* megablocks/layers/moe.py:152-183 + dmoe.py:131-154 (indices_and_bins / indices_and_padded_bins):
 * stable sort of the expert ids on `end_bit` bits, per-expert counts, inclusive bins, and the bins of the
 * counts rounded up to `blocking` (ops/round_up.py:14) when blocking > 0. */
int mbxo_route(const int64_t* top_expert, int64_t n, int64_t num_experts, int end_bit, int64_t blocking,
               int64_t* bin_ids, int64_t* indices, int32_t* tokens_per_expert, int32_t* bins, int32_t* padded_bins) {
  if (mbxo_sort(top_expert, n, end_bit, 32, bin_ids, indices)) return -1;
  mbxo_histogram(top_expert, 1, n, num_experts, tokens_per_expert);
  int64_t acc = 0, pacc = 0;
  for (int64_t e = 0; e < num_experts; ++e) {
    acc += tokens_per_expert[e];
    bins[e] = (int32_t)acc;
    if (blocking > 0) {
      pacc += (tokens_per_expert[e] + blocking - 1) / blocking * blocking;
      padded_bins[e] = (int32_t)pacc;
    }
  }
  return 0;
}
