// Router post-processing: softmax over the experts, top-k selection and the optional p-norm
// renormalisation of the selected weights in one kernel, and their backward in another
// (megablocks/layers/router.py:87-106).  One wave per token; lane l holds experts l, l + 64, ...
#include "common.h"

namespace mbx {
namespace {

constexpr int kTokenThreads = 256;
constexpr int kTokenWaves = kTokenThreads / kWave;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// ||w||_p of the first top_k lanes' values (p > 0)
__device__ __forceinline__ float wave_pnorm(float w, bool live, float p) {
  const float a = fabsf(w);
  float term = 0.f;
  if (live) term = p == 1.f ? a : (p == 2.f ? a * a : powf(a, p));
  const float sum = wave_sum(term);
  return p == 1.f ? sum : (p == 2.f ? sqrtf(sum) : powf(sum, 1.f / p));
}

// scores = softmax(logits) rounded to the storage type (computed in fp32: exp(x - max) / sum, as
// torch's softmax does for 16-bit inputs); the k largest rounded scores in descending order, ties to the
// lower expert index (NaN scores first); weights = those scores, divided by their rounded p-norm if p > 0
// (each of torch's two operations rounds to the storage type).
template <int DT, int R>
__global__ void __launch_bounds__(kTokenThreads)
router_forward_kernel(const void* __restrict__ logits_, int64_t tokens, int num_experts, int top_k, float p,
                      void* __restrict__ scores_, void* __restrict__ weights_, int64_t* __restrict__ indices,
                      int32_t* __restrict__ indices32, float* __restrict__ lse) {
  typedef typename Elem<DT>::type E;
  const E* logits = (const E*)logits_;
  E* scores = (E*)scores_;
  E* weights = (E*)weights_;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t t = (int64_t)blockIdx.x * kTokenWaves + wave; t < tokens; t += (int64_t)gridDim.x * kTokenWaves) {
    const E* row = logits + t * num_experts;
    float x[R];
    float m = -INFINITY;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int e = lane + r * kWave;
      x[r] = e < num_experts ? Elem<DT>::to_f32(row[e]) : -INFINITY;
      m = fmaxf(m, x[r]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      x[r] = lane + r * kWave < num_experts ? expf(x[r] - m) : 0.f;
      sum += x[r];
    }
    sum = wave_sum(sum);
    // logsumexp of the row, the term of the router z-loss (router.py:37): an infinite maximum is the result itself
    if (lse && lane == 0) lse[t] = (m == INFINITY || m == -INFINITY) ? m : m + logf(sum);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int e = lane + r * kWave;
      const E s = Elem<DT>::from_f32(x[r] / sum);
      if (e < num_experts) scores[t * num_experts + e] = s;
      // The selection key: the rounded score; -1 marks "not a candidate" (scores are >= 0).  A NaN score (a NaN
      // or +inf logit makes the whole row NaN) ranks above every number, as torch.topk ranks it, so that the
      // indices written are always experts: +inf, which no score can be, stands for it.
      const float v = Elem<DT>::to_f32(s);
      x[r] = e < num_experts ? (v != v ? INFINITY : v) : -1.f;
    }
    float my_w = 0.f;
    int my_i = 0;
    for (int j = 0; j < top_k; ++j) {
      float best = -1.f;
      int best_e = 0x7fffffff;
#pragma unroll
      for (int r = 0; r < R; ++r)   // ascending expert index: a later equal value does not replace an earlier one
        if (x[r] > best) { best = x[r]; best_e = lane + r * kWave; }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oe = __shfl_xor(best_e, off, 64);
        if (ov > best || (ov == best && oe < best_e)) { best = ov; best_e = oe; }
      }
      if (lane == j) { my_w = best == INFINITY ? NAN : best; my_i = best_e; }
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (lane + r * kWave == best_e) x[r] = -1.f;
    }
    const bool live = lane < top_k;
    if (p > 0.f) {
      const float norm = Elem<DT>::to_f32(Elem<DT>::from_f32(wave_pnorm(my_w, live, p)));
      my_w = my_w / norm;
    }
    if (live) {
      weights[t * top_k + lane] = Elem<DT>::from_f32(my_w);
      indices[t * top_k + lane] = my_i;
      if (indices32) indices32[t * top_k + lane] = my_i;   // what the routing kernels take, without a cast pass
    }
  }
}

// grad_logits = d(loss)/d(logits) given d/d(weights) (and optionally d/d(scores) from other users of the
// scores, e.g. a load-balancing loss): through the p-norm division, the selection (a scatter to the chosen
// experts) and the softmax, in fp32 from the rounded forward values.  grad_lse (optional): d/d(logsumexp of the
// row), whose gradient with respect to the logits is the softmax itself.
template <int DT, int R>
__global__ void __launch_bounds__(kTokenThreads)
router_backward_kernel(const void* __restrict__ grad_weights_, const void* __restrict__ grad_scores_,
                       const void* __restrict__ scores_, const int64_t* __restrict__ indices, int64_t tokens,
                       int num_experts, int top_k, float p, void* __restrict__ grad_logits_,
                       const float* __restrict__ grad_lse) {
  typedef typename Elem<DT>::type E;
  const E* grad_weights = (const E*)grad_weights_;
  const E* grad_scores = (const E*)grad_scores_;
  const E* scores = (const E*)scores_;
  E* grad_logits = (E*)grad_logits_;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t t = (int64_t)blockIdx.x * kTokenWaves + wave; t < tokens; t += (int64_t)gridDim.x * kTokenWaves) {
    float s[R], ds[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int e = lane + r * kWave;
      s[r] = e < num_experts ? Elem<DT>::to_f32(scores[t * num_experts + e]) : 0.f;
      ds[r] = (grad_scores && e < num_experts) ? Elem<DT>::to_f32(grad_scores[t * num_experts + e]) : 0.f;
    }
    if (grad_weights) {
      const bool live = lane < top_k;
      int my_i = live ? (int)indices[t * top_k + lane] : 0;
      if (my_i < 0 || my_i >= num_experts) my_i = 0;
      const float dy = live ? Elem<DT>::to_f32(grad_weights[t * top_k + lane]) : 0.f;
      const float w = live ? Elem<DT>::to_f32(scores[t * num_experts + my_i]) : 0.f;   // the weight before the division
      float dw = dy;
      if (p > 0.f) {
        // y = w / n, n = ||w||_p:  dw_j = dy_j / n - (sum_i dy_i w_i) / n^2 * (w_j / n)^(p - 1)
        const float n = Elem<DT>::to_f32(Elem<DT>::from_f32(wave_pnorm(w, live, p)));
        const float dot = wave_sum(dy * w);
        const float dn = p == 1.f ? 1.f : (p == 2.f ? w / n : powf(w / n, p - 1.f));
        dw = dy / n - dot / (n * n) * dn;
      }
      for (int j = 0; j < top_k; ++j) {
        const int e = __shfl(my_i, j, 64);
        const float v = __shfl(dw, j, 64);
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (lane + r * kWave == e) ds[r] += v;
      }
    }
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) dot += ds[r] * s[r];
    dot = wave_sum(dot);
    const float gl = grad_lse ? grad_lse[t] : 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int e = lane + r * kWave;
      if (e < num_experts) grad_logits[t * num_experts + e] = Elem<DT>::from_f32(s[r] * (ds[r] - dot + gl));
    }
  }
}

static inline unsigned token_grid(int64_t tokens) {
  int64_t blocks = ceil_div(tokens, kTokenWaves);
  if (blocks > 256 * 8) blocks = 256 * 8;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}

#define MBX_ROUTER_DISPATCH(KERNEL, ...)                                                              \
  do {                                                                                                \
    const unsigned grid = token_grid(tokens);                                                         \
    const int per_lane = (num_experts + kWave - 1) / kWave;                                           \
    switch (dtype) {                                                                                  \
      case MBX_BF16:                                                                                  \
        if (per_lane <= 1) KERNEL<MBX_BF16, 1><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);           \
        else if (per_lane <= 2) KERNEL<MBX_BF16, 2><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);      \
        else if (per_lane <= 4) KERNEL<MBX_BF16, 4><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);      \
        else KERNEL<MBX_BF16, 8><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);                         \
        break;                                                                                        \
      case MBX_F16:                                                                                   \
        if (per_lane <= 1) KERNEL<MBX_F16, 1><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);            \
        else if (per_lane <= 2) KERNEL<MBX_F16, 2><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);       \
        else if (per_lane <= 4) KERNEL<MBX_F16, 4><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);       \
        else KERNEL<MBX_F16, 8><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);                          \
        break;                                                                                        \
      default:                                                                                        \
        if (per_lane <= 1) KERNEL<MBX_F32, 1><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);            \
        else if (per_lane <= 2) KERNEL<MBX_F32, 2><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);       \
        else if (per_lane <= 4) KERNEL<MBX_F32, 4><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);       \
        else KERNEL<MBX_F32, 8><<<grid, kTokenThreads, 0, s>>>(__VA_ARGS__);                          \
        break;                                                                                        \
    }                                                                                                 \
  } while (0)

constexpr int kMaxRouterExperts = 8 * kWave;

}  // namespace
}  // namespace mbx

using namespace mbx;

extern "C" {

int mbx_router_forward(const void* logits, int dtype, int64_t tokens, int num_experts, int top_k, float norm_p,
                       void* scores, void* weights, int64_t* indices, int32_t* indices32, float* lse,
                       mbx_stream_t stream) {
  if (tokens < 0 || num_experts <= 0 || top_k <= 0 || top_k > num_experts || !(norm_p >= 0.f)) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (num_experts > kMaxRouterExperts || top_k > kWave) return MBX_EUNSUPPORTED;
  if (tokens == 0) return 0;
  if (!logits || !scores || !weights || !indices) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  MBX_ROUTER_DISPATCH(router_forward_kernel, logits, tokens, num_experts, top_k, norm_p, scores, weights, indices, indices32, lse);
  return launch_status();
}

int mbx_router_backward(const void* grad_weights, const void* grad_scores, const void* scores, const int64_t* indices,
                        int dtype, int64_t tokens, int num_experts, int top_k, float norm_p, void* grad_logits,
                        const float* grad_lse, mbx_stream_t stream) {
  if (tokens < 0 || num_experts <= 0 || top_k <= 0 || top_k > num_experts || !(norm_p >= 0.f)) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (num_experts > kMaxRouterExperts || top_k > kWave) return MBX_EUNSUPPORTED;
  if (tokens == 0) return 0;
  if (!scores || !grad_logits || (grad_weights && !indices)) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  MBX_ROUTER_DISPATCH(router_backward_kernel, grad_weights, grad_scores, scores, indices, tokens, num_experts, top_k,
                      norm_p, grad_logits, grad_lse);
  return launch_status();
}

}  // extern "C"
