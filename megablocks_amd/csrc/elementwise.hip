// Element-wise kernels of the expert MLPs: the gated activation act(a) * b of the GLU experts
// and its backward, one HBM pass each (128-bit loads and stores).
#include "common.h"

namespace mbx {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int DT> struct Pack {  // 16 bytes of storage <-> fp32 values
  static constexpr int N = 16 / (int)sizeof(typename Elem<DT>::type);
  static __device__ __forceinline__ void load(const void* p, int64_t vec, float* f) {
    // every byte of these tensors is touched once per pass and they are far larger than the caches
    const u32x4 v = __builtin_nontemporal_load((const u32x4*)p + vec);
    const typename Elem<DT>::type* e = (const typename Elem<DT>::type*)&v;
#pragma unroll
    for (int i = 0; i < N; ++i) f[i] = Elem<DT>::to_f32(e[i]);
  }
  static __device__ __forceinline__ void store(void* p, int64_t vec, const float* f) {
    u32x4 v;
    typename Elem<DT>::type* e = (typename Elem<DT>::type*)&v;
#pragma unroll
    for (int i = 0; i < N; ++i) e[i] = Elem<DT>::from_f32(f[i]);
    __builtin_nontemporal_store(v, (u32x4*)p + vec);
  }
};

template <int DT>
__device__ __forceinline__ float round_to(float f) { return Elem<DT>::to_f32(Elem<DT>::from_f32(f)); }

enum { ACT_SILU = 0, ACT_GELU_TANH = 1 };

template <int ACT>
__device__ __forceinline__ float act_fwd(float x) {
  if (ACT == ACT_SILU) return x / (1.f + __expf(-x));
  const float t = tanhf(0.7978845608028654f * x * (1.f + 0.044715f * x * x));
  return 0.5f * x * (1.f + t);
}

template <int ACT>
__device__ __forceinline__ float act_grad(float x) {
  if (ACT == ACT_SILU) {
    const float s = 1.f / (1.f + __expf(-x));
    return s * (1.f + x * (1.f - s));
  }
  const float t = tanhf(0.7978845608028654f * x * (1.f + 0.044715f * x * x));
  return 0.5f * x * ((1.f - t * t) * (0.7978845608028654f + 0.1070322243f * x * x)) + 0.5f * (1.f + t);
}

// out = round(round(act(a)) * b): the two roundings of computing act(a) and the product separately
template <int DT, int ACT>
__global__ void __launch_bounds__(256) glu_forward_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                          void* __restrict__ out, int64_t nvec) {
  constexpr int N = Pack<DT>::N;
  int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; v < nvec; v += stride) {
    float fa[N], fb[N], fo[N];
    Pack<DT>::load(a, v, fa);
    Pack<DT>::load(b, v, fb);
#pragma unroll
    for (int i = 0; i < N; ++i) fo[i] = round_to<DT>(act_fwd<ACT>(fa[i])) * fb[i];
    Pack<DT>::store(out, v, fo);
  }
}

// db = g * round(act(a));  da = round(g * b) * act'(a)      (the roundings autograd's two steps make)
template <int DT, int ACT>
__global__ void __launch_bounds__(256) glu_backward_kernel(const void* __restrict__ g, const void* __restrict__ a,
                                                           const void* __restrict__ b, void* __restrict__ da,
                                                           void* __restrict__ db, int64_t nvec) {
  constexpr int N = Pack<DT>::N;
  int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; v < nvec; v += stride) {
    float fg[N], fa[N], fb[N], fda[N], fdb[N];
    Pack<DT>::load(g, v, fg);
    Pack<DT>::load(a, v, fa);
    Pack<DT>::load(b, v, fb);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      fdb[i] = fg[i] * round_to<DT>(act_fwd<ACT>(fa[i]));
      fda[i] = round_to<DT>(fg[i] * fb[i]) * act_grad<ACT>(fa[i]);
    }
    Pack<DT>::store(da, v, fda);
    Pack<DT>::store(db, v, fdb);
  }
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

static inline unsigned ew_grid(int64_t nvec) {
  int64_t blocks = ceil_div(nvec, 256);
  if (blocks > 256 * 8) blocks = 256 * 8;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}

}  // namespace
}  // namespace mbx

using namespace mbx;

#define MBX_DISPATCH_DT_ACT(dtype, act, CALL)                                  \
  switch ((dtype) * 2 + (act)) {                                               \
    case MBX_BF16 * 2 + ACT_SILU: CALL(MBX_BF16, ACT_SILU); break;             \
    case MBX_BF16 * 2 + ACT_GELU_TANH: CALL(MBX_BF16, ACT_GELU_TANH); break;   \
    case MBX_F16 * 2 + ACT_SILU: CALL(MBX_F16, ACT_SILU); break;               \
    case MBX_F16 * 2 + ACT_GELU_TANH: CALL(MBX_F16, ACT_GELU_TANH); break;     \
    case MBX_F32 * 2 + ACT_SILU: CALL(MBX_F32, ACT_SILU); break;               \
    case MBX_F32 * 2 + ACT_GELU_TANH: CALL(MBX_F32, ACT_GELU_TANH); break;     \
    default: return MBX_EINVAL;                                                \
  }

extern "C" {

int mbx_glu_forward(const void* a, const void* b, void* out, int dtype, int act, int64_t numel, mbx_stream_t stream) {
  if (numel < 0 || (act != ACT_SILU && act != ACT_GELU_TANH)) return MBX_EINVAL;
  if (numel == 0) return 0;
  if (!a || !b || !out) return MBX_EINVAL;
  const int per = 16 / dtype_bytes(dtype);
  if (numel % per != 0 || !aligned16(a) || !aligned16(b) || !aligned16(out)) return MBX_EINVAL;
  const int64_t nvec = numel / per;
  hipStream_t s = as_stream(stream);
#define CALL(DT, ACT) glu_forward_kernel<DT, ACT><<<ew_grid(nvec), 256, 0, s>>>(a, b, out, nvec)
  MBX_DISPATCH_DT_ACT(dtype, act, CALL)
#undef CALL
  return launch_status();
}

int mbx_glu_backward(const void* g, const void* a, const void* b, void* da, void* db, int dtype, int act, int64_t numel,
                     mbx_stream_t stream) {
  if (numel < 0 || (act != ACT_SILU && act != ACT_GELU_TANH)) return MBX_EINVAL;
  if (numel == 0) return 0;
  if (!g || !a || !b || !da || !db) return MBX_EINVAL;
  const int per = 16 / dtype_bytes(dtype);
  if (numel % per != 0 || !aligned16(g) || !aligned16(a) || !aligned16(b) || !aligned16(da) || !aligned16(db)) return MBX_EINVAL;
  const int64_t nvec = numel / per;
  hipStream_t s = as_stream(stream);
#define CALL(DT, ACT) glu_backward_kernel<DT, ACT><<<ew_grid(nvec), 256, 0, s>>>(g, a, b, da, db, nvec)
  MBX_DISPATCH_DT_ACT(dtype, act, CALL)
#undef CALL
  return launch_status();
}

}  // extern "C"
