// Grouped GEMM for variable per-expert row counts on gfx950 matrix cores.
//
//   NN: c[r_e] = a[r_e] @ b[e]        NT: c[r_e] = a[r_e] @ b[e]^T       TN: c[e] = a[r_e]^T @ b[r_e]
//
// Two implementations.  The product path is the direct-to-LDS kernels of gmm_dma.h (v_mfma_f32_16x16x32, LDS rings
// filled by buffer_load ... lds, persistent workgroups with an XCD-aware tile schedule).  This file holds their launch
// logic, and, for the shapes they do not take, a register-staged kernel (v_mfma_f32_32x32x16, operand tiles loaded
// into registers, stored to a double-buffered LDS tile) and an element-wise kernel for any shape, alignment and fp32.
// In all of them an operand whose reduction dimension is contiguous in memory ("KC": a in NN/NT, b in NT) is kept as
// [row][k] in LDS and read with 128-bit LDS loads; an operand whose reduction dimension is
// strided ("MC": b in NN, both in TN) is kept as [k][col] and read with the gfx950
// transposing LDS load (ds_read_b64_tr_b16), which hands every lane the four k-consecutive
// values of its column.  The tile -> (expert, row tile) schedule is computed on the device
// from the inclusive row bins, so no host copy of the group sizes is needed and empty
// experts cost nothing (NN/NT) or produce an all-zero block (TN).
#include "common.h"

#include <cstdlib>

namespace mbx {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ f32x16 mfma32(const u32x4& a, const u32x4& b, const f32x16& c) {
  if (DT == MBX_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ f32x4 mfma16(const u32x4& a, const u32x4& b, const f32x4& c) {
  if (DT == MBX_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// One operand of the product as seen by a workgroup.
struct Operand {
  const uint16_t* base;  // element (row, k) of a KC operand is base[row * ld + k];
                         // element (k, col) of an MC operand is base[k * ld + col]
  int64_t ld;
  int r0;      // first row (KC) / column (MC) of the tile in the non-reduction dimension
  int r_lim;   // bound of that dimension (rows are clamped, columns are zero-filled)
};

template <int BM_, int BN_, int BK_, int WM_, int WN_, int PAD_KC_, int PAD_MC_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int PAD_KC = PAD_KC_, PAD_MC = PAD_MC_;
  static constexpr int THREADS = WM * WN * kWave;
  static constexpr int WTM = BM / WM, WTN = BN / WN;   // tile of one wave
  static constexpr int TM = WTM / 32, TN = WTN / 32;    // 32x32 MFMA tiles per wave
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % 16 == 0, "tile shape");
};

// LDS footprint (in elements) of one operand tile with R non-reduction rows/columns.
template <bool MC, int R, int BK, int PAD_KC, int PAD_MC>
struct OperandLds {
  static constexpr int STRIDE = MC ? (R + PAD_MC) : (BK + PAD_KC);
  static constexpr int ELEMS = MC ? BK * STRIDE : R * STRIDE;
};

// Global -> registers: every thread fetches CH 16-byte chunks of the operand tile.
template <bool MC, int R, int BK, int THREADS>
struct Stager {
  static constexpr int CHUNKS = R * BK / 8;
  static constexpr int CH = CHUNKS / THREADS;
  static_assert(CHUNKS % THREADS == 0, "tile must split evenly over the threads");

  // Always loads from an in-bounds (clamped) address and zeroes what lies outside the operand, so
  // the loop body has no branches: the loads of the tile after the last one are redundant, not wild.
  static __device__ __forceinline__ void load(const Operand& op, int k0, int k_begin, int k_end, u32x4 (&reg)[CH]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * THREADS;
      const u32x4 zero = {0u, 0u, 0u, 0u};
      if (!MC) {
        const int r = c / (BK / 8), kc = (c % (BK / 8)) * 8;
        int row = op.r0 + r;
        if (row > op.r_lim - 1) row = op.r_lim - 1;
        int kk = k0 + kc;
        const bool ok = kk < k_end;
        if (kk > k_end - 8) kk = k_end - 8;
        if (kk < k_begin) kk = k_begin;
        const u32x4 v = *(const u32x4*)(op.base + (int64_t)row * op.ld + kk);
        reg[i] = ok ? v : zero;
      } else {
        const int kr = c / (R / 8), rc = (c % (R / 8)) * 8;
        int kk = k0 + kr, col = op.r0 + rc;
        const bool ok = kk < k_end && col < op.r_lim;
        if (kk > k_end - 1) kk = k_end - 1;
        if (kk < k_begin) kk = k_begin;
        if (col > op.r_lim - 8) col = op.r_lim - 8;
        const u32x4 v = *(const u32x4*)(op.base + (int64_t)kk * op.ld + col);
        reg[i] = ok ? v : zero;
      }
    }
  }

  template <int STRIDE>
  static __device__ __forceinline__ void store(uint16_t* lds, const u32x4 (&reg)[CH]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * THREADS;
      if (!MC) {
        const int r = c / (BK / 8), kc = (c % (BK / 8)) * 8;
        *(u32x4*)(lds + r * STRIDE + kc) = reg[i];
      } else {
        const int kk = c / (R / 8), rc = (c % (R / 8)) * 8;
        *(u32x4*)(lds + kk * STRIDE + rc) = reg[i];
      }
    }
  }
};

// LDS -> MFMA operand registers for the 32 rows/columns starting at `r` and k-step `ks`.
template <bool MC, int STRIDE>
__device__ __forceinline__ u32x4 read_frag(const uint16_t* lds, int r, int ks) {
  const int lane = lane_id();
  if (!MC) {
    return *(const u32x4*)(lds + (r + (lane & 31)) * STRIDE + ks * 16 + (lane >> 5) * 8);
  } else {
    const int g = lane >> 4, s = lane & 15;
    const uint16_t* p = lds + (ks * 16 + (g >> 1) * 8 + (s >> 2)) * STRIDE + r + (g & 1) * 16 + (s & 3) * 4;
    typedef __attribute__((address_space(3))) s16x4_t* lds_ptr_t;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p + 4 * STRIDE));
    u32x4 v;
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    v[0] = l2[0]; v[1] = l2[1]; v[2] = h2[0]; v[3] = h2[1];
    return v;
  }
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  const f32x2_t v = {a, b};
  if (DT == MBX_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));  // v_cvt_pk_bf16_f32, RNE
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

// The workgroup-level product: acc += A_tile(k) * B_tile(k) over k in [k_begin, k_end),
// then c[m0.., n0..] = acc for rows < m_lim and columns < n_lim.
template <int DT, bool A_MC, bool B_MC, typename T>
__device__ __forceinline__ void block_gemm(const Operand& opa, const Operand& opb, int k_begin, int k_end,
                                           uint16_t* __restrict__ c, int64_t ldc, int m_lim, int n_lim, uint16_t* lds) {
  typedef OperandLds<A_MC, T::BM, T::BK, T::PAD_KC, T::PAD_MC> LA;
  typedef OperandLds<B_MC, T::BN, T::BK, T::PAD_KC, T::PAD_MC> LB;
  typedef Stager<A_MC, T::BM, T::BK, T::THREADS> SA;
  typedef Stager<B_MC, T::BN, T::BK, T::THREADS> SB;
  constexpr int STAGE = LA::ELEMS + LB::ELEMS;

  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int wm = (wave / T::WN) * T::WTM, wn = (wave % T::WN) * T::WTN;

  f32x16 acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (k_end - k_begin + T::BK - 1) / T::BK;
  constexpr int KS = T::BK / 16;
  static_assert(KS % 2 == 0, "the operand double buffer assumes an even number of k-steps per tile");
  u32x4 ra[SA::CH], rb[SB::CH];
  u32x4 fa[2][T::TM], fb[2][T::TN];   // MFMA operands, double buffered across k-steps

  auto read_frags = [&](const uint16_t* stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i) fa[buf][i] = read_frag<A_MC, LA::STRIDE>(stage, wm + i * 32, ks);
#pragma unroll
    for (int j = 0; j < T::TN; ++j) fb[buf][j] = read_frag<B_MC, LB::STRIDE>(stage + LA::ELEMS, wn + j * 32, ks);
  };
  // operands swapped: the accumulator tile is c^T, so a lane owns runs of four consecutive
  // columns of one row of c and can store them as one 8-byte word.
  auto multiply = [&](int buf) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        acc[i][j] = mfma32<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
      }
  };

  if (nk > 0) {
    SA::load(opa, k_begin, k_begin, k_end, ra);
    SB::load(opb, k_begin, k_begin, k_end, rb);
    SA::template store<LA::STRIDE>(lds, ra);
    SB::template store<LB::STRIDE>(lds + LA::ELEMS, rb);
    __syncthreads();
    read_frags(lds, 0, 0);
  }
  // Per K tile: the global loads of the next tile are issued first and land in registers while
  // k-steps 0..KS-2 run; each k-step first issues the LDS reads of the following k-step, then
  // its MFMAs.  Before the last k-step the staged tile goes to the other LDS buffer, the
  // workgroup synchronises, and the first operands of the next tile are read, so that the
  // barrier and the LDS latency are covered by the MFMAs of the last k-step.
  for (int kt = 0; kt < nk; ++kt) {
    uint16_t* cur = lds + (kt & 1) * STAGE;
    uint16_t* nxt = lds + ((kt + 1) & 1) * STAGE;
    SA::load(opa, k_begin + (kt + 1) * T::BK, k_begin, k_end, ra);
    SB::load(opb, k_begin + (kt + 1) * T::BK, k_begin, k_end, rb);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      read_frags(cur, ks + 1, (ks + 1) & 1);
      multiply(ks & 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    SA::template store<LA::STRIDE>(nxt, ra);
    SB::template store<LB::STRIDE>(nxt + LA::ELEMS, rb);
    __syncthreads();
    read_frags(nxt, 0, KS & 1);
    multiply((KS - 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // accumulator (i, j), register r of lane l holds c[m][n] with
  //   m = opa.r0 + wm + 32 i + (l % 32),  n = opb.r0 + wn + 32 j + 8 (r / 4) + 4 (l / 32) + (r % 4)
  const bool n_vec = (ldc % 4 == 0) && (((uintptr_t)c & 7u) == 0);
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    const int m = opa.r0 + wm + i * 32 + (lane & 31);
    if (m >= m_lim) continue;
    uint16_t* crow = c + (int64_t)m * ldc;
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = opb.r0 + wn + j * 32 + q * 8 + (lane >> 5) * 4;
        const f32x16& v = acc[i][j];
        if (n + 3 < n_lim && n_vec) {
          u32x2 w;
          w[0] = pack2<DT>(v[q * 4 + 0], v[q * 4 + 1]);
          w[1] = pack2<DT>(v[q * 4 + 2], v[q * 4 + 3]);
          *(u32x2*)(crow + n) = w;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (n + t < n_lim) crow[n + t] = (uint16_t)(pack2<DT>(v[q * 4 + t], 0.f) & 0xffffu);
        }
      }
    }
  }
}

// Workgroups are dispatched to the 8 XCDs round-robin by workgroup id, and every XCD has its own
// L2.  The logical tile order is cut into runs of kXcdRun tiles and run r goes to XCD r % 8, so
// the workgroups resident on one XCD at a time form a compact block of tiles (same expert, a few
// row tiles x a few column tiles) whose operand panels are fetched into that L2 once.
constexpr int kXcds = 8;
constexpr int kXcdRun = 32;

__device__ __forceinline__ int xcd_tile_id(int block, int run = kXcdRun) {
  const int xcd = block % kXcds, l = block / kXcds;
  return ((l / run) * kXcds + xcd) * run + (l % run);
}

static inline int64_t xcd_grid(int64_t tiles, int run = kXcdRun) {
  const int64_t q = (int64_t)kXcds * run;
  return (tiles + q - 1) / q * q;
}

// A row bound read from the bins, kept inside [lo, rows]: a table that does not belong to the operands can make
// the result wrong but never an access out of range.
__device__ __forceinline__ int clamp_bound(int v, int lo, int rows) { return v < lo ? lo : (v > rows ? rows : v); }

// ---- NN / NT: row tiles follow the expert bins --------------------------------------
// Logical tile id -> (expert, column tile, row tile inside the expert), row tiles fastest.
template <int DT, bool B_MC, typename T>
__global__ void __launch_bounds__(T::THREADS)
gmm_rows_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
                const int32_t* __restrict__ bins, int num_groups, int rows, int k, int n, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  int id = xcd_tile_id(blockIdx.x);
  int e = 0, start = 0, end = 0, mt = 0;
  for (; e < num_groups; ++e) {
    end = clamp_bound(bins[e], start, rows);
    mt = (end - start + T::BM - 1) / T::BM;
    const int span = mt * tiles_n;
    if (id < span) break;
    id -= span;
    start = end;
  }
  if (e >= num_groups) return;  // surplus workgroup (uniform over the block)
  const int tn = id / mt, tm = id % mt;

  Operand opa, opb;
  opa.base = a; opa.ld = k; opa.r0 = start + tm * T::BM; opa.r_lim = end;
  if (B_MC) { opb.base = b + (int64_t)e * k * n; opb.ld = n; }
  else { opb.base = b + (int64_t)e * n * k; opb.ld = k; }
  opb.r0 = tn * T::BN; opb.r_lim = n;
  block_gemm<DT, false, B_MC, T>(opa, opb, 0, k, c, n, end, n, lds);
}

// ---- TN: one [k, n] product per expert, reduced over the expert's rows ----------------
template <int DT, typename T>
__global__ void __launch_bounds__(T::THREADS)
gmm_tn_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
              const int32_t* __restrict__ bins, int num_groups, int rows, int k, int n, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const int id = xcd_tile_id(blockIdx.x);
  const int per_group = tiles_m * tiles_n;
  const int e = id / per_group;
  if (e >= num_groups) return;
  const int t = id % per_group;
  const int tm = t % tiles_m, tn = t / tiles_m;
  const int start = e > 0 ? clamp_bound(bins[e - 1], 0, rows) : 0, end = clamp_bound(bins[e], start, rows);
  Operand opa, opb;
  opa.base = a; opa.ld = k; opa.r0 = tm * T::BM; opa.r_lim = k;
  opb.base = b; opb.ld = n; opb.r0 = tn * T::BN; opb.r_lim = n;
  block_gemm<DT, true, true, T>(opa, opb, start, end, c + (int64_t)e * k * n, n, k, n, lds);
}

#include "gmm_dma.h"

// ---- any shape, any alignment, fp32 included ------------------------------------------
// c(m, n) = sum_r a(m, r) b(r, n) with element-wise addressing and bounds checks, the products and sums
// in fp32 on the matrix cores (v_mfma_f32_32x32x2_f32 is an IEEE fp32 multiply-add; 16-bit inputs are
// widened exactly).  128 x 128 tile per workgroup, four waves of 64 x 64, K tiles of 16 staged through a
// double-buffered LDS tile [k][128 + 36] per operand (the MFMA wants one k per lane half, 32 consecutive
// rows / columns across the lanes: conflict-free reads).  The next K tile is fetched into registers while
// the current one is multiplied.
constexpr int kGenTile = 128, kGenBK = 16;
// row pitch of the LDS tiles in floats: 36 mod 64 banks apart, so that the 16 k-rows x 4 columns a wave stores
// and the two k-rows x 32 columns a wave reads per instruction fall into (nearly) distinct banks
constexpr int kGenLd = kGenTile + 36;

template <int DT>
__global__ void __launch_bounds__(256)
gmm_generic_kernel(const void* __restrict__ a_, const void* __restrict__ b_, void* __restrict__ c_,
                   const int32_t* __restrict__ bins, int layout, int rows, int k, int n) {
  typedef typename Elem<DT>::type E;
  const E* a = (const E*)a_;
  const E* b = (const E*)b_;
  E* c = (E*)c_;
  __shared__ float as[2][kGenBK][kGenLd], bs[2][kGenBK][kGenLd];
  const int e = blockIdx.z;
  const int start = e > 0 ? clamp_bound(bins[e - 1], 0, rows) : 0, end = clamp_bound(bins[e], start, rows);
  int m_dim, r_begin, r_end;
  if (layout == MBX_TN) { m_dim = k; r_begin = start; r_end = end; }
  else { m_dim = end - start; r_begin = 0; r_end = k; }
  const int m0 = blockIdx.y * kGenTile, n0 = blockIdx.x * kGenTile;
  if (m0 >= m_dim) return;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;

  // Each thread fetches 8 elements of each operand tile; consecutive threads walk the dimension that is
  // contiguous in memory (the reduction index r for a in NN / NT and b in NT, else the row / column).
  const bool a_r_fast = layout != MBX_TN, b_r_fast = layout == MBX_NT;
  const int a_t0 = a_r_fast ? tid / kGenBK : tid % kGenTile, a_r = a_r_fast ? tid % kGenBK : tid / kGenTile;
  const int b_t0 = b_r_fast ? tid / kGenBK : tid % kGenTile, b_r = b_r_fast ? tid % kGenBK : tid / kGenTile;
  // step of the tile index / of r between a thread's 8 elements
  const int a_ts = a_r_fast ? 256 / kGenBK : 0, a_rs = a_r_fast ? 0 : 256 / kGenTile;
  const int b_ts = b_r_fast ? 256 / kGenBK : 0, b_rs = b_r_fast ? 0 : 256 / kGenTile;
  auto a_at = [&](int m, int r) -> float {
    if (m >= m_dim || r >= r_end) return 0.f;
    return Elem<DT>::to_f32(layout == MBX_TN ? a[(int64_t)r * k + m] : a[(int64_t)(start + m) * k + r]);
  };
  auto b_at = [&](int r, int nn) -> float {
    if (r >= r_end || nn >= n) return 0.f;
    if (layout == MBX_TN) return Elem<DT>::to_f32(b[(int64_t)r * n + nn]);
    if (layout == MBX_NN) return Elem<DT>::to_f32(b[((int64_t)e * k + r) * n + nn]);
    return Elem<DT>::to_f32(b[((int64_t)e * n + nn) * k + r]);
  };
  float ra[8], rb[8];
  auto fetch = [&](int r0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ra[i] = a_at(m0 + a_t0 + i * a_ts, r0 + a_r + i * a_rs);
      rb[i] = b_at(r0 + b_r + i * b_rs, n0 + b_t0 + i * b_ts);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      as[buf][a_r + i * a_rs][a_t0 + i * a_ts] = ra[i];
      bs[buf][b_r + i * b_rs][b_t0 + i * b_ts] = rb[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  fetch(r_begin);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int r0 = r_begin; r0 < r_end; r0 += kGenBK) {
    const bool more = r0 + kGenBK < r_end;
    if (more) fetch(r0 + kGenBK);
#pragma unroll
    for (int kk = 0; kk < kGenBK; kk += 2) {
      float fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = as[buf][kk + lane / 32][wm + i * 32 + lane % 32];
        fb[i] = bs[buf][kk + lane / 32][wn + i * 32 + lane % 32];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  // register r of lane l of a 32 x 32 product: row (r / 4) * 8 + (l / 32) * 4 + r % 4, column l % 32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int nn = n0 + wn + j * 32 + lane % 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + (r / 4) * 8 + (lane / 32) * 4 + r % 4;
        if (m < m_dim && nn < n) {
          if (layout == MBX_TN) c[((int64_t)e * k + m) * n + nn] = Elem<DT>::from_f32(acc[i][j][r]);
          else c[(int64_t)(start + m) * n + nn] = Elem<DT>::from_f32(acc[i][j][r]);
        }
      }
    }
}

// ---- GELU backward, in place ---------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_grad(float xv) {   // d/dx gelu_tanh(x), gelu.py:9-13
  const float t = tanhf(0.79788456f * xv * (1.f + 0.044715f * xv * xv));
  return 0.5f * xv * ((1.f - t * t) * (0.79788456f + 0.1070322243f * xv * xv)) + 0.5f * (1.f + t);
}

// elements [first, numel), one per thread and step: the tail of the vector kernel, or everything when the
// buffers are not 16-byte aligned
template <int DT>
__global__ void gelu_backward_kernel(void* __restrict__ g_, const void* __restrict__ x_, int64_t first, int64_t numel) {
  typedef typename Elem<DT>::type E;
  E* g = (E*)g_;
  const E* x = (const E*)x_;
  int64_t i = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < numel; i += stride)
    g[i] = Elem<DT>::from_f32(Elem<DT>::to_f32(g[i]) * gelu_tanh_grad(Elem<DT>::to_f32(x[i])));
}

// 16 bytes per lane and step
template <int DT>
__global__ void __launch_bounds__(256) gelu_backward_vec_kernel(void* __restrict__ g_, const void* __restrict__ x_, int64_t nvec) {
  typedef typename Elem<DT>::type E;
  constexpr int N = 16 / (int)sizeof(E);
  u32x4* g = (u32x4*)g_;
  const u32x4* x = (const u32x4*)x_;
  int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; v < nvec; v += stride) {
    u32x4 gv = g[v];
    const u32x4 xv = x[v];
    E* ge = (E*)&gv;
    const E* xe = (const E*)&xv;
#pragma unroll
    for (int i = 0; i < N; ++i) ge[i] = Elem<DT>::from_f32(Elem<DT>::to_f32(ge[i]) * gelu_tanh_grad(Elem<DT>::to_f32(xe[i])));
    g[v] = gv;
  }
}

// Tile shapes.  256x256x64 with four waves (2x2, 128x128 each) keeps the accumulators in
// 256 registers per lane and needs 144 KiB of the 160 KiB LDS for two stages.
typedef Tile<256, 256, 64, 2, 2, 8, 32> TileBig;
// The tiles of the direct-to-LDS kernels (gmm_dma.h): 256 x 256 x 64, four waves of 128 x 128, three A and two B
// stages of 32 KiB; and the half-height tile (NN / NT only: the row tile follows the expert's row count) for the last
// row tile of an expert when it is at most half full, for the tail of a launch, and for launches of small experts;
// its smaller stages allow a three-deep ring (4 x 16 KiB + 3 x 32 KiB).
typedef dma::Tile<256, 256, 2, 2, 64, 2> TileDma;
typedef dma::Tile<128, 256, 1, 4, 64, 3> TileDmaSmallM;

template <int DT, bool A_MC, bool B_MC, typename T>
constexpr size_t lds_bytes() {
  return 2 * sizeof(uint16_t) *
         (size_t)(OperandLds<A_MC, T::BM, T::BK, T::PAD_KC, T::PAD_MC>::ELEMS + OperandLds<B_MC, T::BN, T::BK, T::PAD_KC, T::PAD_MC>::ELEMS);
}

template <typename K>
int allow_lds(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <int DT, typename T>
int gmm_mfma(const void* a, const void* b, void* c, const int32_t* bins, int num_groups, int64_t rows, int k, int n,
             int layout, hipStream_t s) {
  const uint16_t* ap = (const uint16_t*)a;
  const uint16_t* bp = (const uint16_t*)b;
  uint16_t* cp = (uint16_t*)c;
  if (layout == MBX_TN) {
    const int tiles_m = (int)ceil_div(k, T::BM), tiles_n = (int)ceil_div(n, T::BN);
    constexpr size_t lds = lds_bytes<DT, true, true, T>();
    auto kern = gmm_tn_kernel<DT, T>;
    int rc = allow_lds(kern, lds);
    if (rc) return rc;
    const int64_t grid = xcd_grid((int64_t)tiles_m * tiles_n * num_groups);
    if (grid > 0x7fffffff) return MBX_ERANGE;
    kern<<<(unsigned)grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, (int)rows, k, n, tiles_m, tiles_n);
    return launch_status();
  }
  const int tiles_n = (int)ceil_div(n, T::BN);
  const int64_t max_mt = ceil_div(rows, T::BM) + num_groups;
  const int64_t grid = xcd_grid(max_mt * tiles_n);
  if (grid > 0x7fffffff) return MBX_ERANGE;
  if (layout == MBX_NT) {
    constexpr size_t lds = lds_bytes<DT, false, false, T>();
    auto kern = gmm_rows_kernel<DT, false, T>;
    int rc = allow_lds(kern, lds);
    if (rc) return rc;
    kern<<<(unsigned)grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, (int)rows, k, n, tiles_n);
  } else {
    constexpr size_t lds = lds_bytes<DT, false, true, T>();
    auto kern = gmm_rows_kernel<DT, true, T>;
    int rc = allow_lds(kern, lds);
    if (rc) return rc;
    kern<<<(unsigned)grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, (int)rows, k, n, tiles_n);
  }
  return launch_status();
}

// One persistent workgroup per compute unit (a multiple of 8, so that every XCD gets the same number),
// fewer when there are not that many tiles.
static inline int persistent_grid(int64_t tiles_upper_bound) {
  static int cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < kXcds) n = 256;
    cus[dev] = n / kXcds * kXcds;
  }
  const int64_t need = (tiles_upper_bound + kXcds - 1) / kXcds * kXcds;
  return (int)(need < cus[dev] ? need : cus[dev]);
}

// Launch of the direct-to-LDS kernels (k a multiple of 64 for NN / NT; sizes as dma_sizes_ok() allows).
// TS is the tile the tail of an NN / NT launch is cut into (TS = T: never cut).
// a2 / b2 non-null (NN / NT only): c = a @ b[e] + a2 @ b2[e], the second pair shaped like the first.
// epi / extra (NT, one operand pair only): dma::kEpiAct with the second output, dma::kEpiDact with the second input.
// Rows of `a` gathered on the fly (NT; no epilogue, kEpiAct or kEpiGlu*): see GatherRows.
// Device memory a launch may use for the parts of tiles it cuts along the reduction (gmm_rows_kernel's split-K tail):
// The weighted combine in the epilogue (kEpiCombine): the sorted assignments (top_k = 1: tokens) of the product's rows,
// the weights by token (or null) and their type, the row count of the combined output.
struct CombineRows {
  const int32_t* indices = nullptr;
  const void* weights = nullptr;
  int w_dtype = 0;
  int tokens = 0;
};

// kWorkspaceCounters int32 counters, zero before the launch and zero again after it, then room for fp32 tiles.
constexpr size_t kWorkspaceCounters = 1024, kWorkspacePartBytes = (size_t)256 * 256 * 4, kWorkspaceParts = 320;
struct Workspace {
  void* base = nullptr;
  size_t bytes = 0;
};
struct GatherRows {
  const int32_t* slots = nullptr;      // non-null: a (NT) / b (TN) is [src_rows, .], read through the row map
  const int32_t* src_bins = nullptr;
  int top_k = 1, src_rows = 0;
  // TN only: the table of row offsets the kernel reads (4 bytes per sorted assignment, n_slots of them), and whether an
  // earlier call with the same slots, top_k, src_rows and n has already filled it
  uint32_t* row_table = nullptr;
  int64_t n_slots = 0;
  bool table_ready = false;
};
template <int DT, typename T, typename TS>
int gmm_dma(const void* a, const void* b, void* c, const int32_t* bins, int num_groups, int64_t rows, int k, int n,
            int layout, hipStream_t s, const void* a2 = nullptr, const void* b2 = nullptr, int epi = dma::kEpiNone,
            void* extra = nullptr, void* out2 = nullptr, GatherRows gather = GatherRows(), Workspace ws = Workspace(),
            CombineRows combine = CombineRows()) {
  const uint16_t* ap = (const uint16_t*)a;
  const uint16_t* bp = (const uint16_t*)b;
  const uint16_t* ap2 = (const uint16_t*)a2;
  const uint16_t* bp2 = (const uint16_t*)b2;
  const bool dual = a2 != nullptr && !dma::epi_is_dglu(epi) && !dma::epi_is_glu(epi);
  uint16_t* cp = (uint16_t*)c;
  if (layout == MBX_TN) {
    constexpr size_t lds = T::LDS_BYTES > TS::LDS_BYTES ? T::LDS_BYTES : TS::LDS_BYTES;
    const int tiles_m = (int)ceil_div(k, T::BM), tiles_n = (int)ceil_div(n, T::BN);
    // rows per segment of a reduction: each operand's share stays below 2 GiB (whole K tiles)
    const int64_t seg_rows = (((int64_t)1 << 31) - 1) / ((int64_t)(k > n ? k : n) * 2) / T::BK * T::BK;
    const bool segmented = rows > seg_rows;
    // the last row tile of the product as a TS tile when it is at most half full
    const bool mixed = T::BM != TS::BM && k % T::BM != 0 && k % T::BM <= TS::BM;
    auto kern = mixed ? (segmented ? dma::gmm_tn_kernel<DT, T, TS, true> : dma::gmm_tn_kernel<DT, T, TS, false>)
                      : (segmented ? dma::gmm_tn_kernel<DT, T, T, true> : dma::gmm_tn_kernel<DT, T, T, false>);
    int rc = allow_lds(kern, lds);
    if (rc) return rc;
    // short reductions (few rows per expert): several tiles per workgroup
    const int64_t avg_rows = rows / (num_groups > 0 ? num_groups : 1);
    int chunk = avg_rows >= 1024 ? 1 : avg_rows >= 512 ? 2 : 4;
    // Reductions of a few dozen K tiles still gain from fewer workgroup launches (c3: 2 % of the launch with four
    // tiles per workgroup), but only where an expert brings every XCD many tiles: with the six tiles per expert and
    // XCD of a skewed c4, four to a workgroup leave most compute units idle behind the largest expert (2.4 x slower).
    const dma::TnBlocks shape = dma::tn_block_shape(tiles_m, tiles_n);
    if (avg_rows >= 1024 && avg_rows < 4096 && dma::tn_tiles_per_group(tiles_m, tiles_n, shape) / kXcds >= 64) chunk = 4;
    const int64_t grid = dma::tn_grid(tiles_m, tiles_n, shape, num_groups, chunk);
    if (grid > 0x7fffffff) return MBX_ERANGE;
    // whole experts per XCD (if the kernel finds them balanced): for reductions of a few K tiles only
    const int whole_ok = avg_rows < 1024 ? 1 : 0;
    if (gather.slots) {
      // the rows of b picked through the sorted assignments: the full tile only, one segment
      if (!gather.src_bins || !gather.row_table || gather.top_k <= 0 || gather.n_slots > 0x7fffffff) return MBX_EINVAL;
      if (segmented || !std::is_same<T, TS>::value) return MBX_EUNSUPPORTED;
      if (!gather.table_ready) {
        uint32_t magic = 0;
        int shift = 0;
        dma::gather_divisor(gather.top_k, magic, shift);
        dma::gather_row_table_kernel<<<(unsigned)ceil_div(dma::row_table_entries(gather.n_slots, num_groups), 256), 256, 0, s>>>(
            gather.slots, gather.src_bins, num_groups, (int)gather.n_slots, gather.src_rows, (uint32_t)n * 2u, magic, shift, gather.row_table);
      }
      if constexpr (T::BM == 256 && T::SB == 2) {
        auto gkern = dma::gmm_tn_kernel<DT, T, T, false, true>;
        int grc = allow_lds(gkern, lds);
        if (grc) return grc;
        gkern<<<(unsigned)grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, (int)rows, k, n, tiles_m, tiles_n, shape.bm, shape.bn, chunk, (int)seg_rows, whole_ok, gather.row_table, gather.src_bins, gather.src_rows, (int)gather.n_slots);
        return launch_status();
      } else {
        return MBX_EUNSUPPORTED;
      }
    }
    kern<<<(unsigned)grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, (int)rows, k, n, tiles_m, tiles_n, shape.bm, shape.bn, chunk, (int)seg_rows, whole_ok, nullptr, nullptr, 0, 0);
    return launch_status();
  }
  constexpr size_t lds = T::LDS_BYTES > TS::LDS_BYTES ? T::LDS_BYTES : TS::LDS_BYTES;
  // a [w1 | v1] tile covers half as many output columns
  const int tiles_n = (int)ceil_div(n, dma::epi_is_glu(epi) ? T::BN / 2 : T::BN);
  const int64_t tiles = (ceil_div(rows, T::BM) + num_groups) * tiles_n;   // the row counts are only known on the device
  if (tiles > 0x7fffffff) return MBX_ERANGE;
  const unsigned grid = (unsigned)persistent_grid(tiles);
  // An expert's last row tile, when at most half full, is computed with the half-height tile -- unless a row of tiles is
  // longer than the run of tiles an XCD's workgroups take per round: the half-height tiles of such a row fill whole
  // rounds of some XCDs, those finish early, and from then on the XCD's workgroups are no longer within the few K tiles
  // of each other that the L2 holds (c3's NT launches, 112 and 56 column tiles against runs of 32: L2 misses 5.8 ->
  // 3.3 GB; the launches themselves take 1 % longer for the padding they multiply, the step is 0.7 % shorter, the
  // launches after them running at a higher clock).  With shorter rows of tiles the half-height tile wins (every
  // launch of c2, c4 and c5: 0.7 - 2.8 % per step), and with few row tiles per expert the padding would be a large
  // part of the work.  MBX_FULL_SHORT_FROM=N overrides the column-tile count from which
  // the full tile is used (measurements).
  static const int full_short_from = [] { const char* v = getenv("MBX_FULL_SHORT_FROM"); return v ? atoi(v) : -1; }();
  const int run_tiles = (int)grid / kXcds;
  // ... and only for experts of eight row tiles and more on average, where the padding is a few percent of the work
  const bool long_experts = rows >= (int64_t)num_groups * 8 * T::BM;
  const int half_limit = (full_short_from >= 0 ? tiles_n >= full_short_from : tiles_n > run_tiles && long_experts) ? 0 : TS::BM;
  uint32_t gather_magic = 0;
  int gather_shift = 0;
  if (gather.slots) dma::gather_divisor(gather.top_k, gather_magic, gather_shift);
  // the workspace as the kernel takes it: counters, parts (16-byte aligned), how many parts of a T tile fit
  int32_t* ws_counters = nullptr;
  float* ws_parts = nullptr;
  int ws_capacity = 0;
  if (ws.base && ((uintptr_t)ws.base & 15u) == 0 && ws.bytes > kWorkspaceCounters * sizeof(int32_t) && (int)grid / 2 <= (int)kWorkspaceCounters) {
    ws_counters = (int32_t*)ws.base;
    ws_parts = (float*)((char*)ws.base + kWorkspaceCounters * sizeof(int32_t));
    const size_t fit = (ws.bytes - kWorkspaceCounters * sizeof(int32_t)) / ((size_t)T::BM * T::BN * sizeof(float));
    ws_capacity = (int)(fit > 0x7fffffff ? 0x7fffffff : fit);
    if (ws_capacity < 2) ws_parts = nullptr;
  }
#define MBX_LAUNCH_ROWS_G(B_MC, DUAL, EPI, GATHER)                                                    \
  do {                                                                                                \
    auto kern = dma::gmm_rows_kernel<DT, B_MC, T, TS, DUAL, EPI, GATHER>;                             \
    int rc = allow_lds(kern, lds);                                                                    \
    if (rc) return rc;                                                                                \
    kern<<<grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, rows, k, n, tiles_n, ap2, bp2, (uint16_t*)extra, (uint16_t*)out2,  \
                                       gather.slots, gather.src_bins, gather.top_k, gather.src_rows, gather_magic, gather_shift, half_limit,  \
                                       ws_counters, ws_parts, ws_capacity, combine.weights, combine.w_dtype, combine.tokens);  \
  } while (0)
#define MBX_LAUNCH_ROWS(B_MC, DUAL, EPI) MBX_LAUNCH_ROWS_G(B_MC, DUAL, EPI, false)
  // the combine epilogue takes the sorted assignments where the gathered launches take theirs
#define MBX_LAUNCH_ROWS_C(B_MC, DUAL, EPI)                                                            \
  do {                                                                                                \
    auto kern = dma::gmm_rows_kernel<DT, B_MC, T, TS, DUAL, EPI, false>;                              \
    int rc = allow_lds(kern, lds);                                                                    \
    if (rc) return rc;                                                                                \
    kern<<<grid, T::THREADS, lds, s>>>(ap, bp, cp, bins, num_groups, rows, k, n, tiles_n, ap2, bp2, (uint16_t*)extra, (uint16_t*)out2,  \
                                       combine.indices, nullptr, 1, 0, 0u, 0, half_limit, nullptr, nullptr, 0,          \
                                       combine.weights, combine.w_dtype, combine.tokens);             \
  } while (0)
  if (gather.slots) {
    if (layout != MBX_NT || a2 || !gather.src_bins || gather.top_k <= 0) return MBX_EINVAL;
    switch (epi) {
      case dma::kEpiNone: MBX_LAUNCH_ROWS_G(false, false, dma::kEpiNone, true); break;
      case dma::kEpiAct: if (!extra) return MBX_EINVAL; MBX_LAUNCH_ROWS_G(false, false, dma::kEpiAct, true); break;
      case dma::kEpiGluSilu: if (!extra || !b2 || !out2) return MBX_EINVAL; MBX_LAUNCH_ROWS_G(false, false, dma::kEpiGluSilu, true); break;
      case dma::kEpiGluGelu: if (!extra || !b2 || !out2) return MBX_EINVAL; MBX_LAUNCH_ROWS_G(false, false, dma::kEpiGluGelu, true); break;
      default: return MBX_EINVAL;
    }
    return launch_status();
  }
  if (dma::epi_is_glu(epi)) {
    // b2 is the second matrix of the [w1 | v1] tiles (not a second operand pair)
    if (layout != MBX_NT || !extra || !b2 || !out2 || a2) return MBX_EINVAL;
    if (epi == dma::kEpiGluSilu) MBX_LAUNCH_ROWS(false, false, dma::kEpiGluSilu); else MBX_LAUNCH_ROWS(false, false, dma::kEpiGluGelu);
    return launch_status();
  }
  if (dma::epi_is_dglu(epi)) {
    // a2 carries x2 of the gated activation (not a second operand pair)
    if (layout != MBX_NT || !extra || !a2 || !out2) return MBX_EINVAL;
    if (epi == dma::kEpiDgluSilu) MBX_LAUNCH_ROWS(false, false, dma::kEpiDgluSilu); else MBX_LAUNCH_ROWS(false, false, dma::kEpiDgluGelu);
    return launch_status();
  }
  if (epi == dma::kEpiCombine) {
    // extra is the combined output [tokens, n]; c (the product itself) may be absent
    if (layout != MBX_NN || a2 || !extra || !combine.indices) return MBX_EINVAL;
    MBX_LAUNCH_ROWS_C(true, false, dma::kEpiCombine);
    return launch_status();
  }
  if (epi != dma::kEpiNone) {
    if (layout != MBX_NT || dual || !extra) return MBX_EINVAL;
    if (epi == dma::kEpiAct) MBX_LAUNCH_ROWS(false, false, dma::kEpiAct); else MBX_LAUNCH_ROWS(false, false, dma::kEpiDact);
    return launch_status();
  }
  if (layout == MBX_NT) {
    if (dual) MBX_LAUNCH_ROWS(false, true, dma::kEpiNone); else MBX_LAUNCH_ROWS(false, false, dma::kEpiNone);
  } else {
    if (dual) MBX_LAUNCH_ROWS(true, true, dma::kEpiNone); else MBX_LAUNCH_ROWS(true, false, dma::kEpiNone);
  }
#undef MBX_LAUNCH_ROWS
#undef MBX_LAUNCH_ROWS_C
#undef MBX_LAUNCH_ROWS_G
  return launch_status();
}

template <int DT>
int gmm_generic(const void* a, const void* b, void* c, const int32_t* bins, int num_groups, int64_t rows, int k, int n,
                int layout, hipStream_t s) {
  // The row count of a group is only known on the device: size the grid for the worst case.
  const int64_t m_bound = layout == MBX_TN ? k : rows;
  const int64_t gy = ceil_div(m_bound, kGenTile), gx = ceil_div(n, kGenTile);
  if (gy > 65535 || num_groups > 65535) return MBX_ERANGE;
  if (gy == 0 || gx == 0) return 0;
  gmm_generic_kernel<DT><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)num_groups), 256, 0, s>>>(a, b, c, bins, layout, (int)rows, k, n);
  return launch_status();
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// The direct-to-LDS kernels address with 32-bit byte offsets from a base they set per tile (the tile's first
// row of a and c in NN / NT), per expert (its weights; its [k, n] product in TN) or per segment of an
// expert's rows (TN), so the row count is free; what has to stay below 2 GiB is one expert's weight matrix
// or product and 256 rows of any operand (a 64-row K tile in TN).
static inline bool dma_sizes_ok(int k, int n) {
  const int64_t lim = (int64_t)1 << 31;
  return (int64_t)k * n * 2 < lim && (int64_t)k * 2 * TileDma::BM < lim && (int64_t)n * 2 * TileDma::BM < lim;
}

// NN / NT: whether to tile a launch with the half-height tile only.  With about one such tile per expert
// (up to 144 rows on average) the full tile would mostly multiply padding.  Up to 320 rows the mix of
// full tiles and a half-height last tile moves fewer weight bytes through the compute units (the
// weights are streamed once per row tile), but its tiles cost unequal time, and a launch of fewer than
// three rounds of them does not balance over the statically assigned workgroups.
static inline bool half_height_only(int64_t rows, int num_groups, int n) {
  const int64_t avg = rows / (num_groups > 0 ? num_groups : 1);
  if (avg <= 144) return true;
  if (avg > 320) return false;
  const int64_t mixed_tiles = (ceil_div(rows, TileDma::BM) + num_groups / 2) * ceil_div(n, TileDma::BN);
  return mixed_tiles < 3 * (int64_t)persistent_grid((int64_t)1 << 30);
}

}  // namespace
}  // namespace mbx

using namespace mbx;

extern "C" {

#ifdef MBX_TICKS
// libmbx_ticks.so only: where the kernels of gmm_dma.h put their per-tile time stamps (see there); NULL: nowhere.
int mbx_debug_set_ticks(void* buffer) {
  return (int)hipMemcpyToSymbol(HIP_SYMBOL(dma::g_ticks), &buffer, sizeof(buffer));
}
#endif

size_t mbx_gmm_workspace_bytes(void) { return kWorkspaceCounters * sizeof(int32_t) + kWorkspaceParts * kWorkspacePartBytes; }

static int gmm_dual_ws(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype, const int32_t* bins,
                       int num_groups, int64_t rows, int k, int n, int layout, Workspace ws, mbx_stream_t stream);

static int gmm_ws(const void* a, const void* b, void* c, int dtype, const int32_t* bins, int num_groups, int64_t rows, int k,
                  int n, int layout, Workspace ws, mbx_stream_t stream) {
  if (num_groups < 0 || rows < 0 || k < 0 || n < 0) return MBX_EINVAL;
  if (layout != MBX_NN && layout != MBX_NT && layout != MBX_TN) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (num_groups == 0) return 0;
  if (!bins) return MBX_EINVAL;
  if (rows > 0x7fffffff) return MBX_ERANGE;
  hipStream_t s = as_stream(stream);
  if (layout == MBX_TN) {
    if ((int64_t)k * n == 0) return 0;
    if (!c || (rows > 0 && (!a || !b))) return MBX_EINVAL;
  } else {
    if (rows == 0 || n == 0) return 0;
    if (!c || (k > 0 && (!a || !b))) return MBX_EINVAL;
  }
  // MFMA path: 16-byte global loads need k (and n, where n is the contiguous dimension of an
  // operand) to be multiples of 8 and the bases to be 16-byte aligned.
  bool fast = dtype != MBX_F32 && aligned16(a) && aligned16(b) && k > 0;
  if (layout == MBX_NT) fast = fast && k % 8 == 0;
  if (layout == MBX_NN) fast = fast && k % 8 == 0 && n % 8 == 0;
  if (layout == MBX_TN) fast = fast && k % 8 == 0 && n % 8 == 0;
  if (fast) {
    // direct-to-LDS kernels: whole K tiles (NN / NT); their epilogue writes 16-byte pieces of the output's rows
    bool dma_ok = dma_sizes_ok(k, n) && aligned16(c) && n % 8 == 0;
    if (layout != MBX_TN) dma_ok = dma_ok && k % TileDma::BK == 0;
    if (dma_ok) {
      // TN: the half-height tile only when the product has at most 128 rows (it is slower otherwise)
      const bool small_m = layout == MBX_TN ? k <= TileDmaSmallM::BM : half_height_only(rows, num_groups, n);
      const GatherRows none;
      if (small_m) {
        if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, none, ws);
        return gmm_dma<MBX_F16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, none, ws);
      }
      if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, none, ws);
      return gmm_dma<MBX_F16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, none, ws);
    }
    if (dtype == MBX_BF16) return gmm_mfma<MBX_BF16, TileBig>(a, b, c, bins, num_groups, rows, k, n, layout, s);
    return gmm_mfma<MBX_F16, TileBig>(a, b, c, bins, num_groups, rows, k, n, layout, s);
  }
  switch (dtype) {
    case MBX_BF16: return gmm_generic<MBX_BF16>(a, b, c, bins, num_groups, rows, k, n, layout, s);
    case MBX_F16: return gmm_generic<MBX_F16>(a, b, c, bins, num_groups, rows, k, n, layout, s);
    default: return gmm_generic<MBX_F32>(a, b, c, bins, num_groups, rows, k, n, layout, s);
  }
}

int mbx_gmm(const void* a, const void* b, void* c, int dtype, const int32_t* bins, int num_groups, int64_t rows, int k,
            int n, int layout, mbx_stream_t stream) {
  return gmm_ws(a, b, c, dtype, bins, num_groups, rows, k, n, layout, Workspace(), stream);
}

int mbx_gmm_dual(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype, const int32_t* bins,
                 int num_groups, int64_t rows, int k, int n, int layout, mbx_stream_t stream) {
  return gmm_dual_ws(a, b, a2, b2, c, dtype, bins, num_groups, rows, k, n, layout, Workspace(), stream);
}

int mbx_gmm_ws(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype, const int32_t* bins,
               int num_groups, int64_t rows, int k, int n, int layout, void* workspace, size_t workspace_bytes,
               mbx_stream_t stream) {
  if ((a2 == nullptr) != (b2 == nullptr)) return MBX_EINVAL;
  Workspace ws;
  ws.base = workspace;
  ws.bytes = workspace ? workspace_bytes : 0;
  if (a2) return gmm_dual_ws(a, b, a2, b2, c, dtype, bins, num_groups, rows, k, n, layout, ws, stream);
  return gmm_ws(a, b, c, dtype, bins, num_groups, rows, k, n, layout, ws, stream);
}

static int gmm_dual_ws(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype, const int32_t* bins,
                       int num_groups, int64_t rows, int k, int n, int layout, Workspace ws, mbx_stream_t stream) {
  if (num_groups < 0 || rows < 0 || k < 0 || n < 0) return MBX_EINVAL;
  if (layout != MBX_NN && layout != MBX_NT) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (num_groups == 0 || rows == 0 || n == 0) return 0;
  if (!bins || !c || (k > 0 && (!a || !b || !a2 || !b2))) return MBX_EINVAL;
  if (rows > 0x7fffffff) return MBX_ERANGE;
  // only the direct-to-LDS kernels reduce over two operand pairs: whole K tiles, at least four per pair
  const bool ok = dtype != MBX_F32 && aligned16(a) && aligned16(b) && aligned16(a2) && aligned16(b2) && aligned16(c) &&
                  k % TileDma::BK == 0 && k >= 4 * TileDma::BK && n % 8 == 0 && dma_sizes_ok(k, n);
  if (!ok) return MBX_EUNSUPPORTED;
  hipStream_t s = as_stream(stream);
  const bool small_m = half_height_only(rows, num_groups, n);
  const GatherRows none;
  if (small_m) {
    if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, a2, b2, dma::kEpiNone, nullptr, nullptr, none, ws);
    return gmm_dma<MBX_F16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, a2, b2, dma::kEpiNone, nullptr, nullptr, none, ws);
  }
  if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, a2, b2, dma::kEpiNone, nullptr, nullptr, none, ws);
  return gmm_dma<MBX_F16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, layout, s, a2, b2, dma::kEpiNone, nullptr, nullptr, none, ws);
}

// The NT product with an activation epilogue (epi: dma::kEpiAct / dma::kEpiDact), for the shapes the direct-to-LDS
// kernels take; anything else is MBX_EUNSUPPORTED and the caller runs the product and the element-wise pass.
// (kEpiDglu*: pre2 = x2, out2 = the second output.)
// (kEpiGlu*: b2 = the second matrix, extra = the gated activation, out2 = the second product.)
// gather.slots non-null: `a` is read through the row map (no epilogue, kEpiAct and kEpiGlu* only; `extra` may then be
// null for no epilogue).
static int gmm_nt_epilogue(const void* a, const void* b, void* c, void* extra, int dtype, const int32_t* bins, int num_groups,
                           int64_t rows, int k, int n, int act, int epi, mbx_stream_t stream, const void* pre2 = nullptr,
                           void* out2 = nullptr, const void* b2 = nullptr, GatherRows gather = GatherRows()) {
  if (num_groups < 0 || rows < 0 || k < 0 || n < 0) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  const bool dglu = dma::epi_is_dglu(epi), glu = dma::epi_is_glu(epi);
  const bool plain = epi == dma::kEpiNone;   // gathered rows only
  if (!dglu && !glu && !plain && act != MBX_ACT_GELU_TANH) return MBX_EUNSUPPORTED;
  if (num_groups == 0 || rows == 0 || n == 0) return 0;
  if (!bins || !c || (!extra && !plain) || (k > 0 && (!a || !b)) || (dglu && (!pre2 || !out2)) || (glu && (!out2 || (k > 0 && !b2)))) return MBX_EINVAL;
  if (rows > 0x7fffffff) return MBX_ERANGE;
  bool ok = dtype != MBX_F32 && aligned16(a) && aligned16(b) && aligned16(c) && aligned16(extra) && k > 0 &&
            k % TileDma::BK == 0 && n % 8 == 0 && dma_sizes_ok(k, n) && (!dglu || (aligned16(pre2) && aligned16(out2)));
  // the second matrix is addressed from half a tile before its first row: that much more must fit below 2 GiB
  if (glu) ok = ok && aligned16(b2) && aligned16(out2) && dma_sizes_ok(k, n + TileDma::BN / 2);
  if (!ok) return MBX_EUNSUPPORTED;
  hipStream_t s = as_stream(stream);
  if (half_height_only(rows, num_groups, n)) {
    if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NT, s, pre2, b2, epi, extra, out2, gather);
    return gmm_dma<MBX_F16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NT, s, pre2, b2, epi, extra, out2, gather);
  }
  if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NT, s, pre2, b2, epi, extra, out2, gather);
  return gmm_dma<MBX_F16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NT, s, pre2, b2, epi, extra, out2, gather);
}

int mbx_gmm_act(const void* a, const void* b, void* c, void* c_act, int dtype, const int32_t* bins, int num_groups,
                int64_t rows, int k, int n, int act, mbx_stream_t stream) {
  return gmm_nt_epilogue(a, b, c, c_act, dtype, bins, num_groups, rows, k, n, act, dma::kEpiAct, stream);
}

int mbx_gmm_dact(const void* a, const void* b, const void* pre, void* c, int dtype, const int32_t* bins, int num_groups,
                 int64_t rows, int k, int n, int act, mbx_stream_t stream) {
  return gmm_nt_epilogue(a, b, c, (void*)pre, dtype, bins, num_groups, rows, k, n, act, dma::kEpiDact, stream);
}

int mbx_gmm_glu(const void* a, const void* b1, const void* b2, void* x1, void* x2, void* h, int dtype, const int32_t* bins,
                int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream) {
  if (act != MBX_ACT_SILU && act != MBX_ACT_GELU_TANH) return MBX_EINVAL;
  return gmm_nt_epilogue(a, b1, x1, h, dtype, bins, num_groups, rows, k, n, act,
                         act == MBX_ACT_SILU ? dma::kEpiGluSilu : dma::kEpiGluGelu, stream, nullptr, x2, b2);
}

int mbx_gmm_gather(const void* x, int64_t x_rows, const int32_t* indices, int top_k, const int32_t* x_bins, const void* b1,
                   const void* b2, void* c, void* c2, void* h, int dtype, const int32_t* bins, int num_groups, int64_t rows,
                   int k, int n, int act, mbx_stream_t stream) {
  if (x_rows < 0 || top_k <= 0 || k < 0 || num_groups < 0 || rows < 0 || n < 0) return MBX_EINVAL;
  if (num_groups == 0 || rows == 0 || n == 0) return 0;   // nothing to write (empty outputs may come as NULL)
  if (b2 ? (act != MBX_ACT_SILU && act != MBX_ACT_GELU_TANH) || !c2 || !h : c2 != nullptr) return MBX_EINVAL;
  if (h && !b2 && act != MBX_ACT_GELU_TANH) return MBX_EUNSUPPORTED;
  if (!indices || (k > 0 && !x && x_rows > 0)) return MBX_EINVAL;
  // the row map is indexed with 32 bits and the rows of x are addressed with 31 (bit 31 marks a row of zeros)
  if (x_rows * top_k > 0x7fffffff || x_rows * (int64_t)k * 2 >= ((int64_t)1 << 31)) return MBX_EUNSUPPORTED;
  if (x_rows == 0 && rows > 0) x = b1;   // no row is read; the buffer descriptor still wants an address
  GatherRows gather;
  gather.slots = indices;
  gather.src_bins = x_bins ? x_bins : bins;
  gather.top_k = top_k;
  gather.src_rows = (int)x_rows;
  const int epi = b2 ? (act == MBX_ACT_SILU ? dma::kEpiGluSilu : dma::kEpiGluGelu) : h ? dma::kEpiAct : dma::kEpiNone;
  return gmm_nt_epilogue(x, b1, c, h, dtype, bins, num_groups, rows, k, n, act, epi, stream, nullptr, c2, b2, gather);
}

int mbx_gmm_scatter(const void* a, const void* b, void* c, void* out, int dtype, const int32_t* bins, int num_groups,
                    int64_t rows, int k, int n, const int32_t* indices, const void* weights, int w_dtype, int64_t tokens,
                    mbx_stream_t stream) {
  if (num_groups < 0 || rows < 0 || k < 0 || n < 0 || tokens < 0) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (weights && w_dtype != MBX_BF16 && w_dtype != MBX_F16 && w_dtype != MBX_F32) return MBX_EINVAL;
  if (num_groups == 0 || rows == 0 || n == 0) return 0;
  if (!out || !bins || !indices || (k > 0 && (!a || !b))) return MBX_EINVAL;
  if (rows > 0x7fffffff || tokens > 0x7fffffff) return MBX_ERANGE;
  // the direct-to-LDS NN kernel (16-bit types, whole K tiles, 16-byte pieces of rows); the combined output is addressed
  // with 64 bits
  const bool ok = dtype != MBX_F32 && aligned16(a) && aligned16(b) && (!c || aligned16(c)) && aligned16(out) && k > 0 &&
                  k % TileDma::BK == 0 && n % 8 == 0 && dma_sizes_ok(k, n);
  if (!ok) return MBX_EUNSUPPORTED;
  CombineRows combine;
  combine.indices = indices;
  combine.weights = weights;
  combine.w_dtype = w_dtype;
  combine.tokens = (int)tokens;
  hipStream_t s = as_stream(stream);
  const GatherRows none;
  const Workspace no_ws;
  if (half_height_only(rows, num_groups, n)) {
    if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NN, s, nullptr, nullptr, dma::kEpiCombine, out, nullptr, none, no_ws, combine);
    return gmm_dma<MBX_F16, TileDmaSmallM, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NN, s, nullptr, nullptr, dma::kEpiCombine, out, nullptr, none, no_ws, combine);
  }
  if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NN, s, nullptr, nullptr, dma::kEpiCombine, out, nullptr, none, no_ws, combine);
  return gmm_dma<MBX_F16, TileDma, TileDmaSmallM>(a, b, c, bins, num_groups, rows, k, n, MBX_NN, s, nullptr, nullptr, dma::kEpiCombine, out, nullptr, none, no_ws, combine);
}

size_t mbx_gmm_tn_gather_table_bytes(int64_t x_rows, int top_k, int num_groups) {
  if (x_rows < 0 || top_k <= 0 || num_groups < 0) return 0;
  return (size_t)dma::row_table_entries(x_rows * top_k, num_groups) * 4;
}

int mbx_gmm_tn_gather(const void* a, const void* x, int64_t x_rows, const int32_t* indices, int top_k, const int32_t* x_bins,
                      void* c, int dtype, const int32_t* bins, int num_groups, int64_t rows, int k, int n, void* row_table,
                      size_t row_table_bytes, int table_ready, mbx_stream_t stream) {
  if (x_rows < 0 || top_k <= 0 || k < 0 || n < 0 || num_groups < 0 || rows < 0) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  if (num_groups == 0 || (int64_t)k * n == 0) return 0;
  if (!c || !bins || (x_rows > 0 && (!x || !indices)) || (rows > 0 && !a)) return MBX_EINVAL;
  if (rows > 0x7fffffff) return MBX_ERANGE;
  const int64_t n_slots = x_rows * top_k;
  // the kernel with the full tile, 16-byte pieces of rows, one segment of the reduction, row offsets of 31 bits
  const bool ok = dtype != MBX_F32 && aligned16(a) && aligned16(x) && aligned16(c) && k % 8 == 0 && n % 8 == 0 && dma_sizes_ok(k, n) &&
                  k > TileDmaSmallM::BM && n_slots <= 0x7fffffff && x_rows * (int64_t)n * 2 < ((int64_t)1 << 31) &&
                  rows * (int64_t)(k > n ? k : n) * 2 < ((int64_t)1 << 31);
  if (!ok) return MBX_EUNSUPPORTED;
  if (!row_table || row_table_bytes < mbx_gmm_tn_gather_table_bytes(x_rows, top_k, num_groups) || ((uintptr_t)row_table & 15u)) return MBX_ESCRATCH;
  if (x_rows == 0) x = a ? a : c;   // no row is read; the buffer descriptor still wants an address
  GatherRows gather;
  gather.slots = indices;
  gather.src_bins = x_bins ? x_bins : bins;
  gather.top_k = top_k;
  gather.src_rows = (int)x_rows;
  gather.row_table = (uint32_t*)row_table;
  gather.n_slots = n_slots;
  gather.table_ready = table_ready != 0;
  hipStream_t s = as_stream(stream);
  if (dtype == MBX_BF16) return gmm_dma<MBX_BF16, TileDma, TileDma>(a, x, c, bins, num_groups, rows, k, n, MBX_TN, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, gather);
  return gmm_dma<MBX_F16, TileDma, TileDma>(a, x, c, bins, num_groups, rows, k, n, MBX_TN, s, nullptr, nullptr, dma::kEpiNone, nullptr, nullptr, gather);
}

int mbx_gmm_dglu(const void* a, const void* b, const void* x1, const void* x2, void* d1, void* d2, int dtype,
                 const int32_t* bins, int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream) {
  if (act != MBX_ACT_SILU && act != MBX_ACT_GELU_TANH) return MBX_EINVAL;
  return gmm_nt_epilogue(a, b, d1, (void*)x1, dtype, bins, num_groups, rows, k, n, act,
                         act == MBX_ACT_SILU ? dma::kEpiDgluSilu : dma::kEpiDgluGelu, stream, x2, d2);
}

int mbx_gelu_backward_inplace(void* g, const void* x, int dtype, int64_t numel, mbx_stream_t stream) {
  if (numel < 0) return MBX_EINVAL;
  if (numel == 0) return 0;
  if (!g || !x) return MBX_EINVAL;
  if (dtype != MBX_BF16 && dtype != MBX_F16 && dtype != MBX_F32) return MBX_EINVAL;
  hipStream_t s = as_stream(stream);
  const int per_vec = 16 / dtype_bytes(dtype);
  const int64_t nvec = (aligned16(g) && aligned16(x)) ? numel / per_vec : 0;
  if (nvec > 0) {
    int64_t blocks = ceil_div(nvec, 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    switch (dtype) {
      case MBX_BF16: gelu_backward_vec_kernel<MBX_BF16><<<(unsigned)blocks, 256, 0, s>>>(g, x, nvec); break;
      case MBX_F16: gelu_backward_vec_kernel<MBX_F16><<<(unsigned)blocks, 256, 0, s>>>(g, x, nvec); break;
      default: gelu_backward_vec_kernel<MBX_F32><<<(unsigned)blocks, 256, 0, s>>>(g, x, nvec); break;
    }
  }
  const int64_t first = nvec * per_vec;
  if (first < numel) {
    int64_t blocks = ceil_div(numel - first, 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    switch (dtype) {
      case MBX_BF16: gelu_backward_kernel<MBX_BF16><<<(unsigned)blocks, 256, 0, s>>>(g, x, first, numel); break;
      case MBX_F16: gelu_backward_kernel<MBX_F16><<<(unsigned)blocks, 256, 0, s>>>(g, x, first, numel); break;
      default: gelu_backward_kernel<MBX_F32><<<(unsigned)blocks, 256, 0, s>>>(g, x, first, numel); break;
    }
  }
  return launch_status();
}

}  // extern "C"
