// Grouped-GEMM main loop with direct-to-LDS global loads and a four-stage LDS ring.
//
// Included by gmm.hip (uses its u32x4 / f32x16 types, mfma32, pack2 and the XCD tile mapping).
//
// Why: with 256x256 output tiles a compute unit has to pull 64 bytes of operands per 16
// MFMA-cycles from L2 / Infinity Cache, whose latency under load is a few thousand cycles.  Loads
// that pass through registers can only be one tile ahead (the registers are the limit), which
// leaves the matrix cores idle most of the time.  Here the loads are `buffer_load_dwordx4 ... lds`:
// they write LDS directly, occupy no registers, and three K tiles (96 KiB) are kept in flight per
// compute unit while a fourth is multiplied.
//
// LDS layout of one operand tile (R = 256 rows or columns, BK = 32):
//   KC operand (reduction dim contiguous in memory): [row][32 k] = 64-byte rows, 16-byte chunk c
//     of row r stored at chunk position c ^ ((r >> 2) & 3), so that the 16 lanes a ds_read_b128
//     serves per cycle (16 consecutive rows, same chunk) touch 16 distinct 16-byte bank groups of
//     the 64-bank LDS.
//   MC operand (reduction dim strided): [k][256 cols] = 512-byte rows, 32-byte pair p of row k
//     stored at pair position p ^ (2 (k & 3)), so that the 32 lanes a ds_read_b64_tr_b16 serves per
//     cycle (4 k-rows x two adjacent 32-byte pairs) touch 8 distinct pairs of a 256-byte bank line.
// A wave-wide load instruction fills 1 KiB of LDS in lane order, so the swizzle is applied by
// choosing which global address each lane fetches.  The reads of these tiles are inline asm: the
// compiler would otherwise wait for ALL outstanding LDS-DMA loads before any LDS read.
#pragma once

namespace dma {

constexpr int BK = 32;
constexpr int STAGES = 4;

template <int BM_, int BN_, int WM_, int WN_, int PREFETCH_ = 0>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, PREFETCH = PREFETCH_;
  static constexpr int WAVES = WM * WN, THREADS = WAVES * kWave;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int A_INSTRS = A_BYTES / 1024, B_INSTRS = B_BYTES / 1024;  // wave-wide 1 KiB loads per tile
  // L2 warm-up: per tile and operand, one 4-byte load per 64 bytes of the tile PREFETCH tiles ahead
  static constexpr int PF_INSTRS_A = PREFETCH > 0 ? A_BYTES / 64 / kWave : 0, PF_INSTRS_B = PREFETCH > 0 ? B_BYTES / 64 / kWave : 0;
  static constexpr int LOADS_PER_WAVE = (A_INSTRS + B_INSTRS + PF_INSTRS_A + PF_INSTRS_B) / WAVES;
  static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_BYTES + (PREFETCH > 0 ? 256 * WAVES : 0);
  static_assert(PREFETCH == 0 || (PF_INSTRS_A % WAVES == 0 && PF_INSTRS_B % WAVES == 0), "warm-up loads must split evenly over the waves");
  static_assert(A_INSTRS % WAVES == 0 && B_INSTRS % WAVES == 0, "loads must split evenly over the waves");
  static_assert(WAVES % 2 == 0, "the MC swizzle needs the parity of a wave's load index to be fixed");
};

typedef __attribute__((address_space(3))) char* lds_ptr;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // at most N vector-memory loads of this wave still in flight
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

// ---- LDS reads (inline asm; `addr` is a byte address in LDS) ----
template <int OFF>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// Per-lane byte offset (inside an operand tile) of the MFMA operand of the 32 rows/cols starting
// at `r`, k-step 0.  KC: k-step 1 is the same address with bit 5 flipped.  MC: k-step 1 is +8192.
template <bool MC>
__device__ __forceinline__ uint32_t frag_lane_offset(int r) {
  const int lane = lane_id();
  if (!MC) {
    const int row = lane & 31, xr = (row >> 2) & 3;
    return (uint32_t)((r + row) * 64 + (((lane >> 5) ^ xr) << 4));
  } else {
    const int g = lane >> 4, s = lane & 15;
    const int k = (g >> 1) * 8 + (s >> 2);
    const int pair = (r >> 4) + (g & 1);
    return (uint32_t)(k * 512 + ((pair ^ (2 * ((s >> 2) & 3))) << 5) + ((s & 3) << 3));
  }
}

template <bool MC, int KS>
__device__ __forceinline__ u32x4 read_frag(uint32_t tile_addr, uint32_t lane_off) {
  if (!MC) {
    return lds_read_b128<0>(tile_addr + (lane_off ^ (KS * 32)));
  } else {
    const u32x2 lo = lds_read_tr16_b64<KS * 8192>(tile_addr + lane_off);
    const u32x2 hi = lds_read_tr16_b64<KS * 8192 + 2048>(tile_addr + lane_off);
    u32x4 v;
    v[0] = lo[0]; v[1] = lo[1]; v[2] = hi[0]; v[3] = hi[1];
    return v;
  }
}

// ---- global -> LDS ----
// Byte offset (from the operand's buffer base) fetched by this lane in the wave's first load of
// tile 0; `r0` is the tile origin in the non-reduction dimension, `ld_bytes` the row pitch.
template <bool MC>
__device__ __forceinline__ uint32_t load_lane_offset(int wave, int r0, uint32_t ld_bytes) {
  const int lane = lane_id();
  if (!MC) {  // 16 rows x 4 chunks per instruction
    const int row = lane >> 2, pc = lane & 3;
    const int c = pc ^ ((row >> 2) & 3);
    return (uint32_t)(r0 + row) * ld_bytes + (uint32_t)(c << 4);
  } else {    // 2 k-rows x 32 chunks per instruction; instruction j holds k = 2j, 2j + 1
    const int kl = lane >> 5, pc = lane & 31;
    const int k3 = (2 * (wave & 1) + kl) & 3;          // (2j + kl) & 3 with j = wave (mod 2)
    const int c = ((((pc >> 1) ^ (2 * k3)) << 1) | (pc & 1));
    return (uint32_t)kl * ld_bytes + (uint32_t)(r0 * 2) + (uint32_t)(c << 4);
  }
}

template <bool MC, int INSTRS, int WAVES>
__device__ __forceinline__ void issue_operand(__amdgpu_buffer_rsrc_t rsrc, lds_ptr tile, int wave, uint32_t lane_off,
                                              uint32_t tile_off, uint32_t ld_bytes) {
#pragma unroll
  for (int q = 0; q < INSTRS / WAVES; ++q) {
    const int j = wave + q * WAVES;
    const uint32_t off = lane_off + tile_off + (uint32_t)j * (MC ? 2u : 16u) * ld_bytes;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(tile + j * 1024), 16, (int)off, 0, 0, 0);
  }
}

// Warm-up load: lane l of the wave's q-th instruction touches the 64-byte piece number
// (wave + q * WAVES) * 64 + l of the operand tile.
template <bool MC>
__device__ __forceinline__ uint32_t touch_lane_offset(int piece, int r0, uint32_t ld_bytes) {
  if (!MC) return (uint32_t)(r0 + piece) * ld_bytes;                                  // piece = row (64 bytes of k)
  return (uint32_t)(piece >> 3) * ld_bytes + (uint32_t)(r0 * 2) + (uint32_t)((piece & 7) << 6);  // 8 pieces per k-row
}

struct Args {
  __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b;  // out-of-range bytes read as zero
  uint32_t a_ld_bytes, b_ld_bytes;
  int a_r0, b_r0;                         // tile origin (row of a KC operand / column of an MC operand)
  int nk;                                 // number of 32-wide K tiles
};

// acc (+)= A_tile * B_tile over all K tiles, then c[m][n] = acc for m < m_lim, n < n_lim, where
// m = m_base + (row inside the tile) and n = n_base + (column inside the tile).
template <int DT, bool A_MC, bool B_MC, typename T>
__device__ __forceinline__ void block_gemm(const Args& g, uint16_t* __restrict__ c, int64_t ldc, int m_base, int m_lim,
                                           int n_base, int n_lim, char* lds_generic) {
  const lds_ptr lds = (lds_ptr)lds_generic;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = lane_id();
  const int wm = (wave / T::WN) * T::WTM, wn = (wave % T::WN) * T::WTN;

  f32x16 acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const uint32_t a_lane = load_lane_offset<A_MC>(wave, g.a_r0, g.a_ld_bytes);
  const uint32_t b_lane = load_lane_offset<B_MC>(wave, g.b_r0, g.b_ld_bytes);
  const uint32_t a_step = A_MC ? BK * g.a_ld_bytes : BK * 2;   // bytes per K tile
  const uint32_t b_step = B_MC ? BK * g.b_ld_bytes : BK * 2;
  uint32_t a_touch[T::PF_INSTRS_A / T::WAVES > 0 ? T::PF_INSTRS_A / T::WAVES : 1], b_touch[T::PF_INSTRS_B / T::WAVES > 0 ? T::PF_INSTRS_B / T::WAVES : 1];
  if (T::PREFETCH > 0) {
#pragma unroll
    for (int q = 0; q < T::PF_INSTRS_A / T::WAVES; ++q) a_touch[q] = touch_lane_offset<A_MC>((wave + q * T::WAVES) * kWave + lane, g.a_r0, g.a_ld_bytes);
#pragma unroll
    for (int q = 0; q < T::PF_INSTRS_B / T::WAVES; ++q) b_touch[q] = touch_lane_offset<B_MC>((wave + q * T::WAVES) * kWave + lane, g.b_r0, g.b_ld_bytes);
  }
  auto issue = [&](int kt) {
#ifdef MBX_TUNE_NO_GLOBAL
    return;
#endif
    const lds_ptr stage = lds + (kt % STAGES) * T::STAGE_BYTES;
    issue_operand<A_MC, T::A_INSTRS, T::WAVES>(g.rsrc_a, stage, wave, a_lane, (uint32_t)kt * a_step, g.a_ld_bytes);
    issue_operand<B_MC, T::B_INSTRS, T::WAVES>(g.rsrc_b, stage + T::A_BYTES, wave, b_lane, (uint32_t)kt * b_step, g.b_ld_bytes);
    if (T::PREFETCH > 0) {
      // pull tile kt + PREFETCH into L2; the 4 bytes per lane land in a scratch corner of LDS nobody reads
      const lds_ptr dump = lds + STAGES * T::STAGE_BYTES + wave * 256;
      const uint32_t ka = (uint32_t)(kt + T::PREFETCH) * a_step, kb = (uint32_t)(kt + T::PREFETCH) * b_step;
#pragma unroll
      for (int q = 0; q < T::PF_INSTRS_A / T::WAVES; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(g.rsrc_a, (__attribute__((address_space(3))) void*)dump, 4, (int)(a_touch[q] + ka), 0, 0, 0);
#pragma unroll
      for (int q = 0; q < T::PF_INSTRS_B / T::WAVES; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(g.rsrc_b, (__attribute__((address_space(3))) void*)dump, 4, (int)(b_touch[q] + kb), 0, 0, 0);
    }
  };

  // per-lane LDS offsets of the MFMA operands (KC: one base, tiles at +i*2048; MC: one per tile)
  uint32_t fa_off[A_MC ? T::TM : 1], fb_off[B_MC ? T::TN : 1];
  if (A_MC) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i) fa_off[i] = frag_lane_offset<true>(wm + i * 32);
  } else {
    fa_off[0] = frag_lane_offset<false>(wm);
  }
  if (B_MC) {
#pragma unroll
    for (int j = 0; j < T::TN; ++j) fb_off[j] = T::A_BYTES + frag_lane_offset<true>(wn + j * 32);
  } else {
    fb_off[0] = T::A_BYTES + frag_lane_offset<false>(wn);
  }

  u32x4 fa[2][T::TM], fb[2][T::TN];
#ifdef MBX_TUNE_NO_LDS
#define MBX_READ_FRAGS(KS, BUF, STAGE_ADDR) do { } while (0)
#else
#define MBX_READ_FRAGS(KS, BUF, STAGE_ADDR)                                                                      \
  do {                                                                                                           \
    _Pragma("unroll") for (int i = 0; i < T::TM; ++i)                                                            \
        fa[BUF][i] = A_MC ? read_frag<true, KS>(STAGE_ADDR, fa_off[A_MC ? i : 0])                                \
                          : read_frag<false, KS>(STAGE_ADDR + i * 2048, fa_off[0]);                              \
    _Pragma("unroll") for (int j = 0; j < T::TN; ++j)                                                            \
        fb[BUF][j] = B_MC ? read_frag<true, KS>(STAGE_ADDR, fb_off[B_MC ? j : 0])                                \
                          : read_frag<false, KS>(STAGE_ADDR + j * 2048, fb_off[0]);                              \
  } while (0)
#endif
  // the MFMAs may only start once the operands have arrived: tie them to the wait through "+v"
#define MBX_WAIT_FRAGS(BUF)                                                                                      \
  do {                                                                                                           \
    _Pragma("unroll") for (int i = 0; i < T::TM; ++i) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[BUF][i]));    \
    _Pragma("unroll") for (int j = 0; j < T::TN; ++j) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fb[BUF][j]));    \
  } while (0)
  // operands swapped: the accumulator tile is c^T, so a lane owns runs of four consecutive
  // columns of one row of c and can store them as one 8-byte word
#define MBX_MULTIPLY(BUF)                                                                                        \
  do {                                                                                                           \
    _Pragma("unroll") for (int i = 0; i < T::TM; ++i)                                                            \
      _Pragma("unroll") for (int j = 0; j < T::TN; ++j) acc[i][j] = mfma32<DT>(fb[BUF][j], fa[BUF][i], acc[i][j]); \
  } while (0)

  const int nk = g.nk;
  if (nk > 0) {
    // prologue: fill the ring, wait for tile 0
#pragma unroll
    for (int t = 0; t < STAGES; ++t)
      if (t < nk) issue(t);
    constexpr int L = T::LOADS_PER_WAVE;
    if (nk >= 4) wait_vmcnt<3 * L>();
    else if (nk == 3) wait_vmcnt<2 * L>();
    else if (nk == 2) wait_vmcnt<L>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    MBX_READ_FRAGS(0, 0, lds_base);

    for (int kt = 0; kt < nk; ++kt) {
      const uint32_t cur = lds_base + (uint32_t)(kt % STAGES) * T::STAGE_BYTES;
      const uint32_t nxt = lds_base + (uint32_t)((kt + 1) % STAGES) * T::STAGE_BYTES;
      MBX_WAIT_FRAGS(0);            // operands of k-step 0, read half an iteration ago
      MBX_READ_FRAGS(1, 1, cur);    // k-step 1 arrives under the MFMAs of k-step 0
      __builtin_amdgcn_sched_barrier(0);
      MBX_MULTIPLY(0);
      __builtin_amdgcn_sched_barrier(0);
      MBX_WAIT_FRAGS(1);
      // Tile kt is now entirely in registers.  Once every wave is here and tile kt+1 has landed, the
      // stage of tile kt can be refilled with tile kt+4.
      const int ahead = nk - 2 - kt;  // tiles issued beyond kt+1
      if (ahead >= 2) wait_vmcnt<2 * L>();
      else if (ahead == 1) wait_vmcnt<L>();
      else wait_vmcnt<0>();
      __builtin_amdgcn_s_barrier();
      if (kt + STAGES < nk) issue(kt + STAGES);
      if (kt + 1 < nk) MBX_READ_FRAGS(0, 0, nxt);
      __builtin_amdgcn_sched_barrier(0);
      MBX_MULTIPLY(1);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#undef MBX_READ_FRAGS
#undef MBX_WAIT_FRAGS
#undef MBX_MULTIPLY

  // accumulator (i, j), register r of lane l holds c[m][n] with
  //   m = m_base + wm + 32 i + (l % 32),  n = n_base + wn + 32 j + 8 (r / 4) + 4 (l / 32) + (r % 4)
  const bool n_vec = (ldc % 4 == 0) && (((uintptr_t)c & 7u) == 0);
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    const int m = m_base + wm + i * 32 + (lane & 31);
    if (m >= m_lim) continue;
    uint16_t* crow = c + (int64_t)m * ldc;
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_base + wn + j * 32 + q * 8 + (lane >> 5) * 4;
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

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
}

// ---- NN / NT ----
template <int DT, bool B_MC, typename T>
__global__ void __launch_bounds__(T::THREADS)
gmm_rows_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
                const int32_t* __restrict__ bins, int num_groups, int64_t rows, int k, int n, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  int id = xcd_tile_id(blockIdx.x);
  int e = 0, start = 0, end = 0, mt = 0;
  for (; e < num_groups; ++e) {
    end = bins[e];
    mt = (end - start + T::BM - 1) / T::BM;
    const int span = mt * tiles_n;
    if (id < span) break;
    id -= span;
    start = end;
  }
  if (e >= num_groups) return;
  const int tn = id / mt, tm = id % mt;
  Args g;
  g.rsrc_a = make_rsrc(a, (uint32_t)(rows * k * 2));
  g.a_ld_bytes = (uint32_t)k * 2;
  g.a_r0 = start + tm * T::BM;
  g.rsrc_b = make_rsrc(b + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2));
  g.b_ld_bytes = (uint32_t)(B_MC ? n : k) * 2;
  g.b_r0 = tn * T::BN;
  g.nk = k / BK;
  block_gemm<DT, false, B_MC, T>(g, c, n, g.a_r0, end, g.b_r0, n, lds);
}

// ---- TN ----
template <int DT, typename T>
__global__ void __launch_bounds__(T::THREADS)
gmm_tn_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
              const int32_t* __restrict__ bins, int num_groups, int k, int n, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int id = xcd_tile_id(blockIdx.x);
  const int per_group = tiles_m * tiles_n;
  const int e = id / per_group;
  if (e >= num_groups) return;
  const int t = id % per_group;
  const int tm = t % tiles_m, tn = t / tiles_m;
  const int start = e > 0 ? bins[e - 1] : 0, end = bins[e];
  const int64_t group_rows = end - start;
  Args g;
  // the buffers cover exactly the rows of this expert: later rows read as zero
  g.rsrc_a = make_rsrc(a + (int64_t)start * k, (uint32_t)(group_rows * k * 2));
  g.a_ld_bytes = (uint32_t)k * 2;
  g.a_r0 = tm * T::BM;
  g.rsrc_b = make_rsrc(b + (int64_t)start * n, (uint32_t)(group_rows * n * 2));
  g.b_ld_bytes = (uint32_t)n * 2;
  g.b_r0 = tn * T::BN;
  g.nk = (int)((group_rows + BK - 1) / BK);
  block_gemm<DT, true, true, T>(g, c + (int64_t)e * k * n, n, g.a_r0, k, g.b_r0, n, lds);
}

}  // namespace dma
