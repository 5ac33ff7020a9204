// Grouped-GEMM main loop with direct-to-LDS global loads and LDS rings of K tiles, and the kernels
// that walk the tiles of a launch with it.
//
// Included by gmm.hip (uses its u32x4 / f32x4 types, pack2 and the XCD constants).
//
// Why: with 256x256 output tiles a compute unit has to pull 64 bytes of operands per 16
// MFMA-cycles.  Loads that pass through registers can only run one tile ahead and cost 64
// registers per lane; `buffer_load_dwordx4 ... lds` writes LDS directly, so a whole K tile
// (or several) is in flight while another is multiplied, with no register cost.
//
// The L1 (TCP) of a compute unit handles about 0.35 distinct 128-byte lines per clock no matter how
// few bytes of a line are wanted, so operand rows are fetched 128 bytes at a time: BK = 64 for the
// operands whose reduction dimension is contiguous in memory.
//
// LDS layout of one operand tile (R = 256 rows or columns):
//   KC operand (reduction dim contiguous in memory): [row][BK k], 16-byte chunk c of row r stored
//     at chunk position c ^ swz(r), swz(r) = (r >> 1) & 7 for 128-byte rows (BK 64) and
//     (r >> 2) & 3 for 64-byte rows (BK 32), so that the 16 lanes a ds_read_b128 serves per cycle
//     (16 consecutive rows, same chunk) touch 16 distinct 16-byte bank groups of the 64-bank LDS.
//   MC operand (reduction dim strided): [k][R cols] = 2 R-byte rows (R = 256 or 128), 32-byte pair p of
//     row k stored at pair position p ^ (2 (k & 3)), so that the 32 lanes a ds_read_b64_tr_b16 serves per
//     cycle (4 k-rows x two adjacent 32-byte pairs) touch 8 distinct pairs of a 256-byte bank line.
// A wave-wide load instruction fills 1 KiB of LDS in lane order, so the swizzle is applied by
// choosing which global address each lane fetches.  The reads of these tiles are inline asm: the
// compiler would otherwise wait for ALL outstanding LDS-DMA loads before any LDS read.
#pragma once

#include <type_traits>
#include <utility>

namespace dma {

// The two operands have separate LDS rings: SB stages for the B operand and SA = SB + 1 for the A
// operand.  The extra A stage lets the A loads of a K tile be issued during the k-steps in which no
// B load can be (the B stage to refill is still being read), so that global -> LDS loads leave the
// compute unit at an even rate: the texture-address unit takes some 20 cycles per wave-wide load, is
// shared by the four waves, and a wave whose load has to queue cannot issue its next MFMA either.
// The matrix-core instruction is v_mfma_f32_16x16x32 (16 x 16 product tiles of four accumulator registers per lane,
// reduction length 32): MF names its rows / columns.  It has the peak rate and the LDS bytes per FLOP of the
// 32 x 32 x 16 form and moves half the accumulator registers per FLOP, which under this part's power limit is clock
// (a loop of nothing but these instructions on operands with random mantissas sustains 2.05 GHz where the other
// sustains 1.8); a main loop on the 32 x 32 x 16 form was 4 - 6 % slower on every workload and is gone.
template <int BM_, int BN_, int WM_, int WN_, int BK_, int SB_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, BK = BK_, SB = SB_, SA = SB_ + 1, MF = 16;
  static constexpr int KSTEP = 32;                                             // reduction length of one MFMA
  static constexpr int KS = BK / KSTEP;                                        // MFMA k-steps per tile
  static constexpr int WAVES = WM * WN, THREADS = WAVES * kWave;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / MF, TN = WTN / MF;
  typedef f32x4 Acc;                                                           // one product tile of a lane
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int A_INSTRS = A_BYTES / 1024, B_INSTRS = B_BYTES / 1024;  // wave-wide 1 KiB loads per tile
  static constexpr int LA = A_INSTRS / WAVES, LB = B_INSTRS / WAVES;          // ... per wave
  static constexpr size_t RING_BYTES = (size_t)SA * A_BYTES + (size_t)SB * B_BYTES, EPILOGUE_BYTES = (size_t)BM * (BN * 2 + 16);
  static constexpr size_t LDS_BYTES = RING_BYTES > EPILOGUE_BYTES ? RING_BYTES : EPILOGUE_BYTES;
  static_assert(BK == 64, "K tile");
  static_assert(SB >= 2 && LDS_BYTES <= 160 * 1024, "LDS rings");
  static_assert((BM == 256 || BM == 128) && (BN == 256 || BN == 128), "tile widths the strided-operand LDS layout knows");
  static_assert(A_INSTRS % WAVES == 0 && B_INSTRS % WAVES == 0, "loads must split evenly over the waves");
  static_assert(LA % 2 == 0 && LB % 2 == 0, "the loads of an operand tile are issued in two halves");
  static_assert(WAVES % 2 == 0, "the swizzles need the parity of a wave's load index to be fixed");
  static_assert((SB - 1) * (LA + LB) + LA + LB / 2 < 64, "vmcnt is a 6-bit counter");
};

typedef __attribute__((address_space(3))) char* lds_ptr;

// Measurement build only (libmbx_ticks.so, compiled with -DMBX_TICKS; the library proper has none of this): the first
// lane of a workgroup stamps the phases of every output tile with the constant-rate clock (s_memrealtime, 100 MHz) into
//   g_ticks[(workgroup * kTickTiles + ordinal of the tile in the workgroup) * kTickIds + id]
// id 0: tile starts, 6: its operands are known, 7: the first K tiles are requested, 3: the accumulators are cleared,
// 1: the first K tile has landed, 2: last MFMA done, 4: the tile's last store issued, 5: LDS handed on.
#ifdef MBX_TICKS
__device__ uint64_t* g_ticks;
constexpr int kTickWorkgroups = 16384, kTickTiles = 64, kTickIds = 8;   // the buffer's shape (8 bytes per entry)
__device__ __forceinline__ void tick(int ordinal, int id) {
  if (threadIdx.x == 0 && g_ticks != nullptr && ordinal >= 0 && ordinal < kTickTiles && blockIdx.x < kTickWorkgroups)
    g_ticks[((size_t)blockIdx.x * kTickTiles + ordinal) * kTickIds + id] = __builtin_amdgcn_s_memrealtime();
}
#define MBX_TICK(ordinal, id) tick(ordinal, id)
#else
#define MBX_TICK(ordinal, id) ((void)0)
#endif

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant
// expression in the body (it selects instruction immediates).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

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

// Per-lane byte offset (inside an operand tile) of the MFMA operand of the 16 rows / columns starting at `r`, k-step 0.
// Lane l holds row / column l % 16 and the eight k values 8 (l / 16) ..; k-step s is 32 k further (KC: bits 6.. of the
// address XORed by 64 s; MC: 32 rows of COLS columns).  The MC layout swizzles the 32-byte pair index by
// 2 (k & 3) ^ ((k >> 3) & 1): the two 16-lane groups a transposing read serves per cycle hold k rows 8 apart.
template <bool MC, int BK, int COLS>
__device__ __forceinline__ uint32_t frag_lane_offset(int r) {
  const int lane = lane_id();
  if (!MC) {
    static_assert(BK == 64, "operands are read from 128-byte rows");
    const int row = lane & 15;
    const int swz = (row >> 1) & 7;
    return (uint32_t)((r + row) * (BK * 2) + (((lane >> 4) ^ swz) << 4));
  } else {
    const int g = lane >> 4, s = lane & 15;
    const int k = g * 8 + (s >> 2);
    const int pair = r >> 4;
    return (uint32_t)(k * (COLS * 2) + ((pair ^ (2 * ((s >> 2) & 3)) ^ (g & 1)) << 5) + ((s & 3) << 3));
  }
}

// A fragment of a KC operand, k-step KS.  IMM: constant byte offset of the 16-row fragment inside the operand tile (goes
// into the instruction).
template <int KS, int IMM>
__device__ __forceinline__ u32x4 read_frag_kc(uint32_t tile_addr, uint32_t lane_off) {
  return lds_read_b128<IMM>(tile_addr + (lane_off ^ (KS * 32 * 2)));
}

// ---- global -> LDS ----
// Byte offset (from the operand's buffer base) fetched by this lane in the wave's first load of
// tile 0; `r0` is the tile origin in the non-reduction dimension, `ld_bytes` the row pitch.
// The MC swizzle has the term (k >> 3) & 1 (see frag_lane_offset).  With 256 columns a load holds k = 2 j, 2 j + 1
// for load number j = wave + 4 q of the tile, so that term is the parity of q (`odd`); with 128 columns (k = 4 j ..) it
// is (wave >> 1) & 1.
template <bool MC, int BK, int COLS>
__device__ __forceinline__ uint32_t load_lane_offset(int wave, int r0, uint32_t ld_bytes, bool odd = false) {
  const int lane = lane_id();
  if (!MC) {
    static_assert(BK == 64, "8 rows x 8 chunks per instruction");   // instruction j holds rows 8j .. 8j + 7
    const int row = lane >> 3, pc = lane & 7;
    const int c = pc ^ ((4 * (wave & 1) + (row >> 1)) & 7);     // ((8j + row) >> 1) & 7 with j = wave (mod 2)
    return (uint32_t)(r0 + row) * ld_bytes + (uint32_t)(c << 4);
  } else if (COLS == 256) {   // 2 k-rows x 32 chunks per instruction; instruction j holds k = 2j, 2j + 1
    const int kl = lane >> 5, pc = lane & 31;
    const int k3 = (2 * (wave & 1) + kl) & 3;                     // (2j + kl) & 3 with j = wave (mod 2)
    const int x = (2 * k3) ^ (odd ? 1 : 0);
    const int c = ((((pc >> 1) ^ x) << 1) | (pc & 1));
    return (uint32_t)kl * ld_bytes + (uint32_t)(r0 * 2) + (uint32_t)(c << 4);
  } else {                    // 128 columns: 4 k-rows x 16 chunks per instruction; instruction j holds k = 4j .. 4j + 3
    static_assert(!MC || COLS == 256 || COLS == 128, "strided operand tile width");
    const int kl = lane >> 4, pc = lane & 15;
    const int x = (2 * kl) ^ ((wave >> 1) & 1);
    const int c = ((((pc >> 1) ^ x) << 1) | (pc & 1));
    return (uint32_t)kl * ld_bytes + (uint32_t)(r0 * 2) + (uint32_t)(c << 4);
  }
}

// One wait for all LDS reads in flight, tied to the operand registers of a k-step so that the MFMAs
// that consume them cannot be scheduled above it.
template <int N>
__device__ __forceinline__ void tie_frags(u32x4 (&f)[N]) {   // no instruction: orders later users of f behind the preceding wait
  static_assert(N == 4 || N == 8, "operand registers per k-step");
  if constexpr (N == 8) {
    asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7]));
  } else {
    asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]));
  }
}

template <int NA, int NB>
__device__ __forceinline__ void wait_frags(u32x4 (&a)[NA], u32x4 (&b)[NB]) {
  static_assert(NA <= 8 && NB <= 8 && NA >= 2 && NB >= 2, "operand registers per k-step");
  if constexpr (NA == 8) {   // an asm statement takes at most 30 operands, and "+v" counts twice
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
    tie_frags(b);
  } else if constexpr (NA == 4 && NB == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
  } else if constexpr (NA == 4 && NB == 2) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]));
  } else if constexpr (NA == 2 && NB == 2) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]));
  } else {
    static_for<NA>([&](auto i) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[decltype(i)::value])); });
    static_for<NB>([&](auto i) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(b[decltype(i)::value])); });
  }
}

struct Args {
  __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b;  // out-of-range bytes read as zero
  uint32_t a_ld_bytes, b_ld_bytes;
  int a_r0, b_r0;                         // tile origin (row of a KC operand / column of an MC operand)
  int nk;                                 // number of K tiles
  // A product of two operand pairs, a @ b + a2 @ b2 (same shapes and pitches): K tiles nk1 .. nk-1 come
  // from the second pair.  Used only by the DUAL instantiations.
  __amdgpu_buffer_rsrc_t rsrc_a2, rsrc_b2;
  int nk1;
  // GATHER instantiations: the rows of the A tile are rows of the matrix behind rsrc_a picked by a row map.  Load q of
  // a lane's LA loads of a K tile fetches the 16 bytes at gather_row[q] (+ the K tile's offset); bit 31 set: the row
  // is a row of zeros.
  uint32_t gather_row[8];
  // GATHER_B instantiations (TN): the rows of the B tile (an MC operand: its rows are the reduction) are rows of the
  // matrix behind rsrc_b picked by a row map.  The map comes as a table of byte offsets, one 4-byte entry per row of
  // the reduction (bit 31 flipped: an entry read past the end of the table, i.e. zero, then means "no row"), read
  // through row_table (words of a buffer descriptor over the expert's part of the table).  gather_row / gather_row2:
  // the entries of this lane's loads of K tiles 0 and 1, fetched by the caller while the tile before was computed.
  uint32_t gather_row2[8];
  u32x4 row_table;
  int tick_ordinal = -1;                  // MBX_TICKS builds: which tile of the workgroup this is
};

// Row tables (see Args::row_table) are laid out for the loads that read them: 64 entries per K tile of an expert, in the
// order in which the lanes want them.  Load q (of 8) of wave w (of 4) holds rows 2 j and 2 j + 1 of the K tile,
// j = w + 4 q, lanes 0 .. 31 the first; so the eight entries a lane needs for a K tile (q = 0 .. 7, row parity kl =
// lane / 32) sit together at entries (2 w + kl) 8 .. + 7, and a lane fetches them with two 16-byte loads.
// row_entry_slot(): where the entry of row r of a K tile is; row_of_entry_slot(): its inverse.
constexpr int kRowTableTile = 64;   // entries per K tile
__host__ __device__ constexpr int row_entry_slot(int r) { return (((r >> 1) & 3) * 2 + (r & 1)) * 8 + (r >> 3); }
__host__ __device__ constexpr int row_of_entry_slot(int p) { return 2 * ((p >> 4) + 4 * (p & 7)) + ((p >> 3) & 1); }
// Expert e's part of a table starts at entry (number of assignments before it) + 64 e: room for its last K tile to be
// whole without reaching into the next expert's part.
__host__ __device__ constexpr int64_t row_table_entries(int64_t n_slots, int num_groups) { return n_slots + (int64_t)kRowTableTile * num_groups; }
__device__ __forceinline__ uint32_t row_entry_lane_offset(int wave) { return (uint32_t)(2 * wave + (lane_id() >> 5)) * 32u; }
// The eight entries of this lane for the K tile at byte offset soff of the table (inline asm, so that the compiler
// does not count the loads among those it waits for: the main loop's own waits cover them).
__device__ __forceinline__ void fetch_row_entries(uint32_t (&dst)[8], const u32x4& table, uint32_t voff, uint32_t soff) {
  u32x4 lo, hi;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(lo) : "v"(voff), "s"(table), "s"(soff));
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:16" : "=v"(hi) : "v"(voff), "s"(table), "s"(soff));
#pragma unroll
  for (int q = 0; q < 4; ++q) { dst[q] = lo[q]; dst[4 + q] = hi[q]; }
}

// acc += a-fragment x b-fragment with v_mfma_f32_16x16x32, written as inline asm with the accumulator tied to one
// register tuple ("+a": an AGPR tuple, source and destination): with the builtin, whose destination may differ from
// its accumulator source, the register allocator gave the 64 four-register tiles of a wave other registers at the
// bottom of the main loop than at its top and moved all of them back every iteration (some 400 copies).  The
// compiler does not know that this statement is a matrix-core instruction, so the wait states the instruction set
// asks for around reads and writes of the accumulators by other instructions are put in by hand (mfma16_settle).
template <int DT>
__device__ __forceinline__ void mfma16_acc(f32x4& acc, const u32x4& a, const u32x4& b) {
  if (DT == MBX_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// more wait states than any hazard between a vector-ALU access and a matrix-core access of the same register needs
__device__ __forceinline__ void mfma16_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

// The same product with v_mfma_f32_16x16x32: two k-steps of 32 per K tile, TM x TN = 8 x 8 product tiles of 16 x 16
// per wave (the same 128 x 128 wave tile and 256 accumulator registers; 8 + 8 operand fragments per k-step, double
// buffered: 128 registers).  The one barrier of a K tile sits between its two k-steps, when every wave has both
// k-steps of tile kt in registers: B stage kt % SB is free from then on, A stage kt % SA as well.  Iteration kt issues
//   k-step 0: A tile kt + SB -> A stage (kt - 1) % SA (free since the barrier of iteration kt - 1)
//   barrier:  tile kt + 1 has landed
//   k-step 1: B tile kt + SB -> B stage kt % SB, from the first gaps on
// so that every load has at least a K tile and a half of MFMAs before the barrier that waits for it (a B load issued
// just ahead of the barrier that needs it, as a transcription of the 32 x 32 x 16 schedule had it, stalls every K tile
// for a memory latency).  The prologue loads tiles 0 .. SB - 1 completely.
// GLU: rows BN / 2 .. BN - 1 of the B tile (the second half of every wave's loads of a K tile) come through g.rsrc_b2,
// whose base the caller has set BN / 2 rows before the second matrix: the tile is then [w1 rows | v1 rows] of the same
// BN / 2 output columns, side by side (KC operands only, not with DUAL).
// GATHER: the rows of the A tile (KC operand) are gathered rows of a matrix: each of a lane's LA loads of a K tile gets
// a byte offset of its own (its row's, worked out once per tile from the row map), where the plain tile adds a
// multiple of the row pitch to one lane offset.  The loads are the same 16-byte pieces of 128-byte row segments.
// GATHER_B: the rows of the B tile (MC operand of 256 columns: the reduction runs over its rows) are gathered rows of a
// matrix: each of a lane's LB loads of a K tile takes the byte offset of its row from a table (Args::row_table), which
// it fetches a K tile ahead -- right after the load that used the entry for the K tile before, into the same register.
template <int DT, bool A_MC, bool B_MC, typename T, bool DUAL = false, bool GLU = false, bool GATHER = false, bool GATHER_B = false>
__device__ __forceinline__ void block_multiply16(const Args& g, typename T::Acc (&acc)[T::TM][T::TN], bool clear, char* lds_generic) {
  static_assert(T::KS == 2, "two k-steps of 32 per K tile");
  static_assert(!GLU || (!B_MC && !DUAL && T::LB % 2 == 0), "two matrices side by side in the B tile");
  static_assert(!GATHER || (!A_MC && !DUAL && T::BK == 64), "gathered rows: a KC operand, one operand pair");
  static_assert(!GATHER_B || (B_MC && !DUAL && !GLU && T::BN == 256 && T::SB == 2 && T::LB == 8 && T::WAVES == 4), "gathered rows of a strided operand");
  const lds_ptr lds = (lds_ptr)lds_generic;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wm = (wave / T::WN) * T::WTM, wn = (wave % T::WN) * T::WTN;

  constexpr int BK = T::BK, SA = T::SA, SB = T::SB, LA = T::LA, LB = T::LB;
  constexpr uint32_t B_RING = (uint32_t)SA * T::A_BYTES;
  // a 256-column MC operand takes its lane offsets from the parity of the load's index inside the tile
  constexpr bool A_QDEP = A_MC && T::BM == 256, B_QDEP = B_MC && T::BN == 256;
  static_assert((LA / 2) % 2 == 0 && (LB / 2) % 2 == 0, "every group of loads starts at an even load index");
  const uint32_t a_lane = load_lane_offset<A_MC, BK, T::BM>(wave, g.a_r0, g.a_ld_bytes, false);
  const uint32_t b_lane = load_lane_offset<B_MC, BK, T::BN>(wave, g.b_r0, g.b_ld_bytes, false);
  const uint32_t a_lane1 = A_QDEP ? load_lane_offset<A_MC, BK, T::BM>(wave, g.a_r0, g.a_ld_bytes, true) : a_lane;
  const uint32_t b_lane1 = B_QDEP ? load_lane_offset<B_MC, BK, T::BN>(wave, g.b_r0, g.b_ld_bytes, true) : b_lane;
  const uint32_t a_step = A_MC ? BK * g.a_ld_bytes : BK * 2;   // bytes per K tile
  const uint32_t b_step = B_MC ? BK * g.b_ld_bytes : BK * 2;
  constexpr uint32_t A_ROWS = (uint32_t)(1024 / ((A_MC ? T::BM : BK) * 2)), B_ROWS = (uint32_t)(1024 / ((B_MC ? T::BN : BK) * 2));
  const uint32_t a_jstep = GATHER ? 0u : A_ROWS * g.a_ld_bytes, b_jstep = B_ROWS * g.b_ld_bytes;
  auto scalar_off = [&](bool is_b, int kt, int q) -> uint32_t {
    const uint32_t j = (uint32_t)(wave + q * T::WAVES);
    const uint32_t v = is_b ? (uint32_t)kt * b_step + j * b_jstep : (uint32_t)kt * a_step + j * a_jstep;
    return v | (kt < g.nk ? 0u : 0x80000000u);
  };
  // byte offset of the q-th A load's row and 16-byte piece (bit 31: no such row, the load brings zeros)
  static_assert(!GATHER || LA <= 8, "Args::gather_row");
  uint32_t a_row[GATHER ? LA : 1];
  if constexpr (GATHER) {
#pragma unroll
    for (int q = 0; q < LA; ++q) a_row[q] = g.gather_row[q];
  }
  // GATHER_B: the lane's row offsets for the B loads it issues next (load q: b_row[q]); the column part of the address
  // with the table's bit 31 folded in; where the lane's entries sit in a K tile's part of the table
  uint32_t b_row[GATHER_B ? LB : 1];
  const uint32_t b_col = GATHER_B ? load_lane_offset<B_MC, BK, T::BN>(wave, g.b_r0, 0u, false) + 0x80000000u : 0u;
  const uint32_t b_col1 = GATHER_B ? load_lane_offset<B_MC, BK, T::BN>(wave, g.b_r0, 0u, true) + 0x80000000u : 0u;
  const uint32_t entry_lane = GATHER_B ? row_entry_lane_offset(wave) : 0u;
  if constexpr (GATHER_B) {
#pragma unroll
    for (int q = 0; q < LB; ++q) b_row[q] = g.gather_row[q];
  }
  __amdgpu_buffer_rsrc_t ra = g.rsrc_a, rb = g.rsrc_b;
  const __amdgpu_buffer_rsrc_t rb_upper = GLU ? g.rsrc_b2 : g.rsrc_b;
  auto lds_off = [&](bool is_b, int stage, int q) -> uint32_t {
    return (is_b ? B_RING + (uint32_t)stage * T::B_BYTES : (uint32_t)stage * T::A_BYTES) + (uint32_t)(wave + q * T::WAVES) * 1024u;
  };
  // upper: the load is one of the second half of the wave's B loads of a K tile (GLU only)
  // q: the load's index among the wave's loads of the tile (GATHER, A loads: which row offset)
  auto issue = [&](bool is_b, uint32_t sc, uint32_t dst, bool odd, bool upper, int q) {
    if (is_b) {
      if constexpr (GATHER_B) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)(lds + dst), 16, (int)(b_row[GATHER_B ? q : 0] + (odd ? b_col1 : b_col)), 0, 0, 0);
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(GLU && upper ? rb_upper : rb, (__attribute__((address_space(3))) void*)(lds + dst), 16, (int)((odd ? b_lane1 : b_lane) + sc), 0, 0, 0);
      }
    } else {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void*)(lds + dst), 16, (int)((GATHER ? a_row[GATHER ? q : 0] : odd ? a_lane1 : a_lane) + sc), 0, 0, 0);
    }
  };
  auto issue_group = [&](bool is_b, int kt, int stage, int q0, int count) {   // prologue
    uint32_t sc = scalar_off(is_b, kt, q0), dst = lds_off(is_b, stage, q0);
#pragma unroll
    for (int i = 0; i < count; ++i) {
      issue(is_b, sc, dst, ((q0 + i) & 1) != 0, is_b && q0 + i >= LB / 2, q0 + i);
      sc += T::WAVES * (is_b ? b_jstep : a_jstep);
      dst += T::WAVES * 1024u;
    }
  };

  constexpr int KC_TILE = 16 * BK * 2;   // bytes of a 16-row fragment of a KC operand tile
  uint32_t fa_off[A_MC ? T::TM : 1], fb_off[B_MC ? T::TN : 1];
  if (A_MC) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i) fa_off[i] = frag_lane_offset<true, BK, T::BM>(wm + i * 16);
  } else {
    fa_off[0] = frag_lane_offset<false, BK, T::BM>(wm);
  }
  if (B_MC) {
#pragma unroll
    for (int j = 0; j < T::TN; ++j) fb_off[j] = frag_lane_offset<true, BK, T::BN>(wn + j * 16);
  } else {
    fb_off[0] = frag_lane_offset<false, BK, T::BN>(wn);
  }

  if (A_MC) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i) fa_off[A_MC ? i : 0] += lds_base;
  }
  if (B_MC) {
#pragma unroll
    for (int j = 0; j < T::TN; ++j) fb_off[B_MC ? j : 0] += lds_base + B_RING;
  }

  u32x4 fa[2][T::TM], fb[2][T::TN];
  constexpr int NF = T::TM + T::TN, NP = T::TM * T::TN;
  constexpr int NSA = (A_MC ? 2 : 1) * T::TM, NSB = (B_MC ? 2 : 1) * T::TN, NS = NSA + NSB;   // read instructions per k-step
  static_assert(NS <= NP, "one read per gap");
  // A strided (MC) operand has one lane offset per fragment; adding the stage's address to it for every read would
  // put a vector-ALU instruction right in front of every LDS read, which costs the wave eight cycles each time.  So
  // fa_off / fb_off of such an operand hold absolute addresses in the stage that is read next, and are moved on to
  // the following stage once per K tile (MBX_STEP16's MOVE hook), away from the reads.
  // One read instruction per gap: a fragment of a KC operand is one ds_read_b128, one of an MC operand two
  // transposing reads (its k values 0 .. 3 and 4 .. 7) that take a gap each.  Slot R of a k-step's NS read slots:
#define MBX_READ_SLOT16(KSTEP, BUF, A_ADDR, B_ADDR, R)                                                           \
  do {                                                                                                           \
    if constexpr ((R) < NSA) {                                                                                   \
      if constexpr (A_MC) {                                                                                      \
        constexpr int i_ = (R) / 2, h_ = (R) % 2;                                                                \
        const u32x2 t_ = lds_read_tr16_b64<(KSTEP) * 32 * T::BM * 2 + h_ * 4 * T::BM * 2>(fa_off[A_MC ? i_ : 0]); \
        fa[BUF][i_][2 * h_] = t_[0];                                                                             \
        fa[BUF][i_][2 * h_ + 1] = t_[1];                                                                         \
      } else {                                                                                                   \
        fa[BUF][(R)] = read_frag_kc<KSTEP, (R) * KC_TILE>(A_ADDR, fa_off[0]);                       \
      }                                                                                                          \
    } else if constexpr ((R) < NS) {                                                                             \
      constexpr int r_ = (R) - NSA;                                                                              \
      if constexpr (B_MC) {                                                                                      \
        constexpr int j_ = r_ / 2, h_ = r_ % 2;                                                                  \
        const u32x2 t_ = lds_read_tr16_b64<(KSTEP) * 32 * T::BN * 2 + h_ * 4 * T::BN * 2>(fb_off[B_MC ? j_ : 0]); \
        fb[BUF][j_][2 * h_] = t_[0];                                                                             \
        fb[BUF][j_][2 * h_ + 1] = t_[1];                                                                         \
      } else {                                                                                                   \
        fb[BUF][r_] = read_frag_kc<KSTEP, r_ * KC_TILE>(B_ADDR, fb_off[0]);                         \
      }                                                                                                          \
    }                                                                                                            \
  } while (0)
  constexpr int NMOVE = (A_MC ? T::TM : 0) + (B_MC ? T::TN : 0);
  constexpr int MOVES_PER_GAP = NS + NMOVE > NP ? 2 : 1;
  static_assert(NS * MOVES_PER_GAP + NMOVE <= NP * MOVES_PER_GAP, "the address updates fit behind the reads");
  uint32_t a_delta = 0, b_delta = 0;   // from the stage read now to the next one
#define MBX_MOVE_ONE16(M)                                                                                        \
  do {                                                                                                           \
    if constexpr (A_MC && (M) < T::TM) fa_off[A_MC ? (M) : 0] += a_delta;                                        \
    else if constexpr (B_MC && (M) - (A_MC ? T::TM : 0) >= 0 && (M) < NMOVE) fb_off[B_MC ? (M) - (A_MC ? T::TM : 0) : 0] += b_delta; \
  } while (0)
  // One k-step: NP MFMAs of 16 cycles on register buffer CUR_BUF.  A wave alone on its SIMD issues an independent
  // instruction every four cycles and an MFMA takes two such slots, so the gap behind an MFMA has room for two more
  // before the matrix core runs dry; everything else a k-step has to do is dealt out over the gaps accordingly:
  //   gaps 0 .. NS - 1: the operand reads of the next k-step into the other buffer, one read instruction per gap;
  //   from gap LOAD0 on, every EVERY-th gap: one of the NL global -> LDS loads of operand IS_B at (SC, DST), with the
  //   update of its running offsets in the gap behind it;
  //   the scalar bookkeeping P0 .. P3 (at most three instructions each) in gaps of their own.
#define MBX_STEP16(CUR_BUF, NEXT_KSTEP, NEXT_A, NEXT_B, IS_B, SC, DST, NL, LOAD0, EVERY, P0, P1, P2, P3, P4, MOVE)  \
  do {                                                                                                           \
    static_assert((EVERY) >= 3 && (LOAD0) + ((NL) - 1) * (EVERY) + 2 < NP && (LOAD0) + 3 * (EVERY) + 3 < NP && NS + 1 < NP, "the loads of a k-step and what follows them fit behind its MFMAs"); \
    wait_frags(fa[CUR_BUF], fb[CUR_BUF]);                                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                                           \
    static_for<NP>([&](auto mi_) {                                                                               \
      constexpr int m_ = decltype(mi_)::value;                                                                   \
      constexpr int i_ = m_ / T::TN, j_ = (i_ & 1) ? T::TN - 1 - m_ % T::TN : m_ % T::TN;                        \
      mfma16_acc<DT>(acc[i_][j_], fb[CUR_BUF][j_], fa[CUR_BUF][i_]);                                             \
      MBX_READ_SLOT16(NEXT_KSTEP, (CUR_BUF) ^ 1, NEXT_A, NEXT_B, m_);                                            \
      if constexpr (m_ >= (LOAD0) && (m_ - (LOAD0)) % (EVERY) == 0 && (m_ - (LOAD0)) / (EVERY) < (NL)) {         \
        issue(IS_B, SC, DST, (((m_ - (LOAD0)) / (EVERY)) & 1) != 0, (IS_B) && (m_ - (LOAD0)) / (EVERY) >= (NL) / 2, (m_ - (LOAD0)) / (EVERY)); \
        if constexpr (GATHER_B && (IS_B) && (m_ - (LOAD0)) / (EVERY) == (NL) - 1) {   /* the last B load of the K tile has its address: the entries of the next one */ \
          fetch_row_entries(b_row_next, g.row_table, entry_lane, entry_sc);                                      \
        }                                                                                                        \
      }                                                                                                          \
      if constexpr (m_ > (LOAD0) && (m_ - (LOAD0) - 1) % (EVERY) == 0 && (m_ - (LOAD0) - 1) / (EVERY) < (NL)) {  \
        SC += T::WAVES * ((IS_B) ? b_jstep : a_jstep);                                                           \
        DST += T::WAVES * 1024u;                                                                                 \
      }                                                                                                          \
      if constexpr (m_ == (LOAD0) + 2) P0();                                                                     \
      if constexpr (m_ == (LOAD0) + (EVERY) + 2) P1();                                                           \
      if constexpr (m_ == (LOAD0) + 2 * (EVERY) + 2) P2();                                                       \
      if constexpr (m_ == (LOAD0) + 3 * (EVERY) + 2) P3();                                                       \
      if constexpr (m_ == (NS + 1 > (LOAD0) + 3 * (EVERY) + 3 ? NS + 1 : (LOAD0) + 3 * (EVERY) + 3)) P4();   /* behind the k-step's last read and P3 */ \
      /* the strided operands' read addresses move to the next stage, one per gap, after the k-step's own reads */ \
      if constexpr ((MOVE) && m_ >= NS && (m_ - NS) * MOVES_PER_GAP < NMOVE) {                                    \
        MBX_MOVE_ONE16((m_ - NS) * MOVES_PER_GAP);                                                               \
        if constexpr (MOVES_PER_GAP > 1) MBX_MOVE_ONE16((m_ - NS) * MOVES_PER_GAP + 1);                          \
      }                                                                                                          \
      __builtin_amdgcn_sched_barrier(0);                                                                         \
    });                                                                                                          \
  } while (0)

  const int nk = g.nk;
  constexpr int kEntryLoads = 2;   // fetch_row_entries()
  constexpr int WAIT_PROLOGUE = (SB - 1) * (LA + LB) + (GATHER_B ? kEntryLoads : 0);   // tile 0 has landed (the loads behind it: tile 1's, the entries of tile SB)
  constexpr int WAIT_LOOP = (SB - 2) * (LA + LB) + LA;       // tile kt + 1 has landed: everything up to B tile kt + 1
  static_assert(SB * (LA + LB) < 64, "vmcnt is a 6-bit counter");
  MBX_TICK(g.tick_ordinal, 6);
  uint32_t entry_sc = (uint32_t)(SB + 1) * (kRowTableTile * 4);   // GATHER_B: the table's part of the K tile whose entries the loop fetches next
  uint32_t b_row_next[8];                                           // ... and where they arrive
  if (nk > 0) {
#pragma unroll
    for (int t = 0; t < SB; ++t) {
      issue_group(false, t, t, 0, LA);
      if constexpr (GATHER_B) {
        if (t == 1) {
#pragma unroll
          for (int q = 0; q < LB; ++q) b_row[q] = g.gather_row2[q];
        }
      }
      issue_group(true, t, t, 0, LB);
    }
    if constexpr (GATHER_B) {   // K tile SB's entries, for the first loads of the loop
      fetch_row_entries(b_row_next, g.row_table, entry_lane, (uint32_t)SB * (kRowTableTile * 4));
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  MBX_TICK(g.tick_ordinal, 7);
  if (clear) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
      for (int j = 0; j < T::TN; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  }
  if (nk > 0) {
    MBX_TICK(g.tick_ordinal, 3);
    wait_vmcnt<WAIT_PROLOGUE>();
    __builtin_amdgcn_s_barrier();
    MBX_TICK(g.tick_ordinal, 1);
    mfma16_settle();   // the accumulators were written by vector-ALU instructions
    static_for<NS>([&](auto mi_) { constexpr int m_ = decltype(mi_)::value; MBX_READ_SLOT16(0, 0, lds_base, lds_base + B_RING, m_); });

    constexpr uint32_t A_RING_END = (uint32_t)SA * T::A_BYTES, B_RING_END = B_RING + (uint32_t)SB * T::B_BYTES;
    // Running state, all scalar: the stages being multiplied and the next ones (one iteration ahead); LDS offset and
    // scalar global offset of the first A load of this iteration (tile kt + SB -> stage (kt - 1) % SA) and of the
    // first B load (tile kt + SB -> stage kt % SB).
    uint32_t a_rd = lds_base, b_rd = lds_base + B_RING;
    uint32_t a_rd_next = lds_base + T::A_BYTES, b_rd_next = lds_base + B_RING + T::B_BYTES;
    uint32_t a_dst0 = lds_off(false, SA - 1, 0), b_dst0 = lds_off(true, 0, 0);
    uint32_t a_sc0 = (uint32_t)SB * a_step + (uint32_t)wave * a_jstep, b_sc0 = (uint32_t)SB * b_step + (uint32_t)wave * b_jstep;
    const uint32_t a_dst_end = A_RING_END + (uint32_t)wave * 1024u, b_dst_end = B_RING_END + (uint32_t)wave * 1024u;
    uint32_t past = SB < nk ? 0u : 0x80000000u;
    uint32_t sc_a = a_sc0 | past, dst_a = a_dst0, sc_b = 0, dst_b = 0;
    if (DUAL) ra = SB >= g.nk1 ? g.rsrc_a2 : g.rsrc_a;
    constexpr int A_EVERY = (NP - NF - 3) / LA, B_EVERY = (NP - 4) / LB > 5 ? 5 : (NP - 4) / LB;
    for (int kt = 0; kt < nk; ++kt) {
      // k-step 0: the A loads (offsets set up in the iteration before); p0 / p1 prepare the B loads of k-step 1,
      // p2 moves the A offsets on to K tile kt + SB + 1
      auto p0 = [&]() {
        sc_b = b_sc0 | past;
        dst_b = b_dst0;
      };
      auto p1 = [&]() {
        if (DUAL) rb = kt + SB >= g.nk1 ? g.rsrc_b2 : g.rsrc_b;
        b_sc0 = DUAL && kt + SB + 1 == g.nk1 ? (uint32_t)wave * b_jstep : b_sc0 + b_step;
      };
      auto p2 = [&]() {
        a_sc0 = DUAL && kt + SB + 1 == g.nk1 ? (uint32_t)wave * a_jstep : a_sc0 + a_step;
        a_dst0 += T::A_BYTES;
        a_dst0 = a_dst0 >= a_dst_end ? a_dst0 - A_RING_END : a_dst0;
      };
      auto nop = [&]() {};
      auto p3 = [&]() {
        b_dst0 += T::B_BYTES;
        b_dst0 = b_dst0 >= b_dst_end ? b_dst0 - (uint32_t)SB * T::B_BYTES : b_dst0;
      };
      a_delta = a_rd_next - a_rd;
      b_delta = b_rd_next - b_rd;
      MBX_STEP16(0, 1, a_rd, b_rd, false, sc_a, dst_a, LA, NF, A_EVERY, p0, p1, p2, p3, nop, true);
      wait_frags(fa[1], fb[1]);
      wait_vmcnt<WAIT_LOOP>();
      __builtin_amdgcn_s_barrier();
      if constexpr (GATHER_B) {   // the entries fetched a K tile ago have arrived: they are the ones the loads of k-step 1 use
        asm volatile("" : "+v"(b_row_next[0]), "+v"(b_row_next[1]), "+v"(b_row_next[2]), "+v"(b_row_next[3]),
                          "+v"(b_row_next[4]), "+v"(b_row_next[5]), "+v"(b_row_next[6]), "+v"(b_row_next[7]));
#pragma unroll
        for (int q = 0; q < LB; ++q) b_row[GATHER_B ? q : 0] = b_row_next[q];
      }
      // k-step 1: the B loads from the first gaps on; q0 .. q3 set up the next iteration (its A loads, the stages it
      // reads after the ones this k-step prefetches from)
      auto q0 = [&]() { past = kt + 1 + SB < nk ? 0u : 0x80000000u; };
      auto q1 = [&]() {
        sc_a = a_sc0 | past;
        dst_a = a_dst0;
        if (DUAL) ra = kt + 1 + SB >= g.nk1 ? g.rsrc_a2 : g.rsrc_a;
      };
      uint32_t a_rd_nn = 0, b_rd_nn = 0;
      auto q2 = [&]() {
        a_rd_nn = a_rd_next + T::A_BYTES;
        a_rd_nn = a_rd_nn >= lds_base + A_RING_END ? lds_base : a_rd_nn;
      };
      auto q3 = [&]() {
        b_rd_nn = b_rd_next + T::B_BYTES;
        b_rd_nn = b_rd_nn >= lds_base + B_RING_END ? lds_base + B_RING : b_rd_nn;
      };
      auto q4 = [&]() {   // the reads of this k-step have their addresses: on to the next iteration's stages
        a_rd = a_rd_next;
        b_rd = b_rd_next;
        a_rd_next = a_rd_nn;
        b_rd_next = b_rd_nn;
      };
      MBX_STEP16(1, 0, a_rd_next, b_rd_next, true, sc_b, dst_b, LB, 1, B_EVERY, q0, q1, q2, q3, q4, false);   // past the last tile this reads stale LDS into dead registers
      if constexpr (GATHER_B) entry_sc += kRowTableTile * 4;
    }
    wait_vmcnt<0>();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    mfma16_settle();   // the last products must have reached the accumulators before anything else reads them
  }
#undef MBX_READ_SLOT16
#undef MBX_MOVE_ONE16
#undef MBX_STEP16
}

template <int DT, bool A_MC, bool B_MC, typename T, bool DUAL = false, bool GLU = false, bool GATHER = false, bool GATHER_B = false>
__device__ __forceinline__ void block_multiply(const Args& g, typename T::Acc (&acc)[T::TM][T::TN], bool clear, char* lds) {
  block_multiply16<DT, A_MC, B_MC, T, DUAL, GLU, GATHER, GATHER_B>(g, acc, clear, lds);
}

// ---- activation in the epilogue (tanh-GELU: megablocks/layers/arguments.py:19, megablocks/layers/gelu.py:9-13) ----
// Both are evaluated in fp32 on the value as stored (rounded to the 16-bit type), which is what the reference's
// separate element-wise kernels see, and through one exponential and one reciprocal instead of a library tanh:
//   gelu_tanh(x) = 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)),  tanh(u) = 1 - 2 / (1 + exp(2u)),  u = 0.79788456 (x + 0.044715 x^3)
// Evaluated on the eight values of a 16-byte chunk at a time, stage by stage: a wave alone on its SIMD issues a
// dependent instruction only every eight cycles, an independent one every four, so the eight chains are interleaved.
__device__ __forceinline__ void sigmoid_2u8(const float (&x)[8], float (&x2)[8], float (&s)[8]) {   // s = 1 / (1 + exp(-2u))
  float z[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) x2[i] = x[i] * x[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = -0.102943240f * x2[i] - 2.30220819f;      // -(2 * 0.79788456) (1 + 0.044715 x^2) log2(e)
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = z[i] * x[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = __builtin_amdgcn_exp2f(z[i]);
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = 1.f + z[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = __builtin_amdgcn_rcpf(z[i]);
}
__device__ __forceinline__ void gelu_tanh_fwd8(float (&x)[8]) {                // x <- gelu_tanh(x) = x s
  float x2[8], s[8];
  sigmoid_2u8(x, x2, s);
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = x[i] * s[i];
}
// g <- g * d/dx gelu_tanh(x).  With t = tanh(u) = 2 s - 1 the expression of gelu.py:9-13,
// 0.5 x (1 - t^2) (0.79788456 + 0.1070322243 x^2) + 0.5 (1 + t), is s (1 + x (1 - s) (1.59576912 + 0.2140644486 x^2)).
__device__ __forceinline__ void gelu_tanh_bwd8(float (&g)[8], const float (&x)[8]) {
  float x2[8], s[8], q[8];
  sigmoid_2u8(x, x2, s);
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = 0.2140644486f * x2[i] + 1.59576912f;
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = q[i] * x[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) x2[i] = 1.f - s[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = q[i] * x2[i] + 1.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = s[i] * q[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) g[i] = g[i] * s[i];
}

// What the store of an output tile does besides storing it:
//   kEpiNone      nothing;
//   kEpiAct       also stores gelu_tanh of the (rounded) tile to a second output of the same shape;
//   kEpiDact      multiplies the (rounded) tile by d/dx gelu_tanh of a second input of the same shape before storing it;
//   kEpiDgluSilu, kEpiDgluGelu   the tile g is the gradient of act(x1) * x2 (act = SiLU / tanh-GELU) with x1, x2 two
//                 more inputs of the same shape: stores g * round(act(x1)) and round(g * x2) * act'(x1), two outputs,
//                 and not g itself.
//   kEpiGluSilu, kEpiGluGelu   the tile is [x1 | x2], the same BN / 2 output columns of two products side by side (see
//                 block_multiply16's GLU): stores x1, x2 and round(round(act(x1)) * x2), three outputs.
//   kEpiCombine   also (or only, when c is null) stores every row of the (rounded) tile, multiplied by a weight and
//                 rounded again, to the row of a second output that the row's assignment names: the weighted combine
//                 of megablocks/backend/kernels.py:173-207 for top_k = 1, where a token's output row is one product
//                 row and needs no sum (see Combine).
enum { kEpiNone = 0, kEpiAct = 1, kEpiDact = 2, kEpiDgluSilu = 3, kEpiDgluGelu = 4, kEpiGluSilu = 5, kEpiGluGelu = 6, kEpiCombine = 7 };
constexpr bool epi_is_dglu(int epi) { return epi == kEpiDgluSilu || epi == kEpiDgluGelu; }
constexpr bool epi_is_glu(int epi) { return epi == kEpiGluSilu || epi == kEpiGluGelu; }

// the eight 16-bit values of a 16-byte chunk as fp32 and back (rounded)
template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& v, float (&f)[8]) {
  typedef typename Elem<DT>::type E;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[2 * w] = Elem<DT>::to_f32(__builtin_bit_cast(E, (uint16_t)(v[w] & 0xffffu)));
    f[2 * w + 1] = Elem<DT>::to_f32(__builtin_bit_cast(E, (uint16_t)(v[w] >> 16)));
  }
}
template <int DT>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
  u32x4 r;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = pack2<DT>(f[2 * w], f[2 * w + 1]);
  return r;
}
// The gated activation on a chunk, round(round(act(x1)) * x2): the two roundings of computing act(x1) and the product
// separately (glu.py:89,204).
template <int DT, bool GELU>
__device__ __forceinline__ u32x4 glu_chunk(const u32x4& x1v, const u32x4& x2v) {
  float x[8], b[8], s[8], z[8];
  unpack8<DT>(x1v, x);
  unpack8<DT>(x2v, b);
  if (GELU) {
    sigmoid_2u8(x, z, s);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = -1.44269504f * x[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = __builtin_amdgcn_exp2f(z[i]);
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = 1.f + z[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = __builtin_amdgcn_rcpf(z[i]);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = x[i] * s[i];
  const u32x4 actv = pack8<DT>(z);
  unpack8<DT>(actv, z);
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = z[i] * b[i];
  return pack8<DT>(z);
}
// The backward of the gated activation act(x1) * x2 on a chunk, with the roundings autograd's separate steps make:
//   d2 = g * round(act(x1)),   d1 = round(g * x2) * act'(x1)
// where act(x) = x s and act'(x) = s (1 + x (1 - s) q): SiLU with s = sigmoid(x), q = 1; tanh-GELU with s = sigmoid(2u)
// and q = 1.59576912 + 0.2140644486 x^2 (see gelu_tanh_bwd8).
template <int DT, bool GELU>
__device__ __forceinline__ void dglu_chunk(const u32x4& gv, const u32x4& x1v, const u32x4& x2v, u32x4& d1v, u32x4& d2v) {
  float g[8], x[8], b[8], s[8], q[8], z[8];
  unpack8<DT>(gv, g);
  unpack8<DT>(x1v, x);
  unpack8<DT>(x2v, b);
  if (GELU) {
    sigmoid_2u8(x, z, s);
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = 0.2140644486f * z[i] + 1.59576912f;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = -1.44269504f * x[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = __builtin_amdgcn_exp2f(z[i]);
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = 1.f + z[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = __builtin_amdgcn_rcpf(z[i]);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = x[i] * s[i];                                   // act(x1)
#pragma unroll
  for (int i = 0; i < 8; ++i) b[i] = g[i] * b[i];                                   // g x2
  const u32x4 actv = pack8<DT>(z), gbv = pack8<DT>(b);                              // both rounded to the storage type
  unpack8<DT>(actv, z);
  unpack8<DT>(gbv, b);
#pragma unroll
  for (int i = 0; i < 8; ++i) g[i] = g[i] * z[i];                                   // d2
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = 1.f - s[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = x[i] * z[i];
  if (GELU) {
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = z[i] * q[i];
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = s[i] * z[i] + s[i];                            // act'(x1)
#pragma unroll
  for (int i = 0; i < 8; ++i) b[i] = b[i] * z[i];                                   // d1
  d1v = pack8<DT>(b);
  d2v = pack8<DT>(g);
}
template <int DT>
__device__ __forceinline__ u32x4 gelu_fwd_chunk(const u32x4& v) {
  float x[8];
  unpack8<DT>(v, x);
  gelu_tanh_fwd8(x);
  return pack8<DT>(x);
}
template <int DT>
__device__ __forceinline__ u32x4 gelu_bwd_chunk(const u32x4& gv, const u32x4& xv) {
  float g[8], x[8];
  unpack8<DT>(gv, g);
  unpack8<DT>(xv, x);
  gelu_tanh_bwd8(g, x);
  return pack8<DT>(g);
}

// round(x * w) on the eight values of a chunk, formed the way the permutation kernels' scaled row copy forms it (a
// conversion, a product and a conversion back per element): in fp16 the compiler makes one mixed-precision instruction
// of the three, which rounds once, and the results of the two paths must agree to the bit.
template <int DT>
__device__ __forceinline__ u32x4 scale_chunk(const u32x4& v, float w) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint16_t lo = (uint16_t)(v[i] & 0xffffu), hi = (uint16_t)(v[i] >> 16);
    if (DT == MBX_BF16) {
      r[i] = (uint32_t)f32_to_bf16(bf16_to_f32(lo) * w) | ((uint32_t)f32_to_bf16(bf16_to_f32(hi) * w) << 16);
    } else {
      const _Float16 a = (_Float16)((float)__builtin_bit_cast(_Float16, lo) * w), b = (_Float16)((float)__builtin_bit_cast(_Float16, hi) * w);
      r[i] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
    }
  }
  return r;
}

// Buffer sizes stay below 2 GiB: bit 31 of a byte offset marks a load that must fetch nothing.
__device__ __forceinline__ uint32_t clip_bytes(int64_t bytes) {
  return (uint32_t)(bytes < 0x7fffffff ? bytes : 0x7fffffff);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
}

// c[m][n] = acc for m < m_lim, n < n_lim, where m = m_base + (row inside the tile) and
// n = n_base + (column inside the tile).  Uses the LDS of the operand rings as a staging buffer.  The rows of c must
// start at multiples of 16 bytes (c 16-byte aligned, ldc a multiple of 8: the launch checks both; outputs that are
// not go to the kernels of gmm.hip).
// `extra` (EPI != kEpiNone; laid out like c, same pitch, 16-byte aligned like c): the second output of kEpiAct, the
// second input of kEpiDact, x1 of kEpiDglu*; `pre2` and `out2` (kEpiDglu* only, laid out alike): x2 and the second
// output (c gets round(g x2) act'(x1), out2 gets g round(act(x1))).  These take the staged path only (the launch
// checks pitch and alignment).
// STAGED: the caller has already put the rounded tile into the staging area (stage_product_tile() for every product
// tile, after a barrier of its own); acc is not read.
// kEpiCombine: where the rows of a tile go.  `token` is per thread: the assignment (= token, top_k = 1) of tile row
// threadIdx.x as the caller loaded it before the main loop (not looked at until the store phase, so that nothing waits
// for the load), `row_exists` whether the expert has that row.  A row whose assignment is outside [0, tokens) is not
// combined.  weights (or null: 1) are indexed by token, in the type w_dtype names.
struct Combine {
  uint16_t* out = nullptr;        // [tokens, ldc]
  const void* weights = nullptr;
  int w_dtype = 0, tokens = 0;
  int token = -1;
  bool row_exists = false;
};
__device__ __forceinline__ int combine_token(const Combine& cb) {
  return cb.row_exists && (uint32_t)cb.token < (uint32_t)cb.tokens ? cb.token : -1;
}
__device__ __forceinline__ float combine_weight(const Combine& cb, int token) {
  if (cb.weights == nullptr || token < 0) return 1.f;
  if (cb.w_dtype == 2) return ((const float*)cb.weights)[token];
  const uint16_t raw = ((const uint16_t*)cb.weights)[token];
  return cb.w_dtype == 0 ? Elem<0>::to_f32(__builtin_bit_cast(typename Elem<0>::type, raw)) : Elem<1>::to_f32(__builtin_bit_cast(typename Elem<1>::type, raw));
}

template <int DT, typename T>
__device__ __forceinline__ void stage_product_tile(char* lds_generic, int i, int j, const f32x4& v) {
  const lds_ptr lds = (lds_ptr)lds_generic;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = lane_id();
  const int wm = (wave / T::WN) * T::WTM, wn = (wave % T::WN) * T::WTN;
  constexpr int ROW = T::BN * 2 + 16;
  const int ml = wm + i * T::MF + (lane & 15), nl = wn + j * T::MF + (lane >> 4) * 4;
  u32x2 w;
  w[0] = pack2<DT>(v[0], v[1]);
  w[1] = pack2<DT>(v[2], v[3]);
  *(__attribute__((address_space(3))) u32x2*)(lds + ml * ROW + nl * 2) = w;
}

template <int DT, typename T, int EPI = kEpiNone, bool STAGED = false>
__device__ __forceinline__ void block_store(const typename T::Acc (&acc)[T::TM][T::TN], uint16_t* __restrict__ c, int64_t ldc,
                                            int m_base, int m_lim, int n_base, int n_lim, char* lds_generic,
                                            uint16_t* __restrict__ extra = nullptr, const uint16_t* __restrict__ pre2 = nullptr,
                                            uint16_t* __restrict__ out2 = nullptr, const Combine& combine = Combine()) {
  const lds_ptr lds = (lds_ptr)lds_generic;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = lane_id();
  const int wm = (wave / T::WN) * T::WTM, wn = (wave % T::WN) * T::WTN;
  // kEpiCombine: (token, weight) of tile row threadIdx.x, handed to the lanes that store the row through the LDS
  // behind the staging area; the weight's load (it depends on the token) is under way while the tile is staged
  static_assert(EPI != kEpiCombine || T::EPILOGUE_BYTES + T::BM * 8 <= T::LDS_BYTES, "room for the rows' tokens and weights");
  constexpr uint32_t kPairs = (uint32_t)T::EPILOGUE_BYTES;
  int cb_token = -1;
  float cb_weight = 1.f;
  if constexpr (EPI == kEpiCombine) {
    cb_token = combine_token(combine);
    cb_weight = combine_weight(combine, cb_token);
  }
  // accumulator (i, j), register r of lane l holds c[m][n] with
  //   m = m_base + wm + 16 i + (l % 16),  n = n_base + wn + 16 j + 4 (l / 16) + r
  // i.e. a run of four consecutive columns per lane and product tile.
  constexpr int MF = T::MF;
  const int tile_row = lane & 15, run_col = (lane >> 4) * 4;
  {
    // Staged through LDS (free by now) so that every global store instruction writes whole rows of the
    // tile: 64 lanes x 16 bytes = two 512-byte row segments, instead of 32 scattered 16-byte pieces.
    constexpr int ROW = T::BN * 2 + 16;   // bytes; the 16-byte pad spreads the rows of a column over the banks
    if constexpr (!STAGED) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        const int ml = wm + i * MF + tile_row;
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
          const int nl = wn + j * MF + run_col;
          const typename T::Acc& v = acc[i][j];
          u32x2 w;
          w[0] = pack2<DT>(v[0], v[1]);
          w[1] = pack2<DT>(v[2], v[3]);
          *(__attribute__((address_space(3))) u32x2*)(lds + ml * ROW + nl * 2) = w;
        }
      }
    }
    if constexpr (EPI == kEpiCombine) {
      if (threadIdx.x < T::BM) {   // the tokens, then the weights
        *(__attribute__((address_space(3))) int*)(lds + kPairs + threadIdx.x * 4u) = cb_token;
        *(__attribute__((address_space(3))) float*)(lds + kPairs + (uint32_t)T::BM * 4u + threadIdx.x * 4u) = cb_weight;
      }
    }
    __syncthreads();
    if constexpr (epi_is_glu(EPI)) {
      // The tile is [x1 | x2]: BN / 2 output columns from n_base on.  A lane takes the same 16-byte chunk of both
      // halves of a row: 16 lanes a row, four rows per instruction; it stores the two chunks (to c and out2) and
      // their gated activation (to extra).  Batches of four rows per lane: eight LDS reads in flight, twelve stores.
      static_assert(T::BN == 256, "sixteen chunks per half row");
      constexpr int RPI = 4, ITERS = T::BM / RPI / T::WAVES, BATCH = 4, ROW_STEP = T::WAVES * RPI;
      static_assert(ITERS % BATCH == 0, "store batches");
      const int rl = lane >> 4, ch = lane & 15;
      const int n = n_base + ch * 8;
      const uint32_t rd_addr = lds_base + (uint32_t)((wave * RPI + rl) * ROW + ch * 16);
      int m = m_base + wave * RPI + rl;
      uint32_t off = ((uint32_t)m * (uint32_t)ldc + (uint32_t)n) * 2u;
      const uint32_t off_step = (uint32_t)ROW_STEP * (uint32_t)ldc * 2u;
      char* const cb = (char*)c;
      char* const hb = (char*)extra;
      char* const ob = (char*)out2;
      const bool full_n = n_base + T::BN / 2 <= n_lim;      // uniform
#pragma unroll 1
      for (int b = 0; b < ITERS; b += BATCH) {
        u32x4 v1[BATCH], v2[BATCH], h[BATCH];
        static_for<BATCH>([&](auto ui) {
          constexpr int u = decltype(ui)::value;
          v1[u] = lds_read_b128<u * ROW_STEP * ROW>(rd_addr + (uint32_t)(b * ROW_STEP * ROW));
          v2[u] = lds_read_b128<u * ROW_STEP * ROW + T::BN>(rd_addr + (uint32_t)(b * ROW_STEP * ROW));
        });
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v1[0]), "+v"(v1[1]), "+v"(v1[2]), "+v"(v1[3]), "+v"(v2[0]), "+v"(v2[1]), "+v"(v2[2]), "+v"(v2[3]));
#pragma unroll
        for (int u = 0; u < BATCH; ++u) h[u] = glu_chunk<DT, EPI == kEpiGluGelu>(v1[u], v2[u]);
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          if (m + u * ROW_STEP >= m_lim || n >= n_lim) continue;
          const uint32_t o = off + (uint32_t)u * off_step;
          if (full_n || n + 8 <= n_lim) {
            __builtin_nontemporal_store(v1[u], (u32x4*)(cb + o));
            __builtin_nontemporal_store(v2[u], (u32x4*)(ob + o));
            __builtin_nontemporal_store(h[u], (u32x4*)(hb + o));
          } else {
#pragma unroll
            for (int t = 0; t < 8; ++t)
              if (n + t < n_lim) {
                ((uint16_t*)(cb + o))[t] = (uint16_t)(v1[u][t >> 1] >> ((t & 1) * 16));
                ((uint16_t*)(ob + o))[t] = (uint16_t)(v2[u][t >> 1] >> ((t & 1) * 16));
                ((uint16_t*)(hb + o))[t] = (uint16_t)(h[u][t >> 1] >> ((t & 1) * 16));
              }
          }
        }
        m += BATCH * ROW_STEP;
        off += BATCH * off_step;
      }
      return;
    }
    constexpr int CHUNKS = T::BN / 8;                 // 16-byte chunks per tile row
    constexpr int ROWS_PER_INSTR = kWave / CHUNKS;    // 2 for 256-wide tiles
    const int rl = lane / CHUNKS, ch = lane % CHUNKS;
    const int n = n_base + ch * 8;
    // Eight LDS reads in flight before the first store of a batch (inline asm: the compiler would sink
    // each read to its store, behind the row check).  Like the main loop this part is bound by
    // instruction issue: a tile that is complete in the column direction takes a path with a 32-bit
    // running byte offset and nothing but the row check around each store.  Those stores are
    // non-temporal: the output is not read again by this kernel and need not displace operand panels.
    constexpr bool kDglu = epi_is_dglu(EPI), kPre = EPI == kEpiDact || kDglu;
    constexpr int ITERS = T::BM / ROWS_PER_INSTR / T::WAVES, BATCH = kDglu ? 4 : 8;
    constexpr int ROW_STEP = T::WAVES * ROWS_PER_INSTR;   // rows between consecutive stores of a wave
    static_assert(ITERS % BATCH == 0, "store batches");
    const uint32_t rd_addr = lds_base + (uint32_t)((wave * ROWS_PER_INSTR + rl) * ROW + ch * 16);
    const bool full_n = n_base + T::BN <= n_lim;          // uniform
    int m = m_base + wave * ROWS_PER_INSTR + rl;
    uint32_t off = ((uint32_t)m * (uint32_t)ldc + (uint32_t)n) * 2u;   // outputs are below 2 GiB
    const uint32_t off_step = (uint32_t)ROW_STEP * (uint32_t)ldc * 2u;
    char* const cb = (char*)c;
    char* const eb = (char*)extra;
    const char* const pb = (const char*)pre2;
    char* const ob = (char*)out2;
    // kEpiDact: the chunks of the second input that belong to a batch are fetched one batch ahead (the registers of
    // the accumulators are free by now), so that their latency is behind the arithmetic and the stores of the batch
    // before; rows or columns outside the tile's part of c are not fetched (zeros: their results are not stored)
    // (kEpiDglu*: both inputs, in batches of four, two batches ahead: a batch of four takes less time than a fetch)
    u32x4 pre[kPre ? BATCH : 1], pre_next[kPre ? BATCH : 1], preb[kDglu ? BATCH : 1], preb_next[kDglu ? BATCH : 1];
    u32x4 pre_far[kDglu ? BATCH : 1], preb_far[kDglu ? BATCH : 1];
    // Buffer loads, bounded by the rows this tile may touch: no branch around a load, so the compiler can count the
    // loads in flight (around conditional loads it waits for all of them, the ones fetched ahead included); rows past
    // the end read as zeros, columns past it as whatever follows in the row below — neither is stored.
    const __amdgpu_buffer_rsrc_t pre_rsrc = make_rsrc(kPre ? eb : nullptr, kPre && m_lim > 0 ? clip_bytes((int64_t)m_lim * ldc * 2) : 0u);
    const __amdgpu_buffer_rsrc_t preb_rsrc = make_rsrc(kDglu ? pb : nullptr, kDglu && m_lim > 0 ? clip_bytes((int64_t)m_lim * ldc * 2) : 0u);
    auto fetch_pre = [&](u32x4 (&dst)[kPre ? BATCH : 1], const __amdgpu_buffer_rsrc_t& r, uint32_t off0) {
      if constexpr (kPre) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
          dst[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(off0 + (uint32_t)u * off_step), 0, 0));
      }
    };
    fetch_pre(pre_next, pre_rsrc, off);
    if constexpr (kDglu) {
      fetch_pre(preb_next, preb_rsrc, off);
      fetch_pre(pre_far, pre_rsrc, off + BATCH * off_step);
      fetch_pre(preb_far, preb_rsrc, off + BATCH * off_step);
    }
    // the second output goes where kEpiAct's does (extra) or to out2 (kEpiDglu*: extra is an input there)
    constexpr bool kTwoOut = EPI == kEpiAct || kDglu;
    char* const second = kDglu ? ob : eb;
#pragma unroll 1
    for (int b = 0; b < ITERS; b += BATCH) {
      u32x4 v[BATCH], y[kTwoOut ? BATCH : 1];
      static_for<BATCH>([&](auto ui) {
        constexpr int u = decltype(ui)::value;
        v[u] = lds_read_b128<u * ROW_STEP * ROW>(rd_addr + (uint32_t)(b * ROW_STEP * ROW));
      });
      if constexpr (kPre) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u) pre[u] = pre_next[u];
        if constexpr (kDglu) {
#pragma unroll
          for (int u = 0; u < BATCH; ++u) {
            preb[u] = preb_next[u];
            pre_next[u] = pre_far[u];
            preb_next[u] = preb_far[u];
          }
          fetch_pre(pre_far, pre_rsrc, off + 2 * BATCH * off_step);     // past the tile's rows at the end: not used
          fetch_pre(preb_far, preb_rsrc, off + 2 * BATCH * off_step);
        } else {
          fetch_pre(pre_next, pre_rsrc, off + BATCH * off_step);
        }
      }
      if constexpr (BATCH == 8) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
      } else {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
      }
      if constexpr (EPI == kEpiDact) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u) v[u] = gelu_bwd_chunk<DT>(v[u], pre[u]);
      }
      if constexpr (kDglu) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          const u32x4 gv = v[u];
          dglu_chunk<DT, EPI == kEpiDgluGelu>(gv, pre[u], preb[u], v[u], y[u]);
        }
      }
      if constexpr (EPI == kEpiCombine) {
        // the product's row (where the caller wants it: the backward pass does) and the token's row of the output
        int row_token[BATCH];
        float row_weight[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          const uint32_t at = kPairs + (uint32_t)((wave * ROWS_PER_INSTR + rl + (b + u) * ROW_STEP) * 4);
          row_token[u] = *(const __attribute__((address_space(3))) int*)(lds + at);
          row_weight[u] = *(const __attribute__((address_space(3))) float*)(lds + at + (uint32_t)T::BM * 4u);
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          if (m + u * ROW_STEP >= m_lim || n >= n_lim) continue;
          const int token = row_token[u];
          const float w = row_weight[u];
          const u32x4 scaled = scale_chunk<DT>(v[u], w);
          uint16_t* const dst = (uint16_t*)(cb + (off + (uint32_t)u * off_step));
          uint16_t* const dst2 = token >= 0 ? combine.out + ((int64_t)token * ldc + n) : nullptr;
          if (full_n || n + 8 <= n_lim) {
            if (c != nullptr) __builtin_nontemporal_store(v[u], (u32x4*)dst);
            if (dst2 != nullptr) __builtin_nontemporal_store(scaled, (u32x4*)dst2);
          } else {
#pragma unroll
            for (int t = 0; t < 8; ++t)
              if (n + t < n_lim) {
                if (c != nullptr) dst[t] = (uint16_t)(v[u][t >> 1] >> ((t & 1) * 16));
                if (dst2 != nullptr) dst2[t] = (uint16_t)(scaled[t >> 1] >> ((t & 1) * 16));
              }
          }
        }
      } else if (full_n) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
          if (m + u * ROW_STEP < m_lim) {
            __builtin_nontemporal_store(v[u], (u32x4*)(cb + (off + (uint32_t)u * off_step)));
            if constexpr (EPI == kEpiAct) y[u] = gelu_fwd_chunk<DT>(v[u]);
            if constexpr (kTwoOut) __builtin_nontemporal_store(y[u], (u32x4*)(second + (off + (uint32_t)u * off_step)));
          }
      } else {
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          if (m + u * ROW_STEP >= m_lim || n >= n_lim) continue;
          uint16_t* dst = (uint16_t*)(cb + (off + (uint32_t)u * off_step));
          if constexpr (EPI == kEpiAct) y[u] = gelu_fwd_chunk<DT>(v[u]);
          uint16_t* dst2 = (uint16_t*)(second + (off + (uint32_t)u * off_step));
          if (n + 8 <= n_lim) {
            *(u32x4*)dst = v[u];
            if constexpr (kTwoOut) *(u32x4*)dst2 = y[u];
          } else {
#pragma unroll
            for (int t = 0; t < 8; ++t)
              if (n + t < n_lim) {
                dst[t] = (uint16_t)(v[u][t >> 1] >> ((t & 1) * 16));
                if constexpr (kTwoOut) dst2[t] = (uint16_t)(y[kTwoOut ? u : 0][t >> 1] >> ((t & 1) * 16));
              }
          }
        }
      }
      m += BATCH * ROW_STEP;
      off += BATCH * off_step;
    }
  }
}

// c = A_tile * B_tile over all K tiles (the whole product of one output tile)
template <int DT, bool A_MC, bool B_MC, typename T, bool DUAL = false, int EPI = kEpiNone, bool GATHER = false>
__device__ __forceinline__ void block_gemm(const Args& g, uint16_t* __restrict__ c, int64_t ldc, int m_base, int m_lim,
                                           int n_base, int n_lim, char* lds, uint16_t* __restrict__ extra = nullptr,
                                           const uint16_t* __restrict__ pre2 = nullptr, uint16_t* __restrict__ out2 = nullptr,
                                           const Combine& combine = Combine()) {
  typename T::Acc acc[T::TM][T::TN];
  block_multiply<DT, A_MC, B_MC, T, DUAL, epi_is_glu(EPI), GATHER>(g, acc, true, lds);
  MBX_TICK(g.tick_ordinal, 2);
  block_store<DT, T, EPI>(acc, c, ldc, m_base, m_lim, n_base, n_lim, lds, extra, pre2, out2, combine);
  MBX_TICK(g.tick_ordinal, 4);
}


// ---- workgroups that compute several tiles ----
// An NN / NT launch has one workgroup per compute unit (P of them, a multiple of 8); each walks a
// fixed list of tiles (all tiles of such a launch cost the same).  Workgroup w sits on XCD w % 8 and
// is that XCD's member w / 8; the P / 8 members of an XCD take one run of P / 8 consecutive tiles per
// round, so the tiles an XCD works on at any time are a compact block that shares operand panels in
// that XCD's L2.  Walking the list inside the kernel spares a workgroup launch and an expert lookup
// from scratch per tile, and makes the last, partly filled round visible to the kernel.

// The LDS and the operand registers of the finished tile are dead once every wave is here.
__device__ __forceinline__ void tile_done() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
}

__device__ __forceinline__ int clamp_row(int v, int rows) { return v < 0 ? 0 : (v > rows ? rows : v); }

// ---- NN / NT ----
// Logical tile id -> (expert, column tile, row tile inside the expert).  Lane l of every wave keeps the
// inclusive count of tiles up to its experts (one expert per lane up to 64 experts, else a group of
// consecutive ones), and a tile id is resolved with one ballot, then, with several experts per lane, a short
// search through the bins of that lane's group.
template <int BM>
struct RowTiles {
  // Per lane: one expert up to 64 experts (the lane then keeps its row range too), else a group of per_lane experts.
  int lane_start = 0, lane_end = 0, lane_mt = 0, lane_incl = 0, lane_short_incl = 0;
  int total = 0, total_short = 0;   // all tiles; of these, the short last row tiles that come first in the order
  int per_lane;
  const int32_t* bins;
  int num_groups, tiles_n, rows;
  bool split;              // short last row tiles (at most BM / 2 rows) may be listed apart, ahead of the others

  // row tiles of an expert that are listed with the full ones, and whether a short one is left over
  int apart_from;          // full row tiles an expert must have for its short last tile to be listed apart
  __device__ __forceinline__ int short_tiles(int r) const {
    return split && r > 0 && r % BM > 0 && r % BM <= BM / 2 && r / BM >= apart_from ? 1 : 0;
  }
  __device__ __forceinline__ int long_tiles(int r) const { return r <= 0 ? 0 : (r + BM - 1) / BM - short_tiles(r); }
  // A bin bound as the kernels use it: inside [0, rows] whatever the table holds, so that a table that does not
  // belong to this operand (stale, or of another batch) can make the result wrong but never an access out of range.
  __device__ __forceinline__ int bound(int e) const { return clamp_row(bins[e], rows); }

  __device__ __forceinline__ RowTiles(const int32_t* bins_, int num_groups_, int tiles_n_, int rows_, bool split_, int apart_from_)
      : bins(bins_), num_groups(num_groups_), tiles_n(tiles_n_), rows(rows_), split(split_), apart_from(apart_from_) {
    per_lane = (num_groups + kWave - 1) / kWave;
    const int lane = lane_id();
    const int first = lane * per_lane;
    int span = 0, shorts = 0;
    if (per_lane == 1) {
      if (lane < num_groups) {
        lane_end = bound(lane);
        lane_start = lane > 0 ? bound(lane - 1) : 0;
        lane_mt = long_tiles(lane_end - lane_start);
        shorts = short_tiles(lane_end - lane_start);
      }
      span = lane_mt * tiles_n;
    } else if (first < num_groups) {
      // lane l keeps the tile count of experts l per_lane .. (l + 1) per_lane - 1 and the first row of that group
      lane_start = first > 0 ? bound(first - 1) : 0;
      int start = lane_start;
      for (int e = first; e < first + per_lane && e < num_groups; ++e) {
        const int end = bound(e);
        span += long_tiles(end - start) * tiles_n;
        shorts += short_tiles(end - start);
        start = end;
      }
      lane_mt = span;
    }
    int incl = span, sincl = shorts;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int v = __shfl_up(incl, o, kWave), w = __shfl_up(sincl, o, kWave);
      if (lane >= o) { incl += v; sincl += w; }
    }
    lane_incl = incl;
    lane_short_incl = sincl;
    total_short = __builtin_amdgcn_readlane(sincl, kWave - 1) * tiles_n;
    total = __builtin_amdgcn_readlane(incl, kWave - 1) + total_short;
  }

  // id in [0, total) -> expert, its row range, the row tile and the column tile
  __device__ __forceinline__ void find(int id, int& e, int& start, int& end, int& tm, int& tn) const {
    if (id < total_short) {
      // The short last row tiles that are listed apart, expert by expert, column tiles fastest.  A short tile takes
      // less time than a full one; dealt among the full ones it lets the workgroups of an XCD drift apart, which then
      // no longer find each other's operand panels in the L2.  Apart, the short tile streams its expert's weights on
      // its own, so this is only done for experts with many row tiles (apart_from) and by the launches whose long
      // reductions suffer most from the drift (NN on a Mixtral-shaped layer: L2 misses 4.8 -> 4.0 GB, launch -3 %;
      // NT, with a quarter of the reduction length, was 1.5 % slower apart, and experts of one or two row tiles, which
      // are bound by the weights they stream, 18 %).
      const int j = id / tiles_n;
      tn = id - j * tiles_n;
      const uint64_t hit = __ballot(j < lane_short_incl);
      const int l = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit));
      if (per_lane == 1) {
        e = l;
        start = __builtin_amdgcn_readlane(lane_start, l);
        end = __builtin_amdgcn_readlane(lane_end, l);
      } else {
        // the j-th short tile overall is number `want` among those of lane l's experts
        int want = j - (l > 0 ? __builtin_amdgcn_readlane(lane_short_incl, l > 0 ? l - 1 : 0) : 0);
        start = __builtin_amdgcn_readlane(lane_start, l);
        end = start;
        for (e = l * per_lane; e < num_groups; ++e) {
          end = bound(e);
          if (short_tiles(end - start) && want-- == 0) break;
          start = end;
        }
      }
      tm = long_tiles(end - start);
      return;
    }
    id -= total_short;
    int mt;
    const uint64_t hit = __ballot(id < lane_incl);
    const int l = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit));
    if (per_lane == 1) {
      e = l;
      start = __builtin_amdgcn_readlane(lane_start, l);
      end = __builtin_amdgcn_readlane(lane_end, l);
      mt = __builtin_amdgcn_readlane(lane_mt, l);
      id -= __builtin_amdgcn_readlane(lane_incl, l) - mt * tiles_n;
    } else {
      // the lane's group of experts is searched in the bins (per_lane - 1 steps at most)
      id -= __builtin_amdgcn_readlane(lane_incl, l) - __builtin_amdgcn_readlane(lane_mt, l);
      start = __builtin_amdgcn_readlane(lane_start, l);
      end = start; mt = 0;
      for (e = l * per_lane; e < num_groups; ++e) {
        end = bound(e);
        mt = long_tiles(end - start);
        const int span = mt * tiles_n;
        if (id < span) break;
        id -= span;
        start = end;
      }
    }
    // Inside an expert the tiles are counted in bands of kBand row tiles: rows fastest, then columns, then the
    // next band.  Any 32 consecutive ids of a band are an 8 x 4 block with 12 operand panels, however many row
    // tiles the expert has; counting all its row tiles fastest would make them a 32 x 1 strip with 33.  The
    // last band has the rows that are left, 5 to 12 of them (up to 4 left-over rows join the band before:
    // a band of one row would be a 1 x 32 strip).
    constexpr int kBand = 8;
    const int per_band = kBand * tiles_n;
    const int bands = mt + kBand / 2 - 1 < kBand ? 1 : (mt + kBand / 2 - 1) / kBand;
    const int full = (bands - 1) * per_band;
    if (id < full) {
      const int band = id / per_band, q = id - band * per_band;
      tn = q / kBand;
      tm = band * kBand + q % kBand;
    } else {
      const int left = mt - (bands - 1) * kBand, q = id - full;
      tn = q / left;
      tm = (bands - 1) * kBand + q % left;
    }
  }
};

// T is the main tile.  When the last round would leave at least half of the compute units idle, its
// R tiles are cut into 2 R half tiles of TS (BM / 2 rows, same columns), spread over all XCDs:
// the tail then costs little more than half a round.  TS = T switches this off.
// DUAL: c = a @ b[e] + a2 @ b2[e] in one pass (k is the reduction length of each pair, at least
// (SB + 1) K tiles), as one reduction over 2 k.
// EPI: see block_store; `extra` is its second output / input, [rows, n] like c; kEpiDglu*: `a2` is x2 and `out2` the
// second output, both [rows, n].
// GATHER: `a` is [src_rows, k] and row r of expert e's rows is a[slots[src_start(e) + r] / top_k] while
// src_start(e) + r < src_bins[e], zeros after that (src_start(e) = src_bins[e - 1], 0 for the first expert): the
// product of the rows that megablocks/ops/gather.py:20-38 / padded_gather.py:20-55 would have copied out first.
// half_limit: an expert's last row tile with at most this many rows is computed as a TS tile (TS::BM, or 0: never; the
// launch decides).
// slot / top_k is computed as (slot * top_k_magic) >> (32 + top_k_shift) (see gather_divisor(); top_k = 1: magic 0),
// a division per row and tile being a few hundred dependent instructions on a wave that has its SIMD to itself.
template <int DT, bool B_MC, typename T, typename TS, bool DUAL = false, int EPI = kEpiNone, bool GATHER = false>
__global__ void __launch_bounds__(T::THREADS)
gmm_rows_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
                const int32_t* __restrict__ bins, int num_groups, int64_t rows, int k, int n, int tiles_n,
                const uint16_t* __restrict__ a2, const uint16_t* __restrict__ b2, uint16_t* __restrict__ extra,
                uint16_t* __restrict__ out2, const int32_t* __restrict__ slots, const int32_t* __restrict__ src_bins,
                int top_k, int src_rows, uint32_t top_k_magic, int top_k_shift, int half_limit,
                int32_t* __restrict__ ws_counters, float* ws_parts, int ws_capacity,
                const void* __restrict__ combine_weights, int combine_w_dtype, int combine_tokens) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  static_assert(T::THREADS == TS::THREADS && T::BN == TS::BN && T::BK == TS::BK, "tail tile");
  static_assert(EPI != kEpiCombine || (!GATHER && !DUAL), "the combine: one operand pair, rows as they are");
  static_assert(!(DUAL && (epi_is_dglu(EPI) || epi_is_glu(EPI))), "a2 / b2 are the second operand pair, the epilogue's x2 or the second matrix");
  constexpr int kTileCols = epi_is_glu(EPI) ? T::BN / 2 : T::BN;   // output columns of a tile
  constexpr bool kSplit = T::BM != TS::BM;
  static_assert(!kSplit || T::BM == 2 * TS::BM, "tail tile");
  const int P = gridDim.x, run = P / kXcds;
  const int xcd = blockIdx.x % kXcds, member = blockIdx.x / kXcds;
  const RowTiles<T::BM> tiles(bins, num_groups, tiles_n, (int)rows, kSplit && B_MC, 8);
  const int total = tiles.total;
  const int full_rounds = total / P, rest = total - full_rounds * P;

  Args g;
  g.a_ld_bytes = (uint32_t)k * 2;
  g.b_ld_bytes = (uint32_t)(B_MC ? n : k) * 2;
  const int nk1 = k / T::BK, nk_all = DUAL ? 2 * nk1 : nk1;
  g.nk1 = nk1;
  g.nk = nk_all;
  g.a_r0 = 0;   // the buffers of a and c start at the tile's first row: byte offsets stay small whatever the row count
  // The last, partly filled round.  Its `rest` tiles leave P - rest compute units idle for a whole tile's time, which
  // with long reductions and few rounds is a large part of the launch (a Mixtral-shaped second product: 1088 tiles on
  // 256 compute units, 4.25 rounds).  When at most half of the compute units would be busy:
  //   * with a workspace (kSplitK launches: NN, no epilogue): every tail tile is cut along the reduction into
  //     `ksplit` = P / rest parts, one per workgroup, each a full-size tile over a `ksplit`-th of the K tiles.  A part
  //     writes its fp32 accumulators to the workspace and counts itself in; the workgroup that finds it was the last
  //     adds the parts up in part order (so the sum does not depend on who was last), rounds and stores the tile.
  //     Nobody waits for anybody.  The tail then takes 1 / ksplit of a round plus the reduction;
  //   * else the tail's tiles are cut into two half-height tiles each (TS), which take 0.7 of a full tile's time.
  constexpr bool kSplitK = B_MC && EPI == kEpiNone && !GATHER;
  constexpr int kMaxKSplit = 8, kMinPartTiles = 8;
  int ksplit = 1;
  if constexpr (kSplitK) {
    if (ws_parts != nullptr && rest > 0 && 2 * rest <= P) {
      int s_ = P / rest;
      s_ = s_ > kMaxKSplit ? kMaxKSplit : s_;
      s_ = s_ > nk_all / kMinPartTiles ? nk_all / kMinPartTiles : s_;
      s_ = (int64_t)s_ * rest > ws_capacity ? ws_capacity / rest : s_;
      ksplit = s_ < 2 ? 1 : s_;
    }
  }
  const bool split = ksplit == 1 && kSplit && rest > 0 && 2 * rest <= P;
  const int big_rounds = full_rounds + ((rest > 0 && !split && ksplit == 1) ? 1 : 0);
  // Work items of this workgroup: one tile per round, then (if the tail is cut) one part or one half tile.
  const int items = big_rounds + ((ksplit > 1 || (kSplit && split)) ? 1 : 0);
  // first K tile of part p of a reduction cut into ksplit parts; with two operand pairs a cut within SB K tiles of the
  // pairs' boundary moves onto it (the main loop changes pairs at least SB + 1 K tiles into a call)
  auto part_begin = [&](int p_) -> int {
    int t_ = (int)((int64_t)p_ * nk_all / ksplit);
    if (DUAL && t_ - nk1 < T::SB + 1 && nk1 - t_ < T::SB + 1) t_ = nk1;
    return t_;
  };
  // the tile with first row row0 of expert e (rows start .. end - 1), column tile tn
  auto compute_tile = [&](int e, int end, int tn, int row0, bool use_ts) {
    const uint32_t a_bytes = clip_bytes((rows - row0) * k * 2);   // rows past the tile's are fetched, never stored
    if constexpr (!GATHER) g.rsrc_a = make_rsrc(a + (int64_t)row0 * k, a_bytes);
    g.rsrc_a2 = DUAL ? make_rsrc(a2 + (int64_t)row0 * k, a_bytes) : g.rsrc_a;
    g.rsrc_b = make_rsrc(b + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2));
    g.rsrc_b2 = DUAL ? make_rsrc(b2 + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2)) : g.rsrc_b;
    // the second matrix of a [w1 | v1] tile: rows BN / 2 .. BN - 1 of the tile are its rows b_r0 .. b_r0 + BN / 2 - 1
    if (epi_is_glu(EPI)) g.rsrc_b2 = make_rsrc(b2 + ((int64_t)e * n - T::BN / 2) * k, (uint32_t)(((int64_t)n + T::BN / 2) * k * 2));
    g.b_r0 = tn * kTileCols;
    uint16_t* const c_tile = c + (int64_t)row0 * n;
    uint16_t* const e_tile = EPI != kEpiNone ? extra + (int64_t)row0 * n : nullptr;
    const uint16_t* const p_tile = epi_is_dglu(EPI) ? a2 + (int64_t)row0 * n : nullptr;   // x2 of the gated activation
    uint16_t* const o_tile = epi_is_dglu(EPI) || epi_is_glu(EPI) ? out2 + (int64_t)row0 * n : nullptr;
    // the last row tile of an expert, when at most half full, is computed as a half-height tile as well
    use_ts = kSplit && (use_ts || end - row0 <= half_limit);
    if (use_ts) {
      block_gemm<DT, false, B_MC, TS, DUAL, EPI, GATHER>(g, c_tile, n, 0, end - row0, g.b_r0, n, lds, e_tile, p_tile, o_tile);
    } else {
      block_gemm<DT, false, B_MC, T, DUAL, EPI, GATHER>(g, c_tile, n, 0, end - row0, g.b_r0, n, lds, e_tile, p_tile, o_tile);
    }
    tile_done();
  };
  // item r -> expert, its row range, the column tile, the tile's first row, whether it is a half tile of the split
  // tail; false when the workgroup has no such item (then it has none after it either)
  auto locate = [&](int r, int& e, int& start, int& end, int& tn, int& row0, bool& tail_half) -> bool {
    int id, half = 0;
    tail_half = false;
    if (r < big_rounds) {
      // Rotated by one member per round: where full and half-height tiles alternate along the list, a
      // workgroup would otherwise be dealt the same kind in every round.
      id = (r * kXcds + xcd) * run + (member + r) % run;
      if (id >= total) return false;
    } else {
      const int j = xcd * run + member;   // half tile j: tile j / 2 of the tail, rows half j % 2
      if (j >= 2 * rest) return false;
      id = full_rounds * P + j / 2;
      half = j & 1;
      tail_half = true;
    }
    int tm;
    tiles.find(id, e, start, end, tm, tn);
    row0 = start + tm * T::BM + half * TS::BM;
    return row0 < end;                    // false: the second half of a tile whose rows end in the first (a last item)
  };
  if constexpr (!GATHER) {
    for (int r = 0; r < items; ++r) {
      int id, half = 0;
      bool use_ts = false;
      if (r < big_rounds) {
        id = (r * kXcds + xcd) * run + (member + r) % run;   // as in locate()
        if (id >= total) break;
      } else if (kSplitK && ksplit > 1) {
        if constexpr (kSplitK) {
          // part `part` of tail tile `tile`: consecutive workgroups of an XCD take the same part of consecutive tiles
          const int j = xcd * run + member;
          if (j >= ksplit * rest) break;
          const int tile = j % rest, part = j / rest;
          g.tick_ordinal = r;
          MBX_TICK(r, 0);
          int e, start, end, tm, tn;
          tiles.find(full_rounds * P + tile, e, start, end, tm, tn);
          const int row0 = start + tm * T::BM;
          const int t0 = part_begin(part), t1 = part + 1 < ksplit ? part_begin(part + 1) : nk_all;
          // the operands from K tile t0 on: of the second pair when the part lies in it, with the change of pairs at
          // its place when the part straddles it, never otherwise
          const bool second = DUAL && t0 >= nk1;
          const int kt0 = second ? t0 - nk1 : t0;                      // first K tile inside its pair
          const uint16_t* const pa = (second ? a2 : a) + (int64_t)row0 * k + (int64_t)kt0 * T::BK;
          const uint16_t* const pb = (second ? b2 : b) + (int64_t)e * k * n + (int64_t)kt0 * T::BK * n;
          const int64_t a_left = (rows - row0) * k - (int64_t)kt0 * T::BK, b_left = ((int64_t)k - (int64_t)kt0 * T::BK) * n;
          g.rsrc_a = make_rsrc(pa, clip_bytes(a_left * 2));
          g.rsrc_b = make_rsrc(pb, clip_bytes(b_left * 2));
          g.rsrc_a2 = DUAL ? make_rsrc(a2 + (int64_t)row0 * k, clip_bytes((rows - row0) * k * 2)) : g.rsrc_a;
          g.rsrc_b2 = DUAL ? make_rsrc(b2 + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2)) : g.rsrc_b;
          g.nk = t1 - t0;
          g.nk1 = DUAL && !second && t1 > nk1 ? nk1 - t0 : 0x3fffffff;
          g.b_r0 = tn * kTileCols;
          typename T::Acc acc[T::TM][T::TN];
          block_multiply<DT, false, B_MC, T, DUAL>(g, acc, true, lds);
          MBX_TICK(r, 2);
          g.nk = nk_all;
          g.nk1 = nk1;
          // The part's accumulators as they lie in the registers: 16 bytes per lane and product tile, addressed as a
          // buffer with the lane's offset in a register and the product tile's in a scalar (64-bit addresses per
          // store would take two registers each, which this kernel does not have).  Eight tiles at a time, so that the
          // compiler does not gather all 256 registers of a part in one place.
          constexpr uint32_t kPartBytes = (uint32_t)T::BM * T::BN * 4, kTileStep = (uint32_t)T::THREADS * 16;
          constexpr int kThroughCaches = 0x11;   // cache policy bits sc0 | sc1 of a buffer access: system scope
          const uint32_t lane_off = threadIdx.x * 16u;
          const __amdgpu_buffer_rsrc_t mine = make_rsrc((const char*)ws_parts + (size_t)j * kPartBytes, kPartBytes);
          static_for<T::TM>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
#pragma unroll
            for (int jj = 0; jj < T::TN; ++jj)
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][jj]), mine, (int)lane_off, (int)((i * T::TN + jj) * kTileStep), kThroughCaches);
            __builtin_amdgcn_sched_barrier(0);
          });
          // The parts go between workgroups on different XCDs, whose L2 caches do not see each other: they are stored
          // and loaded past the caches (write-through stores, loads that always miss) instead of between a release
          // and an acquire fence, which here would mean a write-back of the whole L2 by every wave of every part
          // and an invalidation under the workgroups that are still multiplying.  A part is counted in once every
          // wave's stores have been acknowledged; the counter is a device-wide atomic.
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();                       // every wave's share of the part is out; nobody reads the LDS stages any more
          int* const flag = (int*)lds;
          if (threadIdx.x == 0) *flag = __hip_atomic_fetch_add(ws_counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __syncthreads();
          const bool last = *flag == ksplit - 1;  // uniform
          if (last) {
            // The sum of the parts, in part order whoever came last, goes straight to the staging area of the store:
            // one row of product tiles at a time, the parts of up to four workgroups in flight together.
            constexpr int kRowsAtOnce = 1, kTilesAtOnce = kRowsAtOnce * T::TN;   // rows of product tiles per batch of loads
            static_assert(T::TM % kRowsAtOnce == 0, "batches of the reduction");
            static_for<T::TM / kRowsAtOnce>([&](auto ii) {
              constexpr int t0_ = decltype(ii)::value * kTilesAtOnce;         // first product tile of the batch
              f32x4 sum[kTilesAtOnce];
#pragma unroll 1
              for (int p0 = 0; p0 < ksplit; p0 += 4) {
                u32x4 v[4][kTilesAtOnce];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                  if (p0 + u < ksplit) {
                    const __amdgpu_buffer_rsrc_t theirs = make_rsrc((const char*)ws_parts + ((size_t)(p0 + u) * rest + tile) * kPartBytes, kPartBytes);
#pragma unroll
                    for (int t = 0; t < kTilesAtOnce; ++t)
                      v[u][t] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(theirs, (int)lane_off, (int)((t0_ + t) * kTileStep), kThroughCaches));
                  }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                  if (p0 + u < ksplit) {
#pragma unroll
                    for (int t = 0; t < kTilesAtOnce; ++t) {
                      const f32x4 w = __builtin_bit_cast(f32x4, v[u][t]);
                      sum[t] = (p0 == 0 && u == 0) ? w : sum[t] + w;
                    }
                  }
                }
              }
#pragma unroll
              for (int t = 0; t < kTilesAtOnce; ++t) stage_product_tile<DT, T>(lds, (t0_ + t) / T::TN, (t0_ + t) % T::TN, sum[t]);
              __builtin_amdgcn_sched_barrier(0);
            });
            if (threadIdx.x == 0) ws_counters[tile] = 0;   // as the launch found it
            block_store<DT, T, kEpiNone, true>(acc, c + (int64_t)row0 * n, n, 0, end - row0, g.b_r0, n, lds);
          }
          MBX_TICK(r, 4);
          tile_done();
          MBX_TICK(r, 5);
        }
        continue;
      } else {
        const int j = xcd * run + member;
        if (j >= 2 * rest) break;
        id = full_rounds * P + j / 2;
        half = j & 1;
        use_ts = true;
      }
      g.tick_ordinal = r;
      MBX_TICK(r, 0);
      int e, start, end, tm, tn;
      tiles.find(id, e, start, end, tm, tn);
      const int row0 = start + tm * T::BM + half * TS::BM;
      if (row0 >= end) break;
      const uint32_t a_bytes = clip_bytes((rows - row0) * k * 2);   // rows past the tile's are fetched, never stored
      g.rsrc_a = make_rsrc(a + (int64_t)row0 * k, a_bytes);
      g.rsrc_a2 = DUAL ? make_rsrc(a2 + (int64_t)row0 * k, a_bytes) : g.rsrc_a;
      g.rsrc_b = make_rsrc(b + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2));
      g.rsrc_b2 = DUAL ? make_rsrc(b2 + (int64_t)e * k * n, (uint32_t)((int64_t)k * n * 2)) : g.rsrc_b;
      // the second matrix of a [w1 | v1] tile: rows BN / 2 .. BN - 1 of the tile are its rows b_r0 .. b_r0 + BN / 2 - 1
      if (epi_is_glu(EPI)) g.rsrc_b2 = make_rsrc(b2 + ((int64_t)e * n - T::BN / 2) * k, (uint32_t)(((int64_t)n + T::BN / 2) * k * 2));
      g.b_r0 = tn * kTileCols;
      uint16_t* const c_tile = EPI == kEpiCombine && c == nullptr ? nullptr : c + (int64_t)row0 * n;
      uint16_t* const e_tile = EPI != kEpiNone && EPI != kEpiCombine ? extra + (int64_t)row0 * n : nullptr;
      const uint16_t* const p_tile = epi_is_dglu(EPI) ? a2 + (int64_t)row0 * n : nullptr;   // x2 of the gated activation
      uint16_t* const o_tile = epi_is_dglu(EPI) || epi_is_glu(EPI) ? out2 + (int64_t)row0 * n : nullptr;
      // the last row tile of an expert, when at most half full, is computed as a half-height tile as well
      use_ts = kSplit && (use_ts || end - row0 <= half_limit);
      Combine combine;
      if constexpr (EPI == kEpiCombine) {
        // the assignment of tile row threadIdx.x (top_k = 1: the token itself), on its way during the main loop
        combine.out = extra;
        combine.weights = combine_weights;
        combine.w_dtype = combine_w_dtype;
        combine.tokens = combine_tokens;
        const int row = row0 + (int)threadIdx.x;
        combine.row_exists = row < end;
        combine.token = slots[combine.row_exists ? row : end - 1];
      }
      if (use_ts) {
        block_gemm<DT, false, B_MC, TS, DUAL, EPI>(g, c_tile, n, 0, end - row0, g.b_r0, n, lds, e_tile, p_tile, o_tile, combine);
      } else {
        block_gemm<DT, false, B_MC, T, DUAL, EPI>(g, c_tile, n, 0, end - row0, g.b_r0, n, lds, e_tile, p_tile, o_tile, combine);
      }
      tile_done();
      MBX_TICK(r, 5);
    }
  } else {
    // The assignments of a tile's rows are fetched while the tile before it is computed (the tile's loads cannot start
    // without them).  Lane l of wave w issues load w + 4 q of the tile, which holds rows 8 (w + 4 q) + l / 8.
    static_assert(!GATHER || (T::LA >= TS::LA && T::LA <= 8 && T::BK == 64 && T::WAVES == TS::WAVES), "the row map is fetched for the taller tile");
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane_row = lane_id() >> 3;
    const uint32_t piece = load_lane_offset<false, T::BK, T::BM>(wave, 0, 0u, false);   // pitch 0: the piece inside the row
    const int64_t slots_end = (int64_t)src_rows * top_k;
    int next_slot[T::LA];
    auto fetch_slots = [&](int e, int start, int row0) {
      const int src_start = e > 0 ? src_bins[e - 1] : 0, src_end = src_bins[e];
      const int j0 = (src_start < 0 ? 0 : src_start) + (row0 - start);
      const int j1 = (int)(src_end < slots_end ? src_end : slots_end);
#pragma unroll
      for (int q = 0; q < T::LA; ++q) {
        const int j = j0 + 8 * (wave + q * T::WAVES) + lane_row;
        next_slot[q] = j < j1 ? slots[j] : -1;
      }
    };
    g.rsrc_a = make_rsrc(a, clip_bytes((int64_t)src_rows * k * 2));   // the whole source matrix, below 2 GiB
    int e_next, start_next, end_next, tn_next, row0_next;
    bool use_ts_next;
    bool have_next = items > 0 && locate(0, e_next, start_next, end_next, tn_next, row0_next, use_ts_next);
    if (have_next) fetch_slots(e_next, start_next, row0_next);
    for (int r = 0; have_next; ++r) {
      const int e = e_next, end = end_next, tn = tn_next, row0 = row0_next;
      const bool use_ts = use_ts_next;
      // byte offset of the row and 16-byte piece each of this lane's loads of a K tile fetches (bit 31: a row of zeros)
#pragma unroll
      for (int q = 0; q < T::LA; ++q) {
        const uint32_t row = top_k_magic ? __umulhi((uint32_t)next_slot[q], top_k_magic) >> top_k_shift : (uint32_t)next_slot[q];
        g.gather_row[q] = next_slot[q] >= 0 && row < (uint32_t)src_rows ? row * g.a_ld_bytes + piece : 0x80000000u;
      }
      have_next = r + 1 < items && locate(r + 1, e_next, start_next, end_next, tn_next, row0_next, use_ts_next);
      if (have_next) fetch_slots(e_next, start_next, row0_next);
      compute_tile(e, end, tn, row0, use_ts);
    }
  }
}

// n / d for 0 <= n < 2^31 as (n * magic) >> (32 + shift): magic = ceil(2^(31 + l) / d) with l = ceil(log2 d) (at least
// 1) fits 32 bits and gives the exact quotient for every such n; d = 1: magic 0, meaning "no division".
static inline void gather_divisor(int d, uint32_t& magic, int& shift) {
  magic = 0;
  shift = 0;
  if (d <= 1) return;
  int l = 1;
  while ((1 << l) < d) ++l;
  const uint64_t two = (uint64_t)1 << (31 + l);
  magic = (uint32_t)((two + (uint64_t)d - 1) / (uint64_t)d);
  shift = l - 1;
}

// ---- TN ----
// Tiles of one expert's [k, n] product are enumerated in 8 x 4 blocks (8 row tiles x 4 column tiles:
// 12 operand panels per 32 tiles; smaller blocks for products with fewer tiles in a direction), and that
// sequence is cut into 8 equal pieces, one per XCD: XCD x works through piece x of the first expert,
// piece x + 1 of the second, and so on (rotated, so that products of fewer than 8 tiles per expert still
// spread over all XCDs).  The cost of a tile
// is proportional to its expert's row count, so with skewed routing any coarser dealing of tiles to
// XCDs (whose queues are fixed by the workgroup id) leaves some XCDs with several times the work.
// For the same reason the tiles of an XCD are not dealt to workgroups statically: a workgroup takes
// `chunk` consecutive tiles of its XCD's list and the hardware hands out workgroups as compute units
// become free (chunk > 1 when the reductions are short and the per-workgroup overhead shows).
constexpr int kTnBlockM = 8, kTnBlockN = 4;
// XCD of the expert with rank r (0 = most rows) when whole experts are dealt to XCDs: 0 .. 7, 7 .. 0, 0 .. 7, ...
__host__ __device__ static inline int serpentine_xcd(int r) { return ((r / kXcds) & 1) ? kXcds - 1 - r % kXcds : r % kXcds; }
// The block shape of a launch: 8 x 4 when an XCD's eighth of an expert is at least a block (32 tiles); for smaller
// products the shape whose eighths are most compact, so that the workgroups of an XCD, which work on the eighths of
// several experts at a time, fetch few operand panels per tile (a [1408, 2048] product, 6 x 8 tiles: eighths of 3 x 2
// tiles with 5 panels each instead of 6 x 1 with 7).  Chosen by trying every shape: first the fewest tiles in the
// fullest eighth (the XCDs' balance), then the fewest panels over the eight.
struct TnBlocks { int bm, bn; };
static inline int64_t tn_tiles_per_group(int tiles_m, int tiles_n, TnBlocks s) {
  return (int64_t)((tiles_m + s.bm - 1) / s.bm) * ((tiles_n + s.bn - 1) / s.bn) * (s.bm * s.bn);
}
static inline TnBlocks tn_block_shape(int tiles_m, int tiles_n) {
  TnBlocks best{tiles_m < kTnBlockM ? (tiles_m > 0 ? tiles_m : 1) : kTnBlockM, tiles_n < kTnBlockN ? (tiles_n > 0 ? tiles_n : 1) : kTnBlockN};
  const int64_t raw = (int64_t)tiles_m * tiles_n;
  if (raw >= (int64_t)kXcds * kTnBlockM * kTnBlockN || raw <= kXcds) return best;
  // the search takes tens of microseconds: the last few answers are kept (per thread; a layer alternates between two
  // or three shapes)
  struct Known { int tiles_m, tiles_n; TnBlocks shape; };
  static thread_local Known known[8];
  static thread_local int next_slot = 0;
  for (const Known& kn : known)
    if (kn.tiles_m == tiles_m && kn.tiles_n == tiles_n) return kn.shape;
  int64_t best_fullest = -1, best_panels = -1;
  for (int bm = 1; bm <= kTnBlockM && bm <= tiles_m; ++bm) {
    for (int bn = 1; bn <= kTnBlockM && bn <= tiles_n; ++bn) {
      if (bm * bn > kTnBlockM * kTnBlockN) continue;
      const TnBlocks s{bm, bn};
      const int blocks_m = (tiles_m + bm - 1) / bm;
      const int per_group = (int)tn_tiles_per_group(tiles_m, tiles_n, s), per_xcd = (per_group + kXcds - 1) / kXcds;
      int64_t fullest = 0, panels = 0;
      for (int piece = 0; piece < kXcds; ++piece) {
        bool row_seen[256] = {}, col_seen[256] = {};   // raw < 256: fewer than 256 tiles in either direction
        int64_t tiles = 0;
        for (int t = piece * per_xcd; t < (piece + 1) * per_xcd && t < per_group; ++t) {
          const int blk = t / (bm * bn), in = t % (bm * bn);
          const int tm = (blk % blocks_m) * bm + in % bm, tn = (blk / blocks_m) * bn + in / bm;
          if (tm >= tiles_m || tn >= tiles_n) continue;
          ++tiles;
          if (!row_seen[tm]) { row_seen[tm] = true; ++panels; }
          if (!col_seen[tn]) { col_seen[tn] = true; ++panels; }
        }
        fullest = tiles > fullest ? tiles : fullest;
      }
      if (best_fullest < 0 || fullest < best_fullest || (fullest == best_fullest && panels < best_panels)) {
        best_fullest = fullest; best_panels = panels; best = s;
      }
    }
  }
  known[next_slot] = Known{tiles_m, tiles_n, best};
  next_slot = (next_slot + 1) % 8;
  return best;
}
static inline int64_t tn_grid(int tiles_m, int tiles_n, TnBlocks shape, int num_groups, int chunk) {
  const int64_t per_group = tn_tiles_per_group(tiles_m, tiles_n, shape);
  const int64_t per_xcd = (per_group + kXcds - 1) / kXcds;
  const int64_t span = (int64_t)32 * chunk;   // list entries covered by 32 workgroups of an XCD
  // entries of an XCD's list: a piece of every expert, or every tile of its share of the experts (the kernel decides)
  const int64_t pieces = per_xcd * num_groups, whole = (num_groups + kXcds - 1) / kXcds * per_group;
  return ((pieces > whole ? pieces : whole) + span - 1) / span * 32 * kXcds;
}

// One output tile of expert e's product: rows [g.a_r0, g.a_r0 + TT::BM) x columns [g.b_r0, g.b_r0 + TT::BN) of
// c[e] = a[start:end]^T @ b[start:end].
// GATHER: b is the matrix the rows are picked from (its buffer, g.rsrc_b, and the row table, g.row_table /
// g.gather_row / g.gather_row2, are the caller's business).
template <int DT, typename TT, bool SEGMENTED, bool GATHER = false>
__device__ __forceinline__ void tn_tile(Args& g, const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                        uint16_t* __restrict__ c_e, int start, int end, int k, int n, int seg_rows,
                                        char* lds) {
  static_assert(!(GATHER && SEGMENTED), "gathered rows: one segment");
  if constexpr (!SEGMENTED) {
    // the buffers cover exactly the rows of this expert: later rows read as zero
    const int64_t group_rows = end - start;
    g.rsrc_a = make_rsrc(a + (int64_t)start * k, (uint32_t)(group_rows * k * 2));
    if constexpr (!GATHER) g.rsrc_b = make_rsrc(b + (int64_t)start * n, (uint32_t)(group_rows * n * 2));
    g.nk = (int)((group_rows + TT::BK - 1) / TT::BK);
    typename TT::Acc acc[TT::TM][TT::TN];
    block_multiply<DT, true, true, TT, false, false, false, GATHER>(g, acc, true, lds);
    MBX_TICK(g.tick_ordinal, 2);
    block_store<DT, TT>(acc, c_e, n, g.a_r0, k, g.b_r0, n, lds);
    MBX_TICK(g.tick_ordinal, 4);
  } else {
    // The reduction runs over the expert's rows in segments of at most seg_rows rows, each with buffers
    // of its own that cover exactly its rows.
    typename TT::Acc acc[TT::TM][TT::TN];
    int first = start;
    for (;;) {
      const int64_t left = end - first;
      const int64_t seg = left < seg_rows ? left : seg_rows;
      g.rsrc_a = make_rsrc(a + (int64_t)first * k, (uint32_t)(seg * k * 2));
      g.rsrc_b = make_rsrc(b + (int64_t)first * n, (uint32_t)(seg * n * 2));
      g.nk = (int)((seg + TT::BK - 1) / TT::BK);
      block_multiply<DT, true, true, TT>(g, acc, first == start, lds);
      if (left <= seg_rows) break;
      first += seg_rows;
      tile_done();   // the first stages are refilled next
    }
    block_store<DT, TT>(acc, c_e, n, g.a_r0, k, g.b_r0, n, lds);
  }
}

// TS: the tile for the last row tile of a product when at most TS::BM of its rows exist (k % T::BM in
// (0, TS::BM]; half the work; tiles are handed out as compute units become free, so unequal tiles balance);
// TS = T switches this off.
// SEGMENTED: an expert's rows of a or b may reach 2 GiB (the launch passes seg_rows, the number of rows that
// stays below it); otherwise the whole of a and b is smaller than that.
// GATHER: b is [src_rows, n] and row r of expert e's rows of the reduction is b[row of the r-th of its sorted
// assignments], zeros past the expert's last assignment: the weight gradient on the rows that
// megablocks/ops/gather.py:20-38 / padded_gather.py:20-55 would have copied out first (megablocks/layers/mlp.py:456-491,
// glu.py:128-166: `gmm(dsdd_out, x, batch_sizes, trans_a=True)` with x the gathered tokens).  row_table: one entry per
// sorted assignment, the byte offset of its row in b with bit 31 flipped (gather_row_table_kernel); src_bins: the
// inclusive bins of the sorted assignments (`bins` are the row bins of a, which may be padded per expert).
template <int DT, typename T, typename TS, bool SEGMENTED, bool GATHER = false>
__global__ void __launch_bounds__(T::THREADS)
gmm_tn_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b, uint16_t* __restrict__ c,
              const int32_t* __restrict__ bins, int num_groups, int rows, int k, int n, int tiles_m, int tiles_n,
              int bm, int bn, int chunk, int seg_rows, int whole_ok, const uint32_t* __restrict__ row_table,
              const int32_t* __restrict__ src_bins, int src_rows, int n_slots) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  static_assert(!GATHER || (!SEGMENTED && std::is_same<T, TS>::value), "gathered rows: one tile shape, one segment");
  static_assert(T::THREADS == TS::THREADS && T::BN == TS::BN && T::BK == TS::BK, "last-row tile");
  constexpr bool kMixed = T::BM != TS::BM;
  const int blocks_m = (tiles_m + bm - 1) / bm, blocks_n = (tiles_n + bn - 1) / bn;
  const int per_group = blocks_m * blocks_n * (bm * bn);
  const int per_xcd = (per_group + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  // Experts are taken in order of decreasing row count (longest reduction first), so that the tiles
  // of a heavily loaded expert do not start last and leave most of the chip idle at the end.  With at
  // most 64 experts every wave ranks them itself: lane e holds expert e's row count and its rank.
  const bool ranked = num_groups <= kWave;
  int rank = -1;
  // Whole experts per XCD (whole_ok: the host allows it, for short reductions): when the experts, dealt longest first
  // in a serpentine over the XCDs, load every XCD alike (within 1.5 %), XCD x computes all tiles of its experts instead
  // of an eighth of everybody's.  The operand panels of an expert are then fetched into one L2 instead of eight: with
  // a few K tiles per output tile the launch is bound by those fetches and the output's stores together (64 experts
  // of 256 rows, [1024, 4096] products: 0.265 -> 0.247 ms).  Long reductions are not (16 experts of 6190 rows: 2 %
  // slower, the price of the imbalance that is left), so the host does not allow it there.
  bool whole = false;
  if (ranked) {
    const int lane = lane_id();
    const int mine = lane < num_groups ? bins[lane] - (lane > 0 ? bins[lane - 1] : 0) : -1;
    rank = 0;
    for (int o = 0; o < num_groups; ++o) {
      const int other = __shfl(mine, o, kWave);
      rank += (other > mine || (other == mine && o < lane)) ? 1 : 0;
    }
    if (lane >= num_groups) rank = -1;
    if (whole_ok && num_groups >= kXcds) {
      const int home = rank < 0 ? -1 : serpentine_xcd(rank);
      int worst = 0, total = 0;
      for (int x = 0; x < kXcds; ++x) {
        int v = home == x ? (mine > 0 ? mine : 0) : 0;
#pragma unroll
        for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
        worst = v > worst ? v : worst;
        total += v;
      }
      whole = (int64_t)worst * kXcds * 200 <= (int64_t)total * 203;
    }
  }
  whole = __builtin_amdgcn_readfirstlane((int)whole) != 0;
  Args g;
  g.a_ld_bytes = (uint32_t)k * 2;
  g.b_ld_bytes = (uint32_t)n * 2;
  const int64_t items = whole ? (int64_t)((num_groups + kXcds - 1) / kXcds) * per_group : (int64_t)per_xcd * num_groups;   // per XCD
  // A workgroup's `chunk` tiles are 32 apart in its XCD's list: the 32 workgroups an XCD runs at a time are then on 32
  // consecutive tiles (one 8 x 4 block, 12 operand panels) for each of their tiles in turn; with consecutive tiles per
  // workgroup they would be spread over `chunk` blocks at once.
  const int64_t member = blockIdx.x / kXcds;
  const int64_t first = (member / 32) * 32 * chunk + member % 32;
  const int64_t last = first + (int64_t)32 * chunk < items ? first + (int64_t)32 * chunk : items;
  // entry i of this XCD's list -> expert, its rows and the tile; false for the padding of the block enumeration
  // (uniform over the workgroup)
  struct Entry { int e, start, end, tm, tn; };
  auto decode = [&](int64_t i, Entry& t_) -> bool {
    int slot, t;   // position of the expert in the longest-first order, tile slot inside the expert
    if (whole) {
      const int q = (int)(i / per_group);
      slot = q * kXcds + ((q & 1) ? kXcds - 1 - xcd : xcd);
      t = (int)(i % per_group);
      if (slot >= num_groups) return false;
    } else {
      slot = (int)(i / per_xcd);
      t = ((xcd + slot) % kXcds) * per_xcd + (int)(i % per_xcd);
      if (t >= per_group) return false;
    }
    int blk, in;
    if (bm == kTnBlockM && bn == kTnBlockN) {   // the usual case, with constant divisors
      blk = t / (kTnBlockM * kTnBlockN), in = t % (kTnBlockM * kTnBlockN);
      t_.tm = (blk % blocks_m) * kTnBlockM + in % kTnBlockM, t_.tn = (blk / blocks_m) * kTnBlockN + in / kTnBlockM;
    } else {
      blk = t / (bm * bn), in = t % (bm * bn);
      t_.tm = (blk % blocks_m) * bm + in % bm, t_.tn = (blk / blocks_m) * bn + in / bm;
    }
    if (t_.tm >= tiles_m || t_.tn >= tiles_n) return false;
    t_.e = slot;
    if (ranked) t_.e = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(__ballot(rank == slot)));
    // bounds inside [0, rows] and in order whatever the table holds: a wrong table cannot take a load out of range
    t_.start = t_.e > 0 ? clamp_row(bins[t_.e - 1], rows) : 0;
    t_.end = clamp_row(bins[t_.e], rows);
    t_.end = t_.end < t_.start ? t_.start : t_.end;
    return true;
  };
  auto next_tile = [&](int64_t& i, Entry& t_) -> bool {   // the first entry from i on that is a tile
    for (; i < last; i += 32)
      if (decode(i, t_)) return true;
    return false;
  };
  if constexpr (!GATHER) {
    Entry cur;
    for (int64_t i = first; next_tile(i, cur); i += 32) {
      g.tick_ordinal = (int)((i - first) / 32);
      MBX_TICK(g.tick_ordinal, 0);
      g.a_r0 = cur.tm * T::BM;
      g.b_r0 = cur.tn * T::BN;
      uint16_t* const c_e = c + (int64_t)cur.e * k * n;
      if (kMixed && k - g.a_r0 <= TS::BM) {
        tn_tile<DT, TS, SEGMENTED>(g, a, b, c_e, cur.start, cur.end, k, n, seg_rows, lds);
      } else {
        tn_tile<DT, T, SEGMENTED>(g, a, b, c_e, cur.start, cur.end, k, n, seg_rows, lds);
      }
      tile_done();
      MBX_TICK(g.tick_ordinal, 5);
    }
  } else {
    // The row entries of a tile's first two K tiles are fetched while the tile before it is computed (its loads cannot
    // start without them): T::LB entries per K tile and lane, see row_entry_lane_offset().
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t entry_lane = row_entry_lane_offset(wave);
    g.rsrc_b = make_rsrc(b, clip_bytes((int64_t)src_rows * n * 2));   // the whole source matrix, below 2 GiB
    uint32_t ahead[2][T::LB];
    // the expert's part of the table: exactly its assignments, so that an entry past them reads as zero = "no row"
    auto table_of = [&](const Entry& t_) -> u32x4 {
      int xs = t_.e > 0 ? src_bins[t_.e - 1] : 0, xe = src_bins[t_.e];
      xs = xs < 0 ? 0 : (xs > n_slots ? n_slots : xs);
      xe = xe < xs ? xs : (xe > n_slots ? n_slots : xe);
      const uint64_t base = (uint64_t)(uintptr_t)(row_table + xs + (int64_t)kRowTableTile * t_.e);
      u32x4 d;
      d[0] = (uint32_t)base;
      d[1] = (uint32_t)(base >> 32) & 0xffffu;
      d[2] = (uint32_t)((xe - xs + kRowTableTile - 1) / kRowTableTile * kRowTableTile) * 4u;   // whole K tiles
      d[3] = 0x00020000u;
      return d;
    };
    auto fetch_ahead = [&](const u32x4& table) {
      fetch_row_entries(ahead[0], table, entry_lane, 0u);
      fetch_row_entries(ahead[1], table, entry_lane, (uint32_t)kRowTableTile * 4u);
    };
    Entry cur, nxt;
    int64_t i = first;
    bool have = next_tile(i, cur);
    u32x4 table_next = {0u, 0u, 0u, 0x00020000u};
    if (have) {
      table_next = table_of(cur);
      fetch_ahead(table_next);
    }
    bool arrived = false;   // whether a wait since fetch_ahead() has covered its loads
    while (have) {
      g.row_table = table_next;
      // The entries asked for a tile ago have arrived with that tile's main loop, which ends without a load in flight;
      // those of the workgroup's first tile, or behind a tile without rows (no main loop), are waited for here.
      if (!arrived) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int q = 0; q < T::LB; ++q) {
        asm volatile("" : "+v"(ahead[0][q]), "+v"(ahead[1][q]));
        g.gather_row[q] = ahead[0][q];
        g.gather_row2[q] = ahead[1][q];
      }
      int64_t i_next = i + 32;
      const bool have_next = next_tile(i_next, nxt);
      if (have_next) {
        table_next = table_of(nxt);
        fetch_ahead(table_next);
      }
      g.tick_ordinal = (int)((i - first) / 32);
      MBX_TICK(g.tick_ordinal, 0);
      g.a_r0 = cur.tm * T::BM;
      g.b_r0 = cur.tn * T::BN;
      tn_tile<DT, T, false, true>(g, a, b, c + (int64_t)cur.e * k * n, cur.start, cur.end, k, n, seg_rows, lds);
      arrived = g.nk > 0;
      tile_done();
      MBX_TICK(g.tick_ordinal, 5);
      cur = nxt;
      i = i_next;
      have = have_next;
    }
  }
}

// The row table of the GATHER instantiation of gmm_tn_kernel, one thread per entry (see row_entry_slot() for the
// layout): the entry of row r of K tile kt of expert e is the byte offset in the source matrix of the row of the expert's
// (64 kt + r)-th sorted assignment (slot / top_k, as (slot * magic) >> (32 + shift), see gather_divisor()) with bit 31
// flipped; zero -- which reads as bit 31 set: "no row" -- past the expert's assignments and for an assignment outside
// [0, src_rows * top_k).
__global__ void gather_row_table_kernel(const int32_t* __restrict__ slots, const int32_t* __restrict__ src_bins, int num_groups,
                                        int n_slots, int src_rows, uint32_t pitch_bytes, uint32_t top_k_magic, int top_k_shift,
                                        uint32_t* __restrict__ table) {
  const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= row_table_entries(n_slots, num_groups)) return;
  auto bound = [&](int e) -> int { const int v = src_bins[e]; return v < 0 ? 0 : (v > n_slots ? n_slots : v); };
  // the expert whose part holds entry s: the last one that starts at or before it
  int lo = 0, hi = num_groups - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if ((int64_t)bound(mid - 1) + (int64_t)kRowTableTile * mid <= s) lo = mid; else hi = mid - 1;
  }
  const int e = lo;
  const int xs = e > 0 ? bound(e - 1) : 0;
  int xe = bound(e);
  xe = xe < xs ? xs : xe;
  const int64_t local = s - ((int64_t)xs + (int64_t)kRowTableTile * e);
  const int64_t l = local / kRowTableTile * kRowTableTile + row_of_entry_slot((int)(local % kRowTableTile));
  uint32_t v = 0u;
  if (l < xe - xs) {
    const int slot = slots[xs + l];
    const uint32_t row = top_k_magic ? __umulhi((uint32_t)slot, top_k_magic) >> top_k_shift : (uint32_t)slot;
    if (slot >= 0 && row < (uint32_t)src_rows) v = (row * pitch_bytes) ^ 0x80000000u;
  }
  table[s] = v;
}

}  // namespace dma
