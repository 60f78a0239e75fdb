// Grouped W8A8 GEMM, persistent four-wave tile kernel for gfx950 on v_mfma_i32_16x16x64_i8: 256 x 256 output tiles,
// four wavefronts (one per SIMD), 128 x 128 accumulators per wavefront as 8 x 8 blocks of 16 x 16; weights stored
// [E,N,K], packed or [E,K,N].
//
// Why this instruction.  On random int8 operands the chip runs against its power limit and the clock follows what the
// matrix pipe draws; the 16 x 16 x 64 shape draws less for the same multiply-adds than 32 x 32 x 32 (64 products are added
// up inside the array before an accumulator register is touched, instead of 32): a loop of nothing but MFMAs sustains
// 4.1 - 4.3 POP/s with it against 3.5 POP/s.  The design around the MFMAs is that of the 32 x 32 x 32 kernel
// (gmm_tile4_w8a8.hip, kept to be measured against): 128-byte K slabs in two LDS stages, two further slabs in flight
// through staging registers, one barrier per slab, a compile-time K-loop body for the slabs inside a tile and a general
// one for its last slabs, persistent workgroups with the operand stream carried across tiles, epilogue operands brought
// into an LDS table by LDS-direct loads.
//
// What differs:
//   * A fragment is 16 rows x 64 K bytes: lane (m16, g) = (lane % 16, lane / 16) reads row m16 of its block, 16-byte chunk
//     4 h + g of K half h.  x rows are 128 bytes in LDS with chunk c of row r at position c ^ ((r >> 1) & 7): the sixteen
//     lanes of a quarter wave fall into sixteen different 16-byte bank groups.
//   * Weights are the first operand: a lane owns output row m16 of an x block and rows 4 g .. 4 g + 3 of a weight block.
//     Row i of weight block f is column 32 (f / 2) + 8 (i / 4) + 4 (f % 2) + i % 4 of the wave tile, so that the two blocks
//     of a pair give a lane eight consecutive columns: the epilogue stores 16 bytes per lane (bf16 / f16; int32: twice
//     16), 64-byte row pieces per quarter wave, straight from the accumulators, the two halves of a 128-byte line back to
//     back.  Rows past the group fall outside the store descriptor, columns past N are killed in the lane offset.
//     [E,N,K] weights: LDS row rho is column rho, chunk c at position c ^ (bit 1 | bits 3..4 << 1 of rho) -- the rows a
//     quarter wave reads differ in bits 0, 1, 3, 4.  Packed weights: a block (16 columns x 64 K bytes) goes to LDS as it
//     is, odd column groups with bit 2 of the column index flipped; a fragment gathers from two column groups.  Both
//     conflict free.  [E,K,N] weights go through LDS transpose reads (at the kernel's head).
//   * A K half of a slab is multiplied in four steps of 4 x 4 blocks, visited in the order (F0,I0) (F0,I1) (F1,I1) (F1,I0)
//     (F: weight blocks 0..3 / 4..7, I: x blocks 0..3 / 4..7), so that every step needs only four new fragments and two
//     sets of four weight and four x fragments (64 registers) are enough.  A step is 16 MFMAs (256 cycles), four
//     fragment reads, two staging quads written to LDS and two requested.
//   * With 16-cycle MFMAs the order of the memory operations between them decides the K loop's pace (see the slab
//     body): at most one operation behind an MFMA, LDS writes in 8-byte halves.
#include "gmm_common.h"
#include "gmm_kernels.h"
#include "gmm_tile4_common.h"

#include <atomic>
#include <type_traits>

namespace msco {
namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
constexpr int T4M_B = 8;                                         // 16 x 16 blocks per wave tile edge
// LDS: x stages 0 and 1 (32 KiB each), weight stages 0 and 1, two epilogue operand tables, the group table.  [E,K,N]
// weights (WL == 2) lie in LDS as K rows of 256 column bytes at a pitch of 288 bytes (see the kernel's head).
constexpr int T4M_KN_PITCH = 288;
constexpr int t4m_w_stage(int wl) { return wl == 2 ? T4_BK * T4M_KN_PITCH : T4_OP_STAGE; }
constexpr int t4m_param_off(int wl) { return T4_W_BASE + 2 * t4m_w_stage(wl); }
constexpr int t4m_meta_off(int wl) { return t4m_param_off(wl) + 2 * T4_PARAM_BYTES; }   // per group: row end, tiles up to and including it
constexpr int t4m_lds_bytes(int wl) { return t4m_meta_off(wl) + 2 * T4_MAX_E * 4; }
static_assert(t4m_lds_bytes(2) <= 160 * 1024, "LDS of one CU");

}  // namespace

// MODE: output type, 0 bf16, 1 f16, 2 int32 (raw accumulators plus bias).  WL: weight layout, 0 [E,N,K], 1 packed, 2 [E,K,N]
// (N a multiple of 16).  Packed (1 KiB blocks
// of 16 columns x 64 K bytes; a slab of a tile is 16 column groups x 2 blocks, staging quad (u, wave) is block 4 u + wave =
// (column group 2 u + wave / 2, K block wave % 2) and goes to LDS as it is) instead of [E,N,K].  ACT: 0 none, 1 gelu
// (tanh form), 2 v * sigmoid(c v) (silu, fast gelu), 3 relu.
//
// [E,K,N]: rows are N-contiguous and an MFMA operand wants 16 K-contiguous bytes per lane; the LDS transpose read of gfx950
// (ds_read_b64_tr_b8) does that turn on the way out of LDS.  Of a block of 16 lanes, lane i names 8 bytes M[i][0..7];
// lane j receives byte b = M[2 b + j / 8][j % 8].  A slab goes to LDS as it lies in memory -- K rows of 256 columns, one
// staging quad = 4 K rows, lane L row L / 16, 16-column chunk L % 16 -- at a row pitch of 288 bytes, so that the eight K
// rows and two chunks that one block of 16 lanes names fall into sixteen different 16-byte bank groups and every part of
// a fragment address is additive.  The middle dwords of every chunk are swapped on the way in: the first 8 bytes of a
// chunk then are columns 0..3 and 8..11, the second 8 bytes columns 4..7 and 12..15 -- fragment rows 0..7 of an even and of
// an odd weight block (see the head of the file).  K rows 16..31 (mod 32) store the two halves the other way round: the
// two blocks of 16 lanes that read together (K rows 16 apart) then use different banks.  A fragment is two transpose
// reads, 8 K rows apart.
template <int MODE, int WL, int ACT>
__global__ void __launch_bounds__(T4_NW * 64, 1) gmm_w8a8_tile4m_kernel(const GmmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool PK = WL == 1, KN = WL == 2;
  constexpr int W_STAGE = t4m_w_stage(WL), PARAM_OFF = t4m_param_off(WL), META_OFF = t4m_meta_off(WL);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 1, wave_n = wave & 1;

  // ---- this workgroup's share of the tiles (as in gmm_tile4_w8a8.hip) ----------------------------------
  const int n_tiles = (p.n + T4_BN - 1) / T4_BN;
  int *meta_end = reinterpret_cast<int *>(smem + META_OFF);
  int *meta_upto = meta_end + T4_MAX_E;
  int total = 0;
  for (int g0 = 0, carry = 0; g0 < p.e; g0 += 64) {
    int s0, e0;
    group_rows_chunk(p, g0, lane, carry, s0, e0);
    const int rows_g = e0 - s0;
    const int upto = total + wave_scan_add((rows_g > p.rows_lo && rows_g <= p.rows_hi) ? ((rows_g + T4_BM - 1) / T4_BM) * n_tiles : 0, lane);
    if (wave == 0 && g0 + lane < p.e) {
      meta_end[g0 + lane] = e0;
      meta_upto[g0 + lane] = upto;
    }
    total = wave_bcast(upto, 63);
  }
  __syncthreads();
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  const int rounds = (total + (int)gridDim.x - 1) / (int)gridDim.x;
  const int wgs_per_xcd = rounds > 0 ? min((int)gridDim.x / kNumXcd, ((total + rounds - 1) / rounds + kNumXcd - 1) / kNumXcd) : 0;
  if (slot >= wgs_per_xcd) return;
  auto tile_at = [&](int i) -> T4Tile {
    const int l = slot + i * wgs_per_xcd;
    int lane_now = lane;   // laundered: keeps the table addresses out of the registers that live across the K loop
    asm volatile("" : "+v"(lane_now));
    return t4_locate(meta_end, meta_upto, p.e, l < per_xcd ? xcd * per_xcd + l : -1, total, n_tiles, lane_now);
  };
  T4Tile cur = tile_at(0);
  if (!cur.valid) return;

  // K slabs per tile, rounded up to even (the staging parities alternate per slab); slabs past K read zeros
  const int k_slabs = 2 * ((p.k + 2 * T4_BK - 1) / (2 * T4_BK));
  const long long w_elems = (long long)p.k * p.n;
  auto x_rsrc = [&](const T4Tile &t) {
    return t4_rsrc(reinterpret_cast<const int8_t *>(p.x) + (long long)t.m0 * p.k, (long long)(t.g_end - t.m0) * p.k);
  };
  const int k_blocks = (p.k + 63) / 64, col_groups = (p.n + 15) / 16;   // packed layout
  auto w_rsrc = [&](const T4Tile &t) {
    if constexpr (PK) {
      const long long cg_bytes = (long long)k_blocks * 1024;
      return t4_rsrc(p.w + ((long long)t.grp * col_groups + t.n0 / 16) * cg_bytes, (long long)(col_groups - t.n0 / 16) * cg_bytes);
    } else if constexpr (KN) {
      return t4_rsrc(p.w + (long long)t.grp * w_elems + t.n0, w_elems - t.n0);   // (loads use w_rsrc_at: a window per slab)
    } else {
      return t4_rsrc(p.w + (long long)t.grp * w_elems + (long long)t.n0 * p.k, (long long)(p.n - t.n0) * p.k);
    }
  };
  // [E,K,N]: the window of a tile's weights from K row `krow0` on.  A slab's first row cannot go into the scalar offset
  // of the load (the buffer unit range-checks the per-lane offset only, against the whole window): it goes into the
  // base, and the window ends with the expert's matrix, so K rows past K and anything past the tensor read as zeros by
  // the range check alone.  A chunk past N inside the matrix reads the next K row's bytes: columns that are never stored.
  // (base and size of the tile's window are kept as scalars: K N < 2^31, so the size fits 32 bits)
  struct T4Window {
    const int8_t *base;
    int bytes;
  };
  auto w_window = [&](const T4Tile &t) { return T4Window{p.w + (long long)t.grp * w_elems + t.n0, (int)w_elems - t.n0}; };
  auto w_rsrc_at = [&](const T4Window &w, unsigned krow0) {
    const unsigned off = krow0 * (unsigned)p.n;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(w.base + off), 0, max(w.bytes - (int)off, 0), 0x00020000);
  };

  // ---- global -> staging registers: one quad = 1 KiB per wave = 8 rows x 128 B (packed weights: one block) ------------
  const unsigned rows32 = 32u * (unsigned)p.k;
  const unsigned b_step = PK ? 2u * (unsigned)k_blocks * 1024u : KN ? 16u * (unsigned)p.n : rows32;   // staging quad u -> u + 1: two column groups / 16 K rows / 32 rows
  int d_chunk, d_chunk_w;
  unsigned a_voff0, b_voff0;
  // ---- fragment addressing: see the head of the file ------------------------------------------------------
  unsigned x_lane, w_lane, st_x, st_w;
  auto lane_constants = [&]() __attribute__((always_inline)) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int m16 = ln & 15, g4 = ln >> 4;
    const int d_row0 = 8 * wave + (ln >> 3);
    d_chunk = (ln & 7) ^ ((d_row0 >> 1) & 7);
    a_voff0 = (unsigned)d_row0 * (unsigned)p.k + d_chunk * 16;
    // weights [E,N,K]: LDS row rho is column rho of the tile, chunk c at position c ^ sw(rho) with sw(rho) = bit 1 and bits
    // 3..4 of rho (the rows a quarter wave reads differ in bits 0, 1, 3 and 4: see the head of the file)
    d_chunk_w = WL != 0 ? d_chunk : ((ln & 7) ^ (((ln >> 4) & 1) | (wave << 1)));
    b_voff0 = PK   ? (unsigned)(((wave >> 1) * k_blocks + (wave & 1)) * 1024 + ln * 16)
              : KN ? (unsigned)(4 * wave + (ln >> 4)) * (unsigned)p.n + (unsigned)((ln & 15) * 16)   // K row 4 wave + lane / 16 of quad 0, chunk lane % 16
                   : (unsigned)d_row0 * (unsigned)p.k + d_chunk_w * 16;
    const int swz = (m16 >> 1) & 7;
    x_lane = (unsigned)((wave_m * T4_WT + m16) * T4_BK + ((g4 ^ swz) << 4));
    const int w_row = 8 * (m16 >> 2) + (m16 & 3);   // fragment row m16 of blocks 0 and 1 is column w_row, w_row + 4 of the first 32
    if constexpr (PK) {
      // column group w_row / 16 (odd groups lie in LDS with bit 2 of the column swapped), column w_row % 16, chunk g4
      w_lane = (unsigned)(T4_W_BASE + wave_n * 16384 + (m16 >> 3) * 2048 + g4 * 256 + (((w_row & 15) ^ ((m16 >> 3) << 2)) << 4));
    } else if constexpr (KN) {
      // address lane m16 of its block of 16 names K row m16 / 2 of the 16 that lane group g4 multiplies, chunk m16 % 2 of
      // the pair that holds the 32 columns of blocks 0 and 1, the half that holds an even block's columns
      w_lane = (unsigned)(T4_W_BASE + (16 * g4 + (m16 >> 1)) * T4M_KN_PITCH + (wave_n * 8 + (m16 & 1)) * 16 + (g4 & 1) * 8);
    } else {
      w_lane = (unsigned)(T4_W_BASE + (wave_n * T4_WT + w_row) * T4_BK + ((g4 ^ (((m16 >> 1) & 1) | ((m16 >> 2) << 1))) << 4));
    }
    st_x = (unsigned)(wave * 1024 + ln * 16);
    st_w = KN ? T4_W_BASE + (unsigned)((4 * wave + (ln >> 4)) * T4M_KN_PITCH + (ln & 15) * 16)
              : T4_W_BASE + (unsigned)(wave * 1024 + ((PK ? (ln ^ (((wave >> 1) & 1) << 2)) : ln) << 4));
    asm volatile("" : "+v"(st_w));
  };
  lane_constants();

  const std::integral_constant<int, 0> c0;
  const std::integral_constant<int, 1> c1;
  const std::integral_constant<int, 2> c2;
  const std::integral_constant<int, 3> c3;

  v4i acc[T4M_B][T4M_B];   // [f: weight block][i: x block]
  v4i stg[2][2][T4_LD];    // staging quads: [slab parity][operand: 0 x, 1 w][u]
  v4i wf[2][4], xf[2][4];  // two sets of four weight and four x fragments

  T4Tile nxt = cur;        // tile that follows `cur` in this workgroup's walk (loads run ahead into it)
  __amdgpu_buffer_rsrc_t rx_c = x_rsrc(cur), rw_c = w_rsrc(cur), rx_n = rx_c, rw_n = rw_c;
  T4Window ww_c = w_window(cur), ww_n = ww_c;   // ([E,K,N] only)

  // slab s of the current tile, or slab s - k_slabs of the next one
  auto load_one = [&](int s, auto par_c, auto op_c, auto u_c) __attribute__((always_inline)) {
    constexpr int P = decltype(par_c)::value, OP = decltype(op_c)::value, U = decltype(u_c)::value;
#if MSCO_TILE4_ATTR & 8
    if (s >= 2) return;   // (the prologue's slabs 0 and 1 only)
#endif
    const bool ahead = s >= k_slabs;
    const unsigned kbase = (unsigned)(ahead ? s - k_slabs : s) * T4_BK;
    const bool dead = (ahead && !nxt.valid) || kbase + d_chunk * 16 >= (unsigned)p.k;   // K tail, slabs past K, no next tile
    const unsigned kill = dead ? T4_OOB : 0u;
    if constexpr (OP == 0) {
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(ahead ? rx_n : rx_c, (a_voff0 + U * rows32) | kill, kbase, 0);
    } else if constexpr (KN) {
      // K rows 16 U + 4 wave + lane / 16 of the slab, in the window that starts with the slab (rows past K fall outside it)
      const unsigned kill_w = (ahead && !nxt.valid) ? T4_OOB : 0u;
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc_at(ahead ? ww_n : ww_c, kbase), (b_voff0 + U * b_step) | kill_w, 0, 0);
    } else if constexpr (PK) {
      const unsigned kb = 2u * (unsigned)(ahead ? s - k_slabs : s) + (unsigned)(wave & 1);
      const unsigned kill_w = ((ahead && !nxt.valid) || kb >= (unsigned)k_blocks) ? T4_OOB : 0u;
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(ahead ? rw_n : rw_c, (b_voff0 + U * b_step) | kill_w, kbase * 16, 0);
    } else {
      const unsigned kill_n = ((ahead && !nxt.valid) || kbase + d_chunk_w * 16 >= (unsigned)p.k) ? T4_OOB : 0u;
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(ahead ? rw_n : rw_c, (b_voff0 + U * b_step) | kill_n, kbase, 0);
    }
  };
  // LDS address of staging quad (op, u) in stage st (an int or a compile-time constant)
  auto quad_addr = [&](auto st, auto op_c, auto u_c) __attribute__((always_inline)) -> unsigned {
    constexpr int OP = decltype(op_c)::value, U = decltype(u_c)::value;
    if constexpr (OP == 0) return st_x + (unsigned)st * T4_OP_STAGE + U * 4096;
    else return st_w + (unsigned)st * W_STAGE + U * (KN ? 16 * T4M_KN_PITCH : 4096);
  };
  // one 8-byte half (H = 0 first) of staging quad (op, u) to LDS.  [E,K,N] weights: the middle dwords of the chunk
  // change places before the first half leaves, and the K rows of odd quads store their halves the other way round.
  auto put_half = [&](auto st, auto p_c, auto op_c, auto u_c, auto h_c) __attribute__((always_inline)) {
    constexpr int P = decltype(p_c)::value, OP = decltype(op_c)::value, U = decltype(u_c)::value, H = decltype(h_c)::value;
    v4i &v = stg[P][OP][U];
    if constexpr (KN && OP == 1 && H == 0) {
      int y = v.y, z = v.z;
      asm volatile("v_swap_b32 %0, %1" : "+v"(y), "+v"(z));
      v.y = y;
      v.z = z;
    }
    const unsigned addr = quad_addr(st, op_c, u_c) + 8 * ((KN && OP == 1) ? (H ^ (U & 1)) : H);
#if MSCO_TILE4_ATTR & 16
    asm volatile("" ::"v"(v), "v"(addr));
#else
    *reinterpret_cast<v2i *>(smem + addr) = H == 0 ? v2i{v.x, v.y} : v2i{v.z, v.w};
#endif
  };
  // write quad (op, u) of slab s to its LDS stage and refill it with slab s + 2 (the prologue's form: both halves at once)
  auto cycle_one = [&](int s, auto par_c, auto op_c, auto u_c) {
    put_half(s & 1, par_c, op_c, u_c, c0);
    put_half(s & 1, par_c, op_c, u_c, c1);
    load_one(s + 2, par_c, op_c, u_c);
  };
  // fragment B (0..3) of block half BH (blocks 4 BH + B) of K half `half` in LDS stage `stage` (each an int or a
  // compile-time constant: constants end up in the instruction's offset field)
  auto read_x = [&](auto stage, auto half, auto set_c, auto bh_c, auto b_c) __attribute__((always_inline)) {
    constexpr int S = decltype(set_c)::value, BH = decltype(bh_c)::value, B = decltype(b_c)::value;
#if MSCO_TILE4_ATTR & 64
    asm volatile("" : "+v"(xf[S][B]));
    return;
#endif
    xf[S][B] = *reinterpret_cast<const v4i *>(smem + ((x_lane ^ ((unsigned)half << 6)) + (unsigned)stage * T4_OP_STAGE + (4 * BH + B) * 2048));
  };
  // (PART: [E,K,N] fragments are two transpose reads, 0 and 1, each in a slot of its own; the other layouts read in part 0)
  auto read_w = [&](auto stage, auto half, auto set_c, auto bh_c, auto b_c, auto part_c) __attribute__((always_inline)) {
    constexpr int S = decltype(set_c)::value, BH = decltype(bh_c)::value, B = decltype(b_c)::value, PART = decltype(part_c)::value;
#if MSCO_TILE4_ATTR & 64
    if constexpr (PART == 0) asm volatile("" : "+v"(wf[S][B]));
    return;
#endif
    constexpr int F = 4 * BH + B;   // block f lies at 32 (f / 2) + 4 (f % 2) columns
    if constexpr (KN) {
      typedef __attribute__((address_space(3))) v2i *lds_v2i;
      const unsigned addr = (w_lane ^ ((F & 1) << 3)) + (unsigned)stage * W_STAGE + (unsigned)half * (64 * T4M_KN_PITCH) + (F >> 1) * 32 +
                            PART * (8 * T4M_KN_PITCH);
      const v2i got = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(smem + addr));
      if constexpr (PART == 0) { wf[S][B].x = got.x; wf[S][B].y = got.y; }
      else { wf[S][B].z = got.x; wf[S][B].w = got.y; }
    } else if constexpr (PART == 0) {
      if constexpr (PK)
        wf[S][B] = *reinterpret_cast<const v4i *>(smem + ((w_lane ^ ((F & 1) << 6)) + (unsigned)stage * W_STAGE + (unsigned)half * 1024 + (F >> 1) * 4096));
      else
        wf[S][B] = *reinterpret_cast<const v4i *>(smem + ((w_lane ^ ((unsigned)half << 6)) + (unsigned)stage * W_STAGE + (F >> 1) * 4096 + (F & 1) * 512));
    }
  };

  // ---- stream prologue (once per workgroup): slabs 0 and 1 requested; slab 0 and group 0 of slab 1
  // written to LDS and refilled --------------------------------------------------------------------------
  {
    auto for_u = [&](auto fn) {
      fn(std::integral_constant<int, 0>{}); fn(std::integral_constant<int, 1>{}); fn(std::integral_constant<int, 2>{});
      fn(std::integral_constant<int, 3>{}); fn(std::integral_constant<int, 4>{}); fn(std::integral_constant<int, 5>{});
      fn(std::integral_constant<int, 6>{}); fn(std::integral_constant<int, 7>{});
    };
    for_u([&](auto u) { load_one(0, c0, c0, u); });
    for_u([&](auto u) { load_one(0, c0, c1, u); });
    for_u([&](auto u) { load_one(1, c1, c0, u); });
    for_u([&](auto u) { load_one(1, c1, c1, u); });
    for_u([&](auto u) { cycle_one(0, c0, c0, u); });
    for_u([&](auto u) { cycle_one(0, c0, c1, u); });
    cycle_one(1, c1, c0, c0); cycle_one(1, c1, c0, c1);
    cycle_one(1, c1, c1, c0); cycle_one(1, c1, c1, c1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    t4_barrier();
  }
  for (int ti = 0;; ++ti) {
    // the tile after this one: the operand stream crosses into it during the last slabs
    nxt = tile_at(ti + 1);
    if (nxt.valid) { rx_n = x_rsrc(nxt); rw_n = w_rsrc(nxt); ww_n = w_window(nxt); }
    if (ti > 0) lane_constants();

    // Epilogue operands of this tile (scale and bias of its 256 columns, per-token scale of its 256 rows) go straight
    // from memory into this tile's LDS table (two tables, alternating per tile); the K-loop barriers publish them.
    unsigned char *table = smem + PARAM_OFF + (ti & 1) * T4_PARAM_BYTES;
    {
      const unsigned lds = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char *)table + wave * 256;
      const int col = cur.n0 + tid, row = cur.m0 + tid;
      const long long pg = p.scale_per_group ? (long long)cur.grp * p.n : 0;
      if (p.scale_dtype == DT_NONE) {
        reinterpret_cast<float *>(table)[tid] = 1.0f;
      } else {
        const int esz = p.scale_dtype == DT_F32 ? 4 : p.scale_dtype == DT_BF16 ? 2 : 8;
        const long long first = p.scale_is_scalar ? 0 : (pg + cur.n0) * esz;
        const v4i rs = t4_raw_rsrc(reinterpret_cast<const unsigned char *>(p.scale) + first,
                                   p.scale_is_scalar ? esz : (long long)(p.n - cur.n0) * esz);
        const unsigned voff = col < p.n ? (p.scale_is_scalar ? 0u : (unsigned)(tid * esz)) : T4_OOB;
        if (p.scale_dtype == DT_BF16) t4_dma_b16(rs, lds, voff);
        else t4_dma_b32(rs, lds, voff);
      }
      if (p.bias != nullptr) {
        const v4i rb = t4_raw_rsrc(p.bias + pg + cur.n0, (long long)(p.n - cur.n0) * 4);
        t4_dma_b32(rb, lds + 1024, col < p.n ? (unsigned)(tid * 4) : T4_OOB);
      }
      if (p.per_token == nullptr) {
        reinterpret_cast<float *>(table + 2048)[tid] = 1.0f;
      } else {
        const v4i rp = t4_raw_rsrc(p.per_token + cur.m0, (long long)(p.m - cur.m0) * 4);
        t4_dma_b32(rp, lds + 2048, row < cur.g_end ? (unsigned)(tid * 4) : T4_OOB);
      }
    }

    // rows of this tile that exist, and the 16-row blocks of this wave that hold any of them
    const int rows_here = min(T4_BM, cur.g_end - cur.m0);
    const int rows_wave = rows_here - wave_m * T4_WT;
    const int bm_active = max(0, min(T4M_B, (rows_wave + 15) / 16));

    // the fragments of the first step of slab 0: weight blocks 0..3 into set 0, x blocks 0..3 into set 0, K half 0
    read_w(c0, c0, c0, c0, c0, c0); read_w(c0, c0, c0, c0, c1, c0); read_w(c0, c0, c0, c0, c2, c0); read_w(c0, c0, c0, c0, c3, c0);
    read_w(c0, c0, c0, c0, c0, c1); read_w(c0, c0, c0, c0, c1, c1); read_w(c0, c0, c0, c0, c2, c1); read_w(c0, c0, c0, c0, c3, c1);
    read_x(c0, c0, c0, c0, c0); read_x(c0, c0, c0, c0, c1); read_x(c0, c0, c0, c0, c2); read_x(c0, c0, c0, c0, c3);

    {
      // The 16 MFMAs of weight set WS (blocks 4 FH ..) and x set XS (blocks 4 IH ..); behind MFMA k comes slot(k), at most one
      // memory operation.  XM: MFMA k takes x fragment k / 4 and weight fragment k % 4 (else the other way round): the step
      // after one that fetched x fragments runs x-major, so that fragment b is first needed 4 b MFMAs into the step and a
      // fragment read has 240 cycles to arrive.  The MFMAs are written as assembly so that their accumulators are pinned
      // to the accumulation registers (left to the compiler, some blocks get the architectural form of the instruction
      // and the allocator then shuffles and spills accumulators all through the K loop) and declared to touch memory,
      // which keeps every memory operation in its slot (scheduling barriers alone do not: instruction selection has
      // already moved loads by the time they act).  An accumulator block meets its
      // next MFMA 64 instructions later: the compiler's wait counts cover the operands, nothing else needs wait states.
      auto mfma_step = [&](auto xm_c, auto ws_c, auto xs_c, auto fh_c, auto ih_c, auto &&slot) __attribute__((always_inline)) {
        constexpr int WS = decltype(ws_c)::value, XS = decltype(xs_c)::value, FH = decltype(fh_c)::value, IH = decltype(ih_c)::value;
        constexpr bool XM = decltype(xm_c)::value != 0;
        // (plain statements, not a nested lambda: operands of an asm statement do not capture)
#define T4M_WI(K) (XM ? (K) % 4 : (K) / 4)
#define T4M_XI(K) (XM ? (K) / 4 : (K) % 4)
#if MSCO_TILE4_ATTR & 2
#define T4M_MM(K) asm volatile("" ::"v"(wf[WS][T4M_WI(K)]), "v"(xf[XS][T4M_XI(K)]))
#else
#define T4M_MM(K)                                        \
  asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" \
               : "+a"(acc[4 * FH + T4M_WI(K)][4 * IH + T4M_XI(K)]) \
               : "v"(wf[WS][T4M_WI(K)]), "v"(xf[XS][T4M_XI(K)])    \
               : "memory")
#endif
#define T4M_ONE(K)                            \
  T4M_MM(K);                                  \
  slot(std::integral_constant<int, (K)>{});   \
  __builtin_amdgcn_sched_barrier(0)
        __builtin_amdgcn_sched_barrier(0);
        T4M_ONE(0); T4M_ONE(1); T4M_ONE(2); T4M_ONE(3); T4M_ONE(4); T4M_ONE(5); T4M_ONE(6); T4M_ONE(7);
        T4M_ONE(8); T4M_ONE(9); T4M_ONE(10); T4M_ONE(11); T4M_ONE(12); T4M_ONE(13); T4M_ONE(14); T4M_ONE(15);
#undef T4M_ONE
#undef T4M_MM
#undef T4M_WI
#undef T4M_XI
      };
      // One K slab in LDS stage `stage` (`os`: the other stage; ints, or constants in the compile-time loop).  On entry weight
      // blocks 0..3 and x blocks 0..3 of K half 0 are in fragment sets 0 and group 0 of the next slab is in LDS; PAR is the
      // staging parity of the next slab.  fill_a(par, op, u) requests quad (op, u) of the slab three on, fill_b of the slab
      // four on.
      //
      // Eight steps: K half 0 then K half 1, each over the quadrants (F0,I0) (F0,I1) (F1,I1) (F1,I0), so that a step needs
      // four new fragments.  A step also moves two staging quads to LDS and requests their successors.  What a lone wave
      // can issue next to 16-cycle MFMAs was measured on a loop of MFMAs with memory operations woven in: fragment reads
      // and memory requests cost nothing; a 16-byte LDS write costs 12 cycles of MFMA issue by itself and 35 when a read
      // follows one MFMA later, an 8-byte write 4 cycles wherever it stands, two memory operations behind the same MFMA
      // cost as much again (bench.py --probe issue).  So quads go to LDS in halves and no two operations share a slot:
      //   write a.lo, read 0, -, -, write a.hi, read 1, -, request a, write b.lo, read 2, -, -, write b.hi, read 3, -, request b
      // The step before the barrier has its LDS traffic in its first half, so that the wait before the barrier is short.
      // Behind the barrier every wave's part of the next slab is visible and nobody reads this stage any more: group 0 of
      // the slab after next goes there.
      auto slab = [&](auto stage, auto os, auto par_c, auto &&fill_a, auto &&fill_b) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        const std::integral_constant<int, PAR ^ 1> oth;
        // MFMAs of (xm | w set, x set, F half, I half); rd(b): fragment read b of the step; quads 2 g and 2 g + 1 of operand op,
        // staging parity p, to LDS stage st; fill: their successors' requests; early: LDS traffic in the first half
        auto step = [&](auto xm_c, auto ws_c, auto xs_c, auto fh_c, auto ih_c, auto &&rd, auto st, auto p_c, auto op_c, auto g_c, auto &&fill,
                        auto early_c) __attribute__((always_inline)) {
          constexpr int P = decltype(p_c)::value, OP = decltype(op_c)::value, G = decltype(g_c)::value;
          constexpr bool EARLY = decltype(early_c)::value != 0;
          auto wr = [&](auto q_c, auto h_c) __attribute__((always_inline)) {
            put_half(st, p_c, op_c, std::integral_constant<int, 2 * G + decltype(q_c)::value>{}, h_c);
          };
          auto rq = [&](auto q_c) __attribute__((always_inline)) {
            fill(p_c, op_c, std::integral_constant<int, 2 * G + decltype(q_c)::value>{});
          };
          mfma_step(xm_c, ws_c, xs_c, fh_c, ih_c, [&](auto s_c) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            if constexpr (!EARLY) {
              if constexpr (S == 0) wr(c0, c0);
              else if constexpr (S == 1) rd(c0, c0);
              else if constexpr (S == 2) rd(c0, c1);
              else if constexpr (S == 4) wr(c0, c1);
              else if constexpr (S == 5) rd(c1, c0);
              else if constexpr (S == 6) rd(c1, c1);
              else if constexpr (S == 7) rq(c0);
              else if constexpr (S == 8) wr(c1, c0);
              else if constexpr (S == 9) rd(c2, c0);
              else if constexpr (S == 10) rd(c2, c1);
              else if constexpr (S == 12) wr(c1, c1);
              else if constexpr (S == 13) rd(c3, c0);
              else if constexpr (S == 14) rd(c3, c1);
              else if constexpr (S == 15) rq(c1);
            } else {
              if constexpr (S == 0) wr(c0, c0);
              else if constexpr (S == 1) rd(c0, c0);
              else if constexpr (S == 2) wr(c0, c1);
              else if constexpr (S == 3) rd(c1, c0);
              else if constexpr (S == 4) wr(c1, c0);
              else if constexpr (S == 5) rd(c2, c0);
              else if constexpr (S == 6) wr(c1, c1);
              else if constexpr (S == 7) rd(c3, c0);
              else if constexpr (S == 9) rq(c0);
              else if constexpr (S == 11) rq(c1);
            }
          });
        };
        // 1: (F0,I0) of K half 0 from sets (0,0); x blocks 4..7 of K half 0 into set 1
        step(c1, c0, c0, c0, c0, [&](auto b_c, auto part_c) __attribute__((always_inline)) { if constexpr (decltype(part_c)::value == 0) read_x(stage, c0, c1, c1, b_c); }, os, par_c, c0, c1, fill_a, c0);
        // 2: (F0,I1) from (0,1); weight blocks 4..7 of K half 0 into set 1
        step(c1, c0, c1, c0, c1, [&](auto b_c, auto part_c) __attribute__((always_inline)) { read_w(stage, c0, c1, c1, b_c, part_c); }, os, par_c, c1, c1, fill_a, c0);
        // 3: (F1,I1) from (1,1); weight blocks 0..3 of K half 1 into set 0
        step(c0, c1, c1, c1, c1, [&](auto b_c, auto part_c) __attribute__((always_inline)) { read_w(stage, c1, c0, c0, b_c, part_c); }, os, par_c, c0, c2, fill_a, c0);
        // 4: (F1,I0) from (1,0); x blocks 0..3 of K half 1 into set 1
        step(c0, c1, c0, c1, c0, [&](auto b_c, auto part_c) __attribute__((always_inline)) { if constexpr (decltype(part_c)::value == 0) read_x(stage, c1, c1, c0, b_c); }, os, par_c, c1, c2, fill_a, c0);
        // 5: (F0,I0) of K half 1 from (0,1); x blocks 4..7 of K half 1 into set 0
        step(c1, c0, c1, c0, c0, [&](auto b_c, auto part_c) __attribute__((always_inline)) { if constexpr (decltype(part_c)::value == 0) read_x(stage, c1, c0, c1, b_c); }, os, par_c, c0, c3, fill_a, c0);
        // 6: (F0,I1) from (0,0); weight blocks 4..7 of K half 1 into set 1
        step(c1, c0, c0, c0, c1, [&](auto b_c, auto part_c) __attribute__((always_inline)) { read_w(stage, c1, c1, c1, b_c, part_c); }, os, par_c, c1, c3, fill_a,
             std::integral_constant<int, KN ? 0 : 1>{});   // ([E,K,N]: eight reads do not fit the first half)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#if !(MSCO_TILE4_ATTR & 32)
        t4_barrier();
#endif
        // 7: (F1,I1) from (1,0); next slab: weight blocks 0..3 of K half 0 into set 0; x group 0 of the slab after next
        step(c0, c1, c0, c1, c1, [&](auto b_c, auto part_c) __attribute__((always_inline)) { read_w(os, c0, c0, c0, b_c, part_c); }, stage, oth, c0, c0, fill_b, c0);
        // 8: (F1,I0) from (1,1); next slab: x blocks 0..3 of K half 0 into set 0; weight group 0 of the slab after next
        step(c0, c1, c1, c1, c0, [&](auto b_c, auto part_c) __attribute__((always_inline)) { if constexpr (decltype(part_c)::value == 0) read_x(os, c0, c0, c0, b_c); }, stage, oth, c1, c0, fill_b, c0);
      };
      // slab kt, its look-ahead anywhere (next tile, past K)
      auto slab_any = [&](int kt, auto par_c) __attribute__((always_inline)) {
        const int stage = kt & 1;
        slab(stage, stage ^ 1, par_c, [&](auto p_c, auto op_c, auto u_c) __attribute__((always_inline)) { load_one(kt + 3, p_c, op_c, u_c); },
             [&](auto p_c, auto op_c, auto u_c) __attribute__((always_inline)) { load_one(kt + 4, p_c, op_c, u_c); });
      };
      // slab kt in stage ST whose look-ahead stays inside the current tile and inside K; soff3 / soff4: K offsets of the
      // slabs three and four on
      auto slab_inside = [&](auto stage_c, auto par_c, unsigned soff3, unsigned soff4) __attribute__((always_inline)) {
        constexpr int ST = decltype(stage_c)::value;
        const std::integral_constant<int, ST ^ 1> os;
        // ([E,K,N]: one window per slab, made once per slab, and no offset)
        const __amdgpu_buffer_rsrc_t rw3 = KN ? w_rsrc_at(ww_c, soff3) : rw_c, rw4 = KN ? w_rsrc_at(ww_c, soff4) : rw_c;
        auto refill = [&](unsigned soff, __amdgpu_buffer_rsrc_t rw_s, auto p_c, auto op_c, auto u_c) __attribute__((always_inline)) {
          constexpr int P = decltype(p_c)::value, OP = decltype(op_c)::value, U = decltype(u_c)::value;
#if MSCO_TILE4_ATTR & 8
          v4i &q = stg[P][OP][U];   // (named first: operands of an asm statement do not capture)
          asm volatile("" : "+v"(q));
#else
          if constexpr (OP == 0) stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(rx_c, a_voff0 + U * rows32, soff, 0);
          else stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(rw_s, b_voff0 + U * b_step, PK ? soff * 16 : KN ? 0u : soff, 0);
#endif
        };
        slab(stage_c, os, par_c, [&](auto p_c, auto op_c, auto u_c) __attribute__((always_inline)) { refill(soff3, rw3, p_c, op_c, u_c); },
             [&](auto p_c, auto op_c, auto u_c) __attribute__((always_inline)) { refill(soff4, rw4, p_c, op_c, u_c); });
      };
      // slabs whose furthest request (group 0 of the slab five on) ends inside K run the compile-time body, two per round
      const int k_clean = max(0, ((p.k / T4_BK - 4) / 2) * 2);
      int kt = 0;
      {
        // (a zero the compiler cannot see through: a constant vector of zeros gets hoisted out of the tile loop into
        // registers the K loops do not have)
        int zero = 0;
        asm volatile("" : "+v"(zero));
#pragma unroll
        for (int f = 0; f < T4M_B; ++f)
#pragma unroll
          for (int i = 0; i < T4M_B; ++i) acc[f][i] = v4i{zero, zero, zero, zero};
      }
      for (; kt < k_clean; kt += 2) {
        const unsigned kb = (unsigned)kt * T4_BK;
        slab_inside(c0, c1, kb + 3 * T4_BK, kb + 4 * T4_BK);
        slab_inside(c1, c0, kb + 4 * T4_BK, kb + 5 * T4_BK);
      }
      // the last slabs of the tile (their look-ahead runs into the next tile or past K) multiply every block: what
      // lands in blocks without rows is never stored
      for (; kt < k_slabs; kt += 2) {
        slab_any(kt, c1);
        slab_any(kt + 1, c0);
      }
    }
    // ---- fused dequant epilogue ----------------------------------------------------------------------
    // acc[f][i][r] is output row 16 i + m16, column 32 (f / 2) + 8 g + 4 (f % 2) + r of the wave tile (m16 = lane % 16,
    // g = lane / 16).
    // The table was published by the barriers of the slabs since kt == 2.
#if MSCO_TILE4_ATTR & 1
    if (p.m == -12345)
#endif
    {
      int e_lane = lane;   // (laundered: otherwise the addresses below are loop invariant and have to survive the K loop)
      asm volatile("" : "+v"(e_lane));
      const int m16 = e_lane & 15, g4 = e_lane >> 4;
      const int n_base = cur.n0 + wave_n * T4_WT;
      const int m_base = cur.m0 + wave_m * T4_WT;
      const bool has_bias = p.bias != nullptr;
      unsigned *tb_scale = reinterpret_cast<unsigned *>(table) + wave_n * T4_WT + 8 * g4;
      const int *tb_bias = reinterpret_cast<const int *>(table + 1024) + wave_n * T4_WT + 8 * g4;
      const float *tb_pt = reinterpret_cast<const float *>(table + 2048) + wave_m * T4_WT + m16;
      if (p.scale_dtype == DT_BF16) {
        // the table holds raw 16-bit patterns: widen them in place (one entry per thread)
        unsigned *mine = reinterpret_cast<unsigned *>(table) + tid;
        *mine = *mine << 16;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        t4_barrier();
      }
      constexpr bool raw = MODE == 2;
      constexpr int esize = raw ? 4 : 2;
      const unsigned pitch = (unsigned)p.n * esize;
      const int rows_valid = max(0, min(T4_WT, rows_wave));
      // (assembled from scalars read off lane 0: a descriptor the compiler takes for lane-dependent is applied lane
      // group by lane group)
      const unsigned long long out_first =
          (unsigned long long)(reinterpret_cast<unsigned char *>(p.out) + ((long long)m_base * p.n + n_base) * esize);
      const unsigned out_lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)out_first);
      const unsigned out_hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(out_first >> 32));
      const __amdgpu_buffer_rsrc_t rs_out =
          t4_rsrc(reinterpret_cast<void *>(((unsigned long long)out_hi << 32) | out_lo),
                  __builtin_amdgcn_readfirstlane((int)min((long long)rows_valid * pitch, 0x7FFFFFFFll)));
      const unsigned v_lane = (unsigned)m16 * pitch + (unsigned)(8 * g4) * esize;   // row m16, column 8 g of block pair 0, x block 0
      const unsigned row16 = 16u * pitch;
      // this lane's columns: eight of every 32 (block pair j: columns 32 j + 8 g ..), four from each block of the pair
      uint4 sc[T4M_B];
      unsigned voff_p[T4M_B / 2], voff_q[T4M_B / 2];
#pragma unroll
      for (int j = 0; j < T4M_B / 2; ++j) {
        if constexpr (!raw) {
          sc[2 * j] = *reinterpret_cast<const uint4 *>(tb_scale + 32 * j);
          sc[2 * j + 1] = *reinterpret_cast<const uint4 *>(tb_scale + 32 * j + 4);
        }
        const int n_first = n_base + 32 * j + 8 * g4;
        voff_p[j] = (n_first < p.n ? v_lane : T4_OOB) + (unsigned)(32 * j * esize);
        voff_q[j] = (n_first + 4 < p.n ? v_lane : T4_OOB) + (unsigned)((32 * j + 4) * esize);   // (int32 output: second store)
      }
      // accumulators leave the accumulation file here and not earlier
      auto fetch = [&](auto f_c, auto i_c, int (&a4)[4]) __attribute__((always_inline)) {
        constexpr int F = decltype(f_c)::value, I = decltype(i_c)::value;
        v4i &blk = acc[F][I];   // (named first: operands of an asm statement do not capture)
#pragma unroll
        for (int j = 0; j < 4; ++j) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a4[j]) : "a"(blk[j]));
        if (has_bias) {
          const int4 bi = *reinterpret_cast<const int4 *>(tb_bias + 32 * (F / 2) + 4 * (F % 2));
          a4[0] += bi.x; a4[1] += bi.y; a4[2] += bi.z; a4[3] += bi.w;
        }
      };
      auto finish = [&](const int (&a4)[4], const uint4 &s4, float pt_i, unsigned &lo, unsigned &hi) __attribute__((always_inline)) {
        float v[4];
        v[0] = dequant(a4[0], __uint_as_float(s4.x), pt_i); v[1] = dequant(a4[1], __uint_as_float(s4.y), pt_i);
        v[2] = dequant(a4[2], __uint_as_float(s4.z), pt_i); v[3] = dequant(a4[3], __uint_as_float(s4.w), pt_i);
        if constexpr (ACT != 0) {
          // v * sigmoid(t) = v / (1 + 2^(-t log2 e)); t = c v (silu: c = 1, fast gelu: 1.702) or, for the tanh form of
          // gelu, t = v (c1 + c3 v^2) with c1 = 2 sqrt(2 / pi), c3 = 0.044715 c1
          const float slu_k = (p.act_type == ACT_FAST_GELU ? -1.702f : -1.0f) * 1.4426950408889634f;
          constexpr float gelu_k1 = -1.5957691216057308f * 1.4426950408889634f, gelu_k3 = gelu_k1 * 0.044715f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            asm volatile("" : "+v"(v[j]));
            if constexpr (ACT == 3) {
              v[j] = v[j] < 0.0f ? 0.0f : v[j];
            } else if constexpr (ACT == 2) {
              v[j] = v[j] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v[j] * slu_k));
            } else {
              v[j] = v[j] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v[j] * __builtin_fmaf(v[j] * v[j], gelu_k3, gelu_k1)));
            }
            asm volatile("" : "+v"(v[j]));
          }
        }
        if constexpr (MODE == 0) {
          lo = pack_bf16x2(v[0], v[1]);
          hi = pack_bf16x2(v[2], v[3]);
        } else {
          // the float32 product is rounded before the conversion (the golden's order); left visible, multiply and
          // conversion are merged into one mixed-precision instruction that rounds once
#pragma unroll
          for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(v[j]));
          lo = f32_to_f16_rne(v[0]) | ((unsigned)f32_to_f16_rne(v[1]) << 16);
          hi = f32_to_f16_rne(v[2]) | ((unsigned)f32_to_f16_rne(v[3]) << 16);
        }
      };
      // x block i (16 rows): the four block pairs one after the other, so that the two 64-byte halves of an output line
      // (int32: the four quarters) leave the CU back to back
      auto row_block = [&](auto i_c) __attribute__((always_inline)) {
        constexpr int I = decltype(i_c)::value;
        const float pt_i = tb_pt[16 * I];
        static_for<T4M_B / 2>([&](auto j_c) {
          constexpr int J = decltype(j_c)::value;
          int a4[4], b4[4];
          fetch(std::integral_constant<int, 2 * J>{}, i_c, a4);
          fetch(std::integral_constant<int, 2 * J + 1>{}, i_c, b4);
          const unsigned vp = voff_p[J] + (unsigned)I * row16, vq = voff_q[J] + (unsigned)I * row16;
          if constexpr (raw) {
#if MSCO_TILE4_ATTR & 4
            asm volatile("" ::"v"(a4[0]), "v"(a4[1]), "v"(a4[2]), "v"(a4[3]), "v"(vp));
            asm volatile("" ::"v"(b4[0]), "v"(b4[1]), "v"(b4[2]), "v"(b4[3]), "v"(vq));
#else
            __builtin_amdgcn_raw_buffer_store_b128(v4i{a4[0], a4[1], a4[2], a4[3]}, rs_out, vp, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(v4i{b4[0], b4[1], b4[2], b4[3]}, rs_out, vq, 0, 0);
#endif
          } else {
            unsigned r0, r1, r2, r3;
            finish(a4, sc[2 * J], pt_i, r0, r1);
            finish(b4, sc[2 * J + 1], pt_i, r2, r3);
            const v4i r{(int)r0, (int)r1, (int)r2, (int)r3};
#if MSCO_TILE4_ATTR & 4
            asm volatile("" ::"v"(r), "v"(vp));
#else
            __builtin_amdgcn_raw_buffer_store_b128(r, rs_out, vp, 0, 0);
#endif
          }
        });
      };
      if (bm_active == T4M_B) {
        static_for<T4M_B>([&](auto i_c) { row_block(i_c); });
      } else {
        static_for<T4M_B>([&](auto i_c) {
          if (decltype(i_c)::value < bm_active) row_block(i_c);
        });
      }
    }
    if (!nxt.valid) break;
    cur = nxt;
    rx_c = rx_n;
    rw_c = rw_n;
    ww_c = ww_n;
  }
}

template <int MODE, int WL, int ACT>
static hipError_t t4m_launch(const GmmParams &p, unsigned grid, hipStream_t stream) {
  auto kern = gmm_w8a8_tile4m_kernel<MODE, WL, ACT>;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, t4m_lds_bytes(WL));
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(T4_NW * 64), t4m_lds_bytes(WL), stream, p);
  return hipGetLastError();
}

hipError_t launch_tile4m_w8a8(const GmmParams &p, int layout, hipStream_t stream) {
  // layout 0 [E,N,K], 1 packed, 2 [E,K,N] (read in 16-column chunks); the operand stream runs up to four slabs ahead inside
  // one tile; the group table lives in LDS
  if (p.k < 4 * T4_BK || p.e > T4_MAX_E || layout < 0 || layout > 2 || (layout == 2 && p.n % 16 != 0)) return hipErrorInvalidValue;
  const long long n_tiles = (p.n + T4_BN - 1) / T4_BN;
  const long long m_tiles_ub = (p.m + T4_BM - 1) / T4_BM + p.e;   // every non-empty group adds at most one partial tile
  const long long total_ub = m_tiles_ub * n_tiles;
  long long grid = ((total_ub + kNumXcd - 1) / kNumXcd) * kNumXcd;
  if (grid > T4_MAX_WGS) grid = T4_MAX_WGS;
  if (grid <= 0) return hipSuccess;
  const int act = p.act_type == ACT_NONE ? 0 : p.act_type == ACT_RELU ? 3 : (p.act_type == ACT_SILU || p.act_type == ACT_FAST_GELU) ? 2 : 1;
  const unsigned g = (unsigned)grid;
#define MSCO_T4M_BY_ACT(MODE, WL)                                   \
  (act == 0   ? t4m_launch<MODE, WL, 0>(p, g, stream)               \
   : act == 1 ? t4m_launch<MODE, WL, 1>(p, g, stream)               \
   : act == 2 ? t4m_launch<MODE, WL, 2>(p, g, stream)               \
              : t4m_launch<MODE, WL, 3>(p, g, stream))
#define MSCO_T4M_BY_LAYOUT(MODE) (layout == 1 ? MSCO_T4M_BY_ACT(MODE, 1) : layout == 2 ? MSCO_T4M_BY_ACT(MODE, 2) : MSCO_T4M_BY_ACT(MODE, 0))
  switch (p.out_dtype) {
    case DT_BF16: return MSCO_T4M_BY_LAYOUT(0);
    case DT_F16: return MSCO_T4M_BY_LAYOUT(1);
    case DT_I32: return layout == 1 ? t4m_launch<2, 1, 0>(p, g, stream) : layout == 2 ? t4m_launch<2, 2, 0>(p, g, stream) : t4m_launch<2, 0, 0>(p, g, stream);
    default: return hipErrorInvalidValue;
  }
#undef MSCO_T4M_BY_LAYOUT
#undef MSCO_T4M_BY_ACT
}

}  // namespace msco
