// Grouped W8A8 GEMM, persistent register-heavy MFMA tile kernel for gfx950 on v_mfma_i32_32x32x32_i8: 256 x 256
// output tiles, four wavefronts (one per SIMD), 128 x 128 accumulators per wavefront; every weight layout.  The plan
// takes the 16 x 16 x 64 form of the same design (gmm_tile4m_w8a8.hip), which draws less power per multiply-add; this
// one runs only when it is forced (kernel_override 8), to be measured against.
//
// Why this shape.  A wavefront that owns 128 x 128 outputs reads 8 operand fragments from LDS for every
// 16 MFMAs (a 128 x 64 wave tile reads 12), so LDS traffic per multiply-add drops by a third.  The
// 256 int32 accumulators of a lane fill the accumulation register file; operand fragments (two sets)
// and the operand staging registers live in the architectural file.  With one wavefront per SIMD
// nothing else covers a stall, hence:
//
//   * K slab = 128 bytes per row.  Every x row / weight column is requested one full 128-byte line
//     at a time (measured: 64-byte requests cap the operand stream at ~20 B/clk/CU whatever the
//     depth, full lines reach 28 B/clk/CU with two slabs in flight).
//   * Two slabs in flight.  Operands are loaded into staging registers two slabs ahead of their
//     multiply, written to the LDS stage that the last barrier retired, and the registers are refilled
//     right behind the write.  One load, one LDS write and two fragment reads are issued per four
//     MFMAs: a burst of either would stall the in-order issue of the only wave on the SIMD.
//   * One workgroup barrier per slab (2048 MFMA cycles).  Two LDS stages of 64 KiB (x stages 0 and 1, then weight
//     stages 0 and 1, so that stage and block offsets fit the offset field of the LDS instructions).
//   * A wave that is alone on its SIMD issues one instruction about every six cycles, whatever its kind (measured
//     with chains of independent VALU, scalar and no-op instructions), so every address computation, scalar select
//     and wait between the MFMAs costs as much issue time as a memory instruction.  The K loop therefore has two
//     bodies: a steady-state one for slabs whose look-ahead stays inside the tile and inside K (stage, K quarter
//     and staging parity are compile-time constants, every LDS access is a base register plus an immediate, loads
//     need no tail masks: 346 instructions per 128 MFMAs) and a general one for the last slabs, whose loads run into
//     the next tile or past K (546 instructions).
//   * LDS rows are 128 B; 16-byte chunk c of row r sits at chunk position c ^ ((r >> 1) & 7), which
//     makes both the staging writes and the 16-lane fragment reads bank-conflict free.
//   * Persistent workgroups.  A workgroup walks its share of the tiles and the operand stream never
//     drains: the first slabs of the next tile are requested during the last slabs of the current
//     one, so a tile costs its MFMAs plus the epilogue, not a pipeline refill.
//   * Weights are the MFMA's first operand and x the second, so a lane owns output row m and runs of 8
//     consecutive columns; the fused dequant epilogue is staged through a small LDS region next to the
//     ring (32 rows at a time) and stores full 128-byte row segments.
//   * The epilogue is issue bound as well (about 1150 VALU instructions per wave): its stores go through a buffer
//     descriptor over the rows that exist (no predicates, one address add per store) and the LDS round trip of one
//     32-row block hides under the arithmetic of the next.
//   * Partial m-tiles (the last tile of a group) are multiplied in full (a loop variant or branches that skip the
//     32-row blocks without rows make the register allocator shuffle or spill the 256 accumulators); their epilogue
//     only touches the blocks that hold rows.
#include "gmm_common.h"
#include "gmm_kernels.h"
#include "gmm_tile4_common.h"

#include <type_traits>

namespace msco {
namespace {

constexpr int T4_F = 4;                          // 32 x 32 MFMA blocks per wave tile edge
// Attribution builds, never the shipped library: MSCO_TILE4_ATTR is a bit mask that takes one part of the kernel out
// so that timing the rest says what that part costs (results are then wrong on purpose).  1: the epilogue sits behind
// a branch that no launch takes (its code and registers stay); 2: every MFMA becomes an empty statement that keeps
// both operand fragments alive (loads, LDS traffic and barriers unchanged); 4: the epilogue computes everything and
// its output stores become empty statements; 8: the K loop requests no operands from memory (the staging registers keep
// what the prologue brought); 16: staging registers are not written to LDS (loads are still waited for); 32: the K
// loop's workgroup barriers are left out; 64: the K loop reads no operand fragments from LDS (the MFMAs multiply what
// the registers hold).
constexpr int T4_EP_PITCH = 144;                 // epilogue staging: 128 payload bytes per row
constexpr int T4_EP_OFF = T4_PARAM_OFF + 2 * T4_PARAM_BYTES;
constexpr int T4_EP_WAVE = 32 * T4_EP_PITCH;     // one wave stages 32 rows at a time
constexpr int T4_META_OFF = T4_EP_OFF + T4_NW * T4_EP_WAVE;   // per group: row end, tiles up to and including it
constexpr int T4_LDS_BYTES = T4_META_OFF + 2 * T4_MAX_E * 4;
static_assert(T4_LDS_BYTES <= 160 * 1024, "LDS of one CU");

__device__ __forceinline__ int t4_col_of_q(int q) {
  const int g = q >> 3, hh = (q >> 2) & 1, t = q & 3;
  return 16 * (g >> 1) + 8 * hh + 4 * (g & 1) + t;
}


}  // namespace

// MODE: output type, 0 bf16, 1 f16, 2 int32 (raw accumulators plus bias).
// PK: weights in the packed layout (1 KiB blocks of 16 columns x 64 K bytes, byte 16 l + i of block (a, b) =
// w[k = 64 b + 16 (l / 16) + i][n = 16 a + l % 16]) instead of [E,N,K].  A slab of a tile is then 16 column groups x 2
// blocks; staging quad (u, wave) is block 4 u + wave = (column group 2 u + wave / 2, K block wave % 2) and goes to LDS as
// it is, so only the global offsets and the weight fragment addresses differ: MFMA row r of a 32-row block is column
// t4_col_of_q(r), K quarter q is K block q / 2, 16-byte chunks 2 (q % 2) + hh.
// ACT: an activation (p.act_type) follows the dequantisation; a template parameter so that the plain epilogue stays as it
// is (0).  The epilogue is bound by instruction issue, so the common forms get code of their own: 3 relu (one
// instruction per value), 2 v * sigmoid(c v) with a uniform c (silu, fast gelu: five instructions, two of them
// transcendental), 1 the tanh form of gelu (three more for its cubic).
//
// WL: weight layout, 0 [E,N,K], 1 packed, 2 [E,K,N] (N a multiple of 16).  [E,K,N] rows are N-contiguous and an MFMA
// operand wants 16 K-contiguous bytes per lane; the LDS transpose read of gfx950 (ds_read_b64_tr_b8) does that turn on
// the way out of LDS.  Of a block of 16 lanes, lane i names 8 bytes M[i][0..7]; lane j receives byte b = M[2 b + j / 8][j % 8].
// With lanes 2 b and 2 b + 1 pointing at the two 8-byte halves of one 16-column chunk of K row b, lane j gets K rows
// 0 .. 7 of the column at byte j of that chunk, and two such reads (8 K rows apart) make the 16 bytes of the operand in
// natural K order.  So a slab goes to LDS as it lies in memory -- K rows of 256 columns, one staging quad = 4 K rows,
// lane L row L / 16, chunk slot L % 16 -- with two twists: slot s of row r holds chunk s ^ ((r % 8) << 1), so that the
// eight rows of one transpose read (and both 16-lane blocks of a half wave) fall into different banks, and the middle
// two dwords of every chunk are swapped on the way in, so that byte j of a chunk is column t4_col_of_q(j): the
// epilogue's ownership of 8-column runs stays as it is.
template <int MODE, int WL, int ACT>
__global__ void __launch_bounds__(T4_NW * 64, 1) gmm_w8a8_tile4_nk_kernel(const GmmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool PK = WL == 1, KN = WL == 2;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int l32 = lane & 31, hh = lane >> 5;

  // ---- this workgroup's share of the tiles -----------------------------------------------------------
  // Tiles are numbered so that neighbours share operands; every XCD takes a contiguous range and its
  // workgroups walk it with a stride, so the workgroups of an XCD work side by side on neighbours.
  const int n_tiles = (p.n + T4_BN - 1) / T4_BN;
  int *meta_end = reinterpret_cast<int *>(smem + T4_META_OFF);
  int *meta_upto = meta_end + T4_MAX_E;
  int total = 0;
  for (int g0 = 0, carry = 0; g0 < p.e; g0 += 64) {
    int s0, e0;
    group_rows_chunk(p, g0, lane, carry, s0, e0);
    // (groups outside (rows_lo, rows_hi] have no tiles here: a second launch of the small tile kernel takes them)
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
  // As many workgroups as make every round of tiles full: 344 tiles take two rounds either way, and on 176 workgroups
  // instead of 256 the CUs that work share the whole power budget (K = 4096, N = 11008: M = 2048 100.6 -> 94.3 us; M = 1536,
  // 258 tiles on 136 workgroups, 97.9 -> 85.7 us).  The others leave at once.
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
  // (the window ends with the group: the rows of a partial m-tile that belong to the next group read as zeros, cost no
  // memory traffic, and multiplying zeros costs the matrix pipe far less power than multiplying somebody else's rows)
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

  // ---- global -> staging registers -------------------------------------------------------------------
  // One quad = 1 KiB per wave = 8 rows x 128 B; lane L serves row L / 8, chunk position L % 8, so it
  // fetches logical chunk (L % 8) ^ swizzle(row).  The row of quad u is 32 u + 8 wave + d_row, so neither
  // the swizzle ((row >> 1) & 7) nor the MFMA row permutation (row & 31) depends on u.  Everything that
  // can run past a tensor is in the per-lane offset (the only part the buffer unit range-checks).
  // These lane constants are worked out again at the top of every tile from a lane id the compiler cannot see
  // through: kept across the epilogue they would cost it registers, and a spill there stalls the operand stream.
  const unsigned rows32 = 32u * (unsigned)p.k;
  const unsigned b_step = PK ? 2u * (unsigned)k_blocks * 1024u : KN ? 16u * (unsigned)p.n : rows32;   // staging quad u -> u + 1: two column groups / 32 rows / 16 K rows
  int d_chunk;
  unsigned a_voff0, b_voff0;
  // ---- fragment addressing ---------------------------------------------------------------------------
  // lane (l32, hh) reads row l32 of a 32-row block, logical chunk 2 q + hh of K quarter q.  The row
  // swizzle only depends on l32, and the chunk positions of the four quarters differ by an XOR with
  // q << 5 in the byte address.  LDS writes of the staging quads go to st_x / st_w.
  // Every LDS and buffer instruction of the steady-state K loop takes one of these registers and an immediate
  // offset: a wave that is alone on its SIMD issues one instruction about every six cycles whatever its kind, so
  // address arithmetic and scalar bookkeeping between the MFMAs cost as much issue time as the memory instructions.
  unsigned x_lane, w_lane, st_x, st_w;
  auto lane_constants = [&]() {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int q32 = ln & 31, h = ln >> 5;
    const int d_row0 = 8 * wave + (ln >> 3);
    d_chunk = (ln & 7) ^ ((d_row0 >> 1) & 7);
    a_voff0 = (unsigned)d_row0 * (unsigned)p.k + d_chunk * 16;
    const int w_krow = 4 * wave + (ln >> 4);   // [E,K,N]: K row of staging quad 0 that this lane carries
    b_voff0 = PK   ? (unsigned)(((wave >> 1) * k_blocks + (wave & 1)) * 1024 + ln * 16)
              : KN ? (unsigned)w_krow * (unsigned)p.n + (unsigned)(((ln & 15) ^ ((w_krow & 7) << 1)) * 16)
                   : (unsigned)t4_col_of_q(d_row0) * (unsigned)p.k + d_chunk * 16;   // LDS row rho feeds MFMA row rho % 32
    const int swz = (q32 >> 1) & 7;
    x_lane = (unsigned)((wave_m * T4_WT + q32) * T4_BK + ((h ^ swz) << 4));
    // [E,K,N]: address lane i = ln % 16 of its block of 16 points at K row i / 2 (of the 16 that half h of the wave
    // multiplies), half i % 2 of the chunk of this block's 16 columns; fragment f is an XOR with f << 5 away
    w_lane = PK   ? (unsigned)(T4_W_BASE + wave_n * 16384 + (q32 >> 4) * 2048 + h * 256 + (t4_col_of_q(q32) & 15) * 16)
             : KN ? (unsigned)(T4_W_BASE + (h * 16 + ((ln & 15) >> 1)) * 256 +
                               (((wave_n * 8 + ((ln >> 4) & 1)) ^ (((ln & 15) >> 1) << 1)) * 16) + (ln & 1) * 8)
                  : (unsigned)(T4_W_BASE + (wave_n * T4_WT + q32) * T4_BK + ((h ^ swz) << 4));
    st_x = (unsigned)(wave * 1024 + ln * 16);
    st_w = st_x + T4_W_BASE;
    asm volatile("" : "+v"(st_w));
  };
  lane_constants();
  unsigned char *ep_stage = smem + T4_EP_OFF + wave * T4_EP_WAVE;

  const std::integral_constant<int, 0> c0;
  const std::integral_constant<int, 1> c1;
  const std::integral_constant<int, 2> c2;
  const std::integral_constant<int, 3> c3;

  v16i acc[T4_F][T4_F];   // [f: weight block][i: x block]
  v4i stg[2][2][T4_LD];   // staging quads: [slab parity][operand: 0 x, 1 w][u]
  v4i wf[2][T4_F], xf[2][T4_F];

  T4Tile nxt = cur;        // tile that follows `cur` in this workgroup's walk (loads run ahead into it)
  __amdgpu_buffer_rsrc_t rx_c = x_rsrc(cur), rw_c = w_rsrc(cur), rx_n = rx_c, rw_n = rw_c;
  T4Window ww_c = w_window(cur), ww_n = ww_c;   // ([E,K,N] only)

  // slab s of the current tile, or slab s - k_slabs of the next one
  auto load_one = [&](int s, auto par_c, auto op_c, auto u_c) {
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
      // K block 2 slab + wave % 2 of column groups 2 U + wave / 2; blocks past K do not exist (the last one is zero padded)
      const unsigned kb = 2u * (unsigned)(ahead ? s - k_slabs : s) + (unsigned)(wave & 1);
      const unsigned kill_w = ((ahead && !nxt.valid) || kb >= (unsigned)k_blocks) ? T4_OOB : 0u;
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(ahead ? rw_n : rw_c, (b_voff0 + U * b_step) | kill_w, kbase * 16, 0);
    } else {
      stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(ahead ? rw_n : rw_c, (b_voff0 + U * b_step) | kill, kbase, 0);
    }
  };
  // a staging quad on its way to LDS ([E,K,N] weights: the middle dwords of the 16-column chunk change places)
  auto put_quad = [&](unsigned addr, v4i v, auto op_c) {
    if constexpr (KN && decltype(op_c)::value == 1) {
      int y = v.y, z = v.z;
      asm volatile("v_swap_b32 %0, %1" : "+v"(y), "+v"(z));
      v.y = y;
      v.z = z;
    }
#if MSCO_TILE4_ATTR & 16
    asm volatile("" ::"v"(v), "v"(addr));
#else
    *reinterpret_cast<v4i *>(smem + addr) = v;
#endif
  };
  // write quad (op, u) of slab s to its LDS stage and refill it with slab s + 2
  auto cycle_one = [&](int s, auto par_c, auto op_c, auto u_c) {
    constexpr int P = decltype(par_c)::value, OP = decltype(op_c)::value, U = decltype(u_c)::value;
    put_quad((OP == 0 ? st_x : st_w) + (s & 1) * T4_OP_STAGE + U * 4096, stg[P][OP][U], op_c);
    load_one(s + 2, par_c, op_c, u_c);
  };
  // the same for a slab whose successor lies inside the current tile and inside K: WS = stage written, soff = scalar
  // offset of slab s + 2 (bytes of K for x, soff_w for the weights: 16 times that in the packed layout; [E,K,N]: the slab's
  // own window rw_s and no offset)
  auto cycle_clean = [&](auto ws_c, unsigned soff, __amdgpu_buffer_rsrc_t rw_s, unsigned soff_w, auto par_c, auto op_c, auto u_c) {
    constexpr int WS = decltype(ws_c)::value, P = decltype(par_c)::value, OP = decltype(op_c)::value, U = decltype(u_c)::value;
    put_quad((OP == 0 ? st_x : st_w) + WS * T4_OP_STAGE + U * 4096, stg[P][OP][U], op_c);
#if MSCO_TILE4_ATTR & 8
    asm volatile("" : "+v"(stg[P][OP][U]));
#else
    if constexpr (OP == 0) stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(rx_c, a_voff0 + U * rows32, soff, 0);
    else stg[P][OP][U] = __builtin_amdgcn_raw_buffer_load_b128(rw_s, b_voff0 + U * b_step, soff_w, 0);
#endif
  };
  // [E,K,N] weight fragment: two transpose reads, K rows 0 .. 7 and 8 .. 15 of the lane's column
  auto read_tr = [&](unsigned addr) -> v4i {
    typedef int v2i_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) v2i_t *lds_v2i;
    const v2i_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(smem + addr));
    const v2i_t hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(smem + addr + 2048));
    return v4i{lo.x, lo.y, hi.x, hi.y};
  };
  // (qx = q << 5 arrives in a scalar the compiler cannot see through: hoisting the XORs out of the K
  // loop would park eight more addresses in registers that the loop does not have)
  auto read_w = [&](int stage, unsigned qx, auto set_c, auto f_c) {
    constexpr int S = decltype(set_c)::value, F = decltype(f_c)::value;
#if MSCO_TILE4_ATTR & 64
    asm volatile("" : "+v"(wf[S][F]));
    return;
#endif
    if constexpr (PK) {
      // qx = q << 5: K block q / 2 is 1024 bytes on, chunk pair q % 2 another 512
      wf[S][F] = *reinterpret_cast<const v4i *>(smem + stage * T4_OP_STAGE + (w_lane + (qx >> 6) * 1024 + ((qx >> 5) & 1) * 512) + F * 4096);
    } else if constexpr (KN) {
      wf[S][F] = read_tr(stage * T4_OP_STAGE + ((w_lane ^ (unsigned)(F << 5)) + (qx << 8)));   // K quarter q: 32 rows of 256 bytes on
    } else {
      wf[S][F] = *reinterpret_cast<const v4i *>(smem + stage * T4_OP_STAGE + (w_lane ^ qx) + F * 32 * T4_BK);
    }
  };
  auto read_x = [&](int stage, unsigned qx, auto set_c, auto i_c) {
    constexpr int S = decltype(set_c)::value, I = decltype(i_c)::value;
#if MSCO_TILE4_ATTR & 64
    asm volatile("" : "+v"(xf[S][I]));
    return;
#endif
    xf[S][I] = *reinterpret_cast<const v4i *>(smem + stage * T4_OP_STAGE + (x_lane ^ qx) + I * 32 * T4_BK);
  };
  // fragment reads with everything but the registers above known at compile time
  auto read_w_clean = [&](auto stage_c, auto q_c, auto set_c, auto f_c) {
    constexpr int ST = decltype(stage_c)::value, Q = decltype(q_c)::value, S = decltype(set_c)::value, F = decltype(f_c)::value;
#if MSCO_TILE4_ATTR & 64
    asm volatile("" : "+v"(wf[S][F]));
    return;
#endif
    if constexpr (PK) wf[S][F] = *reinterpret_cast<const v4i *>(smem + (w_lane + ST * T4_OP_STAGE + (Q >> 1) * 1024 + (Q & 1) * 512 + F * 4096));
    else if constexpr (KN) wf[S][F] = read_tr((w_lane ^ (unsigned)(F << 5)) + ST * T4_OP_STAGE + Q * 8192);
    else wf[S][F] = *reinterpret_cast<const v4i *>(smem + ((w_lane ^ (unsigned)(Q << 5)) + ST * T4_OP_STAGE + F * 4096));
  };
  auto read_x_clean = [&](auto stage_c, auto q_c, auto set_c, auto i_c) {
    constexpr int ST = decltype(stage_c)::value, Q = decltype(q_c)::value, S = decltype(set_c)::value, I = decltype(i_c)::value;
#if MSCO_TILE4_ATTR & 64
    asm volatile("" : "+v"(xf[S][I]));
    return;
#endif
    xf[S][I] = *reinterpret_cast<const v4i *>(smem + ((x_lane ^ (unsigned)(Q << 5)) + ST * T4_OP_STAGE + I * 4096));
  };
  auto opaque_q = [](int q) {
    unsigned qx = (unsigned)q << 5;
    asm volatile("" : "+s"(qx));
    return qx;
  };

  // ---- stream prologue (once per workgroup): slabs 0 and 1 requested; slab 0 and group 0 of slab 1
  // written to LDS and refilled; quarter-0 fragments of slab 0 read -------------------------------------
  {
    auto for_u = [&](auto fn) {
      fn(std::integral_constant<int, 0>{}); fn(std::integral_constant<int, 1>{}); fn(std::integral_constant<int, 2>{});
      fn(std::integral_constant<int, 3>{}); fn(std::integral_constant<int, 4>{}); fn(std::integral_constant<int, 5>{});
      fn(std::integral_constant<int, 6>{}); fn(std::integral_constant<int, 7>{});
    };
    // (nxt == cur here, and slabs 0 .. 3 are below k_slabs >= 4, so every request goes to `cur`)
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

    // Epilogue operands of this tile (scale and bias of its 256 columns, per-token scale of its 256
    // rows) go straight from memory into this tile's LDS table (two tables, alternating per tile: the
    // other one may still be read by a wave that is finishing the previous epilogue).  The K-loop
    // barriers publish them long before the epilogue reads them.
    unsigned char *table = smem + T4_PARAM_OFF + (ti & 1) * T4_PARAM_BYTES;
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

    // rows of this tile that exist, and the 32-row blocks of this wave that hold any of them
    const int rows_here = min(T4_BM, cur.g_end - cur.m0);
    const int rows_wave = rows_here - wave_m * T4_WT;
    const int fm_active = max(0, min(T4_F, (rows_wave + 31) / 32));

    // The accumulators start at zero.  The matrix pipe clears them itself, a block of sixteen registers per instruction
    // (zero operand, C = 0): 256 single register writes cost a wave that is alone on its SIMD three times as long.
    // (the zero operand is made here, behind an empty asm: a constant vector of zeros would be hoisted out of the tile
    // loop into registers the K loops do not have)
    {
      int zero = 0;
      asm volatile("" : "+v"(zero));
      const v4i z4 = {zero, zero, zero, zero};
      // (the compiler does not know what the statements are, so the wait states between the zero's last write and the
      // first read of it as a matrix operand, and between the last read and the register's next write, are written out;
      // an accumulator block is first added to sixteen MFMAs after it was cleared)
      asm volatile("s_nop 4" ::"v"(z4));
#pragma unroll
      for (int f = 0; f < T4_F; ++f)
#pragma unroll
        for (int i = 0; i < T4_F; ++i)
          asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %1, 0" : "=a"(acc[f][i]) : "v"(z4));
      asm volatile("s_nop 4" ::"v"(z4));
    }
    // quarter-0 fragments of slab 0 (read here rather than behind the previous tile's last slab, so that
    // the epilogue does not have to keep them alive)
    read_w(0, 0, c0, c0); read_w(0, 0, c0, c1); read_w(0, 0, c0, c2); read_w(0, 0, c0, c3);
    read_x(0, 0, c0, c0); read_x(0, 0, c0, c1); read_x(0, 0, c0, c2); read_x(0, 0, c0, c3);

    {
      // The 16 MFMAs of fragment set S; the scheduling groups pin one memory operation of the caller behind each
      // of the first MFMAs.
      auto mfma_quarter = [&](auto set_c) {
        constexpr int S = decltype(set_c)::value;
#pragma unroll
        for (int f = 0; f < T4_F; ++f)
#pragma unroll
          for (int i = 0; i < T4_F; ++i)
#if MSCO_TILE4_ATTR & 2
            asm volatile("" ::"v"(wf[S][f]), "v"(xf[S][i]));
#else
            acc[f][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[S][f], xf[S][i], acc[f][i], 0, 0, 0);
#endif
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);          // MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, KN ? 2 : 1, 0);   // DS read (a transposed weight fragment is two)
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // DS write
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // VMEM read
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // One K quarter: the MFMAs of fragment set CUR; meanwhile the fragments of (rstage, rq) are read
      // into set NXT and staging group G (x and w quads 2 G, 2 G + 1) of slab ss goes to LDS and is
      // refilled.  LDS operations keep their source order; the scheduling groups pin one memory
      // operation behind each of the first MFMAs.
      auto quarter = [&](auto cur_c, auto nxt_c, int rstage, int rq_index, int ss, auto par_c, auto g_c) {
        constexpr int G = decltype(g_c)::value;
        const unsigned rq = opaque_q(rq_index);
        const std::integral_constant<int, 2 * G> ua;
        const std::integral_constant<int, 2 * G + 1> ub;
        read_w(rstage, rq, nxt_c, c0); read_x(rstage, rq, nxt_c, c0);
        cycle_one(ss, par_c, c0, ua);
        read_x(rstage, rq, nxt_c, c1); read_x(rstage, rq, nxt_c, c2);
        cycle_one(ss, par_c, c0, ub);
        read_x(rstage, rq, nxt_c, c3); read_w(rstage, rq, nxt_c, c1);
        cycle_one(ss, par_c, c1, ua);
        read_w(rstage, rq, nxt_c, c2); read_w(rstage, rq, nxt_c, c3);
        cycle_one(ss, par_c, c1, ub);
        mfma_quarter(cur_c);
      };
      // One K slab kt (LDS stage kt & 1).  On entry the quarter-0 fragments are in fragment set 0 and
      // group 0 of slab kt+1 is in LDS; PAR is the staging parity of slab kt+1.
      auto period = [&](int kt, auto par_c) {
        constexpr int PAR = decltype(par_c)::value;
        const std::integral_constant<int, PAR ^ 1> other;
        const int stage = kt & 1;
        quarter(c0, c1, stage, 1, kt + 1, par_c, c1);
        quarter(c1, c0, stage, 2, kt + 1, par_c, c2);
        quarter(c0, c1, stage, 3, kt + 1, par_c, c3);
        // slab kt+1 is in LDS (this wave's part) and the quarter-3 fragments are in registers: after the
        // barrier every wave's part is visible and nobody reads this stage any more
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#if !(MSCO_TILE4_ATTR & 32)
        t4_barrier();
#endif
        quarter(c1, c0, stage ^ 1, 0, kt + 2, other, c0);
      };
      // The same with stage, quarter and parity known at compile time, for slabs whose look-ahead stays inside the
      // current tile and inside K (loads need neither the next tile's descriptors nor a tail mask).
      auto quarter_clean = [&](auto cur_c, auto nxt_c, auto rstage_c, auto rq_c, auto ws_c, unsigned soff, __amdgpu_buffer_rsrc_t rw_s, auto par_c, auto g_c) {
        constexpr int G = decltype(g_c)::value;
        const std::integral_constant<int, 2 * G> ua;
        const std::integral_constant<int, 2 * G + 1> ub;
        const unsigned soff_w = PK ? soff * 16 : KN ? 0u : soff;
        read_w_clean(rstage_c, rq_c, nxt_c, c0); read_x_clean(rstage_c, rq_c, nxt_c, c0);
        cycle_clean(ws_c, soff, rw_s, soff_w, par_c, c0, ua);
        read_x_clean(rstage_c, rq_c, nxt_c, c1); read_x_clean(rstage_c, rq_c, nxt_c, c2);
        cycle_clean(ws_c, soff, rw_s, soff_w, par_c, c0, ub);
        read_x_clean(rstage_c, rq_c, nxt_c, c3); read_w_clean(rstage_c, rq_c, nxt_c, c1);
        cycle_clean(ws_c, soff, rw_s, soff_w, par_c, c1, ua);
        read_w_clean(rstage_c, rq_c, nxt_c, c2); read_w_clean(rstage_c, rq_c, nxt_c, c3);
        cycle_clean(ws_c, soff, rw_s, soff_w, par_c, c1, ub);
        mfma_quarter(cur_c);
      };
      // slab kt in stage ST; soff3 / soff4: K offsets of slabs kt + 3 and kt + 4
      auto period_clean = [&](auto stage_c, auto par_c, unsigned soff3, unsigned soff4) {
        constexpr int ST = decltype(stage_c)::value, PAR = decltype(par_c)::value;
        const std::integral_constant<int, ST ^ 1> other_stage;
        const std::integral_constant<int, PAR ^ 1> other;
        // ([E,K,N]: one window per slab, made once per slab)
        const __amdgpu_buffer_rsrc_t rw3 = KN ? w_rsrc_at(ww_c, soff3) : rw_c, rw4 = KN ? w_rsrc_at(ww_c, soff4) : rw_c;
        quarter_clean(c0, c1, stage_c, c1, other_stage, soff3, rw3, par_c, c1);
        quarter_clean(c1, c0, stage_c, c2, other_stage, soff3, rw3, par_c, c2);
        quarter_clean(c0, c1, stage_c, c3, other_stage, soff3, rw3, par_c, c3);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#if !(MSCO_TILE4_ATTR & 32)
        t4_barrier();
#endif
        quarter_clean(c1, c0, other_stage, c0, stage_c, soff4, rw4, other, c0);
      };
      // iterations whose furthest request (group 0 of slab kt + 5) ends inside K
      const int k_clean = max(0, ((p.k / T4_BK - 4) / 2) * 2);
      int kt = 0;
      for (; kt < k_clean; kt += 2) {
        const unsigned kb = (unsigned)kt * T4_BK;
        period_clean(c0, c1, kb + 3 * T4_BK, kb + 4 * T4_BK);
        period_clean(c1, c0, kb + 4 * T4_BK, kb + 5 * T4_BK);
      }
      // the last slabs of the tile (their look-ahead runs into the next tile or past K) multiply every block: what
      // lands in blocks without rows is never stored
      for (; kt < k_slabs; kt += 2) {
        period(kt, c1);
        period(kt + 1, c0);
      }
    }
    // ---- fused dequant epilogue ----------------------------------------------------------------------
    // acc[f][i][r] is output row 32 i + l32, column 32 f + 16 (r / 8) + 8 hh + (r % 8) of the wave tile.
    // Per 32-row block and 128-byte column piece: dequantise, park in this wave's LDS region (rows of
    // 128 payload bytes at a 144-byte pitch), read back with lanes along columns, store full 128-byte
    // row segments.  The operand ring is live (it already holds the next tile), so only the small
    // region behind it is used.  The table was published by the barriers of the slabs since kt == 2.
#if MSCO_TILE4_ATTR & 1
    if (p.m == -12345)
#endif
    {
      // (lane-derived values are laundered through an empty asm: otherwise every LDS address below is
      // loop invariant, gets computed before the tile loop and has to survive the K loop in a register
      // the K loop does not have)
      int e_l32 = l32, e_hh = hh, e_lane = lane;
      asm volatile("" : "+v"(e_l32), "+v"(e_hh), "+v"(e_lane));
      const int n_base = cur.n0 + wave_n * T4_WT;
      const int m_base = cur.m0 + wave_m * T4_WT;
      const bool has_bias = p.bias != nullptr;
      unsigned *tb_scale = reinterpret_cast<unsigned *>(table) + wave_n * T4_WT;
      const int *tb_bias = reinterpret_cast<const int *>(table + 1024) + wave_n * T4_WT;
      const float *tb_pt = reinterpret_cast<const float *>(table + 2048) + wave_m * T4_WT;
      if (p.scale_dtype == DT_BF16) {
        // the table holds raw 16-bit patterns: widen them in place (one entry per thread)
        unsigned *mine = reinterpret_cast<unsigned *>(table) + tid;
        *mine = *mine << 16;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        t4_barrier();
      }
      // The wave tile leaves in units of one column piece (16-bit outputs: a 64-column half; int32: a 32-column
      // block) x one 32-row block.  A unit is dequantised into four 16-byte vectors per lane, parked in the wave's
      // staging rows and read back with lanes along columns, so that a store covers full 128-byte row segments.
      // The units are software pipelined: the read-back of unit u - 1 is issued before the arithmetic of unit u and
      // stored behind it, so the LDS round trip hides under the arithmetic (a wave's LDS operations execute in
      // order: the staging writes of unit u queue behind that read-back).  Rows past the end of the group fall
      // outside the store descriptor, columns past N are killed in the lane offset: stores need no predicates.
      constexpr bool raw = MODE == 2;
      constexpr int esize = raw ? 4 : 2;
      constexpr int NF = raw ? 1 : 2;                                   // 32-column MFMA blocks in a piece
      constexpr int PIECES = raw ? 4 : 2;
      constexpr int UNITS = PIECES * T4_F;
      const unsigned pitch = (unsigned)p.n * esize;
      const int rows_valid = max(0, min(T4_WT, rows_wave));
      // (assembled from scalars read off lane 0: a descriptor the compiler takes for lane-dependent is applied
      // lane group by lane group)
      const unsigned long long out_first =
          (unsigned long long)(reinterpret_cast<unsigned char *>(p.out) + ((long long)m_base * p.n + n_base) * esize);
      const unsigned out_lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)out_first);
      const unsigned out_hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(out_first >> 32));
      const __amdgpu_buffer_rsrc_t rs_out =
          t4_rsrc(reinterpret_cast<void *>(((unsigned long long)out_hi << 32) | out_lo),
                  __builtin_amdgcn_readfirstlane((int)min((long long)rows_valid * pitch, 0x7FFFFFFFll)));
      const int piece = e_lane & 7;
      const unsigned v_row = (unsigned)(e_lane >> 3) * pitch + piece * 16;
      unsigned char *dst = ep_stage + e_l32 * T4_EP_PITCH + 16 * e_hh * (raw ? 2 : 1);
      const unsigned char *src = ep_stage + (e_lane >> 3) * T4_EP_PITCH + piece * 16;
      unsigned sraw[NF][2][8];
      uint4 q[4], rb[4];
      auto read_back = [&]() {
#pragma unroll
        for (int t = 0; t < 4; ++t) rb[t] = *reinterpret_cast<const uint4 *>(src + 8 * t * T4_EP_PITCH);
      };
      auto store_unit = [&](auto u_c) {
        constexpr int U = decltype(u_c)::value, PIECE = U / T4_F, I = U % T4_F;
        const int n_first = n_base + PIECE * (raw ? 32 : 64) + (raw ? 4 : 8) * piece;
        const unsigned v0 = (n_first < p.n ? v_row : T4_OOB) + PIECE * 128;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#if MSCO_TILE4_ATTR & 4
          {
            const v4i val = __builtin_bit_cast(v4i, rb[t]);
            const unsigned off = v0 + (unsigned)(32 * I + 8 * t) * pitch;
            asm volatile("" ::"v"(val), "v"(off));
          }
#else
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, rb[t]), rs_out, v0 + (unsigned)(32 * I + 8 * t) * pitch, 0, 0);
#endif
      };
      auto load_scales = [&](auto piece_c) {
        constexpr int PIECE = decltype(piece_c)::value;
        if constexpr (!raw) {
#pragma unroll
          for (int ff = 0; ff < NF; ++ff)
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
              const int cw = 32 * (NF * PIECE + ff) + 16 * s2 + 8 * e_hh;
              const uint4 s_lo = *reinterpret_cast<const uint4 *>(tb_scale + cw);
              const uint4 s_hi = *reinterpret_cast<const uint4 *>(tb_scale + cw + 4);
              sraw[ff][s2][0] = s_lo.x; sraw[ff][s2][1] = s_lo.y; sraw[ff][s2][2] = s_lo.z; sraw[ff][s2][3] = s_lo.w;
              sraw[ff][s2][4] = s_hi.x; sraw[ff][s2][5] = s_hi.y; sraw[ff][s2][6] = s_hi.z; sraw[ff][s2][7] = s_hi.w;
            }
        }
      };
      auto compute = [&](auto u_c) __attribute__((always_inline)) {
        constexpr int U = decltype(u_c)::value, PIECE = U / T4_F, I = U % T4_F;
        const float pt = tb_pt[32 * I + e_l32];
#pragma unroll
        for (int ff = 0; ff < NF; ++ff) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            constexpr int f_lo = NF * PIECE;
            const int f = f_lo + ff;
            const int cw = 32 * f + 16 * s2 + 8 * e_hh;          // column inside the wave tile
            // accumulators leave the accumulation file here and not earlier (pinned: read ahead of time they
            // would not fit into the architectural file next to the staging registers)
            int a8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a8[j]) : "a"(acc[f][I][8 * s2 + j]));
            if (has_bias) {
              const int4 b_lo = *reinterpret_cast<const int4 *>(tb_bias + cw);
              const int4 b_hi = *reinterpret_cast<const int4 *>(tb_bias + cw + 4);
              a8[0] += b_lo.x; a8[1] += b_lo.y; a8[2] += b_lo.z; a8[3] += b_lo.w;
              a8[4] += b_hi.x; a8[5] += b_hi.y; a8[6] += b_hi.z; a8[7] += b_hi.w;
            }
            if constexpr (raw) {
              q[2 * s2] = make_uint4(a8[0], a8[1], a8[2], a8[3]);
              q[2 * s2 + 1] = make_uint4(a8[4], a8[5], a8[6], a8[7]);
            } else {
              float v[8];
#pragma unroll
              for (int j = 0; j < 8; ++j) v[j] = dequant(a8[j], __uint_as_float(sraw[ff][s2][j]), pt);
              if constexpr (ACT != 0) {
                // one value after the other (the empty asm statements keep their order): eight exponentials in flight at
                // once would need registers that this kernel does not have
                // v * sigmoid(t) = v / (1 + 2^(-t log2 e)); t = c v (silu: c = 1, fast gelu: 1.702) or, for the tanh form of
                // gelu, t = v (c1 + c3 v^2) with c1 = 2 sqrt(2 / pi), c3 = 0.044715 c1
                const float slu_k = (p.act_type == ACT_FAST_GELU ? -1.702f : -1.0f) * 1.4426950408889634f;
                constexpr float gelu_k1 = -1.5957691216057308f * 1.4426950408889634f, gelu_k3 = gelu_k1 * 0.044715f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
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
              uint4 r;
              if constexpr (MODE == 0) {
                r.x = pack_bf16x2(v[0], v[1]); r.y = pack_bf16x2(v[2], v[3]);
                r.z = pack_bf16x2(v[4], v[5]); r.w = pack_bf16x2(v[6], v[7]);
              } else {
                // the float32 product is rounded before the conversion (the golden's order); left visible,
                // multiply and conversion are merged into one mixed-precision instruction that rounds once
#pragma unroll
                for (int j = 0; j < 8; ++j) asm volatile("" : "+v"(v[j]));
                r.x = f32_to_f16_rne(v[0]) | ((unsigned)f32_to_f16_rne(v[1]) << 16);
                r.y = f32_to_f16_rne(v[2]) | ((unsigned)f32_to_f16_rne(v[3]) << 16);
                r.z = f32_to_f16_rne(v[4]) | ((unsigned)f32_to_f16_rne(v[5]) << 16);
                r.w = f32_to_f16_rne(v[6]) | ((unsigned)f32_to_f16_rne(v[7]) << 16);
              }
              q[2 * ff + s2] = r;
            }
          }
        }
      };
      // staging row of a lane: 16-bit outputs, vector 2 ff + s2 holds columns 32 ff + 16 s2 + 8 hh .. + 8 (bytes 64 ff +
      // 32 s2 + 16 hh); int32, vectors 2 s2 and 2 s2 + 1 hold columns 16 s2 + 8 hh .. + 8 (bytes 64 s2 + 32 hh, + 16)
      auto park = [&]() {
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint4 *>(dst + (raw ? 64 * (j >> 1) + 16 * (j & 1) : 32 * j)) = q[j];
      };
      if (fm_active == T4_F) {
        static_for<UNITS>([&](auto u_c) {
          constexpr int U = decltype(u_c)::value;
          if constexpr (U > 0) read_back();
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (U % T4_F == 0) load_scales(std::integral_constant<int, U / T4_F>{});
          compute(u_c);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (U > 0) store_unit(std::integral_constant<int, (U > 0 ? U - 1 : 0)>{});
          park();
          __builtin_amdgcn_sched_barrier(0);
        });
        read_back();
        store_unit(std::integral_constant<int, UNITS - 1>{});
      } else {
        // partial m-tile: only the 32-row blocks that hold rows, one after the other
        static_for<UNITS>([&](auto u_c) {
          constexpr int U = decltype(u_c)::value;
          if constexpr (U % T4_F == 0) load_scales(std::integral_constant<int, U / T4_F>{});
          if (U % T4_F < fm_active) {
            compute(u_c);
            park();
            read_back();
            store_unit(u_c);
          }
          __builtin_amdgcn_sched_barrier(0);
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
static hipError_t t4_launch(const GmmParams &p, unsigned grid, hipStream_t stream) {
  auto kern = gmm_w8a8_tile4_nk_kernel<MODE, WL, ACT>;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, T4_LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(T4_NW * 64), T4_LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t launch_tile4_w8a8(const GmmParams &p, int layout, hipStream_t stream) {
  // the operand stream runs up to four slabs ahead inside one tile; the group table lives in LDS; [E,K,N] weights
  // (layout 2) are read in 16-column chunks
  if (p.k < 4 * T4_BK || p.e > T4_MAX_E || layout < 0 || layout > 2 || (layout == 2 && p.n % 16 != 0)) return hipErrorInvalidValue;
  const long long n_tiles = (p.n + T4_BN - 1) / T4_BN;
  const long long m_tiles_ub = (p.m + T4_BM - 1) / T4_BM + p.e;   // every non-empty group adds at most one partial tile
  const long long total_ub = m_tiles_ub * n_tiles;
  long long grid = ((total_ub + kNumXcd - 1) / kNumXcd) * kNumXcd;
  if (grid > T4_MAX_WGS) grid = T4_MAX_WGS;
  if (grid <= 0) return hipSuccess;
  const int act = p.act_type == ACT_NONE ? 0 : p.act_type == ACT_RELU ? 3 : (p.act_type == ACT_SILU || p.act_type == ACT_FAST_GELU) ? 2 : 1;
  const unsigned g = (unsigned)grid;
#define MSCO_T4_BY_ACT(MODE, WL)                                   \
  (act == 0   ? t4_launch<MODE, WL, 0>(p, g, stream)               \
   : act == 1 ? t4_launch<MODE, WL, 1>(p, g, stream)               \
   : act == 2 ? t4_launch<MODE, WL, 2>(p, g, stream)               \
              : t4_launch<MODE, WL, 3>(p, g, stream))
#define MSCO_T4_BY_LAYOUT(MODE) (layout == 1 ? MSCO_T4_BY_ACT(MODE, 1) : layout == 2 ? MSCO_T4_BY_ACT(MODE, 2) : MSCO_T4_BY_ACT(MODE, 0))
  switch (p.out_dtype) {
    case DT_BF16: return MSCO_T4_BY_LAYOUT(0);
    case DT_F16: return MSCO_T4_BY_LAYOUT(1);
    case DT_I32: return layout == 1 ? t4_launch<2, 1, 0>(p, g, stream) : layout == 2 ? t4_launch<2, 2, 0>(p, g, stream) : t4_launch<2, 0, 0>(p, g, stream);
    default: return hipErrorInvalidValue;
  }
#undef MSCO_T4_BY_LAYOUT
#undef MSCO_T4_BY_ACT
}

}  // namespace msco
