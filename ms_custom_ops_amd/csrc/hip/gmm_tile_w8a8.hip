// Grouped W8A8 GEMM, MFMA tile kernel (prefill shapes) for gfx950.
//
// One workgroup computes one BM x BN output tile of one group with v_mfma_i32_32x32x32_i8 (the int8
// MFMA that issues at full rate on this part; measured: the 16x16x64 form sustains about half of it).
// The large configuration uses 8 wavefronts (2 x 4, two per SIMD, a 128 x 64 sub-tile of accumulators
// each), so that one wave's LDS reads and barrier waits are covered by the other wave's MFMAs; the
// small configurations use 4 wavefronts (2 x 2).
//
//   * Tile scheduling on the device.  The tile -> (group, m-tile, n-tile) mapping is computed by
//     walking group_list, so the host never reads it; the grid is sized from an upper bound and
//     surplus workgroups exit.  Consecutive tiles (same group, neighbouring n-tiles, all m-tiles of a
//     panel) are dealt to the same XCD so that the x rows of a group and the streamed weight panel
//     stay in that XCD's L2.
//   * Memory.  Operands are read through buffer descriptors (scalar base, one per-lane offset,
//     out-of-range rows read as zero, so no clamping or branching in the loop) in 64-byte K slabs,
//     three slabs ahead of the one being multiplied.  x rows and weights go straight from memory
//     into a 4-stage LDS ring (buffer_load ... lds), so slabs in flight cost no registers.
//   * Weights stored [K,N] lie in LDS as they lie in memory (K rows of BN column bytes) and are turned
//     into K-contiguous MFMA fragments on the way out, by LDS transpose reads.
//   * One LDS-only barrier per slab (it does not wait for the global loads in flight).
//   * Operand roles.  The weights are the MFMA's first operand and x the second, so a lane owns one
//     output row m and, after permuting which weight column feeds which MFMA row, two runs of 8
//     consecutive output columns per 32-column block: the fused dequant epilogue (int32 bias,
//     per-channel scale, per-token scale, bf16/f16 cast) stores 16 bytes per lane and instruction.
//
// LDS layouts (a fragment read is 16 B per lane over 32 consecutive rows, conflict free per 16 lanes):
//   x rows and [N,K] weights: row-major, 64 B per row, 16-byte chunk c of row r stored at chunk
//     position c ^ ((r >> 2) & 3);
//   [K,N] weights: K rows of BN bytes, 16-column chunk c of row r at chunk position c ^ swz_kt<BN>(r).
#include <algorithm>

#include "gmm_common.h"
#include "gmm_kernels.h"

#include <type_traits>

namespace msco {

// rows of BKT bytes in LDS: 16-byte chunk c of row r sits at position c ^ swz<BKT>(r), so that the 16 lanes of a
// fragment read (16 consecutive rows, one logical chunk) cover all 16 slots of a 256-byte LDS cycle
template <int BKT>
__device__ __forceinline__ int swz(int r) { return BKT == 64 ? (r >> 2) & 3 : (r >> 1) & 7; }
// [K,N] slabs read with transpose reads, K rows of BN bytes: a read touches 8 consecutive rows x the chunks of two
// neighbouring 16-lane blocks, and those 16 pieces of 16 bytes have to fall into 16 different bank groups of the
// 256-byte LDS cycle (rows of 128 bytes alias every second row)
template <int BN>
__device__ __forceinline__ int swz_kt(int r) { return BN == 256 ? (r & 7) << 1 : ((r >> 1) & 3) << 1; }

// MFMA output row q (0..31) of a 32 x 32 block <-> weight column inside the block.  Lane half hh holds
// rows q = 8 g + 4 hh + t (g = 0..3, t = 0..3); mapping them to columns 16 (g/2) + 8 hh + 4 (g%2) + t
// gives every lane two runs of 8 consecutive output columns.
__device__ __forceinline__ int col_of_q(int q) {
  const int g = q >> 3, hh = (q >> 2) & 1, t = q & 3;
  return 16 * (g >> 1) + 8 * hh + 4 * (g & 1) + t;
}

// 16 bytes per lane from a buffer straight into LDS: lane L of the wave writes lds_base + 16 L.
// (The address-space cast only exists in the device pass.)
template <int AUX = 0>
__device__ __forceinline__ void buffer_load_lds_b128(__amdgpu_buffer_rsrc_t rsrc, void *lds_base, unsigned voffset,
                                                     unsigned soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (void __attribute__((address_space(3))) *)(lds_base), 16, voffset,
                                           soffset, 0, AUX);
#else
  (void)rsrc; (void)lds_base; (void)voffset; (void)soffset;
#endif
}


// Two LDS transpose reads (ds_read_b64_tr_b8) STRIDE bytes apart, invisible to the compiler's wait-count bookkeeping:
// the compiler takes the builtin for a read that any LDS-direct load in flight may alias and waits for all of them.
// They must be issued before any compiler-visible LDS read whose result is consumed later (LDS operations complete in
// order), and lds_reads_done() must precede the first use of the results.
template <int STRIDE>
__device__ __forceinline__ void lds_read_tr8_pair(const unsigned char *p, uint2 &lo, uint2 &hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  const unsigned a = (unsigned)(unsigned long)(const __attribute__((address_space(3))) unsigned char *)p;
  asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(lo) : "v"(a));
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(a), "n"(STRIDE));
#else
  (void)p; lo = hi = uint2{0, 0};
#endif
}
template <typename T>
__device__ __forceinline__ void lds_reads_done(T &frags) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(frags));
}

// LDS-only barrier: waits for this wave's LDS traffic, not for global loads still in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, long long bytes) {
  const unsigned n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (unsigned)(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// STAGES = depth of the LDS ring of the operands that are loaded straight into LDS (STAGES - 1 slabs in flight)
// PK: weights in the packed layout (1 KiB blocks of 16 columns x 64 K bytes, byte 16 l + i of block (a, b) =
// w[k = 64 b + 16 (l / 16) + i][n = 16 a + l % 16]).  A 64-byte K slab of the tile is then one block per column group:
// the LDS-direct load of a block copies it as it lies, and a weight fragment is read at block (column / 16), chunk
// 2 kk + hh, row (column % 16) -- conflict free without a swizzle.
// KS = 32-byte MFMA K steps per slab (packed weights only for KS = 4): a slab is BKT = 32 KS bytes of K.  With 128-byte
// slabs every x row piece is a whole cache line (64-byte pieces are half lines, and the load path is bound by line
// requests), a column group contributes two consecutive 1 KiB blocks, and there is one barrier per 4 K steps.
// WNT (packed weights): the weight loads carry the non-temporal bit -- planned when the launch streams tens of megabytes
// of weights that at most two m-tiles read (GmmParams::w_nontemporal): a stream that is read once should not push x
// out of the caches.  Whole kilobytes per instruction only: on row-major [E,N,K] weights with 64-byte slabs (half
// lines) the bit costs 15 %.
// KT: the weights are [E,K,N] (N a multiple of 16) and take the LDS-direct path as they lie in
// memory: a slab is BKT K rows of BN column bytes, one wave instruction brings 1024 / BN rows, lane L row L / (BN / 16),
// slot L % (BN / 16), and slot s of row r holds the 16-column chunk s ^ swz_kt<BN>(r).  A weight fragment is two LDS
// transpose reads (ds_read_b64_tr_b8: of a block of 16 lanes, lane i names 8 bytes M[i][0..7] and lane j receives
// byte b = M[2 b + j / 8][j % 8]; with lanes 2 b and 2 b + 1 on the two halves of one chunk of K row b, lane j gets K
// rows 0 .. 7 of the chunk's column j).  MFMA row q of a 32-column block is then column q itself, so a lane owns four
// runs of 4 output columns instead of two of 8 and the epilogue parks 8-byte pieces.
template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, bool PK = false, int KS = 2, bool WNT = false, bool KT = false>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64, 2) gmm_w8a8_tile_kernel(const GmmParams p) {
  static_assert(!WNT || PK || KT, "non-temporal weight loads: whole kilobytes of whole lines per instruction (packed blocks, [K,N] rows)");
  static_assert(KS == 2 || KS == 4, "64- or 128-byte K slabs");
  static_assert(!KT || (!PK && (BN == 128 || BN == 256)), "transpose reads: [K,N] rows of 128 or 256 columns");
  constexpr int BKT = 32 * KS;                      // bytes of K per slab
  constexpr int ROWS_PER_LOAD = 1024 / BKT;         // x rows one wave instruction (1 KiB) brings
  constexpr int KB_PER_SLAB = BKT / 64;             // packed 1 KiB blocks of a column group per slab
  constexpr int NSTAGE = STAGES;
  constexpr int AHEAD = STAGES - 1;                 // slabs requested ahead of the one being multiplied
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int NT = NW * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int FM = WTM / 32, FN = WTN / 32;     // 32 x 32 MFMA blocks per wave
  constexpr int A_LD = BM / ROWS_PER_LOAD / NW;     // 1 KiB pieces (16 or 8 rows) of the x slab per wave
  constexpr int B_LD = BN * BKT / 1024 / NW;        // same for an [N,K] weight slab
  constexpr int A_STAGE = BM * BKT, B_STAGE = BN * BKT;
  constexpr int PANEL = 8;                          // m-tiles that share a streamed weight panel
  constexpr unsigned OOB = 0x80000000u;             // buffer offset that always reads zero
  constexpr int VM_PER_SLAB = A_LD + B_LD;          // vector-memory loads a wave issues per slab
  static_assert(FM >= 1 && FN >= 1 && A_LD >= 1 && B_LD >= 1, "tile shape");
  static_assert(BM % (ROWS_PER_LOAD * NW) == 0 && BN % (16 * NW) == 0, "row blocks per wave");

  // LDS: operand ring, reused by the epilogue staging; behind both, the tile's epilogue operands
  constexpr int LOOP_LDS = NSTAGE * (A_STAGE + B_STAGE);
  constexpr int EPI_LDS = NW * WTM * 144;
  constexpr int PARAM_OFF = LOOP_LDS > EPI_LDS ? LOOP_LDS : EPI_LDS;
  static_assert(BM <= 256 && BN <= 256, "epilogue operand table holds 256 entries");
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char *lds_a = smem;                      // [NSTAGE][BM * BKT], rows of BKT bytes, chunk c at c ^ swz<BKT>(row)
  unsigned char *lds_b = smem + NSTAGE * A_STAGE;   // [NSTAGE][BN * BKT]: rows like x, packed blocks, or K rows of BN bytes ([K,N])

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int l32 = lane & 31, hh = lane >> 5;

  // ---- tile lookup: two wave-parallel passes over group_list (count, then locate) -------------
  // 64 groups per step with prefix scans, so the cost does not grow with the number of experts;
  // every wave does the same work, no LDS or barrier is involved.
  const int n_tiles = (p.n + BN - 1) / BN;
  int total = 0;
  for (int g0 = 0, carry = 0; g0 < p.e; g0 += 64) {
    int s0, e0;
    group_rows_chunk(p, g0, lane, carry, s0, e0);
    const int rows_g = e0 - s0;   // (groups outside (rows_lo, rows_hi] have no tiles in this launch)
    const int t = wave_scan_add((rows_g > p.rows_lo && rows_g <= p.rows_hi) ? ((rows_g + BM - 1) / BM) * n_tiles : 0, lane);
    total += wave_bcast(t, 63);
  }
  // K split across workgroups (small problems): the slices of one tile sit next to each other in the
  // grid, on the same XCD
  constexpr bool CAN_SPLIT = BM * BN <= 128 * 128;   // the plan splits K for the small tile shapes only
  const int split = (CAN_SPLIT && p.split_k > 1) ? p.split_k : 1;
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const int slot = blockIdx.x / kNumXcd;
  const int local = slot / split, ks = slot - local * split;
  if (local >= per_xcd) return;
  const int lid = (blockIdx.x % kNumXcd) * per_xcd + local;
  if (lid >= total) return;

  int grp = 0, g_start = 0, g_end = 0, t_in_group = 0;
  for (int g0 = 0, carry = 0, tiles_before = 0; g0 < p.e; g0 += 64) {
    int s0, e0;
    group_rows_chunk(p, g0, lane, carry, s0, e0);
    const int rows_g = e0 - s0;
    const int tiles = (rows_g > p.rows_lo && rows_g <= p.rows_hi) ? ((rows_g + BM - 1) / BM) * n_tiles : 0;
    const int upto = tiles_before + wave_scan_add(tiles, lane);      // tiles of groups 0 .. g0 + lane
    const int first = __popcll(__ballot(upto <= lid));              // `upto` is non-decreasing: first lane beyond lid
    if (first < 64) {
      grp = g0 + first;
      g_start = wave_bcast(s0, first);
      g_end = wave_bcast(e0, first);
      t_in_group = lid - (wave_bcast(upto, first) - wave_bcast(tiles, first));
      break;
    }
    tiles_before = wave_bcast(upto, 63);
  }
  // order inside a group: panel of PANEL m-tiles, then n-tile, then m-tile inside the panel
  const int m_tiles = (g_end - g_start + BM - 1) / BM;
  const int panel_tiles = PANEL * n_tiles;
  const int panel = t_in_group / panel_tiles;
  const int in_panel = t_in_group - panel * panel_tiles;
  const int panel_m = min(PANEL, m_tiles - panel * PANEL);
  const int nt = in_panel / panel_m;
  const int mt = panel * PANEL + in_panel % panel_m;

  const int m0 = g_start + mt * BM;
  const int n0 = nt * BN;
  const int k_slabs_all = (p.k + BKT - 1) / BKT;
  const int per_slice = (k_slabs_all + split - 1) / split;
  const int k_first = ks * per_slice;                                   // first slab of this workgroup's K slice
  const int k_slabs = max(0, min(k_slabs_all, k_first + per_slice) - k_first);

  // Epilogue operands of this tile (scale and bias of its columns, per-token scale of its rows) are
  // requested now, parked in registers during the main loop and handed over through LDS, so that
  // the epilogue does not start with a chain of global-memory round trips.
  float pre_scale = 1.0f, pre_pt = 1.0f;
  int pre_bias = 0;
  if (tid < 256) {
    if (tid < BN && n0 + tid < p.n) {
      pre_scale = load_scale(p, grp, n0 + tid);
      pre_bias = load_bias(p, grp, n0 + tid);
    }
    if (tid < BM && p.per_token && m0 + tid < g_end) pre_pt = p.per_token[m0 + tid];
  }

  // Buffer descriptors start at this tile's first x row / weight column, so per-lane offsets stay
  // small; anything past the end of the group's rows / the tensor reads as zero (no clamping, no branches in
  // the loop; zeros instead of the next group's rows cost neither memory traffic nor matrix-pipe power).
  const long long w_elems = (long long)p.k * p.n;
  const int8_t *wg = p.w + (long long)grp * w_elems;
  const __amdgpu_buffer_rsrc_t rx =
    make_rsrc(reinterpret_cast<const int8_t *>(p.x) + (long long)m0 * p.k, (long long)(g_end - m0) * p.k);
  const int pk_blocks = (p.k + 63) / 64, pk_groups = (p.n + 15) / 16;   // packed layout: K blocks per column group, column groups
  const __amdgpu_buffer_rsrc_t rw =
    PK   ? make_rsrc(p.w + ((long long)grp * pk_groups + n0 / 16) * pk_blocks * 1024, (long long)(pk_groups - n0 / 16) * pk_blocks * 1024)
    : KT ? make_rsrc(wg + n0, w_elems - n0)
         : make_rsrc(wg + (long long)n0 * p.k, (long long)(p.n - n0) * p.k);

  // ---- operands loaded straight into LDS (x rows, [N,K] weights) -----------------------------
  // One wave instruction fills 1 KiB of LDS = 16 rows x 64 B, lane L writing bytes [16 L, 16 L + 16).
  // With the swizzle, LDS position (row L/4, chunk position L%4) holds logical chunk (L%4) ^ (L/16).
  // Only the per-lane offset is range-checked by the buffer unit, so everything that can run past
  // the tensor (rows, columns, the K tail) lives in the per-lane offset; the scalar offset carries
  // just the slab position inside a row.
  // (general form: lane L writes row L / (BKT/16) of its 1 KiB piece, position L % (BKT/16), which holds logical
  // chunk position ^ swz<BKT>(row); with 128-byte rows the swizzle depends on the piece, so offsets are per piece)
  constexpr int CHUNKS = BKT / 16;
  const int d_row = lane / CHUNKS;
  unsigned a_voff[A_LD];
  int a_chunk[A_LD];                                 // logical chunk of this lane in piece u (for the K tail)
#pragma unroll
  for (int u = 0; u < A_LD; ++u) {
    const int row = (wave * A_LD + u) * ROWS_PER_LOAD + d_row;
    a_chunk[u] = (lane % CHUNKS) ^ swz<BKT>(row);
    a_voff[u] = (unsigned)row * (unsigned)p.k + a_chunk[u] * 16;
  }
  // [N,K] weights: LDS row rho = 32 * block + q feeds MFMA row q of that block and holds weight
  // column 32 * block + col_of_q(q) of the tile.
  unsigned b_voff[B_LD];
  int b_chunk[B_LD];                                 // [N,K] weights: logical chunk of this lane in piece u; [K,N]: its K row
  constexpr int KT_SLOTS = BN / 16, KT_ROWS = 1024 / BN;   // [K,N] slabs: 16-column chunks per K row, K rows per piece
  if constexpr (KT) {
#pragma unroll
    for (int u = 0; u < B_LD; ++u) {
      const int krow = (wave * B_LD + u) * KT_ROWS + lane / KT_SLOTS;   // K row of the slab that this lane brings in piece u
      const int chunk = (lane % KT_SLOTS) ^ swz_kt<BN>(krow);
      b_chunk[u] = krow;                               // (the K tail is a matter of rows here)
      // columns past N read as zero; the K row of the slab goes into the scalar offset, which nobody range-checks
      b_voff[u] = (n0 + chunk * 16 < p.n) ? (unsigned)krow * (unsigned)p.n + chunk * 16 : OOB;
    }
  } else {
#pragma unroll
    for (int u = 0; u < B_LD; ++u) {
      const int blk = wave * B_LD + u;
      const int rho = blk * ROWS_PER_LOAD + d_row;
      b_chunk[u] = (lane % CHUNKS) ^ swz<BKT>(rho);
      if constexpr (PK) b_voff[u] = (unsigned)((blk / KB_PER_SLAB) * pk_blocks * 1024 + lane * 16);   // piece blk: column group blk / KB_PER_SLAB of the tile
      else b_voff[u] = (unsigned)((rho & ~31) + col_of_q(rho & 31)) * (unsigned)p.k + b_chunk[u] * 16;
    }
  }
  auto issue_direct = [&](int kt) {
    const int stage = kt % NSTAGE;
    const unsigned kbase = (k_first + kt) * BKT;
    // K tail, and whole slabs past K (requested by the last steps of the branch-free loop): read as zero
#pragma unroll
    for (int u = 0; u < A_LD; ++u) {
      const int blk = wave * A_LD + u;
      const unsigned kill_a = (kbase + a_chunk[u] * 16 >= (unsigned)p.k) ? OOB : 0u;
      buffer_load_lds_b128(rx, lds_a + stage * A_STAGE + blk * 1024, a_voff[u] | kill_a, kbase);
    }
#pragma unroll
    for (int u = 0; u < B_LD; ++u) {
      const int blk = wave * B_LD + u;
      if constexpr (PK) {
        // K block (k_first + kt) KB_PER_SLAB + blk % KB_PER_SLAB of the column group; blocks past K do not exist
        // (the last one is zero padded)
        const int kblock = (k_first + kt) * KB_PER_SLAB + blk % KB_PER_SLAB;
        const unsigned kill_w = (kblock >= pk_blocks) ? OOB : 0u;
        buffer_load_lds_b128<WNT ? 2 : 0>(rw, lds_b + stage * B_STAGE + blk * 1024, b_voff[u] | kill_w, kblock * 1024);
      } else if constexpr (KT) {
        const unsigned kill_b = (kbase + (unsigned)b_chunk[u] >= (unsigned)p.k) ? OOB : 0u;   // K rows past K
        buffer_load_lds_b128<WNT ? 2 : 0>(rw, lds_b + stage * B_STAGE + blk * 1024, b_voff[u] | kill_b, kbase * (unsigned)p.n);
      } else {
        const unsigned kill_b = (kbase + b_chunk[u] * 16 >= (unsigned)p.k) ? OOB : 0u;
        buffer_load_lds_b128(rw, lds_b + stage * B_STAGE + blk * 1024, b_voff[u] | kill_b, kbase);
      }
    }
  };

  // ---- fragment reads (one 16-byte LDS read per lane and fragment) ----------------------------
  // lane (l32, hh) of k-half kk reads row l32 of its 32-row block, 16-byte chunk c = 2 kk + hh
  auto read_x = [&](int kt, int i, int kk) -> v4i {
    const unsigned char *a = lds_a + (kt % NSTAGE) * A_STAGE;
    const int row = wave_m * WTM + 32 * i + l32;
    return *reinterpret_cast<const v4i *>(a + row * BKT + (((2 * kk + hh) ^ swz<BKT>(row)) << 4));
  };
  auto read_w = [&](int kt, int f, int kk) -> v4i {
    const int rho = wave_n * WTN + 32 * f + l32;
    if constexpr (PK) {
      const unsigned char *b = lds_b + (kt % NSTAGE) * B_STAGE;
      const int col = wave_n * WTN + 32 * f + col_of_q(l32);   // MFMA row l32 of block f is this column of the tile
      // chunk 2 kk + hh of the slab: block (2 kk + hh) / 4 of the column group's blocks in this slab, chunk % 4 inside it
      return *reinterpret_cast<const v4i *>(b + ((col >> 4) * KB_PER_SLAB + ((2 * kk + hh) >> 2)) * 1024 +
                                            ((2 * kk + hh) & 3) * 256 + (col & 15) * 16);
    } else if constexpr (KT) {
      // K rows 32 kk + 16 hh + 8 t + i / 2 (t = 0, 1: the two reads; i = lane % 16), half i % 2 of the chunk that holds the
      // 16 columns of this lane's block of 16
      const int i = lane & 15;
      const int krow = 32 * kk + 16 * hh + (i >> 1);
      const int chunk = (wave_n * WTN + 32 * f) / 16 + ((lane >> 4) & 1);
      const unsigned char *b = lds_b + (kt % NSTAGE) * B_STAGE + krow * BN + ((chunk ^ swz_kt<BN>(krow)) << 4) + (i & 1) * 8;
      uint2 lo, hi;
      lds_read_tr8_pair<8 * BN>(b, lo, hi);   // (the caller orders these reads before its own and waits for them)
      return v4i{(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
    } else {
      const unsigned char *b = lds_b + (kt % NSTAGE) * B_STAGE;
      return *reinterpret_cast<const v4i *>(b + rho * BKT + (((2 * kk + hh) ^ swz<BKT>(rho)) << 4));
    }
  };

  v16i acc[FN][FM];
#pragma unroll
  for (int f = 0; f < FN; ++f)
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[f][i][r] = 0;

  // ---- main loop ---------------------------------------------------------------------------------
  // Slabs t+1 .. t+3 are in flight in the LDS ring while slab t is multiplied.
  //
  // With 8 waves every SIMD hosts two waves, one from each half of the workgroup, and
  // the halves run half a step apart.  While one half issues its 16 MFMAs for slab t, the other half
  // does the memory side of its own step (requests slab t+3, reads its 12 operand fragments from
  // LDS).  Two workgroup barriers per step keep the halves in opposite phases, so the matrix pipe and
  // the LDS / memory pipes are busy at the same time instead of taking turns.  The half that runs
  // behind enters the loop through one extra barrier and the half that runs ahead leaves it through
  // one, so all waves execute the same number.  Four waves keep one phase with one barrier per slab.
  constexpr bool PINGPONG = NW == 8;
  const bool behind = PINGPONG && wave >= NW / 2;
  auto phase_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  // The loop body is branch free: the last steps still request "slabs" t+3 past K, whose offsets are
  // all out of range, so nothing is read and zeros land in a stage nobody reads.  Every path through
  // the loop then issues the same number of loads, which keeps the vmcnt waits exact -- with
  // conditional requests the compiler has to assume the shortest path and waits for the loads it has
  // just issued.
  auto step = [&](int kt) {
    issue_direct(kt + AHEAD);
    v4i xf[KS][FM], wf[KS][FN];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
#pragma unroll
      for (int f = 0; f < FN; ++f) wf[kk][f] = read_w(kt, f, kk);
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
#pragma unroll
      for (int i = 0; i < FM; ++i) xf[kk][i] = read_x(kt, i, kk);
    if constexpr (KT) {
      // hand-issued weight reads: older than every x read, so one wait covers them
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
#pragma unroll
        for (int f = 0; f < FN; ++f) lds_reads_done(wf[kk][f]);
    }
    if constexpr (PINGPONG) {
      wait_vmcnt<(AHEAD - 1) * VM_PER_SLAB>();                // this wave's part of slab t+1 has landed
      __builtin_amdgcn_sched_barrier(0);
      lds_barrier();                                          // fragments are in registers, slab t+1 is published
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(2);
    }
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int i = 0; i < FM; ++i)
          acc[f][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[kk][f], xf[kk][i], acc[f][i], 0, 0, 0);
    if constexpr (PINGPONG) {
      __builtin_amdgcn_s_setprio(0);
      phase_barrier();
    } else {
      wait_vmcnt<(AHEAD - 1) * VM_PER_SLAB>();                // only the loads of younger slabs may be outstanding
      lds_barrier();
    }
  };

  // prologue: slabs 0, 1, 2 requested; slab 0 published
  issue_direct(0);
  issue_direct(1);
  if constexpr (AHEAD > 2) issue_direct(2);
  wait_vmcnt<(AHEAD - 1) * VM_PER_SLAB>();
  lds_barrier();
  if (behind) phase_barrier();

  for (int kt = 0; kt < k_slabs; ++kt) step(kt);
  if (PINGPONG && !behind) phase_barrier();

  // ---- K split: partial tiles meet in the workspace, the last slice to arrive adds them up ----------
  // Every slice parks its accumulators (register by register, so the stores are contiguous across the
  // workgroup), takes a ticket on the tile's counter, and all but the last one leave.  int32 addition
  // is associative, so the result does not depend on the arrival order.  Agent-scope relaxed atomics
  // keep the exchange in L2 without cache-wide fences; the counter resets itself for the next launch.
  if constexpr (CAN_SPLIT) if (split > 1) {
    __shared__ unsigned s_ticket;
    constexpr int TILE_INTS = BM * BN;
    constexpr int WORDS = FN * FM * 8;   // 64-bit words per thread: accumulator registers (r, r + 1) travel together
    typedef long long i64;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + (long long)lid * split * (TILE_INTS / 2);
    i64 *mine = base + (long long)ks * (TILE_INTS / 2) + tid;
#pragma unroll
    for (int f = 0; f < FN; ++f)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const i64 word = (i64)(((unsigned long long)(unsigned)acc[f][i][r + 1] << 32) | (unsigned)acc[f][i][r]);
          __hip_atomic_store(mine + ((f * FM + i) * 8 + r / 2) * NT, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    publish_partials_and_sync();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[lid], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)(split - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[lid], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the other slices, two per memory round trip (the j-th other slice is j, or j + 1 from this one's index on); an
    // odd one out is read alone
    const int others = split - 1;
    for (int j0 = 0; j0 < others; j0 += 2) {
      const bool two = j0 + 1 < others;
      const int sa = j0 < ks ? j0 : j0 + 1, sb = two ? (j0 + 1 < ks ? j0 + 1 : j0 + 2) : sa;
      const i64 *oa = base + (long long)sa * (TILE_INTS / 2) + tid, *ob = base + (long long)sb * (TILE_INTS / 2) + tid;
      i64 ta[WORDS], tb[WORDS];
#pragma unroll
      for (int u = 0; u < WORDS; ++u) ta[u] = __hip_atomic_load(oa + u * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (two) {
#pragma unroll
        for (int u = 0; u < WORDS; ++u) tb[u] = __hip_atomic_load(ob + u * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
#pragma unroll
        for (int u = 0; u < WORDS; ++u) tb[u] = 0;
      }
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const unsigned long long wa = (unsigned long long)ta[(f * FM + i) * 8 + r / 2];
            const unsigned long long wb = (unsigned long long)tb[(f * FM + i) * 8 + r / 2];
            acc[f][i][r] += (int)(unsigned)wa + (int)(unsigned)wb;
            acc[f][i][r + 1] += (int)(unsigned)(wa >> 32) + (int)(unsigned)(wb >> 32);
          }
    }
  }

  float *ep_scale = reinterpret_cast<float *>(smem + PARAM_OFF);
  int *ep_bias = reinterpret_cast<int *>(smem + PARAM_OFF + 1024);
  float *ep_pt = reinterpret_cast<float *>(smem + PARAM_OFF + 2048);
  if (tid < 256) {
    ep_scale[tid] = pre_scale;
    ep_bias[tid] = pre_bias;
    ep_pt[tid] = pre_pt;
  }
  // the epilogue reuses the operand ring: every wave is done reading it and the late zero fills have landed
  wait_vmcnt<0>();
  lds_barrier();

  // ---- fused dequant epilogue --------------------------------------------------------------------
  // acc[f][i][r] is output row 32 i + l32 and column 32 f + 16 (r / 8) + 8 hh + (r % 8) of the wave tile
  // (transpose-read weights, KT: column 32 f + 8 (r / 4) + 4 hh + (r % 4), the MFMA's own row order):
  // lanes run along rows.  Each wave dequantises its values, parks them in a private LDS region
  // (rows of 128 payload bytes at a 144-byte pitch, conflict free both ways) and reads them back with
  // lanes running along columns, so every global store instruction writes 8 full 128-byte row segments.
  static_assert(WTN == 64, "epilogue staging assumes 64-column wave tiles");
  constexpr int EP_PITCH = 144;
  unsigned char *stage = smem + wave * (WTM * EP_PITCH);
  float pt[FM];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    pt[i] = ep_pt[wave_m * WTM + 32 * i + l32];
  }
  // int32 rows are 256 bytes: one 32-column block per pass; 16-bit outputs take a single pass
  auto run_pass = [&](auto raw_c, auto pass_c) {
    constexpr bool raw = decltype(raw_c)::value;
    constexpr int pass = decltype(pass_c)::value;
    constexpr int esize = raw ? 4 : 2;
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      if (raw && f != pass) continue;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        // accumulators 8 s2 .. 8 s2 + 7: one run of 8 columns, or (KT) two runs of 4, eight columns apart
        const int cw = KT ? 32 * f + 16 * s2 + 4 * hh : 32 * f + 16 * s2 + 8 * hh;   // column inside the wave tile
        constexpr int RUN2 = KT ? 8 : 4;                       // first column of accumulators 4 .. 7, relative to cw
        float sc[8];
        int bi[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sc[j] = ep_scale[wave_n * WTN + cw + (j < 4 ? j : RUN2 + j - 4)];
          bi[j] = ep_bias[wave_n * WTN + cw + (j < 4 ? j : RUN2 + j - 4)];
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          unsigned char *dst = stage + (32 * i + l32) * EP_PITCH;
          if (raw) {
            int *d = reinterpret_cast<int *>(dst + (cw - 32 * f) * 4);
            *reinterpret_cast<int4 *>(d) = make_int4(acc[f][i][8 * s2] + bi[0], acc[f][i][8 * s2 + 1] + bi[1],
                                                     acc[f][i][8 * s2 + 2] + bi[2], acc[f][i][8 * s2 + 3] + bi[3]);
            *reinterpret_cast<int4 *>(d + RUN2) = make_int4(acc[f][i][8 * s2 + 4] + bi[4], acc[f][i][8 * s2 + 5] + bi[5],
                                                            acc[f][i][8 * s2 + 6] + bi[6], acc[f][i][8 * s2 + 7] + bi[7]);
          } else {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = dequant(acc[f][i][8 * s2 + j] + bi[j], sc[j], pt[i]);
            if (p.act_type != ACT_NONE) {
#pragma unroll
              for (int j = 0; j < 8; ++j) v[j] = activate(v[j], p.act_type);
            }
            uint4 q;
            if (p.out_dtype == DT_BF16) {
              q.x = pack_bf16x2(v[0], v[1]); q.y = pack_bf16x2(v[2], v[3]);
              q.z = pack_bf16x2(v[4], v[5]); q.w = pack_bf16x2(v[6], v[7]);
            } else {
              q.x = f32_to_f16_rne(v[0]) | ((unsigned)f32_to_f16_rne(v[1]) << 16);
              q.y = f32_to_f16_rne(v[2]) | ((unsigned)f32_to_f16_rne(v[3]) << 16);
              q.z = f32_to_f16_rne(v[4]) | ((unsigned)f32_to_f16_rne(v[5]) << 16);
              q.w = f32_to_f16_rne(v[6]) | ((unsigned)f32_to_f16_rne(v[7]) << 16);
            }
            if constexpr (KT) {
              *reinterpret_cast<uint2 *>(dst + cw * 2) = make_uint2(q.x, q.y);
              *reinterpret_cast<uint2 *>(dst + (cw + RUN2) * 2) = make_uint2(q.z, q.w);
            } else {
              *reinterpret_cast<uint4 *>(dst + cw * 2) = q;
            }
          }
        }
      }
    }
    // read back row-major: lane -> (row = 8 t + lane / 8, 16-byte column piece lane % 8)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int piece = lane & 7;
    const int col = raw ? (32 * pass + 4 * piece) : 8 * piece;   // first column of the piece inside the wave tile
    const int n_first = n0 + wave_n * WTN + col;
#pragma unroll
    for (int t = 0; t < WTM / 8; ++t) {
      const int row = 8 * t + (lane >> 3);
      const int m = m0 + wave_m * WTM + row;
      const uint4 q = *reinterpret_cast<const uint4 *>(stage + row * EP_PITCH + piece * 16);
      if (m < g_end && n_first < p.n) {
        unsigned char *o = reinterpret_cast<unsigned char *>(p.out) + ((long long)m * p.n + n_first) * esize;
        *reinterpret_cast<uint4 *>(o) = q;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  if (p.out_dtype == DT_I32) {
    run_pass(std::true_type{}, std::integral_constant<int, 0>{});
    if constexpr (FN > 1) run_pass(std::true_type{}, std::integral_constant<int, 1>{});
    static_assert(FN <= 2, "int32 epilogue passes");
  } else {
    run_pass(std::false_type{}, std::integral_constant<int, 0>{});
  }
}

// ---- host launcher ---------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES = 4, bool PK = false, int KS = 2, bool WNT = false, bool KT = false>
static hipError_t launch_cfg(const GmmParams &p, hipStream_t stream) {
  constexpr int BKT = 32 * KS;
  const size_t loop_lds = (size_t)STAGES * (BM + BN) * BKT;
  const size_t epi_lds = (size_t)WAVES_M * WAVES_N * (BM / WAVES_M) * 144;   // epilogue staging, 144-byte row pitch
  const size_t lds = (loop_lds > epi_lds ? loop_lds : epi_lds) + 3 * 1024;   // + epilogue operand table
  auto kern = gmm_w8a8_tile_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, PK, KS, WNT, KT>;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const long long n_tiles = (p.n + BN - 1) / BN;
  // every non-empty group adds at most one partial tile; a launch for the small groups only: that many tiles per group
  const long long m_tiles_ub = p.rows_hi < p.m ? std::min<long long>((p.m + BM - 1) / BM + p.e, (long long)p.e * ((p.rows_hi + BM - 1) / BM))
                                               : (p.m + BM - 1) / BM + p.e;
  const long long total_ub = m_tiles_ub * n_tiles;
  const long long grid = ((total_ub + kNumXcd - 1) / kNumXcd) * kNumXcd * (p.split_k > 1 ? p.split_k : 1);
  if (grid <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES_M * WAVES_N * 64), lds, stream, p);
  return hipGetLastError();
}

// The small tile shapes run 128-byte K slabs through a 4-stage ring when the plan says so (GmmParams::wide_k_slabs: the
// workgroups fit one round; measured against 64-byte slabs on M = 256, K = 4096, N = 11008 packed: 26.0 against 28.8 us;
// 3 / 2 stages 26.7 / 34.1).  layout: 0 [E,N,K], 1 packed, 2 [E,K,N] (transpose reads).
template <int BM, int BN>
static hipError_t launch_small(const GmmParams &p, int layout, hipStream_t stream) {
  if (layout == 1 && p.w_nontemporal)
    return p.wide_k_slabs ? launch_cfg<BM, BN, 2, 2, 4, true, 4, true>(p, stream) : launch_cfg<BM, BN, 2, 2, 4, true, 2, true>(p, stream);
  if (layout == 1) return p.wide_k_slabs ? launch_cfg<BM, BN, 2, 2, 4, true, 4>(p, stream) : launch_cfg<BM, BN, 2, 2, 4, true>(p, stream);
  if (layout == 0) return p.wide_k_slabs ? launch_cfg<BM, BN, 2, 2, 4, false, 4>(p, stream) : launch_cfg<BM, BN, 2, 2>(p, stream);
  if (p.w_nontemporal)
    return p.wide_k_slabs ? launch_cfg<BM, BN, 2, 2, 4, false, 4, true, true>(p, stream)
                          : launch_cfg<BM, BN, 2, 2, 4, false, 2, true, true>(p, stream);
  return p.wide_k_slabs ? launch_cfg<BM, BN, 2, 2, 4, false, 4, false, true>(p, stream)
                        : launch_cfg<BM, BN, 2, 2, 4, false, 2, false, true>(p, stream);
}

// nk: weights stored [E,N,K]; packed: the blocked layout; neither: [E,K,N] (N a multiple of 16, which the plan's
// alignment rule guarantees for every MFMA kernel)
hipError_t launch_tile_w8a8(const GmmParams &p, int tile_cfg, bool nk, bool packed, hipStream_t stream) {
  const int layout = packed ? 1 : nk ? 0 : 2;
  if (layout == 2 && p.n % 16 != 0) return hipErrorInvalidValue;
  // the persistent kernel needs at least four 128-byte K slabs per tile and a group table that fits in LDS; what it
  // cannot take runs the eight-wave kernel of the same tile shape
  if (tile_cfg == TILE_256x256_W4 || tile_cfg == TILE_256x256_W4_MFMA32) {
    if (p.k >= 512 && p.e <= 1024)
      return tile_cfg == TILE_256x256_W4 ? launch_tile4m_w8a8(p, layout, stream) : launch_tile4_w8a8(p, layout, stream);
    tile_cfg = TILE_256x256;
  }
  if (tile_cfg == TILE_ROWS256 || tile_cfg == TILE_ROWS128 || tile_cfg == TILE_ROWS160)
    return packed ? launch_rows_w8a8(p, tile_cfg == TILE_ROWS256 ? 16 : tile_cfg == TILE_ROWS160 ? 10 : 8, stream) : hipErrorInvalidValue;
  switch (tile_cfg) {
    case TILE_128x128: return launch_small<128, 128>(p, layout, stream);
    case TILE_64x128: return launch_small<64, 128>(p, layout, stream);
    case TILE_256x256:   // eight waves, two per SIMD
      return layout == 1 ? launch_cfg<256, 256, 2, 4, 4, true>(p, stream)
           : layout == 0 ? launch_cfg<256, 256, 2, 4>(p, stream)
                         : launch_cfg<256, 256, 2, 4, 4, false, 2, false, true>(p, stream);
    case TILE_128x256:   // four waves side by side, 128 x 64 each; two workgroups per CU
      if (layout == 1) {
        if (p.w_nontemporal) return launch_cfg<128, 256, 1, 4, 3, true, 2, true>(p, stream);
        return p.wide_k_slabs ? launch_cfg<128, 256, 1, 4, 3, true, 4>(p, stream) : launch_cfg<128, 256, 1, 4, 3, true>(p, stream);
      }
      if (layout == 2 && p.w_nontemporal) return launch_cfg<128, 256, 1, 4, 3, false, 2, true, true>(p, stream);
      return layout == 0 ? launch_cfg<128, 256, 1, 4, 3>(p, stream) : launch_cfg<128, 256, 1, 4, 3, false, 2, false, true>(p, stream);
    default:
      return hipErrorInvalidValue;
  }
}

const char *tile_cfg_name(int tile_cfg) {
  switch (tile_cfg) {
    case TILE_256x256: return "256x256x64";
    case TILE_128x128: return "128x128";   // (64- or 128-byte K slabs: the plan's wide_k_slabs, whatever the layout)
    case TILE_64x128: return "64x128";
    case TILE_128x256: return "128x256x64";
    case TILE_256x256_W4: return "256x256x128_w4";
    case TILE_256x256_W4_MFMA32: return "256x256x128_w4_mfma32";
    case TILE_ROWS256: return "rows256";
    case TILE_ROWS128: return "rows128";
    case TILE_ROWS160: return "rows160";
    default: return "?";
  }
}

// upper bound of the number of tiles (the real number depends on group_list, which only the device reads)
size_t tile_count_bound(int tile_cfg, int64_t m, int64_t n, int64_t e) {
  int bm, bn;
  tile_cfg_dims(tile_cfg, &bm, &bn);
  // every group that holds rows adds at most one partial m-tile, and at most min(e, m) groups hold rows
  return (size_t)(((m + bm - 1) / bm + (e < m ? e : m)) * ((n + bn - 1) / bn));
}

size_t tile_workspace_bytes(int tile_cfg, int64_t m, int64_t n, int64_t e, int split_k) {
  if (split_k <= 1) return 0;
  int bm, bn;
  tile_cfg_dims(tile_cfg, &bm, &bn);
  return tile_count_bound(tile_cfg, m, n, e) * (size_t)split_k * bm * bn * 4;
}

void tile_cfg_dims(int tile_cfg, int *bm, int *bn) {
  switch (tile_cfg) {
    case TILE_256x256: case TILE_256x256_W4: case TILE_256x256_W4_MFMA32: case TILE_ROWS256: case TILE_ROWS160: *bm = 256; *bn = 256; break;
    case TILE_128x128: *bm = 128; *bn = 128; break;
    case TILE_128x256: case TILE_ROWS128: *bm = 128; *bn = 256; break;
    default: *bm = 64; *bn = 128; break;
  }
}

}  // namespace msco
