// What the persistent four-wave tile kernels share: the tile and LDS ring geometry (256 x 256 output tiles, 128-byte K
// slabs, two LDS stages per operand), buffer descriptors, the LDS-direct loads of the epilogue operands, and the tile
// walk over group_list that is done once per launch and kept in LDS.
#pragma once

#include "gmm_common.h"

#ifndef MSCO_TILE4_ATTR
#define MSCO_TILE4_ATTR 0   // attribution builds only: see gmm_tile4_w8a8.hip
#endif

namespace msco {
namespace {

constexpr int T4_BM = 256, T4_BN = 256;
constexpr int T4_BK = 128;                       // bytes of K per slab and LDS row
constexpr int T4_NW = 4;                         // wavefronts: 2 (m) x 2 (n)
constexpr int T4_WT = 128;                       // wave tile edge
constexpr int T4_OP_STAGE = T4_BM * T4_BK;       // one operand's share of a stage (32 KiB)
constexpr int T4_W_BASE = 2 * T4_OP_STAGE;       // x stages 0 and 1, then weight stages 0 and 1: a stage and a block offset
                                                 // together fit the 16-bit offset field of an LDS instruction
constexpr int T4_RING = 2 * T4_W_BASE;           // 128 KiB
constexpr int T4_LD = T4_BM / 8 / T4_NW;         // staging quads (8 rows x 128 B per wave) per operand and slab
constexpr int T4_PARAM_OFF = T4_RING;            // epilogue operand tables (scale, bias, per-token; two tiles) behind the ring
constexpr int T4_PARAM_BYTES = 3 * 1024;
constexpr int T4_MAX_E = 1024;
constexpr int T4_MAX_WGS = 256;                  // one persistent workgroup per CU
constexpr unsigned T4_OOB = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t t4_rsrc(const void *base, long long bytes) {
  const unsigned n = bytes > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

// Publishes LDS data and retires a stage: the caller has waited for its own LDS traffic.
__device__ __forceinline__ void t4_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Raw buffer descriptor as four scalars (for hand-written buffer instructions).
__device__ __forceinline__ v4i t4_raw_rsrc(const void *base, long long bytes) {
  const unsigned long long a = (unsigned long long)base;
  const unsigned n = bytes > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)(bytes < 0 ? 0 : bytes);
  v4i r;
  r.x = __builtin_amdgcn_readfirstlane((int)(unsigned)a);
  r.y = __builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xFFFFu));
  r.z = __builtin_amdgcn_readfirstlane((int)n);
  r.w = 0x00020000;
  return r;
}

// One dword (or zero-extended 16 bits) per lane from a buffer straight into LDS: lane L writes
// lds_addr + 4 L.  Hand-written so that the compiler's wait-count bookkeeping never sees an LDS
// write in flight (it would make every later LDS read wait for all outstanding loads); the
// counter it does not know about can only make its own waits longer, never shorter, because
// vector memory operations complete in order.
__device__ __forceinline__ void t4_dma_b32(v4i rsrc, unsigned lds_addr, unsigned voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voffset), "s"(rsrc) : "memory");
}
__device__ __forceinline__ void t4_dma_b16(v4i rsrc, unsigned lds_addr, unsigned voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ushort %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voffset), "s"(rsrc) : "memory");
}

// A tile as the whole workgroup sees it (all fields wave-uniform).
struct T4Tile {
  int valid;
  int grp, m0, n0, g_end;
};

// Tile lid -> (group, m-tile, n-tile).  The group walk was done once at kernel start and left in LDS
// (row end and inclusive tile count per group): reading group_list from memory again for every tile
// would put loads into the middle of the operand stream, and vector loads complete in order.
// Order inside a group: panels of 8 m-tiles; inside a panel n-tile major, m-tile minor, so that
// workgroups that run side by side share one streamed weight panel.
__device__ __forceinline__ T4Tile t4_locate(const int *meta_end, const int *meta_upto, int e, int lid, int total,
                                            int n_tiles, int lane) {
  T4Tile t{0, 0, 0, 0, 0};
  if (lid < 0 || lid >= total) return t;
  int g_start = 0, t_in_group = 0;
  for (int g0 = 0; g0 < e; g0 += 64) {
    const int g = g0 + lane;
    const int upto = g < e ? meta_upto[g] : 0x7FFFFFFF;
    const int first = __popcll(__ballot(upto <= lid));              // `upto` is non-decreasing: first group beyond lid
    if (first < 64) {
      const int grp = g0 + first;
      t.grp = grp;
      t.g_end = __builtin_amdgcn_readfirstlane(meta_end[grp]);
      g_start = grp > 0 ? __builtin_amdgcn_readfirstlane(meta_end[grp - 1]) : 0;
      t_in_group = lid - (grp > 0 ? __builtin_amdgcn_readfirstlane(meta_upto[grp - 1]) : 0);
      t.valid = 1;
      break;
    }
  }
  constexpr int PANEL = 8;
  const int m_tiles = (t.g_end - g_start + T4_BM - 1) / T4_BM;
  const int panel_tiles = PANEL * n_tiles;
  const int panel = t_in_group / panel_tiles;
  const int in_panel = t_in_group - panel * panel_tiles;
  const int panel_m = max(1, min(PANEL, m_tiles - panel * PANEL));
  const int nt = in_panel / panel_m;
  const int mt = panel * PANEL + in_panel % panel_m;
  t.m0 = g_start + mt * T4_BM;
  t.n0 = nt * T4_BN;
  return t;
}

}  // namespace
}  // namespace msco
