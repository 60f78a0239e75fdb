// Grouped W8A8 GEMM, MFMA tile kernel (prefill shapes) for gfx950.
//
// One workgroup computes one BM x BN output tile of one group with v_mfma_i32_16x16x64_i8.  The
// large configuration uses 8 wavefronts (2 x 4, two per SIMD, a 128 x 64 sub-tile of accumulators
// each), so that one wave's LDS reads, LDS writes and barrier waits are covered by the other wave's
// MFMAs; the small configurations use 4 wavefronts (2 x 2).
//
//   * Tile scheduling on the device.  The tile -> (group, m-tile, n-tile) mapping is computed by
//     walking group_list, so the host never reads it; the grid is sized from an upper bound and
//     surplus workgroups exit.  Consecutive tiles (same group, neighbouring n-tiles, all m-tiles of a
//     panel) are dealt to the same XCD so that the x rows of a group and the streamed weight panel
//     stay in that XCD's L2.
//   * Memory.  Operands are read through buffer descriptors (scalar base, one per-lane offset,
//     out-of-range rows read as zero, so no clamping or branching in the loop) in 128-byte K slabs.
//     Slab t+1 is in flight in registers while slab t is multiplied out of LDS; it is written to the
//     other LDS stage at the end of the iteration, behind an LDS-only barrier.
//   * Weights stored [K,N] are transposed into K-contiguous MFMA fragments with v_perm_b32 on the
//     way into LDS; weights stored [N,K] are copied as they are.
//   * The dequant epilogue (int32 bias, per-channel scale, per-token scale, bf16/f16 cast) is fused;
//     every lane owns FN consecutive output columns of a row and stores them with one vector store.
//
// LDS layouts (every fragment read is 16 lanes x 16 B over consecutive rows -> conflict free):
//   x rows and [N,K] weights: row-major, 128 B per row, 16-byte chunk c of row r stored at chunk
//     position c ^ swz(r);
//   [K,N] weights: chunk-major, address = (c * BN + slot) * 16.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

constexpr int BK = 128;           // bytes of K per LDS slab

typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int swz_a(int r) { return (r >> 1) & 7; }
__device__ __forceinline__ int swz_b(int r) { return ((r >> 1) ^ (r >> 4)) & 7; }

// LDS-only barrier: waits for this wave's LDS traffic, not for global loads still in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, long long bytes) {
  const unsigned n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (unsigned)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool NK>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64) gmm_w8a8_tile_kernel(const GmmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int FM = WTM / 16, FN = WTN / 16;
  constexpr int ROWS_IT = NT / 8;                   // rows covered by one pass of 16-byte chunk loads
  constexpr int A_IT = BM * 8 / NT;                 // 16-byte chunks of the x slab per thread
  constexpr int B_IT = BN * 8 / NT;                 // same for an [N,K] weight slab
  constexpr int PANEL = 8;                          // m-tiles that share a streamed weight panel
  constexpr unsigned OOB = 0x80000000u;             // buffer offset that always reads zero
  // [K,N] weight slab: 8 K-chunks x BN/4 column groups of 16(k) x 4(n)-byte blocks, one per thread
  static_assert(NT == 2 * BN, "one [K,N] block per thread");
  static_assert(FM >= 1 && FN >= 1 && A_IT >= 1 && B_IT >= 1 && ROWS_IT % 16 == 0, "tile shape");

  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char *lds_a = smem;                      // [2][BM * BK]
  unsigned char *lds_b = smem + 2 * BM * BK;        // [2][BN * BK]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int lane16 = lane & 15, h = lane >> 4;

  // ---- tile lookup: walk group_list twice (count, then locate) -------------------------------
  const int n_tiles = (p.n + BN - 1) / BN;
  int total = 0;
  {
    int prev = 0;
    for (int g = 0; g < p.e; ++g) {
      const int end = group_end(p, g, prev);
      total += ((end - prev + BM - 1) / BM) * n_tiles;
      prev = end;
    }
  }
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const int local = blockIdx.x / kNumXcd;
  if (local >= per_xcd) return;
  const int lid = (blockIdx.x % kNumXcd) * per_xcd + local;
  if (lid >= total) return;

  int grp = 0, g_start = 0, g_end = 0, t_in_group = 0;
  {
    int prev = 0, acc = 0;
    for (int g = 0; g < p.e; ++g) {
      const int end = group_end(p, g, prev);
      const int tiles = ((end - prev + BM - 1) / BM) * n_tiles;
      if (lid < acc + tiles) {
        grp = g; g_start = prev; g_end = end; t_in_group = lid - acc;
        break;
      }
      acc += tiles;
      prev = end;
    }
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
  const int k_slabs = (p.k + BK - 1) / BK;
  const bool k_tail = (p.k % BK) != 0;

  // Buffer descriptors start at this tile's first x row / weight column, so per-lane offsets stay
  // small; anything past the end of the tensor reads as zero (no clamping, no branches in the loop).
  const long long w_elems = (long long)p.k * p.n;
  const int8_t *wg = p.w + (long long)grp * w_elems;
  const __amdgpu_buffer_rsrc_t rx =
    make_rsrc(reinterpret_cast<const int8_t *>(p.x) + (long long)m0 * p.k, (long long)(p.m - m0) * p.k);
  const __amdgpu_buffer_rsrc_t rw = NK ? make_rsrc(wg + (long long)n0 * p.k, (long long)(p.n - n0) * p.k)
                                       : make_rsrc(wg + n0, w_elems - n0);

  // ---- per-thread load / store coordinates ----------------------------------------------------
  const int a_row = tid >> 3, a_c = tid & 7;        // + ROWS_IT rows per iteration
  const unsigned a_voff = (unsigned)a_row * (unsigned)p.k + a_c * 16;
  const unsigned a_lds = a_row * BK + ((a_c ^ swz_a(a_row)) << 4);   // + it * ROWS_IT * BK (swz_a has period 16 rows)
  const unsigned bnk_voff = a_voff;
  const int kn_i = tid % (BN / 4), kn_kc = tid / (BN / 4);
  const unsigned bkn_voff = (unsigned)(16 * kn_kc) * (unsigned)p.n + 4 * kn_i;

  v4u ra[A_IT];
  v4u rb[NK ? B_IT : 1];
  unsigned rkn[NK ? 1 : 16];

  auto load_slab = [&](int kt) {
    const unsigned kbase = kt * BK;
    unsigned av = a_voff, bv = bnk_voff;
    if (k_tail && kbase + a_c * 16 >= (unsigned)p.k) { av = OOB; }
#pragma unroll
    for (int it = 0; it < A_IT; ++it)
      ra[it] = __builtin_amdgcn_raw_buffer_load_b128(rx, av, kbase + it * ROWS_IT * p.k, 0);
    if constexpr (NK) {
#pragma unroll
      for (int it = 0; it < B_IT; ++it)
        rb[it] = __builtin_amdgcn_raw_buffer_load_b128(rw, bv, kbase + it * ROWS_IT * p.k, 0);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) rkn[r] = __builtin_amdgcn_raw_buffer_load_b32(rw, bkn_voff, (kbase + r) * p.n, 0);
    }
  };

  auto store_slab = [&](int buf) {
    unsigned char *a = lds_a + buf * (BM * BK);
    unsigned char *b = lds_b + buf * (BN * BK);
#pragma unroll
    for (int it = 0; it < A_IT; ++it) *reinterpret_cast<v4u *>(a + a_lds + it * ROWS_IT * BK) = ra[it];
    if constexpr (NK) {
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        const int row = a_row + ROWS_IT * it;
        const int wn = row / WTN, nn = row % WTN;
        const int l16 = nn / FN, j = nn % FN;
        const int rho = wn * WTN + j * 16 + (l16 ^ (j & 1));
        *reinterpret_cast<v4u *>(b + rho * BK + ((a_c ^ swz_b(rho)) << 4)) = rb[it];
      }
    } else {
      // 16(k) x 4(n) byte block -> 4 column fragments of 16 K bytes
      v4i frag[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        unsigned c0, c1, c2, c3;
        transpose4x4(rkn[4 * q], rkn[4 * q + 1], rkn[4 * q + 2], rkn[4 * q + 3], c0, c1, c2, c3);
        frag[0][q] = (int)c0; frag[1][q] = (int)c1; frag[2][q] = (int)c2; frag[3][q] = (int)c3;
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int nl = 4 * kn_i + jj;
        const int wn = nl / WTN, nn = nl % WTN;
        const int slot = wn * WTN + (nn % FN) * 16 + nn / FN;
        *reinterpret_cast<v4i *>(b + ((kn_kc * BN + slot) << 4)) = frag[jj];
      }
    }
  };

  // ---- fragment reads (one 16-byte LDS read per lane and fragment) ----------------------------
  auto read_a = [&](int buf, int s, int i) -> v4i {
    const unsigned char *a = lds_a + buf * (BM * BK);
    const int row = wave_m * WTM + 16 * i + lane16;
    return *reinterpret_cast<const v4i *>(a + row * BK + (((4 * s + h) ^ swz_a(row)) << 4));
  };
  auto read_b = [&](int buf, int s, int j) -> v4i {
    const unsigned char *b = lds_b + buf * (BN * BK);
    const int c = 4 * s + h;
    if constexpr (NK) {
      const int rho = wave_n * WTN + 16 * j + (lane16 ^ (j & 1));
      return *reinterpret_cast<const v4i *>(b + rho * BK + ((c ^ swz_b(rho)) << 4));
    } else {
      const int slot = wave_n * WTN + 16 * j + lane16;
      return *reinterpret_cast<const v4i *>(b + ((c * BN + slot) << 4));
    }
  };

  v4i acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

  // ---- main loop ---------------------------------------------------------------------------------
  // registers: slab t+1 in flight | LDS stage t&1: slab t being multiplied | stage (t+1)&1: written at the end
  load_slab(0);
  store_slab(0);
  lds_barrier();
  for (int kt = 0; kt < k_slabs; ++kt) {
    const int buf = kt & 1;
    const bool has_next = kt + 1 < k_slabs;
    if (has_next) load_slab(kt + 1);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      v4i af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = read_a(buf, s, i);
#pragma unroll
      for (int j = 0; j < FN; ++j) bf[j] = read_b(buf, s, j);
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (has_next) {
      // every wave has finished reading stage buf^1 (it was the multiplied stage of iteration t-1,
      // and the barrier below closed that iteration), so it can be overwritten now
      store_slab(buf ^ 1);
    }
    lds_barrier();
  }

  // ---- fused dequant epilogue --------------------------------------------------------------------
  const int nb = n0 + wave_n * WTN + FN * lane16;   // first of this lane's FN consecutive columns
  if (nb >= p.n) return;
  float sc[FN];
  int bi[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int n = min(nb + j, p.n - 1);
    sc[j] = load_scale(p, grp, n);
    bi[j] = load_bias(p, grp, n);
  }
  const bool full = (nb + FN <= p.n);
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + wave_m * WTM + 16 * i + 4 * h + r;
      if (m >= g_end) continue;
      const float pt = p.per_token ? p.per_token[m] : 1.0f;
      const long long base = (long long)m * p.n + nb;
      if (p.out_dtype == DT_I32) {
        int *o = reinterpret_cast<int *>(p.out) + base;
        if (full && (FN % 4 == 0)) {
#pragma unroll
          for (int j = 0; j < FN; j += 4)
            *reinterpret_cast<int4 *>(o + j) = make_int4(acc[i][j][r] + bi[j], acc[i][j + 1][r] + bi[j + 1],
                                                         acc[i][j + 2][r] + bi[j + 2], acc[i][j + 3][r] + bi[j + 3]);
        } else {
#pragma unroll
          for (int j = 0; j < FN; ++j)
            if (nb + j < p.n) o[j] = acc[i][j][r] + bi[j];
        }
      } else {
        unsigned short hv[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const float f = dequant(acc[i][j][r] + bi[j], sc[j], pt);
          hv[j] = (p.out_dtype == DT_BF16) ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
        }
        unsigned short *o = reinterpret_cast<unsigned short *>(p.out) + base;
        if (full && (FN % 8 == 0)) {
#pragma unroll
          for (int j = 0; j < FN; j += 8) {
            uint4 v;
            v.x = hv[j] | ((unsigned)hv[j + 1] << 16);
            v.y = hv[j + 2] | ((unsigned)hv[j + 3] << 16);
            v.z = hv[j + 4] | ((unsigned)hv[j + 5] << 16);
            v.w = hv[j + 6] | ((unsigned)hv[j + 7] << 16);
            *reinterpret_cast<uint4 *>(o + j) = v;
          }
        } else if (full && (FN % 4 == 0)) {
#pragma unroll
          for (int j = 0; j < FN; j += 4) {
            uint2 v;
            v.x = hv[j] | ((unsigned)hv[j + 1] << 16);
            v.y = hv[j + 2] | ((unsigned)hv[j + 3] << 16);
            *reinterpret_cast<uint2 *>(o + j) = v;
          }
        } else {
#pragma unroll
          for (int j = 0; j < FN; ++j)
            if (nb + j < p.n) o[j] = hv[j];
        }
      }
    }
  }
}

// ---- host launcher ---------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, bool NK>
static hipError_t launch_cfg(const GmmParams &p, hipStream_t stream) {
  const size_t lds = 2 * (size_t)(BM + BN) * BK;
  auto kern = gmm_w8a8_tile_kernel<BM, BN, WAVES_M, WAVES_N, NK>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const long long n_tiles = (p.n + BN - 1) / BN;
  const long long m_tiles_ub = (p.m + BM - 1) / BM + p.e;   // every non-empty group adds at most one partial tile
  const long long total_ub = m_tiles_ub * n_tiles;
  const long long grid = ((total_ub + kNumXcd - 1) / kNumXcd) * kNumXcd;
  if (grid <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES_M * WAVES_N * 64), lds, stream, p);
  return hipGetLastError();
}

hipError_t launch_tile_w8a8(const GmmParams &p, int tile_cfg, bool nk, hipStream_t stream) {
  switch (tile_cfg) {
    case TILE_256x256:
      return nk ? launch_cfg<256, 256, 2, 4, true>(p, stream) : launch_cfg<256, 256, 2, 4, false>(p, stream);
    case TILE_128x128:
      return nk ? launch_cfg<128, 128, 2, 2, true>(p, stream) : launch_cfg<128, 128, 2, 2, false>(p, stream);
    case TILE_64x128:
      return nk ? launch_cfg<64, 128, 2, 2, true>(p, stream) : launch_cfg<64, 128, 2, 2, false>(p, stream);
    default:
      return hipErrorInvalidValue;
  }
}

const char *tile_cfg_name(int tile_cfg) {
  switch (tile_cfg) {
    case TILE_256x256: return "256x256x128";
    case TILE_128x128: return "128x128x128";
    case TILE_64x128: return "64x128x128";
    default: return "?";
  }
}

void tile_cfg_dims(int tile_cfg, int *bm, int *bn) {
  switch (tile_cfg) {
    case TILE_256x256: *bm = 256; *bn = 256; break;
    case TILE_128x128: *bm = 128; *bn = 128; break;
    default: *bm = 64; *bn = 128; break;
  }
}

}  // namespace msco
