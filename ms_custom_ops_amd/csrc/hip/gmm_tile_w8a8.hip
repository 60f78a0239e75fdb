// Grouped W8A8 GEMM, MFMA tile kernel (prefill shapes) for gfx950.
//
// One workgroup computes one BM x BN output tile of one group with v_mfma_i32_16x16x64_i8:
//   * the tile -> (group, m-tile, n-tile) mapping is computed on the device by walking group_list,
//     so the host never reads it; the grid is sized from an upper bound and surplus workgroups exit;
//   * consecutive tiles (same group, neighbouring n-tiles, all m-tiles of a panel) are dealt to the
//     same XCD so that the x rows of a group and the streamed weight panel stay in that XCD's L2;
//   * A (x rows) and B (weights) K-slabs of 128 bytes are staged through LDS with a register
//     double buffer (global loads of slab t+1 overlap the MFMAs of slab t);
//   * weights stored [K,N] are transposed to K-contiguous fragments with v_perm_b32 on the way into
//     LDS; weights stored [N,K] are copied as they are;
//   * the dequant epilogue (int32 bias, per-channel scale, per-token scale, bf16/f16 cast) is fused.
//
// LDS layouts (all fragment reads are 16 lanes x 16 B over consecutive rows -> conflict free):
//   A and [N,K] weights: row-major, 128 B per row, 16-B chunk c of row r stored at chunk position
//     c ^ swz(r), swz(r) = ((r >> 1) ^ (r >> 4)) & 7.
//   [K,N] weights: chunk-major, address = (c * BN + slot) * 16.
// Output columns are assigned to MFMA fragments so that lane (l % 16) of fragment j owns column
// FN * (l % 16) + j: every lane ends up with FN consecutive columns of a row and stores them with
// one vector store.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

constexpr int BK = 128;  // bytes of K per LDS slab

__device__ __forceinline__ int swz(int r) { return ((r >> 1) ^ (r >> 4)) & 7; }

template <int BM, int BN, int WAVES_M, int WAVES_N, bool NK>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64) gmm_w8a8_tile_kernel(const GmmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int FM = WTM / 16, FN = WTN / 16;
  constexpr int A_IT = BM * 8 / NT;                 // 16-B chunks of the A slab per thread
  constexpr int B_IT = BN * 8 / NT;                 // same for an [N,K] B slab
  constexpr int KN_BLOCKS = BN;                     // 16x8-byte blocks in a [K,N] B slab
  constexpr int KN_IT = (KN_BLOCKS + NT - 1) / NT;
  constexpr int PANEL = 8;                          // m-tiles that share a streamed weight panel
  static_assert(BM % (WAVES_M * 16) == 0 && BN % (WAVES_N * 16) == 0, "tile shape");
  static_assert(A_IT >= 1 && B_IT >= 1, "tile too small for the workgroup");

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
  const int8_t *xg = reinterpret_cast<const int8_t *>(p.x);
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const int k_slabs = (p.k + BK - 1) / BK;

  // ---- global -> register staging ------------------------------------------------------------
  int4 ra[A_IT];
  int4 rb[NK ? B_IT : 1];
  uint2 rkn[NK ? 1 : KN_IT][16];

  auto load_slab = [&](int kt) {
#pragma unroll
    for (int it = 0; it < A_IT; ++it) {
      const int idx = tid + NT * it;
      const int row = idx >> 3, c = idx & 7;
      const int kk = kt * BK + c * 16;
      const int gr = min(m0 + row, p.m - 1);
      int4 v = make_int4(0, 0, 0, 0);
      if (kk < p.k) v = *reinterpret_cast<const int4 *>(xg + (long long)gr * p.k + kk);
      ra[it] = v;
    }
    if constexpr (NK) {
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        const int idx = tid + NT * it;
        const int row = idx >> 3, c = idx & 7;
        const int kk = min(kt * BK + c * 16, p.k - 16);
        const int gn = min(n0 + row, p.n - 1);
        rb[it] = *reinterpret_cast<const int4 *>(wg + (long long)gn * p.k + kk);
      }
    } else {
#pragma unroll
      for (int it = 0; it < KN_IT; ++it) {
        const int blk = tid + NT * it;
        if (KN_BLOCKS % NT == 0 || blk < KN_BLOCKS) {
          const int i = blk % (BN / 8), kc = blk / (BN / 8);
          const int gn = min(n0 + 8 * i, p.n - 8);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int gk = min(kt * BK + 16 * kc + r, p.k - 1);
            rkn[it][r] = *reinterpret_cast<const uint2 *>(wg + (long long)gk * p.n + gn);
          }
        }
      }
    }
  };

  auto store_slab = [&](int buf) {
    unsigned char *a = lds_a + buf * (BM * BK);
    unsigned char *b = lds_b + buf * (BN * BK);
#pragma unroll
    for (int it = 0; it < A_IT; ++it) {
      const int idx = tid + NT * it;
      const int row = idx >> 3, c = idx & 7;
      *reinterpret_cast<int4 *>(a + row * BK + ((c ^ swz(row)) << 4)) = ra[it];
    }
    if constexpr (NK) {
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        const int idx = tid + NT * it;
        const int row = idx >> 3, c = idx & 7;
        const int wn = row / WTN, nn = row % WTN;
        const int l16 = nn / FN, j = nn % FN;
        const int rho = wn * WTN + j * 16 + (l16 ^ (j & 1));
        *reinterpret_cast<int4 *>(b + rho * BK + ((c ^ swz(rho)) << 4)) = rb[it];
      }
    } else {
#pragma unroll
      for (int it = 0; it < KN_IT; ++it) {
        const int blk = tid + NT * it;
        if (KN_BLOCKS % NT == 0 || blk < KN_BLOCKS) {
          const int i = blk % (BN / 8), kc = blk / (BN / 8);
          v4i frag[8];
          transpose16x8(rkn[it], frag);
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const int nl = 8 * i + jj;
            const int wn = nl / WTN, nn = nl % WTN;
            const int slot = wn * WTN + (nn % FN) * 16 + nn / FN;
            *reinterpret_cast<v4i *>(b + ((kc * BN + slot) << 4)) = frag[jj];
          }
        }
      }
    }
  };

  // ---- main loop -------------------------------------------------------------------------------
  v4i acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

  load_slab(0);
  store_slab(0);
  __syncthreads();

  for (int kt = 0; kt < k_slabs; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < k_slabs) load_slab(kt + 1);

    const unsigned char *a = lds_a + buf * (BM * BK);
    const unsigned char *b = lds_b + buf * (BN * BK);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c = 4 * s + h;
      v4i af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int row = wave_m * WTM + 16 * i + lane16;
        af[i] = *reinterpret_cast<const v4i *>(a + row * BK + ((c ^ swz(row)) << 4));
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (NK) {
          const int rho = wave_n * WTN + 16 * j + (lane16 ^ (j & 1));
          bf[j] = *reinterpret_cast<const v4i *>(b + rho * BK + ((c ^ swz(rho)) << 4));
        } else {
          const int slot = wave_n * WTN + 16 * j + lane16;
          bf[j] = *reinterpret_cast<const v4i *>(b + ((c * BN + slot) << 4));
        }
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }

    if (kt + 1 < k_slabs) store_slab(buf ^ 1);
    __syncthreads();
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
#pragma unroll
        for (int j = 0; j < FN; ++j)
          if (full || nb + j < p.n) o[j] = acc[i][j][r] + bi[j];
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
  constexpr int NT = WAVES_M * WAVES_N * 64;
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
  long long total_ub = m_tiles_ub * n_tiles;
  long long grid = ((total_ub + kNumXcd - 1) / kNumXcd) * kNumXcd;
  if (grid <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, stream, p);
  return hipGetLastError();
}

hipError_t launch_tile_w8a8(const GmmParams &p, int tile_cfg, bool nk, hipStream_t stream) {
  switch (tile_cfg) {
    case TILE_256x256:
      return nk ? launch_cfg<256, 256, 2, 2, true>(p, stream) : launch_cfg<256, 256, 2, 2, false>(p, stream);
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
