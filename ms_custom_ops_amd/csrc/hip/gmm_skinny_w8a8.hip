// Grouped W8A8 GEMM, skinny (decode) kernel for gfx950: HBM-bound weight streaming.
//
// A workgroup owns (group g, 128-column strip, K split ks).  Its waves take interleaved 64-row
// K blocks of the strip, so the reduction over K is split across wavefronts:
//   * each wave streams its 64 x 128 byte weight blocks straight from HBM into registers (row
//     segments of 128 contiguous bytes), turns them into K-contiguous MFMA fragments with
//     v_perm_b32 ([K,N] storage) or uses them as loaded ([N,K] storage), and multiplies them with a
//     16-row x fragment (rows beyond the group are clamped and never stored) using
//     v_mfma_i32_16x16x64_i8;
//   * the waves' int32 partial tiles are added through LDS; with split_k > 1 the workgroups'
//     partial tiles go to the workspace and the last workgroup to arrive (arrival counter) adds
//     them and runs the epilogue.  int32 addition is associative, so the result is bit-exact
//     whatever the arrival order;
//   * empty groups exit before touching their weights.
// Groups with more than 16 rows are processed in 16-row chunks that re-stream the strip (from L2);
// split_k > 1 is only planned when M <= 16, so a workgroup then has exactly one chunk.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

constexpr int SK_WAVES = 4;
constexpr int SK_THREADS = SK_WAVES * 64;
constexpr int SK_PREFETCH = 2;  // weight blocks in flight per wave

template <bool NK>
__device__ __forceinline__ void skinny_load_block(const GmmParams &p, const int8_t *wg, int n0, int k0, int lane16,
                                                  int h, uint2 (&rr)[16], v4i (&bf)[8]) {
  if constexpr (NK) {
    const int kk = min(k0 + 16 * h, p.k - 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int nrow = min(n0 + 8 * lane16 + j, p.n - 1);
      bf[j] = *reinterpret_cast<const v4i *>(wg + (long long)nrow * p.k + kk);
    }
  } else {
    const int col = min(n0 + 8 * lane16, p.n - 8);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int krow = min(k0 + 16 * h + r, p.k - 1);
      rr[r] = *reinterpret_cast<const uint2 *>(wg + (long long)krow * p.n + col);
    }
  }
}

template <bool NK>
__global__ void __launch_bounds__(SK_THREADS, 2) gmm_w8a8_skinny_kernel(const GmmParams p) {
  __shared__ int red[SK_WAVES][kSkinnyRows][kSkinnyCols + 4];
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lane16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, grp = blockIdx.y, ks = blockIdx.z;

  int g_start = 0, g_end = 0;
  for (int g = 0; g <= grp; ++g) {
    g_start = g_end;
    g_end = group_end(p, g, g_start);
  }
  const int rows = g_end - g_start;
  if (rows <= 0) return;

  const int n0 = strip * kSkinnyCols;
  const int8_t *xg = reinterpret_cast<const int8_t *>(p.x);
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const int k_blocks = (p.k + 63) / 64;
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const int chunks = (rows + kSkinnyRows - 1) / kSkinnyRows;

  for (int mc = 0; mc < chunks; ++mc) {
    v4i acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = v4i{0, 0, 0, 0};
    const int mrow = min(g_start + mc * kSkinnyRows + lane16, g_end - 1);
    const int8_t *xrow = xg + (long long)mrow * p.k;

    // software pipeline: SK_PREFETCH blocks of weights in flight per wave
    uint2 rr[SK_PREFETCH][16];
    v4i bq[SK_PREFETCH][8];
    v4i aq[SK_PREFETCH];
    int kb = kb_begin + wave;
#pragma unroll
    for (int s = 0; s < SK_PREFETCH; ++s) {
      const int kbs = kb + s * SK_WAVES;
      if (kbs < kb_end) {
        const int k0 = kbs * 64;
        skinny_load_block<NK>(p, wg, n0, k0, lane16, h, rr[s], bq[s]);
        const int kk = k0 + 16 * h;
        aq[s] = (kk < p.k) ? *reinterpret_cast<const v4i *>(xrow + kk) : v4i{0, 0, 0, 0};
      }
    }
    for (; kb < kb_end; kb += SK_PREFETCH * SK_WAVES) {
#pragma unroll
      for (int s = 0; s < SK_PREFETCH; ++s) {
        const int kbs = kb + s * SK_WAVES;
        if (kbs < kb_end) {
          v4i bf[8];
          if constexpr (NK) {
#pragma unroll
            for (int j = 0; j < 8; ++j) bf[j] = bq[s][j];
          } else {
            transpose16x8(rr[s], bf);
          }
          const v4i af = aq[s];
          // refill this pipeline slot before the MFMAs so the loads overlap them
          const int kbn = kbs + SK_PREFETCH * SK_WAVES;
          if (kbn < kb_end) {
            const int k0 = kbn * 64;
            skinny_load_block<NK>(p, wg, n0, k0, lane16, h, rr[s], bq[s]);
            const int kk = k0 + 16 * h;
            aq[s] = (kk < p.k) ? *reinterpret_cast<const v4i *>(xrow + kk) : v4i{0, 0, 0, 0};
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, bf[j], acc[j], 0, 0, 0);
        }
      }
    }

    // ---- reduce the waves' partial tiles through LDS ------------------------------------------
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][4 * h + r][8 * lane16 + j] = acc[j][r];
    __syncthreads();

    const int row = tid >> 4, c8 = (tid & 15) * 8;
    int v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int s = 0;
#pragma unroll
      for (int w = 0; w < SK_WAVES; ++w) s += red[w][row][c8 + j];
      v[j] = s;
    }
    const int m = g_start + mc * kSkinnyRows + row;
    const bool row_ok = (m < g_end);
    bool do_epilogue = true;

    if (p.split_k > 1) {
      // ---- cross-workgroup reduction through the workspace ------------------------------------
      const long long tile = (long long)grp * p.n_strips + strip;
      int *mine = p.partial + ((tile * p.split_k + ks) * kSkinnyRows + row) * kSkinnyCols + c8;
      // Partial tiles and the arrival counter are exchanged with agent-scope atomic accesses: they
      // bypass the per-XCD L2 for this data only, so no cache-wide write-back / invalidate fence is
      // needed.  The stores are complete (vmcnt == 0) before the counter is bumped.
      if (row_ok) {
#pragma unroll
        for (int j = 0; j < 8; ++j) __hip_atomic_store(mine + j, v[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      do_epilogue = (s_ticket == (unsigned)(p.split_k - 1));
      if (do_epilogue) {
        if (row_ok) {
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = 0;
          for (int s = 0; s < p.split_k; ++s) {
            const int *src = p.partial + ((tile * p.split_k + s) * kSkinnyRows + row) * kSkinnyCols + c8;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] += __hip_atomic_load(src + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }

    if (do_epilogue && row_ok) {
      const int nb = n0 + c8;
      if (nb < p.n) {
        const float pt = p.per_token ? p.per_token[m] : 1.0f;
        const long long base = (long long)m * p.n + nb;
        if (p.out_dtype == DT_I32) {
          int *o = reinterpret_cast<int *>(p.out) + base;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (nb + j < p.n) o[j] = v[j] + load_bias(p, grp, nb + j);
        } else {
          unsigned short hv[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int n = min(nb + j, p.n - 1);
            const float f = dequant(v[j] + load_bias(p, grp, n), load_scale(p, grp, n), pt);
            hv[j] = (p.out_dtype == DT_BF16) ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
          }
          unsigned short *o = reinterpret_cast<unsigned short *>(p.out) + base;
          if (nb + 8 <= p.n) {
            uint4 q;
            q.x = hv[0] | ((unsigned)hv[1] << 16);
            q.y = hv[2] | ((unsigned)hv[3] << 16);
            q.z = hv[4] | ((unsigned)hv[5] << 16);
            q.w = hv[6] | ((unsigned)hv[7] << 16);
            *reinterpret_cast<uint4 *>(o) = q;
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (nb + j < p.n) o[j] = hv[j];
          }
        }
      }
    }
    __syncthreads();  // red[] is reused by the next chunk
  }
}

size_t skinny_workspace_bytes(int64_t m, int64_t n, int64_t e, int split_k, bool fp32_partials) {
  (void)m; (void)fp32_partials;
  if (split_k <= 1) return 0;
  const int64_t strips = (n + kSkinnyCols - 1) / kSkinnyCols;
  // one 16 x 128 tile of 4-byte partial sums plus 16 row sums (weight-only path) per (group, strip, split)
  return (size_t)(e * strips * split_k * (kSkinnyRows * kSkinnyCols + kSkinnyRows) * 4);
}

size_t skinny_counter_count(int64_t n, int64_t e) {
  const int64_t strips = (n + kSkinnyCols - 1) / kSkinnyCols;
  return (size_t)(e * strips);
}

hipError_t launch_skinny_w8a8(const GmmParams &p, bool nk, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const dim3 grid((unsigned)p.n_strips, (unsigned)p.e, (unsigned)p.split_k);
  if (nk) {
    hipLaunchKernelGGL(gmm_w8a8_skinny_kernel<true>, grid, dim3(SK_THREADS), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_w8a8_skinny_kernel<false>, grid, dim3(SK_THREADS), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace msco
