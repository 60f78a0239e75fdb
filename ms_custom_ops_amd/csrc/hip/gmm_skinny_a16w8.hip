// Grouped weight-only (bf16/f16 activations x int8 weights) GEMM, skinny decode kernel for gfx950.
//
// Same work decomposition as the W8A8 skinny kernel: a workgroup owns (group, 128-column strip,
// K split), its waves take interleaved 64-row K blocks and stream the int8 weights [K,N] from HBM.
// The int8 bytes are turned into exact bf16/f16 values of (w + 128) in registers
// (v_cvt_f32_ubyteN on w ^ 0x80, then a 16-bit pack), multiplied with v_mfma_f32_16x16x32_{bf16,f16}
// and accumulated in float32.  A second MFMA against an all-ones fragment yields sum_k x[m,k], so
// the per-channel antiquant offset and the +128 bias fold into the epilogue:
//
//   out[m,n] = s[g,n] * ( sum_k x[m,k]*(w[k,n]+128)  +  (o[g,n] - 128) * sum_k x[m,k] )
//            = sum_k x[m,k] * (w[k,n] + o[g,n]) * s[g,n]
//
// Partial sums are combined in a fixed order (wave 0..3, then split 0..S-1), so results are
// reproducible run to run.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

constexpr int AW_WAVES = 4;
constexpr int AW_THREADS = AW_WAVES * 64;
constexpr int AW_TILE_FLOATS = kSkinnyRows * kSkinnyCols + kSkinnyRows;  // tile + row sums

typedef _Float16 v8h __attribute__((ext_vector_type(8)));

template <bool BF16>
__device__ __forceinline__ unsigned pack2(float lo, float hi) {
  if constexpr (BF16) {
    // both values are integers below 256: the upper 16 bits of the float32 pattern are the exact bf16
    return perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
  } else {
    return __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
}

template <bool BF16>
__device__ __forceinline__ v4f mfma16(const v4i &a, const v4i &b, const v4f &c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0,
                                                   0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
}

template <bool BF16>
__device__ __forceinline__ float half_like_to_f32(unsigned short b) {
  return BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}

template <bool BF16>
__global__ void __launch_bounds__(AW_THREADS, 2) gmm_a16w8_skinny_kernel(const GmmParams p) {
  __shared__ float red[AW_WAVES][kSkinnyRows][kSkinnyCols + 4];
  __shared__ float red_rs[AW_WAVES][kSkinnyRows];
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
  const unsigned short *xg = reinterpret_cast<const unsigned short *>(p.x);
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const int k_blocks = (p.k + 63) / 64;
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const int chunks = (rows + kSkinnyRows - 1) / kSkinnyRows;
  const unsigned ones = BF16 ? 0x3F803F80u : 0x3C003C00u;
  const v4i ones_frag = v4i{(int)ones, (int)ones, (int)ones, (int)ones};
  const int col = min(n0 + 8 * lane16, p.n - 8);

  for (int mc = 0; mc < chunks; ++mc) {
    v4f acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
    v4f rs = v4f{0.f, 0.f, 0.f, 0.f};
    const int mrow = min(g_start + mc * kSkinnyRows + lane16, g_end - 1);
    const unsigned short *xrow = xg + (long long)mrow * p.k;

    uint2 rr[2][16];
    v4i aq[2][2];
    auto load_block = [&](int kb, int slot) {
      const int k0 = kb * 64 + 16 * h;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int krow = min(k0 + r, p.k - 1);
        rr[slot][r] = *reinterpret_cast<const uint2 *>(wg + (long long)krow * p.n + col);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int kk = k0 + 8 * t;
        aq[slot][t] = (kk < p.k) ? *reinterpret_cast<const v4i *>(xrow + kk) : v4i{0, 0, 0, 0};
      }
    };

    int kb = kb_begin + wave;
    if (kb < kb_end) load_block(kb, 0);
    if (kb + AW_WAVES < kb_end) load_block(kb + AW_WAVES, 1);
    for (; kb < kb_end; kb += 2 * AW_WAVES) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int kbs = kb + s * AW_WAVES;
        if (kbs < kb_end) {
          // int8 -> 16-bit float fragments: bfrag[j][t] holds k rows 8t..8t+7 of column j
          v4i bfrag[8][2];
#pragma unroll
          for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int r = 8 * t + 2 * q;
              const unsigned lo0 = rr[s][r].x ^ 0x80808080u, lo1 = rr[s][r + 1].x ^ 0x80808080u;
              const unsigned hi0 = rr[s][r].y ^ 0x80808080u, hi1 = rr[s][r + 1].y ^ 0x80808080u;
#pragma unroll
              for (int b = 0; b < 4; ++b) {
                bfrag[b][t][q] = (int)pack2<BF16>((float)((lo0 >> (8 * b)) & 0xFFu), (float)((lo1 >> (8 * b)) & 0xFFu));
                bfrag[4 + b][t][q] =
                  (int)pack2<BF16>((float)((hi0 >> (8 * b)) & 0xFFu), (float)((hi1 >> (8 * b)) & 0xFFu));
              }
            }
          }
          const v4i a0 = aq[s][0], a1 = aq[s][1];
          const int kbn = kbs + 2 * AW_WAVES;
          if (kbn < kb_end) load_block(kbn, s);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            acc[j] = mfma16<BF16>(a0, bfrag[j][0], acc[j]);
            acc[j] = mfma16<BF16>(a1, bfrag[j][1], acc[j]);
          }
          rs = mfma16<BF16>(a0, ones_frag, rs);
          rs = mfma16<BF16>(a1, ones_frag, rs);
        }
      }
    }

    // ---- reduce across waves in a fixed order ----------------------------------------------------
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][4 * h + r][8 * lane16 + j] = acc[j][r];
    if (lane16 == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) red_rs[wave][4 * h + r] = rs[r];
    }
    __syncthreads();

    const int row = tid >> 4, c8 = (tid & 15) * 8;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float s = red[0][row][c8 + j];
#pragma unroll
      for (int w = 1; w < AW_WAVES; ++w) s += red[w][row][c8 + j];
      v[j] = s;
    }
    float xs = red_rs[0][row];
#pragma unroll
    for (int w = 1; w < AW_WAVES; ++w) xs += red_rs[w][row];

    const int m = g_start + mc * kSkinnyRows + row;
    const bool row_ok = (m < g_end);
    bool do_epilogue = true;

    if (p.split_k > 1) {
      const long long tile = (long long)grp * p.n_strips + strip;
      float *base = reinterpret_cast<float *>(p.partial) + (tile * p.split_k + ks) * AW_TILE_FLOATS;
      if (row_ok) {
        float *mine = base + row * kSkinnyCols + c8;
#pragma unroll
        for (int j = 0; j < 8; ++j) __hip_atomic_store(mine + j, v[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (c8 == 0)
          __hip_atomic_store(base + kSkinnyRows * kSkinnyCols + row, xs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      do_epilogue = (s_ticket == (unsigned)(p.split_k - 1));
      if (do_epilogue) {
        if (row_ok) {
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = 0.f;
          xs = 0.f;
          for (int s = 0; s < p.split_k; ++s) {
            const float *src = reinterpret_cast<const float *>(p.partial) + (tile * p.split_k + s) * AW_TILE_FLOATS;
#pragma unroll
            for (int j = 0; j < 8; ++j)
              v[j] += __hip_atomic_load(src + row * kSkinnyCols + c8 + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            xs += __hip_atomic_load(src + kSkinnyRows * kSkinnyCols + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }

    if (do_epilogue && row_ok) {
      const int nb = n0 + c8;
      if (nb < p.n) {
        const unsigned short *sc = reinterpret_cast<const unsigned short *>(p.aq_scale);
        const unsigned short *of = reinterpret_cast<const unsigned short *>(p.aq_offset);
        unsigned short hv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int n = min(nb + j, p.n - 1);
          const float s = sc ? half_like_to_f32<BF16>(sc[(long long)grp * p.n + n]) : 1.0f;
          const float o = of ? half_like_to_f32<BF16>(of[(long long)grp * p.n + n]) : 0.0f;
          const float f = fmaf(o - 128.0f, xs, v[j]) * s;
          hv[j] = (p.out_dtype == DT_BF16) ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
        }
        unsigned short *o16 = reinterpret_cast<unsigned short *>(p.out) + (long long)m * p.n + nb;
        if (nb + 8 <= p.n) {
          uint4 q;
          q.x = hv[0] | ((unsigned)hv[1] << 16);
          q.y = hv[2] | ((unsigned)hv[3] << 16);
          q.z = hv[4] | ((unsigned)hv[5] << 16);
          q.w = hv[6] | ((unsigned)hv[7] << 16);
          *reinterpret_cast<uint4 *>(o16) = q;
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (nb + j < p.n) o16[j] = hv[j];
        }
      }
    }
    __syncthreads();
  }
}

hipError_t launch_skinny_a16w8(const GmmParams &p, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const dim3 grid((unsigned)p.n_strips, (unsigned)p.e, (unsigned)p.split_k);
  if (p.x_dtype == DT_BF16) {
    hipLaunchKernelGGL(gmm_a16w8_skinny_kernel<true>, grid, dim3(AW_THREADS), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_a16w8_skinny_kernel<false>, grid, dim3(AW_THREADS), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace msco
