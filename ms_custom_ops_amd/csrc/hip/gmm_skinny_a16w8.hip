// Grouped weight-only (bf16/f16 activations x int8 weights) GEMM, skinny decode kernel for gfx950.
//
// Same work decomposition as the 4-wave W8A8 skinny kernel: a workgroup owns one 16-row chunk of one
// group, one 256-column strip and one K slice; its waves take interleaved 32-row blocks and stream
// the int8 weights [K,N] from HBM with 16-byte loads (4 rows x 256 contiguous bytes per instruction).
// The int8 bytes are turned into exact bf16/f16 values of (w + 128) in registers
// (v_cvt_f32_ubyteN on w ^ 0x80 picks the column byte, then a 16-bit pack -- no byte transposes are
// needed), multiplied with v_mfma_f32_16x16x32_{bf16,f16} and accumulated in float32.  One more MFMA
// per block against an all-ones fragment yields sum_k x[m,k], so the per-channel antiquant offset
// and the +128 bias fold into the epilogue:
//
//   out[m,n] = s[g,n] * ( sum_k x[m,k]*(w[k,n]+128)  +  (o[g,n] - 128) * sum_k x[m,k] )
//            = sum_k x[m,k] * (w[k,n] + o[g,n]) * s[g,n]
//
// Partial sums are combined in a fixed order (wave 0..3, then K slice 0..S-1), so results are
// reproducible run to run.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

namespace {
constexpr int AW_WAVES = 4;
constexpr int AW_THREADS = AW_WAVES * 64;
constexpr int AW_COLS = kSkinnyCols;                              // 256
constexpr int AW_TILE_WORDS = kSkinnyRows * AW_COLS / 2 + 128;    // 64-bit words: tile + 4 row sums per lane slot
typedef long long i64;
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
}  // namespace

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

// byte `B` (0..3) of w as float
template <int B>
__device__ __forceinline__ float ubyte_f32(unsigned w) {
  return (float)((w >> (8 * B)) & 0xFFu);   // v_cvt_f32_ubyteB
}

template <bool BF16, int B>
__device__ __forceinline__ v4i column_frag(const unsigned (&w)[8]) {
  v4i f;
#pragma unroll
  for (int q = 0; q < 4; ++q) f[q] = (int)pack2<BF16>(ubyte_f32<B>(w[2 * q]), ubyte_f32<B>(w[2 * q + 1]));
  return f;
}

template <bool BF16>
__global__ void __launch_bounds__(AW_THREADS, 4) gmm_a16w8_skinny_kernel(const GmmParams p) {
  // wave w, pass q: red[w][jj][lane] holds acc[8q + jj] (rows 4h..4h+3 of one column); later the output tile
  __shared__ __align__(16) v4f red[AW_WAVES][8][64];
  __shared__ __align__(16) v4f red_rs[AW_WAVES][64];
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, kSkinnyRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * kSkinnyRows;
  const int chunk_rows = min(kSkinnyRows, g_end - m0);

  const int n0 = strip * AW_COLS;
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(wg, (long long)p.k * p.n);   // planned only when K * N < 2^31
  const int k_blocks = (p.k + 31) / 32;
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const unsigned short *xrow =
    reinterpret_cast<const unsigned short *>(p.x) + (long long)min(m0 + c16, g_end - 1) * p.k;
  const unsigned ones = BF16 ? 0x3F803F80u : 0x3C003C00u;
  const v4i ones_frag = v4i{(int)ones, (int)ones, (int)ones, (int)ones};

  // accumulator j of this lane: column n0 + 16 c + j, rows 4h..4h+3
  v4f acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
  v4f rs = v4f{0.f, 0.f, 0.f, 0.f};
  const bool cols_ok = n0 + 16 * c16 < p.n;   // N % 16 == 0: the lane's 16 columns are all inside or all outside

  for (int kb = kb_begin + wave; kb < kb_end; kb += AW_WAVES) {
    const int k0 = kb * 32 + 8 * h;             // K % 8 == 0: 8 K rows all inside or all outside
    const bool k_ok = k0 < p.k;
    const unsigned voff = (k_ok && cols_ok) ? (unsigned)(k0 * p.n + n0 + 16 * c16) : kBufferOob;
    v4i r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, voff, i * p.n, kStreamAux);
    const v4i a = k_ok ? *reinterpret_cast<const v4i *>(xrow + k0) : v4i{0, 0, 0, 0};
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      unsigned w[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = (unsigned)r[i][c4] ^ 0x80808080u;   // w + 128 as unsigned bytes
      acc[4 * c4 + 0] = mfma16<BF16>(a, column_frag<BF16, 0>(w), acc[4 * c4 + 0]);
      acc[4 * c4 + 1] = mfma16<BF16>(a, column_frag<BF16, 1>(w), acc[4 * c4 + 1]);
      acc[4 * c4 + 2] = mfma16<BF16>(a, column_frag<BF16, 2>(w), acc[4 * c4 + 2]);
      acc[4 * c4 + 3] = mfma16<BF16>(a, column_frag<BF16, 3>(w), acc[4 * c4 + 3]);
    }
    rs = mfma16<BF16>(a, ones_frag, rs);
  }

  // ---- add the four waves' tiles through LDS in wave order: thread (wave, lane) ends up with
  // columns j = 8q + wave + 4u (q, u = 0..1) of its own lane position, rows 4h..4h+3 --------------
  v4f v[4];
  red_rs[wave][lane] = rs;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    if (q) __syncthreads();
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) red[wave][jj][lane] = acc[8 * q + jj];
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      v4f s = red[0][wave + 4 * u][lane];
#pragma unroll
      for (int w = 1; w < AW_WAVES; ++w) s += red[w][wave + 4 * u][lane];
      v[2 * q + u] = s;
    }
  }
  // row sums of x for rows 4h..4h+3 (every column of the MFMA result holds the same sum)
  v4f xs = red_rs[0][lane];
#pragma unroll
  for (int w = 1; w < AW_WAVES; ++w) xs += red_rs[w][lane];
  const bool rows_ok = 4 * h < chunk_rows;

  if (p.split_k > 1) {
    // cross-workgroup reduction as in the W8A8 kernel; float32 partials, added in slice order.
    // slice s: word e (0..7) of thread t at (s * AW_TILE_WORDS + e * 256 + t); row sums of wave 0's
    // lanes at (s * AW_TILE_WORDS + 2048 + 2 * lane + {0, 1})
    const long long tile = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * AW_TILE_WORDS;
    auto pack = [](float lo, float hi) {
      return (i64)(((unsigned long long)__float_as_uint(hi) << 32) | __float_as_uint(lo));
    };
    if (rows_ok) {
      i64 *mine = base + (long long)ks * AW_TILE_WORDS;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        __hip_atomic_store(mine + e * AW_THREADS + tid, pack(v[e >> 1][2 * (e & 1)], v[e >> 1][2 * (e & 1) + 1]),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (wave == 0) {
        __hip_atomic_store(mine + 2048 + 2 * lane, pack(xs[0], xs[1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + 2048 + 2 * lane + 1, pack(xs[2], xs[3]), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    publish_partials_and_sync();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (rows_ok) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v4f{0.f, 0.f, 0.f, 0.f};
      xs = v4f{0.f, 0.f, 0.f, 0.f};
      for (int s0 = 0; s0 < p.split_k; s0 += 4) {
        i64 t[4][10];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int s = min(s0 + u, p.split_k - 1);
          const i64 *src = base + (long long)s * AW_TILE_WORDS;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            t[u][e] = __hip_atomic_load(src + e * AW_THREADS + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          t[u][8] = __hip_atomic_load(src + 2048 + 2 * lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          t[u][9] = __hip_atomic_load(src + 2048 + 2 * lane + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < p.split_k) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              v[e >> 1][2 * (e & 1)] += __uint_as_float((unsigned)(unsigned long long)t[u][e]);
              v[e >> 1][2 * (e & 1) + 1] += __uint_as_float((unsigned)((unsigned long long)t[u][e] >> 32));
            }
            xs[0] += __uint_as_float((unsigned)(unsigned long long)t[u][8]);
            xs[1] += __uint_as_float((unsigned)((unsigned long long)t[u][8] >> 32));
            xs[2] += __uint_as_float((unsigned)(unsigned long long)t[u][9]);
            xs[3] += __uint_as_float((unsigned)((unsigned long long)t[u][9] >> 32));
          }
      }
    }
  }

  // ---- epilogue: v[2q + u] = rows 4h..4h+3 of column j = 8q + wave + 4u -----------------------
  unsigned short(*tile_out)[AW_COLS + 8] = reinterpret_cast<unsigned short(*)[AW_COLS + 8]>(&red[0][0][0]);
  __syncthreads();   // every wave is done reading red[]
  const unsigned short *sc = reinterpret_cast<const unsigned short *>(p.aq_scale);
  const unsigned short *of = reinterpret_cast<const unsigned short *>(p.aq_offset);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int j = 8 * (e >> 1) + wave + 4 * (e & 1);
    const int cl = 16 * c16 + j;
    const int n = n0 + cl;
    if (n < p.n && rows_ok) {
      const float s = sc ? half_like_to_f32<BF16>(sc[(long long)grp * p.n + n]) : 1.0f;
      const float o = of ? half_like_to_f32<BF16>(of[(long long)grp * p.n + n]) : 0.0f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float f = fmaf(o - 128.0f, xs[r], v[e][r]) * s;
        tile_out[4 * h + r][cl] = half_out(p, f);
      }
    }
  }
  __syncthreads();
  // whole-row stores: 16 rows x 32 pieces of 8 columns, two pieces per thread
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int item = tid + AW_THREADS * u;
    const int row = item >> 5, c8 = (item & 31) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && n < p.n) {
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

size_t a16w8_workspace_bytes(int64_t m, int64_t n, int64_t e, int split_k) {
  if (split_k <= 1) return 0;
  return skinny_counter_count(m, n, e, AW_COLS) * (size_t)split_k * AW_TILE_WORDS * 8;
}

hipError_t launch_skinny_a16w8(const GmmParams &p, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, kSkinnyRows), (unsigned)p.split_k);
  if (p.x_dtype == DT_BF16) {
    hipLaunchKernelGGL(gmm_a16w8_skinny_kernel<true>, grid, dim3(AW_THREADS), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_a16w8_skinny_kernel<false>, grid, dim3(AW_THREADS), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace msco
