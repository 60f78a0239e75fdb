// Grouped W8A8 GEMM, skinny (decode) kernel for gfx950: HBM-bound weight streaming.
//
// A workgroup (4 waves) owns one 16-row chunk of one group, one 256-column strip of the weights and
// one slice of K.  Measured on MI355X, a strip walk reaches the bandwidth of a plain contiguous read
// only when every row segment a wave touches is at least 256 bytes and when about a thousand
// workgroups are in flight, which fixes the shape:
//   * [K,N] storage: a wave takes 32-row blocks; lane (c, h) loads 16 bytes (columns 16c..16c+15)
//     of rows 8h..8h+7, so one load instruction covers 4 rows x 256 contiguous bytes.  4x4 byte
//     transposes (v_perm_b32) turn them into the K-contiguous operand of v_mfma_i32_16x16x32_i8;
//   * [N,K] storage: a wave takes 64-row K blocks; lane (c, h) loads 16 K-bytes of row 16j + c for
//     j = 0..15 and feeds them unchanged to v_mfma_i32_16x16x64_i8; neighbouring waves take
//     neighbouring K blocks, so the workgroup reads whole 256-byte row segments;
//   * the x fragment (rows beyond the chunk are clamped and never stored) is the other operand; the
//     work is bandwidth bound, the MFMA is only the cheapest way to do the dot products;
//   * the four waves' int32 partial tiles are added through LDS.  With split_k > 1 every workgroup
//     then publishes its 16 x 256 partial tile to the workspace and bumps the tile's arrival
//     counter; the last one to arrive adds all slices and runs the epilogue.  int32 addition is
//     associative, so the result is bit-exact whatever the arrival order.  Counters reset themselves;
//   * the epilogue dequantises in registers, stages the 16 x 256 output tile in LDS and writes whole
//     rows; empty chunks exit before touching their weights.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

namespace {
constexpr int SK_WAVES = 4;
constexpr int SK_THREADS = SK_WAVES * 64;
constexpr int SK_COLS = kSkinnyCols;                  // 256
constexpr int SK_TILE_INTS = kSkinnyRows * SK_COLS;   // one partial tile
typedef long long i64;
}  // namespace

template <bool NK>
__global__ void __launch_bounds__(SK_THREADS, NK ? 3 : 4) gmm_w8a8_skinny_kernel(const GmmParams p) {
  constexpr int KB = NK ? 64 : 32;  // K rows per wave block
  // wave w, pass q: red[w][jj][lane] holds acc[8q + jj] (rows 4h..4h+3 of one column); later the output tile
  __shared__ __align__(16) v4i red[SK_WAVES][8][64];
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: scalar loop control
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, kSkinnyRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * kSkinnyRows;
  const int chunk_rows = min(kSkinnyRows, g_end - m0);

  const int n0 = strip * SK_COLS;
  const int8_t *xg = reinterpret_cast<const int8_t *>(p.x);
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(wg, (long long)p.k * p.n);  // planned only when K * N < 2^31
  const int k_blocks = (p.k + KB - 1) / KB;
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const int8_t *xrow = xg + (long long)min(m0 + c16, g_end - 1) * p.k;

  // column of accumulator j in this lane: [K,N]: n0 + 16 c + j (a lane owns 16 consecutive columns);
  // [N,K]: n0 + 16 j + c (a load instruction covers 16 consecutive weight rows)
  v4i acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = v4i{0, 0, 0, 0};

  // N % 16 == 0: the 16 columns 16c..16c+15 of the strip are all inside N or all outside
  const bool cols_ok = n0 + 16 * c16 < p.n;
  for (int kb = kb_begin + wave; kb < kb_end; kb += SK_WAVES) {
    if constexpr (NK) {
      const int k0 = kb * 64 + 16 * h;  // K % 16 == 0: 16 K bytes all inside or all outside
      const bool k_ok = k0 < p.k;
      v4i b[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int n = n0 + 16 * j + c16;
        const unsigned voff = (k_ok && n < p.n) ? (unsigned)(n * p.k + k0) : kBufferOob;
        b[j] = __builtin_amdgcn_raw_buffer_load_b128(rw, voff, 0, 0);
      }
      const v4i a = k_ok ? *reinterpret_cast<const v4i *>(xrow + k0) : v4i{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[j], acc[j], 0, 0, 0);
    } else {
      const int k0 = kb * 32 + 8 * h;  // K % 8 == 0: 8 K rows all inside or all outside
      const bool k_ok = k0 < p.k;
      const unsigned voff = (k_ok && cols_ok) ? (unsigned)(k0 * p.n + n0 + 16 * c16) : kBufferOob;
      v4i r[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, voff, i * p.n, kStreamAux);
      const i64 a = k_ok ? *reinterpret_cast<const i64 *>(xrow + k0) : 0;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        unsigned lo[4], hi[4];
        transpose4x4(r[0][c4], r[1][c4], r[2][c4], r[3][c4], lo[0], lo[1], lo[2], lo[3]);
        transpose4x4(r[4][c4], r[5][c4], r[6][c4], r[7][c4], hi[0], hi[1], hi[2], hi[3]);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const i64 b = (i64)(((unsigned long long)hi[u] << 32) | lo[u]);
          acc[4 * c4 + u] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, acc[4 * c4 + u], 0, 0, 0);
        }
      }
    }
  }

  // ---- add the four waves' tiles through LDS: thread (wave, lane) ends up with columns
  // j = 8q + wave + 4u (q, u = 0..1) of its own lane position, rows 4h..4h+3 -----------------------
  v4i v[4];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    if (q) __syncthreads();
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) red[wave][jj][lane] = acc[8 * q + jj];
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      v4i s = red[0][wave + 4 * u][lane];
#pragma unroll
      for (int w = 1; w < SK_WAVES; ++w) s += red[w][wave + 4 * u][lane];
      v[2 * q + u] = s;
    }
  }
  const bool rows_ok = 4 * h < chunk_rows;  // at least one of the lane's 4 rows is part of the chunk

  if (p.split_k > 1) {
    // ---- cross-workgroup reduction through the workspace --------------------------------------
    // Partial tiles and the arrival counter are exchanged with agent-scope atomic accesses: they
    // bypass the per-XCD L2 for this data only, so no cache-wide write-back / invalidate fence is
    // needed.  Every wavefront waits for its own stores (vmcnt == 0) before the barrier that precedes the counter bump.  A tile is kept in
    // the threads' own fragment order: slice s, 64-bit word e of thread t at ((s * 8 + e) * 256 + t).
    const long long tile = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * (SK_TILE_INTS / 2);
    if (rows_ok) {
      i64 *mine = base + (long long)ks * (SK_TILE_INTS / 2) + tid;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const i64 word = (i64)(((unsigned long long)(unsigned)v[e >> 1][2 * (e & 1) + 1] << 32) |
                               (unsigned)v[e >> 1][2 * (e & 1)]);
        __hip_atomic_store(mine + e * SK_THREADS, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    publish_partials_and_sync();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (rows_ok) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v4i{0, 0, 0, 0};
      // batches of 4 slices: 32 independent loads in flight, then the adds
      for (int s0 = 0; s0 < p.split_k; s0 += 4) {
        i64 t[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int s = min(s0 + u, p.split_k - 1);
          const i64 *src = base + (long long)s * (SK_TILE_INTS / 2) + tid;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            t[u][e] = __hip_atomic_load(src + e * SK_THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < p.split_k) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              v[e >> 1][2 * (e & 1)] += (int)(unsigned)(unsigned long long)t[u][e];
              v[e >> 1][2 * (e & 1) + 1] += (int)(unsigned)((unsigned long long)t[u][e] >> 32);
            }
          }
      }
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------
  // v[2q + u] = rows 4h..4h+3 of column j = 8q + wave + 4u
  float pt[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) pt[r] = (p.per_token && 4 * h + r < chunk_rows) ? p.per_token[m0 + 4 * h + r] : 1.0f;
  unsigned short(*tile_out)[SK_COLS + 8] = reinterpret_cast<unsigned short(*)[SK_COLS + 8]>(&red[0][0][0]);
  __syncthreads();  // every wave is done reading red[]
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int j = 8 * (e >> 1) + wave + 4 * (e & 1);
    const int cl = NK ? 16 * j + c16 : 16 * c16 + j;  // column inside the strip
    const int n = n0 + cl;
    if (n < p.n && rows_ok) {
      const int bias = load_bias(p, grp, n);
      if (p.out_dtype == DT_I32) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * h + r < chunk_rows)
            reinterpret_cast<int *>(p.out)[(long long)(m0 + 4 * h + r) * p.n + n] = v[e][r] + bias;
      } else {
        const float sc = load_scale(p, grp, n);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float f = dequant(v[e][r] + bias, sc, pt[r]);
          tile_out[4 * h + r][cl] = half_out(p, f);
        }
      }
    }
  }
  if (p.out_dtype == DT_I32) return;
  __syncthreads();
  // whole-row stores: 16 rows x 32 pieces of 8 columns, two pieces per thread
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int item = tid + SK_THREADS * u;
    const int row = item >> 5, c8 = (item & 31) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && n < p.n) {  // N % 16 == 0: 8 columns all inside or all outside
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Variant for small weight sets (few strips): the whole problem must be in flight at once, because
// with less than one workgroup per CU a wave that walks several blocks one after the other pays one
// HBM round trip per block.  One workgroup of 16 waves per CU owns a 128-column strip and a K slice;
// every wave keeps up to four 32-row blocks (two 64-row blocks for [N,K]) in flight, so for K = 4096
// split two ways all weight bytes are requested before the first one is consumed.  The K split
// across workgroups stays small (at most 256 workgroups in total), which keeps the last arriver's
// reduction to a single round of loads.
namespace {
constexpr int W16_WAVES = 16;
constexpr int W16_THREADS = W16_WAVES * 64;
constexpr int W16_COLS = 128;
constexpr int W16_REDUCERS = 512;                       // threads that own a piece of the 16 x 128 tile
constexpr int W16_TILE_WORDS = kSkinnyRows * W16_COLS / 2;   // 64-bit words of one partial tile
constexpr size_t W16_LDS = (size_t)8 * W16_WAVES * 64 * sizeof(v4i);   // red[j][source wave][lane]
}  // namespace

template <bool NK>
__global__ void __launch_bounds__(W16_THREADS) gmm_w8a8_skinny16_kernel(const GmmParams p) {
  constexpr int KB = NK ? 64 : 32;
  constexpr int DEPTH = NK ? 2 : 4;
  extern __shared__ __align__(16) unsigned char smem16[];
  v4i *red = reinterpret_cast<v4i *>(smem16);
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: scalar loop control
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, kSkinnyRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * kSkinnyRows;
  const int chunk_rows = min(kSkinnyRows, g_end - m0);

  const int n0 = strip * W16_COLS;
  const int8_t *wg = p.w + (long long)grp * p.k * p.n;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(wg, (long long)p.k * p.n);
  const int k_blocks = (p.k + KB - 1) / KB;
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const int8_t *xrow = reinterpret_cast<const int8_t *>(p.x) + (long long)min(m0 + c16, g_end - 1) * p.k;

  // Epilogue operands of the tile piece this thread will own after the reduction (wave j < 8 owns
  // column j of every lane position), requested now so their latency hides behind the weight stream.
  const int ep_cl = NK ? 16 * wave + c16 : 8 * c16 + wave;
  const int ep_n = n0 + ep_cl;
  int ep_bias = 0;
  float ep_scale = 1.0f, ep_pt[4] = {1.0f, 1.0f, 1.0f, 1.0f};
  if (tid < W16_REDUCERS && ep_n < p.n) {
    ep_bias = load_bias(p, grp, ep_n);
    ep_scale = load_scale(p, grp, ep_n);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (p.per_token && 4 * h + r < chunk_rows) ep_pt[r] = p.per_token[m0 + 4 * h + r];
  }

  // column of accumulator j in this lane: [K,N]: n0 + 8 c + j; [N,K]: n0 + 16 j + c
  v4i acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = v4i{0, 0, 0, 0};
  const bool cols_ok = n0 + 8 * c16 < p.n;   // N % 16 == 0: the lane's 8 columns are all inside or all outside

  uint2 rk[DEPTH][8];   // [K,N]: rows 8h..8h+7, 8 column bytes each
  v4i bn[DEPTH][8];     // [N,K]: 16 K bytes of weight rows 16j + c
  i64 ak[DEPTH];
  v4i an[DEPTH];
  auto load_block = [&](int kb, int s) {
    if constexpr (NK) {
      const int k0 = kb * 64 + 16 * h;
      const bool k_ok = k0 < p.k;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int n = n0 + 16 * j + c16;
        const unsigned voff = (k_ok && n < p.n) ? (unsigned)(n * p.k + k0) : kBufferOob;
        bn[s][j] = __builtin_amdgcn_raw_buffer_load_b128(rw, voff, 0, 0);
      }
      an[s] = k_ok ? *reinterpret_cast<const v4i *>(xrow + k0) : v4i{0, 0, 0, 0};
    } else {
      const int k0 = kb * 32 + 8 * h;
      const bool k_ok = k0 < p.k;
      const unsigned voff = (k_ok && cols_ok) ? (unsigned)(k0 * p.n + n0 + 8 * c16) : kBufferOob;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        rk[s][i] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(rw, voff, i * p.n, kStreamAux));
      ak[s] = k_ok ? *reinterpret_cast<const i64 *>(xrow + k0) : 0;
    }
  };

  int kb = kb_begin + wave;
#pragma unroll
  for (int s = 0; s < DEPTH; ++s)
    if (kb + s * W16_WAVES < kb_end) load_block(kb + s * W16_WAVES, s);
  for (; kb < kb_end; kb += DEPTH * W16_WAVES) {
#pragma unroll
    for (int s = 0; s < DEPTH; ++s) {
      const int kbs = kb + s * W16_WAVES;
      if (kbs < kb_end) {
        const int kbn = kbs + DEPTH * W16_WAVES;
        if constexpr (NK) {
          const v4i a = an[s];
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bn[s][j], acc[j], 0, 0, 0);
          if (kbn < kb_end) load_block(kbn, s);
        } else {
          const i64 a = ak[s];
#pragma unroll
          for (int c4 = 0; c4 < 2; ++c4) {
            unsigned lo[4], hi[4];
            if (c4 == 0) {
              transpose4x4(rk[s][0].x, rk[s][1].x, rk[s][2].x, rk[s][3].x, lo[0], lo[1], lo[2], lo[3]);
              transpose4x4(rk[s][4].x, rk[s][5].x, rk[s][6].x, rk[s][7].x, hi[0], hi[1], hi[2], hi[3]);
            } else {
              transpose4x4(rk[s][0].y, rk[s][1].y, rk[s][2].y, rk[s][3].y, lo[0], lo[1], lo[2], lo[3]);
              transpose4x4(rk[s][4].y, rk[s][5].y, rk[s][6].y, rk[s][7].y, hi[0], hi[1], hi[2], hi[3]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const i64 b = (i64)(((unsigned long long)hi[u] << 32) | lo[u]);
              acc[4 * c4 + u] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, acc[4 * c4 + u], 0, 0, 0);
            }
          }
          if (kbn < kb_end) load_block(kbn, s);
        }
      }
    }
  }

  // ---- add the 16 waves' tiles through LDS: wave j < 8 ends up with column j of every lane position
#pragma unroll
  for (int j = 0; j < 8; ++j) red[(j * W16_WAVES + wave) * 64 + lane] = acc[j];
  __syncthreads();
  const bool reducer = tid < W16_REDUCERS;
  v4i v = v4i{0, 0, 0, 0};
  if (reducer) {
#pragma unroll
    for (int sw = 0; sw < W16_WAVES; ++sw) v += red[(wave * W16_WAVES + sw) * 64 + lane];
  }
  const bool rows_ok = reducer && 4 * h < chunk_rows;

  if (p.split_k > 1) {
    // cross-workgroup reduction, as in the 4-wave kernel; slice s, word e of reducer t at ((s * 2 + e) * 512 + t)
    const long long tile = ((long long)grp * p.max_chunks + mc) * gridDim.x + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * W16_TILE_WORDS;
    if (rows_ok) {
      i64 *mine = base + (long long)ks * W16_TILE_WORDS + tid;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const i64 word = (i64)(((unsigned long long)(unsigned)v[2 * e + 1] << 32) | (unsigned)v[2 * e]);
        __hip_atomic_store(mine + e * W16_REDUCERS, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    publish_partials_and_sync();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (rows_ok) {
      v = v4i{0, 0, 0, 0};
      for (int s0 = 0; s0 < p.split_k; s0 += 8) {   // 16 independent loads in flight, then the adds
        i64 t[8][2];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int s = min(s0 + u, p.split_k - 1);
          const i64 *src = base + (long long)s * W16_TILE_WORDS + tid;
#pragma unroll
          for (int e = 0; e < 2; ++e)
            t[u][e] = __hip_atomic_load(src + e * W16_REDUCERS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < p.split_k) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              v[2 * e] += (int)(unsigned)(unsigned long long)t[u][e];
              v[2 * e + 1] += (int)(unsigned)((unsigned long long)t[u][e] >> 32);
            }
          }
      }
    }
  }

  // ---- epilogue: reducer (wave j, lane) holds rows 4h..4h+3 of column j of its lane position
  unsigned short(*tile_out)[W16_COLS + 8] = reinterpret_cast<unsigned short(*)[W16_COLS + 8]>(smem16);
  __syncthreads();   // every wave is done reading red[]
  if (rows_ok && ep_n < p.n) {
    if (p.out_dtype == DT_I32) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (4 * h + r < chunk_rows)
          reinterpret_cast<int *>(p.out)[(long long)(m0 + 4 * h + r) * p.n + ep_n] = v[r] + ep_bias;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float f = dequant(v[r] + ep_bias, ep_scale, ep_pt[r]);
        tile_out[4 * h + r][ep_cl] = half_out(p, f);
      }
    }
  }
  if (p.out_dtype == DT_I32) return;
  __syncthreads();
  if (tid < 256) {   // whole-row stores: 16 rows x 16 pieces of 8 columns
    const int row = tid >> 4, c8 = (tid & 15) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && n < p.n) {
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

// one arrival counter per (group, 16-row chunk, strip of `cols` columns)
size_t skinny_counter_count(int64_t m, int64_t n, int64_t e, int cols) {
  const int64_t strips = (n + cols - 1) / cols;
  const int64_t max_chunks = (m + kSkinnyRows - 1) / kSkinnyRows;
  return (size_t)(e * (max_chunks > 0 ? max_chunks : 1) * strips);
}

size_t skinny_workspace_bytes(int64_t m, int64_t n, int64_t e, int split_k, int cols) {
  if (split_k <= 1) return 0;
  // one 16 x cols tile of 4-byte partial sums per (tile, K slice)
  return skinny_counter_count(m, n, e, cols) * (size_t)split_k * kSkinnyRows * cols * 4;
}

hipError_t launch_skinny_w8a8(const GmmParams &p, bool nk, bool wide16, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  if (wide16) {
    auto kern = nk ? gmm_w8a8_skinny16_kernel<true> : gmm_w8a8_skinny16_kernel<false>;
    static std::atomic<bool> attr_done[2];   // zero-initialised; the attribute call is idempotent, so a race between first launches repeats it at worst
    if (!attr_done[nk]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)W16_LDS);
      if (e != hipSuccess) return e;
      attr_done[nk] = true;
    }
    const dim3 grid((unsigned)((p.n + W16_COLS - 1) / W16_COLS), chunk_slots(p, kSkinnyRows), (unsigned)p.split_k);
    hipLaunchKernelGGL(kern, grid, dim3(W16_THREADS), W16_LDS, stream, p);
    return hipGetLastError();
  }
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, kSkinnyRows), (unsigned)p.split_k);
  if (nk) {
    hipLaunchKernelGGL(gmm_w8a8_skinny_kernel<true>, grid, dim3(SK_THREADS), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_w8a8_skinny_kernel<false>, grid, dim3(SK_THREADS), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace msco
