// Grouped decode kernels for weights in the packed layout (gfx950): HBM-bound weight streaming at the
// rate of a plain contiguous read.
//
// Packed layout of one group's weights (K x N int8): ceil(N/16) column groups, each ceil(K/64) blocks of
// 1024 bytes, zero outside K x N.  Byte 16 l + i (l = 0..63, i = 0..15) of block (a, b) is
//     w[k = 64 b + 16 (l / 16) + i][n = 16 a + (l % 16)],
// so one 16-byte load per lane of 1024 consecutive bytes IS the B operand of v_mfma_i32_16x16x64_i8
// (lane l: column l % 16, K bytes 16 (l / 16) ..), and the blocks of a column group and the column groups
// of a strip follow each other in memory.  Measured on MI355X a workgroup whose waves take neighbouring
// 1 KiB pieces of one contiguous region streams at about 7 TB/s, against 6.2 TB/s for the best walk of
// 256-byte row segments of a row-major matrix and 5.5 TB/s for any walk of a [N,K] matrix whose row pitch
// is a power of two -- which is why this layout exists.
//
// Work decomposition (both kernels): a workgroup (4 waves) owns one 16-row chunk of one group, one strip
// of up to 16 column groups (256 columns; fewer for small weight sets, so that every CU gets a strip without
// splitting K) and one K slice of at most 128 blocks.  It walks its strip in memory
// order: column group after column group, wave w taking blocks w, w + 4, ... of the slice, eight loads in
// flight per wave across column-group boundaries.  A wave meets the same K blocks in every column group,
// so its x fragments are loaded once and stay in registers; the inner step is one 16-byte load and one
// MFMA, nothing else.  Per column group a wave parks its partial tile in LDS; afterwards the four waves'
// tiles are added in wave order.  K split across workgroups, arrival counter and epilogue are those of the
// row-major decode kernels.
//
// Further down: the multi-row forms for groups of more than 16 rows (W8A8 on packed weights; weight-only on packed and
// on row-major [E,K,N] weights, the latter two with the chunk's x -- and where it pays the weights -- staged in LDS).
#include <type_traits>
#include <utility>

#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

namespace {
constexpr int ST_WAVES = 4;
constexpr int ST_THREADS = ST_WAVES * 64;
constexpr int ST_COLS = kSkinnyCols;                  // 256 columns = 16 column groups per strip
constexpr int ST_GROUPS = ST_COLS / 16;
constexpr int ST_TILE_INTS = kSkinnyRows * ST_COLS;   // one partial tile
constexpr size_t ST_LDS = (size_t)ST_WAVES * ST_GROUPS * 64 * 16 + 16;   // red[wave][column group][lane] + ticket
typedef long long i64;
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

__host__ __device__ inline long long packed_group_bytes(long long k, long long n) {
  return ((n + 15) / 16) * ((k + 63) / 64) * 1024;
}
}  // namespace

// ---- packing -------------------------------------------------------------------------------------------
// One thread per 16 destination bytes.  NK: source [E,N,K] (16 K-contiguous bytes), else [E,K,N].
template <bool NK>
__global__ void __launch_bounds__(256) pack_weight_kernel(const int8_t *src, int8_t *dst, long long e, int k, int n) {
  const long long per_group = packed_group_bytes(k, n) / 16;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= e * per_group) return;
  const long long g = idx / per_group, r = idx % per_group;
  const int l = (int)(r & 63);
  const long long blk = r >> 6;
  const int kblocks = (k + 63) / 64;
  const int a = (int)(blk / kblocks), b = (int)(blk % kblocks);
  const int col = 16 * a + (l & 15), k0 = 64 * b + 16 * (l >> 4);
  const int8_t *s = src + g * (long long)k * n;
  int8_t v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int kk = k0 + i;
    v[i] = (col < n && kk < k) ? (NK ? s[(long long)col * k + kk] : s[(long long)kk * n + col]) : (int8_t)0;
  }
  *reinterpret_cast<uint4 *>(dst + idx * 16) = *reinterpret_cast<const uint4 *>(v);
}

hipError_t launch_pack_weight(const void *src, void *dst, long long e, long long k, long long n, bool src_nk,
                              hipStream_t stream) {
  const long long total = e * (packed_group_bytes(k, n) / 16);
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (src_nk) {
    hipLaunchKernelGGL(pack_weight_kernel<true>, dim3(grid), dim3(256), 0, stream, static_cast<const int8_t *>(src),
                       static_cast<int8_t *>(dst), e, (int)k, (int)n);
  } else {
    hipLaunchKernelGGL(pack_weight_kernel<false>, dim3(grid), dim3(256), 0, stream, static_cast<const int8_t *>(src),
                       static_cast<int8_t *>(dst), e, (int)k, (int)n);
  }
  return hipGetLastError();
}

size_t packed_weight_bytes(int64_t k, int64_t n) { return (size_t)packed_group_bytes(k, n); }

// ---- W8A8 ----------------------------------------------------------------------------------------------
// NB = K blocks a wave meets per column group (the slice has at most 4 NB blocks); 4, 8, 16 or 32.
// XLDS: the chunk's x rows reach the waves through LDS.  Read straight from memory, a wave's fragment load touches 16
// rows x 64 bytes = 16 half lines, twice the line requests of a weight load of the same size, and the request rate of
// the load path is what bounds these kernels; staged, the workgroup reads every x line once with whole-line requests
// (four rows x 256 contiguous bytes per wave instruction) and the waves pick their fragments out of LDS.
template <int NB, bool XLDS>
__global__ void __launch_bounds__(ST_THREADS, 2) gmm_w8a8_stream_kernel(const GmmParams p) {
  extern __shared__ __align__(16) unsigned char st_smem[];
  v4i(*red)[ST_GROUPS][64] = reinterpret_cast<v4i(*)[ST_GROUPS][64]>(st_smem);   // [wave][column group][lane]
  unsigned *s_ticket = reinterpret_cast<unsigned *>(st_smem + ST_LDS - 16);
#ifndef MSCO_STREAM_DEPTH
#define MSCO_STREAM_DEPTH 8
#endif
  constexpr int D = NB < MSCO_STREAM_DEPTH ? NB : MSCO_STREAM_DEPTH;   // loads in flight per wave

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, kSkinnyRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * kSkinnyRows;
  const int chunk_rows = min(kSkinnyRows, g_end - m0);

  const int n0 = strip * p.strip_groups * 16;
  const int col_groups = (p.n + 15) / 16, k_blocks = (p.k + 63) / 64;
  const int cg_count = min(p.strip_groups, col_groups - strip * p.strip_groups);   // column groups of this strip that exist
  const long long group_bytes = (long long)col_groups * k_blocks * 1024;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(p.w + (long long)grp * group_bytes, group_bytes);   // planned only below 2^31
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);

  // the wave's blocks kb_begin + wave + 4 j: x fragments (zero past the slice or past K, which also cancels
  // whatever a masked weight load returns) and byte offsets inside a column group
  v4i xf[NB];
  unsigned voff[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int kb = kb_begin + wave + ST_WAVES * j;
    voff[j] = kb < kb_end ? (unsigned)(kb * 1024 + lane * 16) : kBufferOob;
  }
  v4i xtmp[XLDS ? NB : 1];
  const int st_row = tid >> 4, st_col = tid & 15;                      // staging: 16 threads per row, 256 bytes per pass
  const int slice_bytes = (kb_end - kb_begin) * 64, x_pitch = slice_bytes + 64;   // the pad spreads the 16 rows of a fragment read over all banks
  if constexpr (XLDS) {
    const int8_t *srow = reinterpret_cast<const int8_t *>(p.x) + (long long)min(m0 + st_row, g_end - 1) * p.k + kb_begin * 64;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int off = (st_col + 16 * j) * 16;
      xtmp[j] = (off < slice_bytes && kb_begin * 64 + off < p.k) ? *reinterpret_cast<const v4i *>(srow + off) : v4i{0, 0, 0, 0};
    }
  } else {
    const int8_t *xrow = reinterpret_cast<const int8_t *>(p.x) + (long long)min(m0 + c16, g_end - 1) * p.k;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int kb = kb_begin + wave + ST_WAVES * j;
      const int k0 = kb * 64 + 16 * h;   // K % 16 == 0: 16 K bytes all inside or all outside
      const bool ok = kb < kb_end && k0 < p.k;
      xf[j] = ok ? *reinterpret_cast<const v4i *>(xrow + k0) : v4i{0, 0, 0, 0};
    }
  }

  v4i ring[D];
  const int cg_base = strip * p.strip_groups * k_blocks * 1024;   // byte offset of the strip's first column group
  auto issue = [&](int cg, auto j_c, auto slot_c) {
    constexpr int J = decltype(j_c)::value, SLOT = decltype(slot_c)::value;
    const unsigned vo = cg < cg_count ? voff[J] : kBufferOob;
    ring[SLOT] = __builtin_amdgcn_raw_buffer_load_b128(rw, vo, cg_base + cg * k_blocks * 1024, kStreamAux);
  };
  static_for<NB>([&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    if constexpr (J < D) issue(0, j_c, j_c);
  });
  if constexpr (XLDS) {
    // (the x rows were requested before the weights, so waiting for them does not wait for the weight stream; the
    // staging area is the reduction area of the end of the kernel: the second barrier keeps a wave that is already
    // parking its first partial tile from overwriting fragments another wave has not read yet)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int off = (st_col + 16 * j) * 16;
      if (off < slice_bytes) *reinterpret_cast<v4i *>(st_smem + st_row * x_pitch + off) = xtmp[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int kb_rel = wave + ST_WAVES * j;
      xf[j] = kb_rel * 64 < slice_bytes ? *reinterpret_cast<const v4i *>(st_smem + c16 * x_pitch + kb_rel * 64 + 16 * h) : v4i{0, 0, 0, 0};
    }
    __syncthreads();
  }
  // epilogue operands of this thread's outputs (column groups wave + 4 e, rows 4 h .. 4 h + 3), requested behind the
  // first weight loads so that they are in registers long before the stream ends: a memory round trip after the
  // reduction is as long as a tenth of the whole kernel on a 45 MB weight set
  const bool rows_ok = 4 * h < chunk_rows;  // at least one of the lane's 4 rows is part of the chunk
  int ep_bias[4];
  float ep_scale[4], pt[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int n = n0 + 16 * (wave + 4 * e) + c16;
    const bool live = wave + 4 * e < cg_count && n < p.n && rows_ok;
    ep_bias[e] = live ? load_bias(p, grp, n) : 0;
    ep_scale[e] = (live && p.out_dtype != DT_I32) ? load_scale(p, grp, n) : 1.0f;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) pt[r] = (p.per_token && 4 * h + r < chunk_rows) ? p.per_token[m0 + 4 * h + r] : 1.0f;
  for (int cg = 0; cg < cg_count; ++cg) {
    v4i a0 = v4i{0, 0, 0, 0}, a1 = v4i{0, 0, 0, 0};
    static_for<NB>([&](auto j_c) {
      constexpr int J = decltype(j_c)::value;
      constexpr int SLOT = J % D;
      if constexpr (J & 1) a1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[J], ring[SLOT], a1, 0, 0, 0);
      else a0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[J], ring[SLOT], a0, 0, 0, 0);
      if constexpr (J + D < NB) issue(cg, std::integral_constant<int, J + D>{}, std::integral_constant<int, SLOT>{});
      else issue(cg + 1, std::integral_constant<int, J + D - NB>{}, std::integral_constant<int, SLOT>{});
    });
    red[wave][cg][lane] = a0 + a1;
  }
  __syncthreads();

  // ---- the four waves' tiles, added in wave order: thread (wave, lane) ends up with column groups
  // wave + 4 e (e = 0..3) of its lane position, rows 4h..4h+3, column 16 (wave + 4 e) + c ----------------
  v4i v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int cg = wave + 4 * e;
    v4i s = v4i{0, 0, 0, 0};
    if (cg < cg_count) {
      s = red[0][cg][lane];
#pragma unroll
      for (int w = 1; w < ST_WAVES; ++w) s += red[w][cg][lane];
    }
    v[e] = s;
  }

  if (p.split_k > 1) {
    // cross-workgroup reduction through the workspace with agent-scope relaxed atomics (no cache-wide
    // fences); slice s, 64-bit word e of thread t at ((s * 8 + e) * 256 + t); the last arriver adds up
    const long long tile = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * (ST_TILE_INTS / 2);
    if (rows_ok) {
      i64 *mine = base + (long long)ks * (ST_TILE_INTS / 2) + tid;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const i64 word = (i64)(((unsigned long long)(unsigned)v[e >> 1][2 * (e & 1) + 1] << 32) |
                               (unsigned)v[e >> 1][2 * (e & 1)]);
        __hip_atomic_store(mine + e * ST_THREADS, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    publish_partials_and_sync();
    if (tid == 0) *s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (rows_ok) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v4i{0, 0, 0, 0};
      for (int s0 = 0; s0 < p.split_k; s0 += 4) {
        i64 t[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int s = min(s0 + u, p.split_k - 1);
          const i64 *src = base + (long long)s * (ST_TILE_INTS / 2) + tid;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            t[u][e] = __hip_atomic_load(src + e * ST_THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

  // ---- epilogue: v[e] = rows 4h..4h+3 of column 16 (wave + 4 e) + c ---------------------------------------
  unsigned short(*tile_out)[ST_COLS + 8] = reinterpret_cast<unsigned short(*)[ST_COLS + 8]>(st_smem);
  __syncthreads();  // every wave is done reading red[]
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int cl = 16 * (wave + 4 * e) + c16;  // column inside the strip
    const int n = n0 + cl;
    if (wave + 4 * e < cg_count && n < p.n && rows_ok) {
      const int bias = ep_bias[e];
      if (p.out_dtype == DT_I32) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * h + r < chunk_rows)
            reinterpret_cast<int *>(p.out)[(long long)(m0 + 4 * h + r) * p.n + n] = v[e][r] + bias;
      } else {
        const float sc = ep_scale[e];
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
    const int item = tid + ST_THREADS * u;
    const int row = item >> 5, c8 = (item & 31) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && c8 < 16 * cg_count && n < p.n) {  // N % 16 == 0: 8 columns all inside or all outside
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

int stream_blocks_per_wave(int64_t k, int split_k) {
  const int64_t k_blocks = (k + 63) / 64;
  const int64_t per_split = (k_blocks + split_k - 1) / split_k;
  return (int)((per_split + ST_WAVES - 1) / ST_WAVES);
}

template <int NB, bool XLDS>
static hipError_t stream_launch_w8a8(const GmmParams &p, const dim3 &grid, hipStream_t stream) {
  auto kern = gmm_w8a8_stream_kernel<NB, XLDS>;
  // the x staging area (16 rows of at most 4 NB blocks of 64 bytes, 64 bytes of padding per row) shares the LDS of the
  // reduction area
  constexpr size_t lds = XLDS ? (ST_LDS > (size_t)16 * (4 * NB * 64 + 64) + 16 ? ST_LDS : (size_t)16 * (4 * NB * 64 + 64) + 16) : ST_LDS;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(ST_THREADS), lds, stream, p);
  return hipGetLastError();
}

hipError_t launch_stream_w8a8(const GmmParams &p, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const int nb = stream_blocks_per_wave(p.k, p.split_k);
  if (nb > 32 || p.strip_groups < 1 || p.strip_groups > ST_GROUPS) return hipErrorInvalidValue;   // the plan splits K until a slice has at most 128 blocks
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, kSkinnyRows), (unsigned)p.split_k);
  if (nb > 16) return stream_launch_w8a8<32, false>(p, grid, stream);   // (a 128-block slice of 16 rows would need 128 KiB of LDS)
  if (p.x_via_lds) {
    if (nb > 8) return stream_launch_w8a8<16, true>(p, grid, stream);
    if (nb > 4) return stream_launch_w8a8<8, true>(p, grid, stream);
    return stream_launch_w8a8<4, true>(p, grid, stream);
  }
  if (nb > 8) return stream_launch_w8a8<16, false>(p, grid, stream);
  if (nb > 4) return stream_launch_w8a8<8, false>(p, grid, stream);
  return stream_launch_w8a8<4, false>(p, grid, stream);
}

// ---- W8A8, more than 16 rows per group (packed weights) -----------------------------------------------------
// Same streaming idea for 16 TCH rows per workgroup (TCH = 2, 4, 8): a workgroup owns one chunk of 16 TCH rows of one
// group, a strip of four column groups (64 columns) and one K slice; wave w takes K blocks w, w + 4, ...  Per K block
// a wave loads its TCH x fragments (16 rows x 64 K bytes each) and the four weight blocks and issues 4 TCH MFMAs into
// accumulators that stay in registers for the whole slice.  At the end the four waves add their tiles into one LDS
// tile with ds_add (int32: exact in any order), K slices of different workgroups meet in the workspace as in the
// kernels above, and the epilogue stages the 16 TCH x 64 output tile in LDS for whole-row stores.  Operand delivery
// from L2 bounds this kernel, not the matrix pipe: per K block a wave moves (TCH + 4) KiB for 4 TCH MFMAs.
namespace {
constexpr int SM_GROUPS = 4;                    // column groups per strip
constexpr int SM_COLS = SM_GROUPS * 16;
template <int TCH>
struct SmShape {
  static constexpr int kRows = 16 * TCH;
  static constexpr int kFrags = SM_GROUPS * TCH;              // 16 x 16 int32 fragments of the tile
  static constexpr int kTileInts = kRows * SM_COLS;
  static constexpr size_t kLds = (size_t)kTileInts * 4 + 16;   // int32 tile (later the 16-bit output tile) + ticket
};
}  // namespace

template <int TCH>
__global__ void __launch_bounds__(ST_THREADS, 2) gmm_w8a8_streamm_kernel(const GmmParams p) {
  using S = SmShape<TCH>;
  extern __shared__ __align__(16) unsigned char st_smem[];
  int *tile = reinterpret_cast<int *>(st_smem);   // fragment (cg, t), lane, r at ((cg * TCH + t) * 64 + lane) * 4 + r
  unsigned *s_ticket = reinterpret_cast<unsigned *>(st_smem + S::kLds - 16);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, S::kRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * S::kRows;
  const int chunk_rows = min(S::kRows, g_end - m0);

  for (int i = tid; i < S::kTileInts / 4; i += ST_THREADS) reinterpret_cast<v4i *>(tile)[i] = v4i{0, 0, 0, 0};

  const int n0 = strip * SM_COLS;
  const int col_groups = (p.n + 15) / 16, k_blocks = (p.k + 63) / 64;
  const int cg_count = min(SM_GROUPS, col_groups - strip * SM_GROUPS);
  const long long group_bytes = (long long)col_groups * k_blocks * 1024;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(p.w + (long long)grp * group_bytes, group_bytes);
  const __amdgpu_buffer_rsrc_t rx = buffer_over(p.x, (long long)p.m * p.k);   // planned only when M * K < 2^31
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);
  const int cg_base = strip * SM_GROUPS * k_blocks * 1024;

  // row of fragment t in this lane (clamped into the group: rows past the chunk are computed and never stored)
  unsigned xoff[TCH];
#pragma unroll
  for (int t = 0; t < TCH; ++t) xoff[t] = (unsigned)(min(m0 + 16 * t + c16, g_end - 1) * p.k + 16 * h);

  v4i acc[SM_GROUPS][TCH];
#pragma unroll
  for (int cg = 0; cg < SM_GROUPS; ++cg)
#pragma unroll
    for (int t = 0; t < TCH; ++t) acc[cg][t] = v4i{0, 0, 0, 0};

  auto fetch = [&](int kb, v4i (&xf)[TCH], v4i (&wv)[SM_GROUPS]) {
    const bool live = kb < kb_end;
    const bool k_ok = live && kb * 64 + 16 * h < p.k;   // K % 16 == 0: 16 K bytes all inside or all outside
#pragma unroll
    for (int cg = 0; cg < SM_GROUPS; ++cg)
      wv[cg] = __builtin_amdgcn_raw_buffer_load_b128(rw, (live && cg < cg_count) ? (unsigned)(kb * 1024 + lane * 16) : kBufferOob,
                                                     cg_base + cg * k_blocks * 1024, kStreamAux);
#pragma unroll
    for (int t = 0; t < TCH; ++t)
      xf[t] = __builtin_amdgcn_raw_buffer_load_b128(rx, k_ok ? xoff[t] + (unsigned)(kb * 64) : kBufferOob, 0, 0);
  };
  auto multiply = [&](const v4i (&xf)[TCH], const v4i (&wv)[SM_GROUPS]) {
#pragma unroll
    for (int cg = 0; cg < SM_GROUPS; ++cg)
#pragma unroll
      for (int t = 0; t < TCH; ++t) acc[cg][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[t], wv[cg], acc[cg][t], 0, 0, 0);
  };
  {
    // two K blocks in flight per wave: the loads of the next block are issued before this one is multiplied
    v4i xa[TCH], wa[SM_GROUPS], xb[TCH], wb[SM_GROUPS];
    int kb = kb_begin + wave;
    fetch(kb, xa, wa);
    for (; kb < kb_end; kb += 2 * ST_WAVES) {
      fetch(kb + ST_WAVES, xb, wb);   // past the slice: masked, zeros
      multiply(xa, wa);
      fetch(kb + 2 * ST_WAVES, xa, wa);
      multiply(xb, wb);
    }
  }

  __syncthreads();   // the tile is zeroed
#pragma unroll
  for (int cg = 0; cg < SM_GROUPS; ++cg)
#pragma unroll
    for (int t = 0; t < TCH; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        __hip_atomic_fetch_add(tile + ((cg * TCH + t) * 64 + lane) * 4 + r, acc[cg][t][r], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
  __syncthreads();

  // thread tid owns fragments f = j * 4 + wave (j = 0..TCH-1) at its lane position: rows 16 t + 4 h + r, column 16 cg + c
  constexpr int OWN = S::kFrags / ST_WAVES;   // = TCH
  v4i v[OWN];
#pragma unroll
  for (int j = 0; j < OWN; ++j) v[j] = reinterpret_cast<const v4i *>(tile)[(j * ST_WAVES + wave) * 64 + lane];

  if (p.split_k > 1) {
    // slice s, fragment word (j, half) of thread t at ((s * OWN + j) * 2 + half) * 256 + t, 64-bit words
    const long long tile_id = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile_id * p.split_k * (S::kTileInts / 2);
    i64 *mine = base + (long long)ks * (S::kTileInts / 2) + tid;
#pragma unroll
    for (int j = 0; j < OWN; ++j)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const i64 word = (i64)(((unsigned long long)(unsigned)v[j][2 * hf + 1] << 32) | (unsigned)v[j][2 * hf]);
        __hip_atomic_store(mine + (j * 2 + hf) * ST_THREADS, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    publish_partials_and_sync();
    if (tid == 0) *s_ticket = __hip_atomic_fetch_add(&p.counters[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int j = 0; j < OWN; ++j) v[j] = v4i{0, 0, 0, 0};
    for (int s = 0; s < p.split_k; ++s) {
      const i64 *src = base + (long long)s * (S::kTileInts / 2) + tid;
      i64 t2[OWN][2];
#pragma unroll
      for (int j = 0; j < OWN; ++j)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
          t2[j][hf] = __hip_atomic_load(src + (j * 2 + hf) * ST_THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int j = 0; j < OWN; ++j)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          v[j][2 * hf] += (int)(unsigned)(unsigned long long)t2[j][hf];
          v[j][2 * hf + 1] += (int)(unsigned)((unsigned long long)t2[j][hf] >> 32);
        }
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------------------
  unsigned short(*tile_out)[SM_COLS + 8] = reinterpret_cast<unsigned short(*)[SM_COLS + 8]>(st_smem);
  __syncthreads();   // every thread holds its part of the int32 tile: the LDS tile can be reused
#pragma unroll
  for (int j = 0; j < OWN; ++j) {
    const int f = j * ST_WAVES + wave, cg = f / TCH, t = f % TCH;
    const int cl = 16 * cg + c16, n = n0 + cl;
    if (cg < cg_count && n < p.n) {
      const int bias = load_bias(p, grp, n);
      const float sc = p.out_dtype == DT_I32 ? 1.0f : load_scale(p, grp, n);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 16 * t + 4 * h + r;
        if (row < chunk_rows) {
          if (p.out_dtype == DT_I32) {
            reinterpret_cast<int *>(p.out)[(long long)(m0 + row) * p.n + n] = v[j][r] + bias;
          } else {
            const float f32 = dequant(v[j][r] + bias, sc, p.per_token ? p.per_token[m0 + row] : 1.0f);
            tile_out[row][cl] = half_out(p, f32);
          }
        }
      }
    }
  }
  if (p.out_dtype == DT_I32) return;
  __syncthreads();
  // whole-row stores: 16 TCH rows x 8 pieces of 8 columns
  for (int item = tid; item < S::kRows * 8; item += ST_THREADS) {
    const int row = item >> 3, c8 = (item & 7) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && c8 < 16 * cg_count && n < p.n) {
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

int streamm_chunk_rows(int tch) { return 16 * tch; }
size_t streamm_tile_bytes(int tch) { return (size_t)16 * tch * SM_COLS * 4; }

template <int TCH>
static hipError_t streamm_launch(const GmmParams &p, const dim3 &grid, hipStream_t stream) {
  hipLaunchKernelGGL(gmm_w8a8_streamm_kernel<TCH>, grid, dim3(ST_THREADS), SmShape<TCH>::kLds, stream, p);
  return hipGetLastError();
}

// tch = 16-row fragments per chunk (2, 4 or 8); p.max_chunks counts chunks of 16 tch rows, p.n_strips strips of 64 columns
hipError_t launch_streamm_w8a8(const GmmParams &p, int tch, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, 16 * tch), (unsigned)p.split_k);
  if (tch == 8) return streamm_launch<8>(p, grid, stream);
  if (tch == 4) return streamm_launch<4>(p, grid, stream);
  if (tch == 2) return streamm_launch<2>(p, grid, stream);
  return hipErrorInvalidValue;
}

// ---- weight-only (bf16 / f16 activations) ------------------------------------------------------------------
// The 16 K bytes a lane holds of a block feed two v_mfma_f32_16x16x32_{bf16,f16}: bytes 0..7 and bytes 8..15, each
// turned into exact 16-bit values of (w + 128) (v_cvt_f32_ubyteN on w ^ 0x80, then a 16-bit pack).  The x fragments
// follow the same K order: for block b, lane (c, q), step s the 8 values x[c][64 b + 16 q + 8 s ..].  As in the
// row-major weight-only kernel the row sums of x (one MFMA against ones per fragment, once per workgroup) fold the
// offset and the +128 into the epilogue:  out = s * (sum_k x (w + 128) + (o - 128) sum_k x).
namespace {
constexpr int SA_TILE_WORDS = kSkinnyRows * ST_COLS / 2 + 128;   // 64-bit words: partial tile + 4 row sums per lane slot
constexpr size_t SA_LDS = (size_t)ST_WAVES * ST_GROUPS * 64 * 16 + (size_t)ST_WAVES * 64 * 16 + 16;

template <bool BF16>
__device__ __forceinline__ unsigned sa_pack2(float lo, float hi) {
  if constexpr (BF16) {
    // both values are integers below 256: the upper 16 bits of the float32 pattern are the exact bf16
    return perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
  } else {
    return __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
}
template <int B>
__device__ __forceinline__ float sa_ubyte(unsigned w) {
  return (float)((w >> (8 * B)) & 0xFFu);   // v_cvt_f32_ubyteB
}
// 8 consecutive K bytes (two dwords, already + 128) -> the 8 16-bit values of one MFMA operand
template <bool BF16>
__device__ __forceinline__ v4i sa_frag(unsigned lo, unsigned hi) {
  v4i f;
  f[0] = (int)sa_pack2<BF16>(sa_ubyte<0>(lo), sa_ubyte<1>(lo));
  f[1] = (int)sa_pack2<BF16>(sa_ubyte<2>(lo), sa_ubyte<3>(lo));
  f[2] = (int)sa_pack2<BF16>(sa_ubyte<0>(hi), sa_ubyte<1>(hi));
  f[3] = (int)sa_pack2<BF16>(sa_ubyte<2>(hi), sa_ubyte<3>(hi));
  return f;
}
template <bool BF16>
__device__ __forceinline__ v4f sa_mfma(const v4i &a, const v4i &b, const v4f &c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
}
template <bool BF16>
__device__ __forceinline__ float sa_half_like(unsigned short b) {
  return BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}
}  // namespace

template <bool BF16, int NB>
__global__ void __launch_bounds__(ST_THREADS, 2) gmm_a16w8_stream_kernel(const GmmParams p) {
  extern __shared__ __align__(16) unsigned char st_smem[];
  v4f(*red)[ST_GROUPS][64] = reinterpret_cast<v4f(*)[ST_GROUPS][64]>(st_smem);   // [wave][column group][lane]
  v4f(*red_rs)[64] = reinterpret_cast<v4f(*)[64]>(st_smem + (size_t)ST_WAVES * ST_GROUPS * 64 * 16);
  unsigned *s_ticket = reinterpret_cast<unsigned *>(st_smem + SA_LDS - 16);
  constexpr int D = NB < 8 ? NB : 8;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x, ks = blockIdx.z;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, kSkinnyRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * kSkinnyRows;
  const int chunk_rows = min(kSkinnyRows, g_end - m0);

  const int n0 = strip * p.strip_groups * 16;
  const int col_groups = (p.n + 15) / 16, k_blocks = (p.k + 63) / 64;
  const int cg_count = min(p.strip_groups, col_groups - strip * p.strip_groups);
  const long long group_bytes = (long long)col_groups * k_blocks * 1024;
  const __amdgpu_buffer_rsrc_t rw = buffer_over(p.w + (long long)grp * group_bytes, group_bytes);
  const int per_split = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb_begin = ks * per_split;
  const int kb_end = min(k_blocks, kb_begin + per_split);

  // x fragments of the wave's blocks, through a descriptor over the chunk's rows (zeros past the slice or past K): all
  // requested before anything waits -- a load under a condition would be waited for on the spot (vmcnt(0)), one
  // memory round trip per fragment before the first weight is asked for
  const __amdgpu_buffer_rsrc_t rx = buffer_over(reinterpret_cast<const unsigned short *>(p.x) + (long long)m0 * p.k,
                                                2ll * chunk_rows * p.k);
  const unsigned x_row_byte = 2u * (unsigned)min(c16, chunk_rows - 1) * (unsigned)p.k;
  v4i xf[NB][2];
  unsigned voff[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int kb = kb_begin + wave + ST_WAVES * j;
    const int k0 = kb * 64 + 16 * h;   // K % 16 == 0: the 16 K positions are all inside or all outside
    const bool ok = kb < kb_end && k0 < p.k;
    xf[j][0] = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? x_row_byte + 2u * (unsigned)k0 : kBufferOob, 0, 0);
    xf[j][1] = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? x_row_byte + 2u * (unsigned)k0 + 16u : kBufferOob, 0, 0);
    voff[j] = kb < kb_end ? (unsigned)(kb * 1024 + lane * 16) : kBufferOob;
  }

  v4i ring[D];
  const int cg_base = strip * p.strip_groups * k_blocks * 1024;
  auto issue = [&](int cg, auto j_c, auto slot_c) {
    constexpr int J = decltype(j_c)::value, SLOT = decltype(slot_c)::value;
    const unsigned vo = cg < cg_count ? voff[J] : kBufferOob;
    ring[SLOT] = __builtin_amdgcn_raw_buffer_load_b128(rw, vo, cg_base + cg * k_blocks * 1024, kStreamAux);
  };
  static_for<NB>([&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    if constexpr (J < D) issue(0, j_c, j_c);
  });
  // antiquant scale and offset of this thread's output columns (column groups wave + 4 e), requested behind the first
  // weight loads (16-bit elements: the word that holds them, branch-free; decoded in the epilogue)
  const bool rows_ok = 4 * h < chunk_rows;
  unsigned sc_word[4], of_word[4];
  {
    const __amdgpu_buffer_rsrc_t rs_sc = buffer_over(p.aq_scale, p.aq_scale ? 2ll * p.e * p.n : 0);
    const __amdgpu_buffer_rsrc_t rs_of = buffer_over(p.aq_offset, p.aq_offset ? 2ll * p.e * p.n : 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int n = n0 + 16 * (wave + 4 * e) + c16;
      const bool live = wave + 4 * e < cg_count && n < p.n && rows_ok;
      const unsigned byte = 2u * (unsigned)((long long)grp * p.n + n);
      sc_word[e] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_sc, live ? (byte & ~3u) : kBufferOob, 0, 0);
      of_word[e] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_of, live ? (byte & ~3u) : kBufferOob, 0, 0);
    }
  }
  for (int cg = 0; cg < cg_count; ++cg) {
    v4f a0 = v4f{0.f, 0.f, 0.f, 0.f}, a1 = v4f{0.f, 0.f, 0.f, 0.f};
    static_for<NB>([&](auto j_c) {
      constexpr int J = decltype(j_c)::value;
      constexpr int SLOT = J % D;
      const v4i r = ring[SLOT];
      const unsigned d0 = (unsigned)r[0] ^ 0x80808080u, d1 = (unsigned)r[1] ^ 0x80808080u;   // w + 128 as unsigned bytes
      const unsigned d2 = (unsigned)r[2] ^ 0x80808080u, d3 = (unsigned)r[3] ^ 0x80808080u;
      a0 = sa_mfma<BF16>(xf[J][0], sa_frag<BF16>(d0, d1), a0);
      a1 = sa_mfma<BF16>(xf[J][1], sa_frag<BF16>(d2, d3), a1);
      if constexpr (J + D < NB) issue(cg, std::integral_constant<int, J + D>{}, std::integral_constant<int, SLOT>{});
      else issue(cg + 1, std::integral_constant<int, J + D - NB>{}, std::integral_constant<int, SLOT>{});
      // the refill stays behind the step that freed its slot: left to itself the scheduler gathers the next column
      // group's loads at the end of the loop body, and the wave's load queue runs empty once per column group
      __builtin_amdgcn_sched_barrier(0);
    });
    red[wave][cg][lane] = a0 + a1;
  }
  // row sums of x over the wave's K blocks (for the offset term), by the matrix pipe against a fragment of ones
  const unsigned ones = BF16 ? 0x3F803F80u : 0x3C003C00u;
  const v4i ones_frag = v4i{(int)ones, (int)ones, (int)ones, (int)ones};
  v4f rs = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    rs = sa_mfma<BF16>(xf[j][0], ones_frag, rs);
    rs = sa_mfma<BF16>(xf[j][1], ones_frag, rs);
  }
  red_rs[wave][lane] = rs;
  __syncthreads();

  // the four waves' tiles and row sums, added in wave order (reproducible run to run)
  v4f v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int cg = wave + 4 * e;
    v4f s = v4f{0.f, 0.f, 0.f, 0.f};
    if (cg < cg_count) {
      s = red[0][cg][lane];
#pragma unroll
      for (int w = 1; w < ST_WAVES; ++w) s += red[w][cg][lane];
    }
    v[e] = s;
  }
  v4f xs = red_rs[0][lane];
#pragma unroll
  for (int w = 1; w < ST_WAVES; ++w) xs += red_rs[w][lane];

  if (p.split_k > 1) {
    // float32 partials through the workspace, added in slice order by the last arriver.  Slice s: word e (0..7) of
    // thread t at (s * SA_TILE_WORDS + e * 256 + t); row sums of wave 0's lanes at (... + 2048 + 2 lane + {0, 1})
    const long long tile = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * SA_TILE_WORDS;
    auto pack = [](float lo, float hi) {
      return (i64)(((unsigned long long)__float_as_uint(hi) << 32) | __float_as_uint(lo));
    };
    if (rows_ok) {
      i64 *mine = base + (long long)ks * SA_TILE_WORDS;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        __hip_atomic_store(mine + e * ST_THREADS + tid, pack(v[e >> 1][2 * (e & 1)], v[e >> 1][2 * (e & 1) + 1]),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (wave == 0) {
        __hip_atomic_store(mine + 2048 + 2 * lane, pack(xs[0], xs[1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + 2048 + 2 * lane + 1, pack(xs[2], xs[3]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    publish_partials_and_sync();
    if (tid == 0) *s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*s_ticket != (unsigned)(p.split_k - 1)) return;
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
          const i64 *src = base + (long long)s * SA_TILE_WORDS;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            t[u][e] = __hip_atomic_load(src + e * ST_THREADS + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

  // ---- epilogue: v[e] = rows 4h..4h+3 of column 16 (wave + 4 e) + c --------------------------------------------
  unsigned short(*tile_out)[ST_COLS + 8] = reinterpret_cast<unsigned short(*)[ST_COLS + 8]>(st_smem);
  __syncthreads();   // every wave is done reading red[]
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int cl = 16 * (wave + 4 * e) + c16;
    const int n = n0 + cl;
    if (wave + 4 * e < cg_count && n < p.n && rows_ok) {
      const bool upper = ((long long)grp * p.n + n) & 1;   // which half of its word the element is
      const float s = p.aq_scale ? sa_half_like<BF16>((unsigned short)(upper ? sc_word[e] >> 16 : sc_word[e])) : 1.0f;
      const float o = p.aq_offset ? sa_half_like<BF16>((unsigned short)(upper ? of_word[e] >> 16 : of_word[e])) : 0.0f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float f = fmaf(o - 128.0f, xs[r], v[e][r]) * s;
        tile_out[4 * h + r][cl] = half_out(p, f);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int item = tid + ST_THREADS * u;
    const int row = item >> 5, c8 = (item & 31) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && c8 < 16 * cg_count && n < p.n) {
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

size_t stream_a16w8_tile_bytes() { return (size_t)SA_TILE_WORDS * 8; }

template <bool BF16, int NB>
static hipError_t stream_launch_a16w8(const GmmParams &p, const dim3 &grid, hipStream_t stream) {
  auto kern = gmm_a16w8_stream_kernel<BF16, NB>;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)SA_LDS);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(ST_THREADS), SA_LDS, stream, p);
  return hipGetLastError();
}

hipError_t launch_stream_a16w8(const GmmParams &p, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  const int nb = stream_blocks_per_wave(p.k, p.split_k);
  if (nb > 16 || p.strip_groups < 1 || p.strip_groups > ST_GROUPS) return hipErrorInvalidValue;   // slices of at most 64 blocks
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, kSkinnyRows), (unsigned)p.split_k);
  const bool bf = p.x_dtype == DT_BF16;
  if (nb > 8) return bf ? stream_launch_a16w8<true, 16>(p, grid, stream) : stream_launch_a16w8<false, 16>(p, grid, stream);
  if (nb > 4) return bf ? stream_launch_a16w8<true, 8>(p, grid, stream) : stream_launch_a16w8<false, 8>(p, grid, stream);
  return bf ? stream_launch_a16w8<true, 4>(p, grid, stream) : stream_launch_a16w8<false, 4>(p, grid, stream);
}

// ---- weight-only, more than 16 rows per group (packed weights) ------------------------------------------------
// A workgroup owns one chunk of 16 TCH rows of one group (TCH = 2, 4; 128-row chunks have the kernel below) and a strip
// of 4 G column groups (G = 2, 4: 128 or 256 columns) over all of K; wave w owns column groups w G .. w G + G - 1 of the
// strip and walks every K block, so its accumulators are complete sums: no K split, no reduction between waves, the same float32 summation order run to run.
// Per K block the workgroup brings the chunk's x slab (16 TCH rows x 64 K, 16-bit) into LDS once -- every wave needs
// all of it, and 16-bit x is twice the bytes of the weights it meets -- while each wave requests its G weight blocks,
// converts them to 16-bit operands once and uses them for all TCH row fragments (2 G TCH MFMAs, plus 2 TCH against ones
// for the row sums that fold the offset into the epilogue).  A group's weights are streamed once per 16 TCH rows
// instead of once per 16.  LDS rows of 128 payload bytes at a 144-byte pitch: the 16 lanes of a fragment read (16
// consecutive rows, one 16-byte chunk) fall into 16 different bank groups.
//
// KN (32-row chunks only; larger chunks of this layout have the kernel below): the weights are row-major [E,K,N] instead
// of packed.  Then the workgroup also brings the strip's weight slab (64 K
// rows x 64 G column bytes, whole lines) into LDS as it lies in memory, and a wave gets the operand of a 16 x 16 x 32
// MFMA with one LDS transpose read (ds_read_b64_tr_b8: of a block of 16 lanes, lane i names 8 bytes M[i][0..7] and lane j
// receives byte b = M[2 b + j / 8][j % 8]; with lanes 2 b and 2 b + 1 on the two halves of the 16 column bytes of K row
// b, lane j of block q holds K rows 8 q .. 8 q + 7 of column j): lane group q then multiplies K positions 32 s + 8 q ..
// of step s, and reads x chunk 4 s + q instead of 2 q + s.  Weight rows sit at a pitch of 64 G + 16 bytes (the 8 rows
// of a block's read, and the two blocks of a half wave, in different bank groups).
namespace {
template <int TCH, int G, bool KN = false>
struct SamShape {
  static constexpr int kRows = 16 * TCH;
  static constexpr int kCols = 64 * G;                         // 4 waves x G column groups x 16
  static constexpr int kPitch = 144;                           // bytes of an x row in LDS (64 K x 2 bytes + 16)
  static constexpr int kStage = kRows * kPitch;                // one K block of the chunk's x
  static constexpr int kPieces = kRows * 8 / ST_THREADS;       // 16-byte pieces of a slab per thread
  static constexpr int kWPitch = kCols + 16;                   // [E,K,N]: bytes of a weight K row in LDS
  static constexpr int kWStage = KN ? 64 * kWPitch : 0;        // [E,K,N]: one K block of the strip's weights
  static constexpr int kWPieces = 64 * kCols / 16 / ST_THREADS;   // its 16-byte pieces per thread (= G)
  static constexpr int kSlabs = 2 * (kStage + kWStage);        // two stages of operands
  static constexpr size_t kOut = (size_t)kRows * (kCols + 8) * 2;   // 16-bit output tile of the epilogue
  static constexpr size_t kLds = kSlabs > kOut ? kSlabs : kOut;
  static_assert(kPieces >= 1 && kWPieces == G, "slab pieces per thread");
};
}  // namespace

template <bool BF16, int TCH, int G, bool KN = false>
__global__ void __launch_bounds__(ST_THREADS, 2) gmm_a16w8_rows_kernel(const GmmParams p) {
  using S = SamShape<TCH, G, KN>;
  extern __shared__ __align__(16) unsigned char st_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int strip = blockIdx.x;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, S::kRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * S::kRows;
  const int chunk_rows = min(S::kRows, g_end - m0);

  const int n0 = strip * S::kCols;
  const int col_groups = (p.n + 15) / 16, k_blocks = (p.k + 63) / 64;
  const int cg0 = strip * 4 * G + wave * G;                          // this wave's first column group
  const int cg_count = max(0, min(G, col_groups - cg0));
  const long long group_bytes = KN ? (long long)p.k * p.n : (long long)col_groups * k_blocks * 1024;
  // ([E,K,N]: the window starts at the strip's first column and ends with the expert's matrix; every offset goes into
  // the range-checked per-lane part, so K rows past K read as zeros, and a chunk past N reads bytes of the next K row
  // into columns that are never stored)
  const __amdgpu_buffer_rsrc_t rw = KN ? buffer_over(p.w + (long long)grp * group_bytes + n0, group_bytes - n0)
                                       : buffer_over(p.w + (long long)grp * group_bytes, group_bytes);
  // (a window over the chunk's rows: 16-bit x can be twice as many bytes as a 32-bit window holds)
  const __amdgpu_buffer_rsrc_t rx = buffer_over(reinterpret_cast<const unsigned short *>(p.x) + (long long)m0 * p.k,
                                                2ll * chunk_rows * p.k);
  unsigned char *w_smem = st_smem + 2 * S::kStage;   // [E,K,N]: the two weight stages behind the two x stages

  // the slab pieces this thread carries: piece i = tid + 256 u is row i / 8 (clamped into the chunk: rows past it are
  // computed at most and never stored), 16-byte chunk i % 8 of the block's 128 bytes
  unsigned x_src[S::kPieces], x_dst[S::kPieces];
#pragma unroll
  for (int u = 0; u < S::kPieces; ++u) {
    const int i = tid + ST_THREADS * u, row = i >> 3, chunk = i & 7;
    x_src[u] = 2u * (unsigned)min(row, chunk_rows - 1) * (unsigned)p.k + 16u * (unsigned)chunk;
    x_dst[u] = (unsigned)(row * S::kPitch + chunk * 16);
  }
  auto load_x = [&](int kb, v4i (&xr)[S::kPieces]) {
#pragma unroll
    for (int u = 0; u < S::kPieces; ++u) {
      const int chunk = (tid + ST_THREADS * u) & 7;
      const bool ok = kb < k_blocks && kb * 64 + 8 * chunk < p.k;   // K % 16 == 0: a chunk's 8 K positions are all inside or all outside
      xr[u] = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? x_src[u] + (unsigned)(kb * 128) : kBufferOob, 0, 0);
    }
  };
  auto store_x = [&](int stage, const v4i (&xr)[S::kPieces]) {
#pragma unroll
    for (int u = 0; u < S::kPieces; ++u) *reinterpret_cast<v4i *>(st_smem + stage * S::kStage + x_dst[u]) = xr[u];
  };
  // packed: this wave's G blocks of K block kb, straight into the registers they are multiplied from.  [E,K,N]: this
  // thread's G pieces of the strip's slab (piece i = tid + 256 u: K row i / (4 G), 16-byte chunk i % (4 G)), on their way to LDS
  auto load_w = [&](int kb, v4i (&wv)[G]) {
#pragma unroll
    for (int cg = 0; cg < G; ++cg) {
      if constexpr (KN) {
        const int i = tid + ST_THREADS * cg, row = i / (4 * G), chunk = i % (4 * G);
        const bool ok = kb < k_blocks && n0 + 16 * chunk < p.n;
        wv[cg] = __builtin_amdgcn_raw_buffer_load_b128(rw, ok ? (unsigned)(kb * 64 + row) * (unsigned)p.n + 16u * (unsigned)chunk : kBufferOob,
                                                       0, kStreamAux);
      } else {
        wv[cg] = __builtin_amdgcn_raw_buffer_load_b128(rw, (kb < k_blocks && cg < cg_count) ? (unsigned)(kb * 1024 + lane * 16) : kBufferOob,
                                                       (cg0 + cg) * k_blocks * 1024, kStreamAux);
      }
    }
  };
  auto store_w = [&](int stage, const v4i (&wv)[G]) {
    if constexpr (KN) {
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int i = tid + ST_THREADS * u, row = i / (4 * G), chunk = i % (4 * G);
        *reinterpret_cast<v4i *>(w_smem + stage * S::kWStage + row * S::kWPitch + chunk * 16) = wv[u];
      }
    }
  };

  v4f acc[G][TCH], rs[TCH];
#pragma unroll
  for (int t = 0; t < TCH; ++t) {
    rs[t] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int cg = 0; cg < G; ++cg) acc[cg][t] = v4f{0.f, 0.f, 0.f, 0.f};
  }
  const unsigned ones = BF16 ? 0x3F803F80u : 0x3C003C00u;
  const v4i ones_frag = v4i{(int)ones, (int)ones, (int)ones, (int)ones};
  // x fragments as in the 16-row kernel: lane (c, q), step s holds the 8 values x[16 t + c][64 b + 16 q + 8 s ..], i.e.
  // chunk 2 q + s of row 16 t + c.  (A block that was not loaded reads as w + 128 = 128: its x is zeros, it adds nothing.)
  // LIVE = row fragments that hold rows of the chunk (a compile-time count: the others are neither read nor multiplied)
  auto multiply = [&](auto live_c, int stage, const v4i (&wv)[G]) {
    constexpr int LIVE = decltype(live_c)::value;
    v4i xf[LIVE][2];
#pragma unroll
    for (int t = 0; t < LIVE; ++t)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
        xf[t][s2] = *reinterpret_cast<const v4i *>(st_smem + stage * S::kStage + (16 * t + c16) * S::kPitch + (KN ? 4 * s2 + h : 2 * h + s2) * 16);
#pragma unroll
    for (int cg = 0; cg < G; ++cg) {
      unsigned d0, d1, d2, d3;   // w + 128 as unsigned bytes: the lane's 8 K positions of step 0, then of step 1
      if constexpr (KN) {
        typedef int v2i_t __attribute__((ext_vector_type(2)));
        typedef __attribute__((address_space(3))) v2i_t *lds_v2i;
        const unsigned char *src = w_smem + stage * S::kWStage + (8 * h + (c16 >> 1)) * S::kWPitch + 16 * (wave * G + cg) + (c16 & 1) * 8;
        const v2i_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(src));
        const v2i_t hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(src + 32 * S::kWPitch));
        d0 = (unsigned)lo.x ^ 0x80808080u; d1 = (unsigned)lo.y ^ 0x80808080u;
        d2 = (unsigned)hi.x ^ 0x80808080u; d3 = (unsigned)hi.y ^ 0x80808080u;
      } else {
        d0 = (unsigned)wv[cg][0] ^ 0x80808080u; d1 = (unsigned)wv[cg][1] ^ 0x80808080u;
        d2 = (unsigned)wv[cg][2] ^ 0x80808080u; d3 = (unsigned)wv[cg][3] ^ 0x80808080u;
      }
      const v4i w0 = sa_frag<BF16>(d0, d1), w1 = sa_frag<BF16>(d2, d3);
#pragma unroll
      for (int t = 0; t < LIVE; ++t) {
        acc[cg][t] = sa_mfma<BF16>(xf[t][0], w0, acc[cg][t]);
        acc[cg][t] = sa_mfma<BF16>(xf[t][1], w1, acc[cg][t]);
      }
    }
#pragma unroll
    for (int t = 0; t < LIVE; ++t) {
      rs[t] = sa_mfma<BF16>(xf[t][0], ones_frag, rs[t]);
      rs[t] = sa_mfma<BF16>(xf[t][1], ones_frag, rs[t]);
    }
  };

  // slab 0 to LDS, slab 1 and the weights of blocks 0 and 1 on their way
  v4i xr[S::kPieces], wa[G], wb[G];
  load_x(0, xr);
  load_w(0, wa);
  // antiquant scale and offset of this lane's G output columns, requested behind the first operand loads (16-bit
  // elements: the word that holds them, branch-free; decoded in the epilogue)
  unsigned sc_word[G], of_word[G];
  {
    const __amdgpu_buffer_rsrc_t rs_sc = buffer_over(p.aq_scale, p.aq_scale ? 2ll * p.e * p.n : 0);
    const __amdgpu_buffer_rsrc_t rs_of = buffer_over(p.aq_offset, p.aq_offset ? 2ll * p.e * p.n : 0);
#pragma unroll
    for (int cg = 0; cg < G; ++cg) {
      const int n = 16 * (cg0 + cg) + c16;
      const bool live = cg < cg_count && n < p.n;
      const unsigned byte = 2u * (unsigned)((long long)grp * p.n + n);
      sc_word[cg] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_sc, live ? (byte & ~3u) : kBufferOob, 0, 0);
      of_word[cg] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_of, live ? (byte & ~3u) : kBufferOob, 0, 0);
    }
  }
  // (LDS-only barrier: __syncthreads would also wait for the operand loads that are in flight on purpose)
  auto slab_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  store_x(0, xr);
  load_x(1, xr);
  if constexpr (KN) {   // (the weights take the same road as x: registers -> LDS, one block ahead of the multiply)
    store_w(0, wa);
    load_w(1, wa);
  }
  slab_barrier();
  // One barrier per K block: the slab of block kb + 1 is written to the other stage (which every wave finished reading
  // before the last barrier) while block kb is multiplied, and the requests run two blocks ahead.
  // One copy of the loop per number of row fragments that hold rows (the last chunk of a group is rarely full, and on
  // 64- and 128-row chunks the matrix pipe is what bounds this kernel); 32-row chunks keep one loop (two copies measured
  // slower there, 87 against 80 us at 64 tokens).  Written out rather than wrapped in a lambda: called through one, the
  // same loop came out of the scheduler 8 % slower.
  const int live = (TCH <= 2) ? TCH : (chunk_rows + 15) / 16;   // 1 .. TCH, the same for the whole workgroup
#define MSCO_ROWS_LOOP(LIVE)                                               \
  if constexpr (LIVE <= TCH) {                                             \
    if (live == LIVE) {                                                    \
      const std::integral_constant<int, (LIVE <= TCH ? LIVE : 1)> live_c;  \
      for (int kb = 0; kb < k_blocks; kb += 2) {                           \
        if constexpr (!KN) load_w(kb + 1, wb);                             \
        multiply(live_c, 0, wa);                                           \
        store_x(1, xr);                                                    \
        load_x(kb + 2, xr);                                                \
        if constexpr (KN) { store_w(1, wa); load_w(kb + 2, wa); }          \
        slab_barrier();                                                    \
        if constexpr (!KN) load_w(kb + 2, wa);                             \
        multiply(live_c, 1, KN ? wa : wb); /* (past K: zeros times 128) */ \
        store_x(0, xr);                                                    \
        load_x(kb + 3, xr);                                                \
        if constexpr (KN) { store_w(0, wa); load_w(kb + 3, wa); }          \
        slab_barrier();                                                    \
      }                                                                    \
    }                                                                      \
  }
  MSCO_ROWS_LOOP(1) MSCO_ROWS_LOOP(2) MSCO_ROWS_LOOP(3) MSCO_ROWS_LOOP(4)
#undef MSCO_ROWS_LOOP

  // ---- epilogue: out = s * (sum_k x (w + 128) + (o - 128) sum_k x); lane (c, h) holds rows 16 t + 4 h + r of column
  // 16 cg + c of its wave's column groups.  The output tile is staged in LDS (the slabs are done with) for whole-row stores.
  unsigned short(*tile_out)[S::kCols + 8] = reinterpret_cast<unsigned short(*)[S::kCols + 8]>(st_smem);
#pragma unroll
  for (int cg = 0; cg < G; ++cg) {
    const int n = 16 * (cg0 + cg) + c16, cl = 16 * (wave * G + cg) + c16;
    if (cg < cg_count && n < p.n) {
      const bool upper = ((long long)grp * p.n + n) & 1;   // which half of its word the element is
      const float sc = p.aq_scale ? sa_half_like<BF16>((unsigned short)(upper ? sc_word[cg] >> 16 : sc_word[cg])) : 1.0f;
      const float of = p.aq_offset ? sa_half_like<BF16>((unsigned short)(upper ? of_word[cg] >> 16 : of_word[cg])) : 0.0f;
#pragma unroll
      for (int t = 0; t < TCH; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = 16 * t + 4 * h + r;
          if (row < chunk_rows) tile_out[row][cl] = half_out(p, fmaf(of - 128.0f, rs[t][r], acc[cg][t][r]) * sc);
        }
    }
  }
  __syncthreads();
  // whole-row stores: 16 TCH rows x pieces of 8 columns
  constexpr int ROW_PIECES = S::kCols / 8;
  for (int item = tid; item < S::kRows * ROW_PIECES; item += ST_THREADS) {
    const int row = item / ROW_PIECES, c8 = (item % ROW_PIECES) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && n < p.n) {   // N % 16 == 0: 8 columns all inside or all outside
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

template <bool BF16, int TCH, int G, bool KN = false>
static hipError_t rows_launch_a16w8(const GmmParams &p, const dim3 &grid, hipStream_t stream) {
  using S = SamShape<TCH, G, KN>;
  auto kern = gmm_a16w8_rows_kernel<BF16, TCH, G, KN>;
  if constexpr (S::kLds > 64 * 1024) {
    static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::kLds);
      if (e != hipSuccess) return e;
      attr_set = true;
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(ST_THREADS), S::kLds, stream, p);
  return hipGetLastError();
}

// ---- weight-only, 64- and 128-row chunks on [E,K,N] weights, 128-row chunks on packed weights: 32 x 32 x 16 MFMAs ----
// The 16 x 16 x 32 forms above run at half the rate of the 32 x 32 forms, and a 128-row chunk of them fills the register
// file at 128 columns.  Here a workgroup owns a chunk of 32 TR rows (TR = 2, 4) and a strip of 128 GP columns; wave w owns
// the GP blocks of 32 columns w GP .. w GP + GP - 1 and all rows, again over all of K.  Both slabs go through LDS as they
// lie in memory.  Of a 16-K step, lane l of an x fragment holds row l % 32, K positions 8 (l / 32) .. + 7 (one 16-byte read),
// and of a weight fragment column l % 32 at the same K positions: one transpose read, with the four blocks of 16 lanes
// on (K half, column half) = (l / 32, l / 16 % 2).  Weight rows sit at a pitch of 128 GP + 32 bytes: the 8 rows and the
// two column halves a pass reads fall into 16 different bank groups.  PK: packed weights.  A block of 16 columns x 64 K
// keeps its lane order in LDS, and the same fragment is a plain 8-byte read (no transpose: a packed lane already holds 16
// consecutive K positions of one column).
// The row sums of x come from the vector unit instead of an MFMA against ones (which would cost a quarter of the matrix
// time here): a thread adds up the 8 values of every slab piece it carries to LDS (always the same row), and 8 neighbouring
// threads combine their sums at the end.
namespace {
typedef float v16f __attribute__((ext_vector_type(16)));
template <int TR, int GP, bool PK = false>
struct Rows32Shape {
  static constexpr int kRows = 32 * TR;
  static constexpr int kCols = 128 * GP;                       // 4 waves x GP blocks of 32 columns
  static constexpr int kPitch = 144;                           // bytes of an x row in LDS (64 K x 2 bytes + 16)
  static constexpr int kStage = kRows * kPitch;                // one K block of the chunk's x
  static constexpr int kPieces = kRows * 8 / ST_THREADS;       // 16-byte pieces of an x slab per thread
  static constexpr int kWPitch = kCols + 32;                   // bytes of a weight K row in LDS
  static constexpr int kWBlock = 1024 + 8;                     // packed: bytes of a 16-column block in LDS
  static constexpr int kWStage = PK ? (kCols / 16) * kWBlock : 64 * kWPitch;   // one K block of the strip's weights
  static constexpr int kWPieces = 64 * kCols / 16 / ST_THREADS;   // its 16-byte pieces per thread (= 2 GP)
  static constexpr int kSlabs = 2 * (kStage + kWStage);        // two stages of operands
  static constexpr int kOut = kRows * (kCols + 8) * 2;         // 16-bit output tile of the epilogue
  static constexpr int kTile = kSlabs > kOut ? kSlabs : kOut;
  static constexpr size_t kLds = (size_t)kTile + kRows * 4 + 16;   // + the chunk's row sums of x + the K split's ticket
  static constexpr size_t kSliceWords = (size_t)kRows * kCols / 2 + kRows / 2;   // 64-bit words of a K slice's partial tile
  static_assert(kPieces >= 1 && kWPieces == 2 * GP, "slab pieces per thread");
};
template <bool BF16>
__device__ __forceinline__ v16f rows32_mfma(const v4i &a, const v4i &b, const v16f &c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
}
// the sum of the 8 16-bit values of a slab piece, in float32, element 0 first
template <bool BF16>
__device__ __forceinline__ float rows32_sum8(const v4i &v) {
  float s = 0.f;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned w = (unsigned)v[d];
    s += sa_half_like<BF16>((unsigned short)w);
    s += sa_half_like<BF16>((unsigned short)(w >> 16));
  }
  return s;
}
}  // namespace

template <bool BF16, int TR, int GP, bool PK = false>
__global__ void __launch_bounds__(ST_THREADS, 2) gmm_a16w8_rows32_kernel(const GmmParams p) {
  using S = Rows32Shape<TR, GP, PK>;
  extern __shared__ __align__(16) unsigned char st_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, kh = lane >> 5;
  const int strip = blockIdx.x;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, S::kRows, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * S::kRows;
  const int chunk_rows = min(S::kRows, g_end - m0);

  const int n0 = strip * S::kCols;
  const int k_blocks = (p.k + 63) / 64, col_groups = (p.n + 15) / 16;
  // K slice of this workgroup (grid.z slices of whole blocks; one past the end of K adds zeros)
  const int ks = blockIdx.z, slice_blocks = (k_blocks + p.split_k - 1) / p.split_k;
  const int kb0 = ks * slice_blocks, kb_end = min(k_blocks, kb0 + slice_blocks);
  const long long group_bytes = PK ? (long long)col_groups * k_blocks * 1024 : (long long)p.k * p.n;
  // (windows as in the kernel above: the weights from the strip's first column to the end of the expert's matrix, K rows
  // past K read as zeros -- packed: the expert's blocks; x over the chunk's rows)
  const __amdgpu_buffer_rsrc_t rw = PK ? buffer_over(p.w + (long long)grp * group_bytes, group_bytes)
                                       : buffer_over(p.w + (long long)grp * group_bytes + n0, group_bytes - n0);
  const __amdgpu_buffer_rsrc_t rx = buffer_over(reinterpret_cast<const unsigned short *>(p.x) + (long long)m0 * p.k,
                                                2ll * chunk_rows * p.k);
  unsigned char *w_smem = st_smem + 2 * S::kStage;

  // x slab piece u of this thread: row tid / 8 + 32 u, 16-byte chunk tid % 8 of the block's 128 bytes (rows past the chunk
  // lie outside the window and read as zeros)
  const int x_chunk = tid & 7;
  const unsigned x_src = 2u * (unsigned)(tid >> 3) * (unsigned)p.k + 16u * (unsigned)x_chunk;
  const unsigned x_dst = (unsigned)((tid >> 3) * S::kPitch + x_chunk * 16);
  float x_sum[S::kPieces];
#pragma unroll
  for (int u = 0; u < S::kPieces; ++u) x_sum[u] = 0.f;
  auto load_x = [&](int kb, v4i (&xr)[S::kPieces]) {
    const bool ok = kb < kb_end && kb * 64 + 8 * x_chunk < p.k;   // K % 16 == 0: a chunk's 8 K positions are all inside or all outside
#pragma unroll
    for (int u = 0; u < S::kPieces; ++u)
      xr[u] = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? x_src + (unsigned)(64 * u) * (unsigned)p.k + (unsigned)(kb * 128) : kBufferOob, 0, 0);
  };
  auto store_x = [&](int stage, const v4i (&xr)[S::kPieces]) {   // (every piece passes here once: its share of the row sum)
#pragma unroll
    for (int u = 0; u < S::kPieces; ++u) {
      *reinterpret_cast<v4i *>(st_smem + stage * S::kStage + x_dst + 32 * u * S::kPitch) = xr[u];
      x_sum[u] += rows32_sum8<BF16>(xr[u]);
    }
  };
  // weight slab piece i = tid + 256 u: K row i / (8 GP), 16-byte chunk i % (8 GP) of the strip's columns.  Packed: lane
  // i % 64 of the strip's block i / 64 = wave + 4 u (a block is 16 columns x 64 K, lane (q, c) holding K positions 16 q ..
  // 16 q + 15 of column c), kept in LDS at a pitch of 1024 + 8 bytes, hence written in two halves
  auto load_w = [&](int kb, v4i (&wv)[S::kWPieces]) {
#pragma unroll
    for (int u = 0; u < S::kWPieces; ++u) {
      if constexpr (PK) {
        const int cg = strip * (8 * GP) + wave + 4 * u;
        wv[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, (kb < kb_end && cg < col_groups) ? (unsigned)(kb * 1024 + lane * 16) : kBufferOob,
                                                      min(cg, col_groups - 1) * k_blocks * 1024, kStreamAux);
      } else {
        const int i = tid + ST_THREADS * u, row = i / (8 * GP), chunk = i % (8 * GP);
        const bool ok = kb < kb_end && n0 + 16 * chunk < p.n;
        wv[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, ok ? (unsigned)(kb * 64 + row) * (unsigned)p.n + 16u * (unsigned)chunk : kBufferOob,
                                                      0, kStreamAux);
      }
    }
  };
  auto store_w = [&](int stage, const v4i (&wv)[S::kWPieces]) {
#pragma unroll
    for (int u = 0; u < S::kWPieces; ++u) {
      if constexpr (PK) {
        typedef int v2i_t __attribute__((ext_vector_type(2)));
        unsigned char *dst = w_smem + stage * S::kWStage + (wave + 4 * u) * S::kWBlock + lane * 16;
        *reinterpret_cast<v2i_t *>(dst) = v2i_t{wv[u][0], wv[u][1]};
        *reinterpret_cast<v2i_t *>(dst + 8) = v2i_t{wv[u][2], wv[u][3]};
      } else {
        const int i = tid + ST_THREADS * u, row = i / (8 * GP), chunk = i % (8 * GP);
        *reinterpret_cast<v4i *>(w_smem + stage * S::kWStage + row * S::kWPitch + chunk * 16) = wv[u];
      }
    }
  };

  v16f acc[GP][TR];
#pragma unroll
  for (int gp = 0; gp < GP; ++gp)
#pragma unroll
    for (int t = 0; t < TR; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[gp][t][v] = 0.f;

  // this lane's corner of the two slabs: x row l % 32 at chunk l / 32; of the weights the 8 bytes it names for a transpose
  // read (K row 8 (l / 32) + (l % 16) / 2, column half l / 16 % 2, byte half l % 2 of the wave's first block)
  const unsigned x_lane = (unsigned)(c32 * S::kPitch + kh * 16);
  // (packed: of block 2 (w GP + gp) + (l % 32) / 16, the lane of K group s and column l % 16, its half l / 32 -- a plain
  // 8-byte read; the 8-byte skew between blocks puts the two blocks of a pass into different banks)
  const unsigned w_lane = PK ? (unsigned)((2 * wave * GP + (c32 >> 4)) * S::kWBlock + (c32 & 15) * 16 + 8 * kh)
                             : (unsigned)((8 * kh + ((lane & 15) >> 1)) * S::kWPitch + 32 * wave * GP + 16 * ((lane >> 4) & 1) + 8 * (lane & 1));
  // LIVE = 32-row fragments that hold rows of the chunk (a compile-time count: the others are neither read nor multiplied)
  auto multiply = [&](auto live_c, int stage) {
    constexpr int LIVE = decltype(live_c)::value;
    typedef int v2i_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) v2i_t *lds_v2i;
    const unsigned char *xs = st_smem + stage * S::kStage + x_lane;
    const unsigned char *ws = w_smem + stage * S::kWStage + w_lane;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      v4i xf[LIVE];
#pragma unroll
      for (int t = 0; t < LIVE; ++t) xf[t] = *reinterpret_cast<const v4i *>(xs + 32 * t * S::kPitch + 32 * s);
#pragma unroll
      for (int gp = 0; gp < GP; ++gp) {
        v2i_t w8;
        if constexpr (PK) w8 = *reinterpret_cast<const v2i_t *>(ws + 256 * s + 2 * S::kWBlock * gp);
        else w8 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(ws + 16 * s * S::kWPitch + 32 * gp));
        const v4i wf = sa_frag<BF16>((unsigned)w8.x ^ 0x80808080u, (unsigned)w8.y ^ 0x80808080u);   // w + 128, exact in 16 bits
#pragma unroll
        for (int t = 0; t < LIVE; ++t) acc[gp][t] = rows32_mfma<BF16>(xf[t], wf, acc[gp][t]);
      }
    }
  };

  v4i xr[S::kPieces], wr[S::kWPieces];
  load_x(kb0, xr);
  load_w(kb0, wr);
  // antiquant scale and offset of this lane's GP output columns (16-bit elements: the word that holds them)
  unsigned sc_word[GP], of_word[GP];
  {
    const __amdgpu_buffer_rsrc_t rs_sc = buffer_over(p.aq_scale, p.aq_scale ? 2ll * p.e * p.n : 0);
    const __amdgpu_buffer_rsrc_t rs_of = buffer_over(p.aq_offset, p.aq_offset ? 2ll * p.e * p.n : 0);
#pragma unroll
    for (int gp = 0; gp < GP; ++gp) {
      const int n = n0 + 32 * (wave * GP + gp) + c32;
      const unsigned byte = 2u * (unsigned)((long long)grp * p.n + n);
      sc_word[gp] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_sc, n < p.n ? (byte & ~3u) : kBufferOob, 0, 0);
      of_word[gp] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_of, n < p.n ? (byte & ~3u) : kBufferOob, 0, 0);
    }
  }
  // (LDS-only barrier: __syncthreads would also wait for the operand loads that are in flight on purpose)
  auto slab_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  store_x(0, xr);
  load_x(kb0 + 1, xr);
  store_w(0, wr);
  load_w(kb0 + 1, wr);
  slab_barrier();
  // One barrier per K block, the requests two blocks ahead, one copy of the loop per number of live row fragments.
  const int live = (chunk_rows + 31) / 32;   // 1 .. TR, the same for the whole workgroup
#define MSCO_ROWS32_LOOP(LIVE)                                             \
  if constexpr (LIVE <= TR) {                                              \
    if (live == LIVE) {                                                    \
      const std::integral_constant<int, (LIVE <= TR ? LIVE : 1)> live_c;   \
      for (int kb = kb0; kb < kb_end; kb += 2) {                           \
        multiply(live_c, 0);                                               \
        store_x(1, xr);                                                    \
        load_x(kb + 2, xr);                                                \
        store_w(1, wr);                                                    \
        load_w(kb + 2, wr);                                                \
        slab_barrier();                                                    \
        multiply(live_c, 1); /* (past K: zeros times anything finite) */   \
        store_x(0, xr);                                                    \
        load_x(kb + 3, xr);                                                \
        store_w(0, wr);                                                    \
        load_w(kb + 3, wr);                                                \
        slab_barrier();                                                    \
      }                                                                    \
    }                                                                      \
  }
  MSCO_ROWS32_LOOP(1) MSCO_ROWS32_LOOP(2) MSCO_ROWS32_LOOP(3) MSCO_ROWS32_LOOP(4)
#undef MSCO_ROWS32_LOOP

  // ---- row sums: the 8 chunks of a row sit with 8 neighbouring threads
  float *row_sum = reinterpret_cast<float *>(st_smem + S::kTile);
#pragma unroll
  for (int u = 0; u < S::kPieces; ++u) {
    float v = x_sum[u];
    v += __shfl_xor(v, 1);
    v += __shfl_xor(v, 2);
    v += __shfl_xor(v, 4);
    if ((tid & 7) == 0) row_sum[(tid + ST_THREADS * u) >> 3] = v;
  }
  __syncthreads();

  if (p.split_k > 1) {
    // float32 partials through the workspace, added in slice order by the last arriver: 64-bit word i of thread t at
    // i * 256 + t (accumulator elements 2 i, 2 i + 1 in (gp, t, element) order), the row sums behind them
    typedef long long i64;
    constexpr int WORDS = GP * TR * 8;
    unsigned *s_ticket = reinterpret_cast<unsigned *>(st_smem + S::kTile + S::kRows * 4);
    const long long tile = ((long long)grp * p.max_chunks + mc) * p.n_strips + strip;
    i64 *base = reinterpret_cast<i64 *>(p.partial) + tile * p.split_k * (long long)S::kSliceWords;
    i64 *mine = base + (long long)ks * (long long)S::kSliceWords;
    auto pack = [](float lo, float hi) { return (i64)(((unsigned long long)__float_as_uint(hi) << 32) | __float_as_uint(lo)); };
#pragma unroll
    for (int gp = 0; gp < GP; ++gp)
#pragma unroll
      for (int t = 0; t < TR; ++t)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          __hip_atomic_store(mine + ((gp * TR + t) * 8 + i) * ST_THREADS + tid, pack(acc[gp][t][2 * i], acc[gp][t][2 * i + 1]),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid < S::kRows / 2)
      __hip_atomic_store(mine + WORDS * ST_THREADS + tid, pack(row_sum[2 * tid], row_sum[2 * tid + 1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    publish_partials_and_sync();
    if (tid == 0) *s_ticket = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*s_ticket != (unsigned)(p.split_k - 1)) return;
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // (as many loads in flight as the registers hold -- every round is a round trip to memory: blocks of up to 32 words,
    // two slices at a time where the accumulators leave room)
    constexpr int WB = WORDS < 32 ? WORDS : 32, NS = WORDS >= 64 ? 1 : 2;
#pragma unroll
    for (int gp = 0; gp < GP; ++gp)
#pragma unroll
      for (int t = 0; t < TR; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[gp][t][v] = 0.f;
#pragma unroll
    for (int b0 = 0; b0 < WORDS; b0 += WB) {
      for (int s0 = 0; s0 < p.split_k; s0 += NS) {
        i64 w[NS][WB];
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const i64 *src = base + (long long)min(s0 + u, p.split_k - 1) * (long long)S::kSliceWords + b0 * ST_THREADS + tid;
#pragma unroll
          for (int i = 0; i < WB; ++i) w[u][i] = __hip_atomic_load(src + i * ST_THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < NS; ++u)
          if (s0 + u < p.split_k) {
#pragma unroll
            for (int i = 0; i < WB; ++i) {
              const int word = b0 + i;   // (gp TR + t) 8 + pair
              acc[word / (8 * TR)][(word / 8) % TR][2 * (word % 8)] += __uint_as_float((unsigned)(unsigned long long)w[u][i]);
              acc[word / (8 * TR)][(word / 8) % TR][2 * (word % 8) + 1] += __uint_as_float((unsigned)((unsigned long long)w[u][i] >> 32));
            }
          }
      }
    }
    if (tid < S::kRows / 2) {   // (these threads read their two row sums above, before the barrier)
      float lo = 0.f, hi = 0.f;
      for (int s0 = 0; s0 < p.split_k; s0 += 8) {   // (eight loads in flight: one round trip for any split the plan makes)
        i64 w[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          w[u] = __hip_atomic_load(base + (long long)min(s0 + u, p.split_k - 1) * (long long)S::kSliceWords + WORDS * ST_THREADS + tid,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < p.split_k) {
            lo += __uint_as_float((unsigned)(unsigned long long)w[u]);
            hi += __uint_as_float((unsigned)((unsigned long long)w[u] >> 32));
          }
      }
      row_sum[2 * tid] = lo;
      row_sum[2 * tid + 1] = hi;
    }
    __syncthreads();
  }

  // ---- epilogue: out = s * (sum_k x (w + 128) + (o - 128) sum_k x); lane l holds column l % 32 of its wave's blocks and
  // rows 32 t + 8 j + 4 (l / 32) + r in accumulator element 4 j + r.  The output tile is staged in LDS (the slabs are
  // done with) for whole-row stores.
  unsigned short(*tile_out)[S::kCols + 8] = reinterpret_cast<unsigned short(*)[S::kCols + 8]>(st_smem);
  float sc[GP], of[GP];
#pragma unroll
  for (int gp = 0; gp < GP; ++gp) {
    const int n = n0 + 32 * (wave * GP + gp) + c32;
    const bool upper = ((long long)grp * p.n + n) & 1;   // which half of its word the element is
    sc[gp] = p.aq_scale ? sa_half_like<BF16>((unsigned short)(upper ? sc_word[gp] >> 16 : sc_word[gp])) : 1.0f;
    of[gp] = (p.aq_offset ? sa_half_like<BF16>((unsigned short)(upper ? of_word[gp] >> 16 : of_word[gp])) : 0.0f) - 128.0f;
  }
#pragma unroll
  for (int t = 0; t < TR; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row0 = 32 * t + 8 * j + 4 * kh;
      if (row0 < chunk_rows) {
        // (rows past the chunk and columns past N land in the tile as well: the row stores below leave them out)
        const v4f xs4 = *reinterpret_cast<const v4f *>(&row_sum[row0]);
#pragma unroll
        for (int gp = 0; gp < GP; ++gp) {
          const int cl = 32 * (wave * GP + gp) + c32;
#pragma unroll
          for (int r = 0; r < 4; ++r) tile_out[row0 + r][cl] = half_out(p, fmaf(of[gp], xs4[r], acc[gp][t][4 * j + r]) * sc[gp]);
        }
      }
    }
  __syncthreads();
  // whole-row stores: pieces of 8 columns
  constexpr int ROW_PIECES = S::kCols / 8;
  for (int item = tid; item < S::kRows * ROW_PIECES; item += ST_THREADS) {
    const int row = item / ROW_PIECES, c8 = (item % ROW_PIECES) * 8;
    const int n = n0 + c8;
    if (row < chunk_rows && n < p.n) {   // N % 16 == 0: 8 columns all inside or all outside
      const uint4 q = *reinterpret_cast<const uint4 *>(&tile_out[row][c8]);
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + row) * p.n + n) = q;
    }
  }
}

template <bool BF16, int TR, int GP, bool PK = false>
static hipError_t rows32_launch_a16w8(const GmmParams &p, const dim3 &grid, hipStream_t stream) {
  using S = Rows32Shape<TR, GP, PK>;
  auto kern = gmm_a16w8_rows32_kernel<BF16, TR, GP, PK>;
  if constexpr (S::kLds > 64 * 1024) {
    static std::atomic<bool> attr_set{false};   // (idempotent, as above)
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::kLds);
      if (e != hipSuccess) return e;
      attr_set = true;
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(ST_THREADS), S::kLds, stream, p);
  return hipGetLastError();
}

// workspace bytes of one (chunk, strip, K slice) partial tile of the 128-row kernel: accumulators and row sums
size_t rows32_a16w8_slice_bytes(int strip_groups) { return ((size_t)128 * 16 * strip_groups + 128) * 4; }

// tch = 16-row fragments per chunk (2, 4 or 8); p.max_chunks counts chunks of 16 tch rows; p.strip_groups = column groups
// per strip (8 or 16: strips of 128 or 256 columns), p.n_strips strips
hipError_t launch_streamm_a16w8(const GmmParams &p, int tch, bool packed, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  if (!packed && p.n % 16 != 0) return hipErrorInvalidValue;   // [E,K,N] rows of whole 16-column chunks
  if ((p.strip_groups != 8 && p.strip_groups != 16) || (tch != 2 && tch != 4 && tch != 8) || p.split_k < 1 ||
      (p.split_k > 1 && tch != 8))   // (a K split: 128-row chunks only)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)p.n_strips, chunk_slots(p, 16 * tch), (unsigned)p.split_k);
  const bool bf = p.x_dtype == DT_BF16;
  const bool wide = p.strip_groups == 16;
#define MSCO_ROWS_BY(TCH)                                                                                                   \
  (bf ? (wide ? rows_launch_a16w8<true, TCH, 4>(p, grid, stream) : rows_launch_a16w8<true, TCH, 2>(p, grid, stream))      \
      : (wide ? rows_launch_a16w8<false, TCH, 4>(p, grid, stream) : rows_launch_a16w8<false, TCH, 2>(p, grid, stream)))
  if (!packed) {   // 32-row chunks on 16 x 16 x 32 MFMAs, 64- and 128-row chunks on 32 x 32 x 16
#define MSCO_ROWS32_BY(TR)                                                                                                  \
  (bf ? (wide ? rows32_launch_a16w8<true, TR, 2>(p, grid, stream) : rows32_launch_a16w8<true, TR, 1>(p, grid, stream))    \
      : (wide ? rows32_launch_a16w8<false, TR, 2>(p, grid, stream) : rows32_launch_a16w8<false, TR, 1>(p, grid, stream)))
    if (tch == 8) return MSCO_ROWS32_BY(4);
    if (tch == 4) return MSCO_ROWS32_BY(2);
#undef MSCO_ROWS32_BY
    return wide ? (bf ? rows_launch_a16w8<true, 2, 4, true>(p, grid, stream) : rows_launch_a16w8<false, 2, 4, true>(p, grid, stream))
                : (bf ? rows_launch_a16w8<true, 2, 2, true>(p, grid, stream) : rows_launch_a16w8<false, 2, 2, true>(p, grid, stream));
  }
  if (tch == 8)   // 128-row chunks: the 32 x 32 x 16 kernel, the packed blocks through LDS
    return wide ? (bf ? rows32_launch_a16w8<true, 4, 2, true>(p, grid, stream) : rows32_launch_a16w8<false, 4, 2, true>(p, grid, stream))
                : (bf ? rows32_launch_a16w8<true, 4, 1, true>(p, grid, stream) : rows32_launch_a16w8<false, 4, 1, true>(p, grid, stream));
  return tch == 4 ? MSCO_ROWS_BY(4) : MSCO_ROWS_BY(2);
#undef MSCO_ROWS_BY
}

}  // namespace msco
