// MoE routing (stable counting sort of (token, k) entries by expert + activation gather) and weighted
// un-permutation for gfx950.  Both are HBM-bound row copies around a small integer problem:
//
//   init_routing   up to 16384 entries, plain row copy: ONE launch (route_fused_kernel): every workgroup counts all expert
//                  ids itself, places its own 32 entries and copies their rows.  Otherwise (more entries, or the
//                  quantising gather) the steps below; 1-3 are one launch for up to 16 blocks, every block repeating
//                  the small steps 1 and 2 for itself
//                  1. per block of 1024 entries: histogram of the expert ids (LDS atomics)
//                  2. one workgroup: per expert, exclusive scan over the blocks, then over the experts;
//                     writes the count / cumulative-count output
//                  3. per block, sixteen wavefronts rank 64 consecutive entries each among equal expert ids with
//                     ballots; a prefix over the sixteen chunks keeps the flat order, so the sort is stable
//                  4. one workgroup per output row copies x[token] with 16-byte loads and stores
//   unpermute      one workgroup per token: 16 bytes of every selected row per lane, the running sum kept
//                  in the element type and rounded exactly where the golden rounds it
#include "msco_moe.h"

#include <hip/hip_runtime.h>

#include "gmm_common.h"

// Rows that are read or written once go past the caches' retention (non-temporal): measured on MI355X the
// un-permutation of 4096 x 8 float16 rows of 7168 runs at 5.3 TB/s with it and 4.8 TB/s without.
typedef unsigned msco_v4u __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ uint4 msco_nt_load(const uint4 *p) {
  const msco_v4u v = __builtin_nontemporal_load(reinterpret_cast<const msco_v4u *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
static __device__ __forceinline__ void msco_nt_store(uint4 *p, const uint4 &v) {
  __builtin_nontemporal_store(msco_v4u{v.x, v.y, v.z, v.w}, reinterpret_cast<msco_v4u *>(p));
}
#define MSCO_ROW_LOAD(p) msco_nt_load(p)
#define MSCO_ROW_STORE(p, v) msco_nt_store(p, v)

namespace msco {
namespace {

constexpr int kRouteBlock = 1024;   // entries per histogram / ranking block
constexpr int kMaxExperts = 1024;

__device__ __forceinline__ int clamp_expert(int e, int expert_num) { return e < 0 ? 0 : (e >= expert_num ? expert_num - 1 : e); }

__global__ void __launch_bounds__(256) route_hist_kernel(const int *expert_idx, int *block_hist, long long n, int expert_num) {
  __shared__ int hist[kMaxExperts];
  for (int e = threadIdx.x; e < expert_num; e += 256) hist[e] = 0;
  __syncthreads();
  const long long first = (long long)blockIdx.x * kRouteBlock;
#pragma unroll
  for (int u = 0; u < kRouteBlock / 256; ++u) {
    const long long i = first + u * 256 + threadIdx.x;
    if (i < n) atomicAdd(&hist[clamp_expert(expert_idx[i], expert_num)], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < expert_num; e += 256) block_hist[(long long)blockIdx.x * expert_num + e] = hist[e];
}

// block_hist[b][e] becomes the first output position of block b's entries of expert e
__global__ void __launch_bounds__(1024) route_scan_kernel(int *block_hist, int *count_or_cumsum, int *before_capacity,
                                                          int blocks, int expert_num, int flag) {
  __shared__ int total[kMaxExperts];
  __shared__ int base[kMaxExperts];
  const int e = threadIdx.x;
  int running = 0;
  if (e < expert_num) {
    for (int b = 0; b < blocks; ++b) {
      const int v = block_hist[(long long)b * expert_num + e];
      block_hist[(long long)b * expert_num + e] = running;
      running += v;
    }
    total[e] = running;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int j = 0; j < expert_num; ++j) {
      base[j] = acc;
      acc += total[j];
    }
  }
  __syncthreads();
  if (e < expert_num) {
    const int b0 = base[e];
    for (int b = 0; b < blocks; ++b) block_hist[(long long)b * expert_num + e] += b0;
    if (count_or_cumsum != nullptr && flag == 1) count_or_cumsum[e] = b0 + total[e];
    if (count_or_cumsum != nullptr && flag == 2) count_or_cumsum[e] = total[e];
    if (before_capacity != nullptr) before_capacity[e] = 0;
  }
}

// One block of 1024 entries, sixteen wavefronts of 64 consecutive entries each.  A wavefront ranks its entries among
// equal expert ids with ballots (one round per distinct id in the chunk) and leaves the chunk's per-expert counts
// in LDS; a prefix over the sixteen chunks turns the counts into first positions; rank + first position is the
// output row.  Chunks, and positions inside a chunk, are taken in flat order, so the sort is stable.
// (block_first: this block's row of first positions, in global memory or in LDS; e: the entry's expert id, -1 for none)
__device__ __forceinline__ void rank_block(int *chunk_first, const int *block_first, long long i, bool live, int e,
                                           int *expanded_row_idx, int *sorted_src, int expert_num) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int *mine = chunk_first + wave * expert_num;
  for (int x = lane; x < expert_num; x += 64) mine[x] = 0;
  unsigned long long todo = __ballot(live);
  int rank = 0;
  while (todo) {
    const int leader = __ffsll((long long)todo) - 1;
    const int e0 = __shfl(e, leader);
    const unsigned long long same = __ballot(e == e0) & todo;
    if (e == e0) rank = __popcll(same & ((1ull << lane) - 1ull));
    if (lane == leader) mine[e0] = __popcll(same);      // after the zero fill above: one wavefront's LDS operations stay in order
    todo &= ~same;
  }
  __syncthreads();
  for (int x = threadIdx.x; x < expert_num; x += 1024) {
    int running = block_first[x];
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int c = chunk_first[w * expert_num + x];
      chunk_first[w * expert_num + x] = running;
      running += c;
    }
  }
  __syncthreads();
  if (live) {
    const int dest = mine[e] + rank;
    expanded_row_idx[i] = dest;
    sorted_src[dest] = (int)i;
  }
}

__global__ void __launch_bounds__(1024) route_rank_kernel(const int *expert_idx, const int *block_first, int *expanded_row_idx,
                                                          int *sorted_src, long long n, int expert_num) {
  extern __shared__ int chunk_first[];   // [16][expert_num]
  const long long i = (long long)blockIdx.x * kRouteBlock + threadIdx.x;
  const bool live = i < n;
  const int e = live ? clamp_expert(expert_idx[i], expert_num) : -1;
  rank_block(chunk_first, block_first + (long long)blockIdx.x * expert_num, i, live, e, expanded_row_idx, sorted_src, expert_num);
}

// Histogram, scan and ranking in one launch for problems of at most kSmallBlocks blocks: every block histograms all
// entries itself (a few thousand LDS atomics) instead of waiting for the other blocks, then ranks its own 1024.  At
// this size the three launches above cost more in launch gaps than in work.
constexpr int kSmallBlocks = 16;
__global__ void __launch_bounds__(1024) route_small_kernel(const int *expert_idx, int *count_or_cumsum, int *before_capacity,
                                                           int *expanded_row_idx, int *sorted_src, long long n, int expert_num,
                                                           int flag) {
  extern __shared__ int lds[];   // first[blocks][expert_num], chunk_first[16][expert_num], total[expert_num], base[expert_num]
  const int blocks = gridDim.x;
  int *first = lds;
  int *chunk_first = first + blocks * expert_num;
  int *total = chunk_first + 16 * expert_num;
  int *base = total + expert_num;
  for (int x = threadIdx.x; x < blocks * expert_num; x += 1024) first[x] = 0;
  __syncthreads();
  // (all of a thread's ids are requested before the first is used: one memory round trip instead of one per block)
  int my_e = -1;
  int ids[kSmallBlocks];
#pragma unroll
  for (int b = 0; b < kSmallBlocks; ++b) {
    const long long i = (long long)b * kRouteBlock + threadIdx.x;
    ids[b] = b < blocks && i < n ? expert_idx[i] : -1;
  }
#pragma unroll
  for (int b = 0; b < kSmallBlocks; ++b) {
    const long long i = (long long)b * kRouteBlock + threadIdx.x;
    if (b < blocks && i < n) {
      const int e = clamp_expert(ids[b], expert_num);
      atomicAdd(&first[b * expert_num + e], 1);
      if (b == (int)blockIdx.x) my_e = e;
    }
  }
  __syncthreads();
  const int e = threadIdx.x;
  if (e < expert_num) {
    int running = 0;
    for (int b = 0; b < blocks; ++b) {
      const int v = first[b * expert_num + e];
      first[b * expert_num + e] = running;
      running += v;
    }
    total[e] = running;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int j = 0; j < expert_num; ++j) {
      base[j] = acc;
      acc += total[j];
    }
  }
  __syncthreads();
  if (e < expert_num) {
    first[blockIdx.x * expert_num + e] += base[e];
    if (blockIdx.x == 0) {
      if (count_or_cumsum != nullptr && flag == 1) count_or_cumsum[e] = base[e] + total[e];
      if (count_or_cumsum != nullptr && flag == 2) count_or_cumsum[e] = total[e];
      if (before_capacity != nullptr) before_capacity[e] = 0;
    }
  }
  __syncthreads();
  const long long i = (long long)blockIdx.x * kRouteBlock + threadIdx.x;
  rank_block(chunk_first, first + blockIdx.x * expert_num, i, my_e >= 0, my_e, expanded_row_idx, sorted_src, expert_num);
}

// ---- per-row dynamic int8 quantisation (tests/st/test_grouped_matmul_w4.py:83-89), shared by the gather kernels ----
//   scale = float32(max |x[t, :]|) / 127,   q[h] = int8(rint(float32(x[t, h]) / scale))
// |x| is ordered like its bit pattern without the sign, so the maximum is taken on 15-bit integers and converted once.
template <bool BF16>
__device__ __forceinline__ float rq_widen(unsigned short b) { return BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b); }
__device__ __forceinline__ void rq_fold(unsigned &mx, const uint4 &v) {
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    mx = max(mx, w[i] & 0x7FFFu);
    mx = max(mx, (w[i] >> 16) & 0x7FFFu);
  }
}
// The golden rounds the correctly rounded quotient x / scale to an integer.  A correctly rounded division costs a
// dozen instructions per element; x * (1 / scale) is within 2^-22 * 128 of that quotient, so unless it lands within
// 1e-4 of a half-integer (then the division is done properly) both round to the same integer.
__device__ __forceinline__ int rq_to_int(float f, float scale, float inv) {
  const float r = f * inv;
  const float n = rintf(r);
  if (fabsf(r - n) > 0.4999f) return (int)rintf(f / scale);
  return (int)n;
}
// eight elements -> eight int8; `nonzero`: the row's maximum is not zero (a row of zeros has scale 0: the golden divides
// 0 by 0 there; it gets zeros)
template <bool BF16>
__device__ __forceinline__ uint2 rq_quantise(const uint4 &v, float scale, float inv, bool nonzero) {
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  unsigned q[2] = {0, 0};
  if (nonzero) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int lo = rq_to_int(rq_widen<BF16>((unsigned short)(w[i] & 0xFFFFu)), scale, inv);
      const int hi = rq_to_int(rq_widen<BF16>((unsigned short)(w[i] >> 16)), scale, inv);
      q[i >> 1] |= ((unsigned)(lo & 0xFF) | ((unsigned)(hi & 0xFF) << 8)) << (16 * (i & 1));
    }
  }
  return make_uint2(q[0], q[1]);
}

// Routing in ONE launch for up to kFusedMaxEntries entries: every workgroup owns kFusedRows consecutive entries (its
// slice), finds their output rows by itself and copies their rows.  For that it counts, over ALL entries, how many carry
// each expert id (total) and how many of those lie before its slice (before): the output row of entry i with id e is
//     (entries with a smaller id) + (entries with id e before the slice) + (entries with id e inside the slice before i),
// which is the position a stable sort gives it.  The counting is redundant across workgroups (a few thousand LDS
// atomics each, on `rep` interleaved copies of the tables so that the lanes of a wavefront rarely meet on one address),
// but nothing waits for another workgroup, so the sort, the index outputs and the row copy need no second launch.
#ifndef MSCO_FUSED_ROWS
#define MSCO_FUSED_ROWS 32
#endif
constexpr int kFusedRows = MSCO_FUSED_ROWS;   // 16, 32 or 64: one to four rows per wavefront
constexpr int kFusedThreads = 1024;   // sixteen wavefronts: the counting is a chain of dependent LDS atomics per wavefront, four per SIMD overlap them
constexpr int kFusedIdsPerThread = 16;
constexpr long long kFusedMaxEntries = (long long)kFusedThreads * kFusedIdsPerThread;   // 16384
__global__ void __launch_bounds__(kFusedThreads) route_fused_kernel(const unsigned char *x, const int *expert_idx,
                                                                    unsigned char *expanded_x,
                                                                    int *expanded_row_idx, int *count_or_cumsum,
                                                                    int *before_capacity, long long n, int expert_num, int flag,
                                                                    long long row_bytes, int k, int rep) {
  extern __shared__ int lds[];   // total[rep][expert_num], before[rep][expert_num], base[expert_num], wave_sum[16], dest[kFusedRows]
  int *total = lds;
  int *before = total + rep * expert_num;
  int *base = before + rep * expert_num;
  int *wave_sum = base + expert_num;
  int *dest = wave_sum + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long long start = (long long)blockIdx.x * kFusedRows;
  for (int i = tid; i < 2 * rep * expert_num; i += kFusedThreads) lds[i] = 0;
  // all of a thread's ids are requested before the first is used: entries 4 (tid + 1024 j) .. + 3 (ids past n read as 0,
  // by the range check of the buffer load, and are skipped by their index; only the vector offset is range-checked)
  const __amdgpu_buffer_rsrc_t rs_ids = buffer_over(expert_idx, n * 4);
  v4i ids[kFusedIdsPerThread / 4];
  static_for<kFusedIdsPerThread / 4>([&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    ids[J] = __builtin_amdgcn_raw_buffer_load_b128(rs_ids, (unsigned)(16 * (tid + kFusedThreads * J)), 0, 0);
  });
  __syncthreads();
  const int copy = (lane & (rep - 1)) * expert_num;   // rep is a power of two
  static_for<kFusedIdsPerThread / 4>([&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    const long long i0 = 4ll * (tid + kFusedThreads * J);
    static_for<4>([&](auto u_c) {
      constexpr int U = decltype(u_c)::value;
      if (i0 + U < n) {
        const int e = clamp_expert(ids[J][U], expert_num);
        atomicAdd(&total[copy + e], 1);
        if (i0 + U < start) atomicAdd(&before[copy + e], 1);
      }
    });
  });
  __syncthreads();
  // fold the copies; exclusive scan of the totals over the experts (one expert per thread)
  int tsum = 0, bsum = 0;
  if (tid < expert_num) {
    for (int r = 0; r < rep; ++r) {
      tsum += total[r * expert_num + tid];
      bsum += before[r * expert_num + tid];
    }
    before[tid] = bsum;   // copy 0 now holds the folded value (a thread touches only its own expert)
  }
  const int incl = wave_scan_add(tsum, lane);
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  int offset = incl - tsum;
  for (int w = 0; w < wave; ++w) offset += wave_sum[w];
  if (tid < expert_num) {
    base[tid] = offset;
    if (blockIdx.x == 0) {
      if (count_or_cumsum != nullptr && flag == 1) count_or_cumsum[tid] = offset + tsum;
      if (count_or_cumsum != nullptr && flag == 2) count_or_cumsum[tid] = tsum;
      if (before_capacity != nullptr) before_capacity[tid] = 0;
    }
  }
  __syncthreads();
  // the slice's entries, one per lane of wavefront 0: rank among equal ids inside the slice by ballots
  if (wave == 0) {
    const long long i = start + lane;
    const bool live = lane < kFusedRows && i < n;
    const int e = live ? clamp_expert(expert_idx[i], expert_num) : -1;
    unsigned long long todo = __ballot(live);
    int rank = 0;
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const int e0 = __shfl(e, leader);
      const unsigned long long same = __ballot(e == e0) & todo;
      if (e == e0) rank = __popcll(same & ((1ull << lane) - 1ull));
      todo &= ~same;
    }
    if (live) {
      const int d = base[e] + before[e] + rank;
      dest[lane] = d;
      expanded_row_idx[i] = d;
    }
  }
  __syncthreads();
  // copy the rows: wavefront w takes the slice's rows w, w + 16, ...; a lane's vectors of all of them in flight together
  const long long vecs = row_bytes / 16;
  constexpr int RPW = kFusedRows / 16;   // rows per wavefront
  for (long long v0 = 0; v0 < vecs; v0 += 64 * 4) {
    uint4 buf[RPW][4];
    static_for<4 * RPW>([&](auto q_c) {
      constexpr int RR = decltype(q_c)::value / 4, C = decltype(q_c)::value % 4;
      const long long i = start + wave + 16 * RR;
      const uint4 *src = reinterpret_cast<const uint4 *>(x + (i < n ? i / k : 0) * row_bytes);
      const long long v = v0 + lane + 64 * C;
      buf[RR][C] = (i < n && v < vecs) ? src[v] : make_uint4(0, 0, 0, 0);
    });
    static_for<4 * RPW>([&](auto q_c) {
      constexpr int RR = decltype(q_c)::value / 4, C = decltype(q_c)::value % 4;
      const long long i = start + wave + 16 * RR;
      const long long v = v0 + lane + 64 * C;
      if (i < n && v < vecs) {
        uint4 *dst = reinterpret_cast<uint4 *>(expanded_x + (long long)dest[wave + 16 * RR] * row_bytes);
        dst[v] = buf[RR][C];   // kept cacheable: the matmul reads it next
      }
    });
  }
}

__global__ void __launch_bounds__(256) route_gather_kernel(const unsigned char *x, const int *sorted_src, unsigned char *expanded_x,
                                                           long long row_bytes, int k) {
  const long long j = blockIdx.x;
  const long long token = sorted_src[j] / k;
  const uint4 *src = reinterpret_cast<const uint4 *>(x + token * row_bytes);
  uint4 *dst = reinterpret_cast<uint4 *>(expanded_x + j * row_bytes);
  for (long long v = threadIdx.x; v < row_bytes / 16; v += 256) dst[v] = src[v];   // kept cacheable: the matmul reads it next
}

// The gather with per-row dynamic int8 quantisation on the way (tests/st/test_grouped_matmul_w4.py:83-89):
//   scale = float32(max |x[t, :]|) / 127,   q[h] = int8(rint(float32(x[t, h]) / scale))
// One workgroup per output row, 16 bytes (8 elements) per lane and step.  Up to four steps a lane keeps its elements
// in registers between the maximum and the division; longer rows are read again (they are L2 hits).  |x| is ordered
// like its bit pattern without the sign, so the maximum is taken on 15-bit integers and converted once.
template <bool BF16>
__global__ void __launch_bounds__(256) route_gather_quant_kernel(const unsigned short *x, const int *sorted_src, signed char *expanded_x,
                                                                 float *expanded_scale, long long hidden, int k) {
  __shared__ unsigned wave_max[4];
  const long long j = blockIdx.x;
  const long long token = sorted_src[j] / k;
  const uint4 *src = reinterpret_cast<const uint4 *>(x + token * hidden);
  uint2 *dst = reinterpret_cast<uint2 *>(expanded_x + j * hidden);
  const long long vecs = hidden / 8;
  constexpr int KEEP = 4;
  uint4 kept[KEEP];
  unsigned mx = 0;
  auto fold = [&](const uint4 &v) { rq_fold(mx, v); };
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const long long v = threadIdx.x + u * 256;
    kept[u] = v < vecs ? src[v] : make_uint4(0, 0, 0, 0);
    fold(kept[u]);
  }
  for (long long v = threadIdx.x + KEEP * 256; v < vecs; v += 256) fold(src[v]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = max(mx, (unsigned)__shfl_xor((int)mx, o));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
  const float scale = rq_widen<BF16>((unsigned short)mx) / 127.0f;
  if (threadIdx.x == 0) expanded_scale[j] = scale;
  const float inv = 1.0f / scale;
  auto quantise = [&](const uint4 &v) { return rq_quantise<BF16>(v, scale, inv, mx != 0); };
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const long long v = threadIdx.x + u * 256;
    if (v < vecs) dst[v] = quantise(kept[u]);
  }
  for (long long v = threadIdx.x + KEEP * 256; v < vecs; v += 256) dst[v] = quantise(src[v]);
}

// float32 -> element type with round to nearest even, and back
template <bool BF16>
__device__ __forceinline__ unsigned short to_elem(float f) {
  return BF16 ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
}
template <bool BF16>
__device__ __forceinline__ float from_elem(unsigned short b) {
  return BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

// K: top_k as a compile-time constant (the row indices, the probabilities and the K row pieces of a pass are then all
// requested before the first one is used; with a run-time loop every step waits for two dependent loads), 0: any top_k
// kUnpermuteU: 2048-element pieces of the row a workgroup takes together (all their row vectors are requested before
// the first is used: with many tokens, four pieces measured 91 us where one piece takes 97 us at 4096 x top-8 x 7168)
template <bool BF16, int K, int kUnpermuteU>
__global__ void __launch_bounds__(256) unpermute_kernel(const unsigned short *permuted, const int *sorted_indices,
                                                        const unsigned short *probs, unsigned short *out, int top_k_arg,
                                                        long long hidden) {
  const long long token = blockIdx.x;
  const int top_k = K > 0 ? K : top_k_arg;
  constexpr int KK = K > 0 ? K : 1;
  long long rows[KK];
  unsigned short pbs[KK];
  if constexpr (K > 0) {
#pragma unroll
    for (int kk = 0; kk < K; ++kk) {
      rows[kk] = sorted_indices[token * K + kk];
      pbs[kk] = probs[token * K + kk];
    }
  }
  // blockIdx.y walks the row in pieces of kUnpermuteU x 2048 elements: one pass per workgroup, so nothing waits for a
  // previous pass; a thread requests its kUnpermuteU x K vectors before it uses the first
  for (long long v0 = (long long)blockIdx.y * kUnpermuteU * 256 + threadIdx.x; v0 * 8 < hidden; v0 += (long long)gridDim.y * kUnpermuteU * 256) {
    uint4 all_pieces[kUnpermuteU][KK];
    if constexpr (K > 0) {
#pragma unroll
      for (int u = 0; u < kUnpermuteU; ++u)
#pragma unroll
        for (int kk = 0; kk < K; ++kk) {
          const long long hu = (v0 + u * 256) * 8;
          all_pieces[u][kk] = hu < hidden ? MSCO_ROW_LOAD(reinterpret_cast<const uint4 *>(permuted + rows[kk] * hidden + hu)) : make_uint4(0, 0, 0, 0);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnpermuteU; ++u) {
    const long long h0 = (v0 + u * 256) * 8;
    if (h0 >= hidden) break;
    uint4 *pieces = all_pieces[u];
    // running sums, kept as the float32 value of the already rounded element
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
    auto step = [&](int kk) {
      unsigned short pbits;
      uint4 q;
      if constexpr (K > 0) {
        pbits = pbs[kk];
        q = pieces[kk];
      } else {
        pbits = probs[token * top_k + kk];
        q = MSCO_ROW_LOAD(reinterpret_cast<const uint4 *>(permuted + (long long)sorted_indices[token * top_k + kk] * hidden + h0));
      }
      const unsigned w[4] = {q.x, q.y, q.z, q.w};
      // The golden rounds the product to the element type, then the running sum (both computed in float32).
      // The two steps are kept apart -- no fused multiply-add, no mixed-precision merge -- by empty asm statements.
      if constexpr (!BF16) {
        // float16: the packed half multiply rounds the exact product once, which is what rounding the (exact)
        // float32 product gives; the sum goes through float32 because numpy's does (double rounding included)
        const h2_t p2 = {__builtin_bit_cast(_Float16, pbits), __builtin_bit_cast(_Float16, pbits)};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          h2_t prod = __builtin_bit_cast(h2_t, w[d]) * p2;
          asm volatile("" : "+v"(prod));
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            float sum = acc[2 * d + u] + (float)prod[u];
            asm volatile("" : "+v"(sum));
            acc[2 * d + u] = (float)(_Float16)sum;
          }
        }
      } else {
        const float p = bf16_bits_to_f32(pbits);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const unsigned short v = (unsigned short)(w[j >> 1] >> (16 * (j & 1)));
          float prod = p * bf16_bits_to_f32(v);
          asm volatile("" : "+v"(prod));
          float sum = acc[j] + bf16_bits_to_f32(f32_to_bf16_rne(prod));
          asm volatile("" : "+v"(sum));
          acc[j] = bf16_bits_to_f32(f32_to_bf16_rne(sum));
        }
      }
        };
    if constexpr (K > 0) {
#pragma unroll
      for (int kk = 0; kk < K; ++kk) step(kk);
    } else {
      for (int kk = 0; kk < top_k; ++kk) step(kk);
    }
    unsigned short ob[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) ob[j] = to_elem<BF16>(acc[j]);   // exact: acc already holds an element-type value
    uint4 o;
    o.x = ob[0] | ((unsigned)ob[1] << 16); o.y = ob[2] | ((unsigned)ob[3] << 16);
    o.z = ob[4] | ((unsigned)ob[5] << 16); o.w = ob[6] | ((unsigned)ob[7] << 16);
    MSCO_ROW_STORE(reinterpret_cast<uint4 *>(out + token * hidden + h0), o);
    }
  }
}

long long route_blocks(long long n) { return (n + kRouteBlock - 1) / kRouteBlock; }

}  // namespace
}  // namespace msco

extern "C" {

size_t msco_moe_init_routing_v2_workspace_bytes(int64_t num_rows, int64_t k, int64_t expert_num) {
  if (num_rows <= 0 || k <= 0 || expert_num <= 0) return 0;
  const long long n = num_rows * k;
  // per-block expert histograms / first positions, then the source entry of every output row
  return (size_t)(msco::route_blocks(n) * expert_num + n) * sizeof(int32_t);
}

// quant_dtype: MSCO_DT_NONE copies rows of elem_bytes-wide elements; MSCO_DT_F16 / MSCO_DT_BF16 quantises rows of that
// type to int8 and writes their scales
static int route_and_gather(const void *x, const int32_t *expert_idx, void *expanded_x, float *expanded_scale,
                            int32_t *expanded_row_idx, int32_t *expert_tokens_count_or_cumsum,
                            int32_t *expert_tokens_before_capacity, void *workspace, size_t workspace_bytes, int64_t num_rows,
                            int64_t hidden, int64_t k, int64_t expert_num, int32_t elem_bytes, int32_t quant_dtype,
                            int32_t count_or_cumsum_flag, void *stream) {
  using namespace msco;
  if (num_rows < 0 || hidden <= 0 || k <= 0 || expert_num <= 0 || expert_num > kMaxExperts) return MSCO_ERR_SHAPE;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) return MSCO_ERR_UNSUPPORTED;
  if (quant_dtype != MSCO_DT_NONE && quant_dtype != MSCO_DT_F16 && quant_dtype != MSCO_DT_BF16) return MSCO_ERR_UNSUPPORTED;
  if ((hidden * elem_bytes) % 16 != 0) return MSCO_ERR_SHAPE;
  if (count_or_cumsum_flag < 0 || count_or_cumsum_flag > 2) return MSCO_ERR_INVALID_ARG;
  const long long n = num_rows * k;
  if (n > 0x7FFFFFFFll) return MSCO_ERR_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n == 0) {   // no entries: the count outputs are all zero (the scan kernel over zero blocks writes just that)
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, static_cast<int *>(nullptr), expert_tokens_count_or_cumsum,
                       expert_tokens_before_capacity, 0, (int)expert_num, (int)count_or_cumsum_flag);
    return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
  }
  if (x == nullptr || expert_idx == nullptr || expanded_x == nullptr || expanded_row_idx == nullptr) return MSCO_ERR_INVALID_ARG;
  if (quant_dtype != MSCO_DT_NONE && expanded_scale == nullptr) return MSCO_ERR_INVALID_ARG;
  if (count_or_cumsum_flag != 0 && expert_tokens_count_or_cumsum == nullptr) return MSCO_ERR_INVALID_ARG;
  if (workspace == nullptr || workspace_bytes < msco_moe_init_routing_v2_workspace_bytes(num_rows, k, expert_num))
    return MSCO_ERR_WORKSPACE;
  if (quant_dtype == MSCO_DT_NONE && n <= kFusedMaxEntries) {
    // small problems: the sort and the row copy in one launch, no workspace traffic.  (The quantising gather stays a
    // launch of its own: it is bound by its arithmetic, and one workgroup per row overlaps that better -- fused the
    // same way it measured 27.5 us against 24.4 us.)
    int rep = 8;
    while (rep > 1 && rep * expert_num > 512) rep /= 2;
    const size_t lds_bytes = (size_t)(2 * rep * expert_num + expert_num + 16 + kFusedRows) * sizeof(int);
    hipLaunchKernelGGL(route_fused_kernel, dim3((unsigned)((n + kFusedRows - 1) / kFusedRows)), dim3(kFusedThreads), lds_bytes, s,
                       static_cast<const unsigned char *>(x), expert_idx, static_cast<unsigned char *>(expanded_x), expanded_row_idx,
                       expert_tokens_count_or_cumsum, expert_tokens_before_capacity, n, (int)expert_num, (int)count_or_cumsum_flag,
                       (long long)hidden * elem_bytes, (int)k, rep);
    return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
  }
  const long long blocks = route_blocks(n);
  int *block_hist = static_cast<int *>(workspace);
  int *sorted_src = block_hist + blocks * expert_num;
  const size_t small_lds = (size_t)(blocks + 16 + 2) * expert_num * sizeof(int);
  if (blocks <= kSmallBlocks && small_lds <= 64 * 1024) {
    hipLaunchKernelGGL(route_small_kernel, dim3((unsigned)blocks), dim3(1024), small_lds, s, expert_idx, expert_tokens_count_or_cumsum,
                       expert_tokens_before_capacity, expanded_row_idx, sorted_src, n, (int)expert_num, (int)count_or_cumsum_flag);
  } else {
    hipLaunchKernelGGL(route_hist_kernel, dim3((unsigned)blocks), dim3(256), 0, s, expert_idx, block_hist, n, (int)expert_num);
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, block_hist, expert_tokens_count_or_cumsum,
                       expert_tokens_before_capacity, (int)blocks, (int)expert_num, (int)count_or_cumsum_flag);
    hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)blocks), dim3(1024), (size_t)16 * expert_num * sizeof(int), s, expert_idx,
                       block_hist, expanded_row_idx, sorted_src, n, (int)expert_num);
  }
  if (quant_dtype == MSCO_DT_NONE) {
    hipLaunchKernelGGL(route_gather_kernel, dim3((unsigned)n), dim3(256), 0, s, static_cast<const unsigned char *>(x), sorted_src,
                       static_cast<unsigned char *>(expanded_x), (long long)hidden * elem_bytes, (int)k);
  } else if (quant_dtype == MSCO_DT_BF16) {
    hipLaunchKernelGGL(route_gather_quant_kernel<true>, dim3((unsigned)n), dim3(256), 0, s, static_cast<const unsigned short *>(x),
                       sorted_src, static_cast<signed char *>(expanded_x), expanded_scale, (long long)hidden, (int)k);
  } else {
    hipLaunchKernelGGL(route_gather_quant_kernel<false>, dim3((unsigned)n), dim3(256), 0, s, static_cast<const unsigned short *>(x),
                       sorted_src, static_cast<signed char *>(expanded_x), expanded_scale, (long long)hidden, (int)k);
  }
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

int msco_moe_init_routing_v2(const void *x, const int32_t *expert_idx, void *expanded_x, int32_t *expanded_row_idx,
                             int32_t *expert_tokens_count_or_cumsum, int32_t *expert_tokens_before_capacity,
                             void *workspace, size_t workspace_bytes, int64_t num_rows, int64_t hidden, int64_t k,
                             int64_t expert_num, int32_t elem_bytes, int32_t count_or_cumsum_flag, void *stream) {
  return route_and_gather(x, expert_idx, expanded_x, nullptr, expanded_row_idx, expert_tokens_count_or_cumsum,
                          expert_tokens_before_capacity, workspace, workspace_bytes, num_rows, hidden, k, expert_num, elem_bytes,
                          MSCO_DT_NONE, count_or_cumsum_flag, stream);
}

int msco_moe_init_routing_v2_quant(const void *x, const int32_t *expert_idx, int8_t *expanded_x, float *expanded_scale,
                                   int32_t *expanded_row_idx, int32_t *expert_tokens_count_or_cumsum,
                                   int32_t *expert_tokens_before_capacity, void *workspace, size_t workspace_bytes,
                                   int64_t num_rows, int64_t hidden, int64_t k, int64_t expert_num, int32_t x_dtype,
                                   int32_t count_or_cumsum_flag, void *stream) {
  if (x_dtype != MSCO_DT_F16 && x_dtype != MSCO_DT_BF16) return MSCO_ERR_UNSUPPORTED;
  return route_and_gather(x, expert_idx, expanded_x, expanded_scale, expanded_row_idx, expert_tokens_count_or_cumsum,
                          expert_tokens_before_capacity, workspace, workspace_bytes, num_rows, hidden, k, expert_num, 2, x_dtype,
                          count_or_cumsum_flag, stream);
}

int msco_moe_token_unpermute(const void *permuted_tokens, const int32_t *sorted_indices, const void *probs, void *out,
                             int64_t num_tokens, int64_t top_k, int64_t hidden, int32_t dtype, void *stream) {
  using namespace msco;
  if (num_tokens < 0 || top_k <= 0 || top_k > 64 || hidden <= 0 || hidden % 8 != 0) return MSCO_ERR_SHAPE;
  if (dtype != MSCO_DT_F16 && dtype != MSCO_DT_BF16) return MSCO_ERR_UNSUPPORTED;
  if (num_tokens == 0) return MSCO_OK;
  if (num_tokens > 0x7FFFFFFFll) return MSCO_ERR_SHAPE;
  if (permuted_tokens == nullptr || sorted_indices == nullptr || probs == nullptr || out == nullptr) return MSCO_ERR_INVALID_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const auto *pt = static_cast<const unsigned short *>(permuted_tokens);
  const auto *pr = static_cast<const unsigned short *>(probs);
  auto *o = static_cast<unsigned short *>(out);
  // enough tokens to fill the chip with one workgroup per four pieces: fewer, larger workgroups; else one per piece
  const int u = (num_tokens >= 1024 && top_k <= 8) ? 4 : 1;
  const long long piece = 2048ll * u;
  const dim3 grid((unsigned)num_tokens, (unsigned)((hidden + piece - 1) / piece > 16 ? 16 : (hidden + piece - 1) / piece)), block(256);
  const bool bf = dtype == MSCO_DT_BF16;
#define MSCO_UNPERMUTE(K)                                                                                               \
  do {                                                                                                                  \
    if (u == 4) {                                                                                                       \
      if (bf) hipLaunchKernelGGL((unpermute_kernel<true, K, 4>), grid, block, 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);  \
      else hipLaunchKernelGGL((unpermute_kernel<false, K, 4>), grid, block, 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);    \
    } else {                                                                                                            \
      if (bf) hipLaunchKernelGGL((unpermute_kernel<true, K, 1>), grid, block, 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);  \
      else hipLaunchKernelGGL((unpermute_kernel<false, K, 1>), grid, block, 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);    \
    }                                                                                                                   \
  } while (0)
  switch (top_k) {
    case 1: MSCO_UNPERMUTE(1); break;
    case 2: MSCO_UNPERMUTE(2); break;
    case 4: MSCO_UNPERMUTE(4); break;
    case 8: MSCO_UNPERMUTE(8); break;
    default: MSCO_UNPERMUTE(0); break;
  }
#undef MSCO_UNPERMUTE
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

}  // extern "C"
