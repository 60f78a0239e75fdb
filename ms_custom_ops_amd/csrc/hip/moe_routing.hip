// MoE routing (stable counting sort of (token, k) entries by expert + activation gather) and weighted
// un-permutation for gfx950.  Both are HBM-bound row copies around a small integer problem:
//
//   init_routing   up to 16384 entries: ONE launch (route_fused_kernel): every workgroup counts all expert ids itself,
//                  places its own 32 entries and moves their rows (plain copy, or per-row dynamic int8 quantisation);
//                  a wavefront owns consecutive entries, so the k entries of a token cost one read (and one
//                  quantisation) of its row.  More entries take four launches:
//                  1. per block of 1024 entries: histogram of the expert ids (LDS atomics)
//                  2. one workgroup: per expert, exclusive scan over the blocks (runs of blocks in parallel), then over
//                     the experts; writes the count / cumulative-count output
//                  3. per block, sixteen wavefronts rank 64 consecutive entries each among equal expert ids (one ballot
//                     per bit of the id); a prefix over the sixteen chunks keeps the flat order, so the sort is stable
//                  4. one wavefront per token moves (or quantises) its row once and writes it to its k rows
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

// The lanes of the wavefront that carry the same id as this one, among the live lanes: one ballot per bit of the id
// (ids below 2^bits), whatever the number of distinct ids in the wavefront.
__device__ __forceinline__ unsigned long long wave_match(int e, bool live, int bits) {
  unsigned long long same = __ballot(live);
  for (int k = 0; k < bits; ++k) {
    const bool bit = (e >> k) & 1;
    const unsigned long long b = __ballot(bit);
    same &= bit ? b : ~b;
  }
  return same;
}
__device__ __forceinline__ int id_bits(int expert_num) { return expert_num > 1 ? 32 - __clz(expert_num - 1) : 0; }

// block_hist[b][e] becomes the first position of block b's entries of expert e among the entries of that expert;
// expert_base[e] the number of entries of smaller experts (the ranking adds the two).  One workgroup: thread (g, e) owns
// expert e in the g-th of G = 1024 / expert_num runs of consecutive blocks, sums its run, the runs of an expert are
// scanned in LDS, and the thread walks its run again writing the running positions -- loads in batches of eight ahead of
// their stores (in place: a load behind a store would wait for it).
__global__ void __launch_bounds__(1024) route_scan_kernel(int *block_hist, int *expert_base, int *count_or_cumsum,
                                                          int *before_capacity, int blocks, int expert_num, int flag) {
  __shared__ int part[1024];
  __shared__ int wave_sum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int groups = 1024 / expert_num;                 // expert_num <= 1024
  const int e = tid % expert_num, g = tid / expert_num;
  const int per = (blocks + groups - 1) / groups;
  const int b_lo = min(blocks, g * per), b_hi = g < groups ? min(blocks, b_lo + per) : b_lo;
  int sum = 0;
#pragma unroll 8
  for (int b = b_lo; b < b_hi; ++b) sum += block_hist[(long long)b * expert_num + e];
  part[tid] = sum;
  __syncthreads();
  int total = 0;
  if (tid < expert_num) {
    for (int r = 0; r < groups; ++r) {
      const int v = part[r * expert_num + tid];
      part[r * expert_num + tid] = total;
      total += v;
    }
  }
  const int incl = wave_scan_add(total, lane);
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  if (tid < expert_num) {
    int base = incl - total;
    for (int w = 0; w < wave; ++w) base += wave_sum[w];
    if (expert_base != nullptr) expert_base[tid] = base;
    if (count_or_cumsum != nullptr && flag == 1) count_or_cumsum[tid] = base + total;
    if (count_or_cumsum != nullptr && flag == 2) count_or_cumsum[tid] = total;
    if (before_capacity != nullptr) before_capacity[tid] = 0;
  }
  int running = part[tid];
  for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = b0 + u < b_hi ? block_hist[(long long)(b0 + u) * expert_num + e] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (b0 + u < b_hi) block_hist[(long long)(b0 + u) * expert_num + e] = running;
      running += v[u];
    }
  }
}

// One block of 1024 entries, sixteen wavefronts of 64 consecutive entries each.  A wavefront ranks its entries among
// equal expert ids with ballots (one round per distinct id in the chunk) and leaves the chunk's per-expert counts
// in LDS; a prefix over the sixteen chunks turns the counts into first positions; rank + first position is the
// output row.  Chunks, and positions inside a chunk, are taken in flat order, so the sort is stable.
// (block_first: this block's row of first positions, in global memory or in LDS; expert_base: what to add to them per
// expert, or null; e: the entry's expert id, -1 for none)
__device__ __forceinline__ void rank_block(int *chunk_first, const int *block_first, const int *expert_base, long long i,
                                           bool live, int e, int *expanded_row_idx, int expert_num) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int *mine = chunk_first + wave * expert_num;
  for (int x = lane; x < expert_num; x += 64) mine[x] = 0;
  const unsigned long long same = wave_match(e, live, id_bits(expert_num));
  const int rank = __popcll(same & ((1ull << lane) - 1ull));
  if (live && rank == 0) mine[e] = __popcll(same);      // after the zero fill above: one wavefront's LDS operations stay in order
  __syncthreads();
  for (int x = threadIdx.x; x < expert_num; x += 1024) {
    int running = block_first[x] + (expert_base != nullptr ? expert_base[x] : 0);
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int c = chunk_first[w * expert_num + x];
      chunk_first[w * expert_num + x] = running;
      running += c;
    }
  }
  __syncthreads();
  if (live) expanded_row_idx[i] = mine[e] + rank;
}

__global__ void __launch_bounds__(1024) route_rank_kernel(const int *expert_idx, const int *block_first, const int *expert_base,
                                                          int *expanded_row_idx, long long n, int expert_num) {
  extern __shared__ int chunk_first[];   // [16][expert_num]
  const long long i = (long long)blockIdx.x * kRouteBlock + threadIdx.x;
  const bool live = i < n;
  const int e = live ? clamp_expert(expert_idx[i], expert_num) : -1;
  rank_block(chunk_first, block_first + (long long)blockIdx.x * expert_num, expert_base, i, live, e, expanded_row_idx, expert_num);
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
// dozen instructions per element.  r = x * (1 / scale) differs from that quotient by at most 1.5 * 2^-23 * 127.5 < 2.3e-5
// (two roundings here, one there), so unless r lies within kRqMargin = 5e-5 of a half-integer both round to the same
// integer.  Adding 1.5 * 2^23 rounds r to that integer (nearest, ties to even, like rint) in the low mantissa bits: its
// low byte is the int8.  Elements too close to a half-integer (1e-4 of them) are done again with the division.
// eight elements -> eight int8; `nonzero`: the row's maximum is not zero (a row of zeros has scale 0: the golden divides
// 0 by 0 there; it gets zeros)
constexpr float kRqMargin = 5e-5f;
template <bool BF16>
__device__ __forceinline__ uint2 rq_quantise(const uint4 &v, float scale, float inv, bool nonzero) {
  constexpr float kRound = 12582912.0f;   // 1.5 * 2^23
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  float f[8], d[8];
  unsigned b[8];
  float worst = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = BF16 ? __uint_as_float(w[i] << 16) : f16_bits_to_f32((unsigned short)(w[i] & 0xFFFFu));
    f[2 * i + 1] = BF16 ? __uint_as_float(w[i] & 0xFFFF0000u) : f16_bits_to_f32((unsigned short)(w[i] >> 16));
  }
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    const float r0 = f[e] * inv, r1 = f[e + 1] * inv;
    const float t0 = r0 + kRound, t1 = r1 + kRound;
    b[e] = __float_as_uint(t0);
    b[e + 1] = __float_as_uint(t1);
    d[e] = r0 - (t0 - kRound);
    d[e + 1] = r1 - (t1 - kRound);
    worst = fmaxf(fmaxf(fabsf(d[e]), fabsf(d[e + 1])), worst);
  }
  if (!(worst <= 0.5f - kRqMargin)) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (!(fabsf(d[e]) <= 0.5f - kRqMargin)) b[e] = (unsigned)(int)rintf(f[e] / scale);
    }
  }
  // bytes 0 of b[0..3] and of b[4..7] side by side (v_perm_b32: selector 0-3 picks a byte of the second operand, 4-7 of the first)
  unsigned q[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const unsigned p01 = __builtin_amdgcn_perm(b[4 * h + 1], b[4 * h], 0x0c0c0400u);
    const unsigned p23 = __builtin_amdgcn_perm(b[4 * h + 3], b[4 * h + 2], 0x0c0c0400u);
    q[h] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
  }
  return nonzero ? make_uint2(q[0], q[1]) : make_uint2(0, 0);
}

// ---- one wavefront moves one source row to `copies` destination rows ----
// The k entries of a token are neighbours in the flat entry order, so a wavefront that owns consecutive entries reads
// (and quantises) a token's row once and writes it k times: half the loads and half the arithmetic at top-2.

// Rows are read and written through buffer descriptors over exactly one row (the row's address is the same for the whole
// wavefront: callers derive it from a wavefront index made scalar with readfirstlane): what lies past the row's end
// reads as zeros and is not written, so no lane ever branches around a load (a conditional load costs a full
// `s_waitcnt vmcnt(0)` where its value meets the zero of the other path).
typedef unsigned rq_v4u __attribute__((ext_vector_type(4)));
typedef unsigned rq_v2u __attribute__((ext_vector_type(2)));
typedef int rq_v2i __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 row_load16(__amdgpu_buffer_rsrc_t rs, long long byte_offset) {
  const unsigned off = byte_offset > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)byte_offset;   // (past any row: zeros)
  const rq_v4u v = __builtin_bit_cast(rq_v4u, __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void row_store16(__amdgpu_buffer_rsrc_t rs, long long byte_offset, const uint4 &v) {
  const unsigned off = byte_offset > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)byte_offset;
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, rq_v4u{v.x, v.y, v.z, v.w}), rs, off, 0, 0);
}
__device__ __forceinline__ void row_store8(__amdgpu_buffer_rsrc_t rs, long long byte_offset, const uint2 &v) {
  const unsigned off = byte_offset > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)byte_offset;
  __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(rq_v2i, rq_v2u{v.x, v.y}), rs, off, 0, 0);
}

// the first KV vectors per lane of a row (lane + 64 u), requested together; zeros past the row's end
template <int KV>
__device__ __forceinline__ void wave_load_row(uint4 (&kept)[KV], __amdgpu_buffer_rsrc_t src, int lane, long long first_byte = 0) {
  static_for<KV>([&](auto u_c) {
    constexpr int U = decltype(u_c)::value;
    kept[U] = row_load16(src, first_byte + 16ll * (lane + 64 * U));
  });
}

// `first`: what wave_load_row brought of this row; dest_row(j): the j-th destination row
template <int KV, typename DestFn>
__device__ __forceinline__ void wave_copy_row(const uint4 (&first)[KV], __amdgpu_buffer_rsrc_t src, int lane, int copies,
                                              DestFn dest_row, unsigned char *expanded_x, long long row_bytes) {
  for (int j = 0; j < copies; ++j) {
    const __amdgpu_buffer_rsrc_t dst = buffer_over(expanded_x + (long long)dest_row(j) * row_bytes, row_bytes);
    static_for<KV>([&](auto u_c) {
      constexpr int U = decltype(u_c)::value;
      row_store16(dst, 16ll * (lane + 64 * U), first[U]);   // kept cacheable: the matmul reads it next
    });
  }
  for (long long b0 = 1024ll * KV; b0 < row_bytes; b0 += 1024ll * KV) {
    uint4 buf[KV];
    wave_load_row(buf, src, lane, b0);
    for (int j = 0; j < copies; ++j) {
      const __amdgpu_buffer_rsrc_t dst = buffer_over(expanded_x + (long long)dest_row(j) * row_bytes, row_bytes);
      static_for<KV>([&](auto u_c) {
        constexpr int U = decltype(u_c)::value;
        row_store16(dst, b0 + 16ll * (lane + 64 * U), buf[U]);
      });
    }
  }
}

// The same with the per-row dynamic int8 quantisation on the way: the row's maximum needs no LDS (one wavefront holds
// the whole row); a lane keeps KEEP vectors of the row in registers (64 lanes x KEEP x 16 bytes in one pass), what lies
// beyond is read again for the division (L2 hits).  Zeros past the row's end change neither the maximum nor anything
// that is stored.
template <bool BF16, int KEEP, typename DestFn>
__device__ __forceinline__ void wave_quantise_row(const uint4 (&kept)[KEEP], __amdgpu_buffer_rsrc_t src, int lane, int copies,
                                                  DestFn dest_row, signed char *expanded_x, float *expanded_scale,
                                                  long long hidden) {
  const long long row_bytes = 2 * hidden;
  unsigned mx = 0;
  static_for<KEEP>([&](auto u_c) { rq_fold(mx, kept[decltype(u_c)::value]); });
  for (long long b = 1024ll * KEEP; b < row_bytes; b += 1024) rq_fold(mx, row_load16(src, b + 16 * lane));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = max(mx, (unsigned)__shfl_xor((int)mx, o));
  const float scale = rq_widen<BF16>((unsigned short)mx) / 127.0f;
  const float inv = 1.0f / scale;
  if (lane == 0) {
    for (int j = 0; j < copies; ++j) expanded_scale[dest_row(j)] = scale;
  }
  // two vectors at a time, to every copy (the quantised row never exists as a whole in registers).  A lane's eight
  // bytes and its neighbour's are consecutive in the row: the even lane of a pair takes both lanes' bytes of the first
  // vector and the odd lane both of the second, so that every lane stores 16 bytes (rows of a multiple of 16 bytes).
  const bool wide = (hidden & 15) == 0;
  const long long pair_byte = 512 * (lane & 1) + 16 * (lane >> 1);
  static_for<KEEP / 2>([&](auto p_c) {
    constexpr int P = decltype(p_c)::value;
    const uint2 qa = rq_quantise<BF16>(kept[2 * P], scale, inv, mx != 0);
    const uint2 qb = rq_quantise<BF16>(kept[2 * P + 1], scale, inv, mx != 0);
    if (wide) {
      const bool odd = lane & 1;
      const unsigned sx = odd ? qa.x : qb.x, sy = odd ? qa.y : qb.y;
      const unsigned rx = (unsigned)__builtin_amdgcn_update_dpp(0, (int)sx, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
      const unsigned ry = (unsigned)__builtin_amdgcn_update_dpp(0, (int)sy, 0xB1, 0xF, 0xF, true);
      const uint4 out = odd ? make_uint4(rx, ry, qb.x, qb.y) : make_uint4(qa.x, qa.y, rx, ry);
      for (int j = 0; j < copies; ++j)
        row_store16(buffer_over(expanded_x + (long long)dest_row(j) * hidden, hidden), 1024ll * P + pair_byte, out);
    } else {
      for (int j = 0; j < copies; ++j) {
        const __amdgpu_buffer_rsrc_t dst = buffer_over(expanded_x + (long long)dest_row(j) * hidden, hidden);
        row_store8(dst, 8ll * (lane + 128 * P), qa);
        row_store8(dst, 8ll * (lane + 128 * P + 64), qb);
      }
    }
  });
  for (long long b = 1024ll * KEEP; b < row_bytes; b += 1024) {
    const uint2 q = rq_quantise<BF16>(row_load16(src, b + 16 * lane), scale, inv, mx != 0);
    for (int j = 0; j < copies; ++j)
      row_store8(buffer_over(expanded_x + (long long)dest_row(j) * hidden, hidden), (b >> 1) + 8 * lane, q);
  }
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
// QUANT: 0 copies rows of row_bytes bytes; 1 / 2 quantise float16 / bfloat16 rows to int8 and write their scales.
template <int QUANT>
__global__ void __launch_bounds__(kFusedThreads) route_fused_kernel(const unsigned char *x, const int *expert_idx,
                                                                    unsigned char *expanded_x, float *expanded_scale,
                                                                    int *expanded_row_idx, int *count_or_cumsum,
                                                                    int *before_capacity, long long n, int expert_num, int flag,
                                                                    long long row_bytes, int k, int rep) {
  extern __shared__ int lds[];   // total[rep][expert_num], before[rep][expert_num], base[expert_num], wave_sum[16], dest[kFusedRows]
  int *total = lds;
  int *before = total + rep * expert_num;
  int *base = before + rep * expert_num;
  int *wave_sum = base + expert_num;
  int *dest = wave_sum + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long long start = (long long)blockIdx.x * kFusedRows;
  constexpr int RPW = kFusedRows / 16;   // consecutive entries per wavefront
  constexpr int KV = 8;                  // vectors of a row per lane and pass
  const long long entry0 = start + RPW * wave;
  for (int i = tid; i < 2 * rep * expert_num; i += kFusedThreads) lds[i] = 0;
  // all of a thread's ids are requested before the first is used: entries 4 (tid + 1024 j) .. + 3 (ids past n read as 0,
  // by the range check of the buffer load, and are skipped by their index; only the vector offset is range-checked)
  const __amdgpu_buffer_rsrc_t rs_ids = buffer_over(expert_idx, n * 4);
  v4i ids[kFusedIdsPerThread / 4];
  static_for<kFusedIdsPerThread / 4>([&](auto j_c) {
    constexpr int J = decltype(j_c)::value;
    ids[J] = __builtin_amdgcn_raw_buffer_load_b128(rs_ids, (unsigned)(16 * (tid + kFusedThreads * J)), 0, 0);
  });
  // the slice's own ids for the ranking by wavefront 0, requested now: a load issued where they are needed would put a
  // memory round trip between two barriers (other lanes ask beyond the list and get zeros)
  const int slice_id = __builtin_amdgcn_raw_buffer_load_b32(
      rs_ids, wave == 0 && lane < kFusedRows && start + lane < n ? (unsigned)(4 * (start + lane)) : 0xFFFFFFFCu, 0, 0);
  // The plain copy requests the row of the wavefront's first entry right behind the ids (loads return in order: the
  // counting must not wait for it): where it comes from is known from the entry's index alone (token = entry / k), only
  // where it goes has to wait for the counting below.  (Measured: 0.4 us less for the copy at 8192 entries of 4 KiB; the
  // quantising variant is 0.7 us slower with it.)
  constexpr bool kPreload = QUANT == 0;
  uint4 row0[KV];
  if constexpr (kPreload) {
    wave_load_row(row0, buffer_over(x + (long long)(entry0 < n ? (unsigned)entry0 / (unsigned)k : 0u) * row_bytes, entry0 < n ? row_bytes : 0),
                  lane);
  }
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
    const int e = live ? clamp_expert(slice_id, expert_num) : -1;
    const int rank = __popcll(wave_match(e, live, id_bits(expert_num)) & ((1ull << lane) - 1ull));
    if (live) {
      const int d = base[e] + before[e] + rank;
      dest[lane] = d;
      expanded_row_idx[i] = d;
    }
  }
  __syncthreads();
  // move the rows: wavefront w takes the slice's entries RPW w .. RPW w + RPW - 1; neighbours of one token share a pass
  int r = 0;
  while (r < RPW) {
    const long long i = entry0 + r;
    if (i >= n) break;
    const unsigned token = (unsigned)i / (unsigned)k;   // (entries fit 31 bits: 32-bit divisions)
    int copies = 1;
    while (r + copies < RPW && i + copies < n && (unsigned)(i + copies) / (unsigned)k == token) ++copies;
    const int first = RPW * wave + r;
    auto dest_row = [&](int j) { return __builtin_amdgcn_readfirstlane(dest[first + j]); };
    const __amdgpu_buffer_rsrc_t src = buffer_over(x + (long long)token * row_bytes, row_bytes);
    if (r != 0 || !kPreload) wave_load_row(row0, src, lane);
    if constexpr (QUANT == 0) {
      wave_copy_row(row0, src, lane, copies, dest_row, expanded_x, row_bytes);
    } else {
      wave_quantise_row<QUANT == 2>(row0, src, lane, copies, dest_row, reinterpret_cast<signed char *>(expanded_x),
                                    expanded_scale, row_bytes / 2);
    }
    r += copies;
  }
}

// The row movement behind the sort for problems beyond the single launch: one wavefront per token reads its row once and
// writes it to the k rows expanded_row_idx names for it.
__global__ void __launch_bounds__(256) route_scatter_kernel(const unsigned char *x, const int *expanded_row_idx,
                                                            unsigned char *expanded_x, long long num_rows, long long row_bytes,
                                                            int k) {
  const int lane = threadIdx.x & 63;
  const long long token = (long long)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (token >= num_rows) return;
  const int *dests = expanded_row_idx + token * k;
  const __amdgpu_buffer_rsrc_t src = buffer_over(x + token * row_bytes, row_bytes);
  uint4 first[8];
  wave_load_row(first, src, lane);
  wave_copy_row(first, src, lane, k, [&](int j) { return __builtin_amdgcn_readfirstlane(dests[j]); }, expanded_x, row_bytes);
}

// Per-row dynamic int8 quantisation on the way to the sorted rows, for problems beyond the single launch: one wavefront
// per token quantises its row once and writes it to the k rows expanded_row_idx names for it.
template <bool BF16>
__global__ void __launch_bounds__(256) route_scatter_quant_kernel(const unsigned short *x, const int *expanded_row_idx,
                                                                  signed char *expanded_x, float *expanded_scale,
                                                                  long long num_rows, long long hidden, int k) {
  const int lane = threadIdx.x & 63;
  const long long token = (long long)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (token >= num_rows) return;
  const int *dests = expanded_row_idx + token * k;
  const __amdgpu_buffer_rsrc_t src = buffer_over(x + token * hidden, 2 * hidden);
  uint4 kept[16];
  wave_load_row(kept, src, lane);
  wave_quantise_row<BF16>(kept, src, lane, k, [&](int j) { return __builtin_amdgcn_readfirstlane(dests[j]); }, expanded_x,
                          expanded_scale, hidden);
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
  // per-block expert histograms / first positions, then the first position of every expert
  return (size_t)(msco::route_blocks(n) + 1) * expert_num * sizeof(int32_t);
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
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, static_cast<int *>(nullptr), static_cast<int *>(nullptr),
                       expert_tokens_count_or_cumsum, expert_tokens_before_capacity, 0, (int)expert_num, (int)count_or_cumsum_flag);
    return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
  }
  if (x == nullptr || expert_idx == nullptr || expanded_x == nullptr || expanded_row_idx == nullptr) return MSCO_ERR_INVALID_ARG;
  if (quant_dtype != MSCO_DT_NONE && expanded_scale == nullptr) return MSCO_ERR_INVALID_ARG;
  if (count_or_cumsum_flag != 0 && expert_tokens_count_or_cumsum == nullptr) return MSCO_ERR_INVALID_ARG;
  if (workspace == nullptr || workspace_bytes < msco_moe_init_routing_v2_workspace_bytes(num_rows, k, expert_num))
    return MSCO_ERR_WORKSPACE;
  if (n <= kFusedMaxEntries) {
    // small problems: the sort and the row movement in one launch, no workspace traffic
    int rep = 8;
    while (rep > 1 && rep * expert_num > 512) rep /= 2;
    const size_t lds_bytes = (size_t)(2 * rep * expert_num + expert_num + 16 + kFusedRows) * sizeof(int);
    const dim3 grid((unsigned)((n + kFusedRows - 1) / kFusedRows)), block(kFusedThreads);
#define MSCO_ROUTE_FUSED(Q)                                                                                                  \
    hipLaunchKernelGGL(route_fused_kernel<Q>, grid, block, lds_bytes, s, static_cast<const unsigned char *>(x), expert_idx,   \
                       static_cast<unsigned char *>(expanded_x), expanded_scale, expanded_row_idx,                            \
                       expert_tokens_count_or_cumsum, expert_tokens_before_capacity, n, (int)expert_num,                      \
                       (int)count_or_cumsum_flag, (long long)hidden * (quant_dtype == MSCO_DT_NONE ? elem_bytes : 2), (int)k, rep)
    if (quant_dtype == MSCO_DT_NONE) MSCO_ROUTE_FUSED(0);
    else if (quant_dtype == MSCO_DT_F16) MSCO_ROUTE_FUSED(1);
    else MSCO_ROUTE_FUSED(2);
#undef MSCO_ROUTE_FUSED
    return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
  }
  const long long blocks = route_blocks(n);
  int *block_hist = static_cast<int *>(workspace);
  int *expert_base = block_hist + blocks * expert_num;
  hipLaunchKernelGGL(route_hist_kernel, dim3((unsigned)blocks), dim3(256), 0, s, expert_idx, block_hist, n, (int)expert_num);
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, block_hist, expert_base, expert_tokens_count_or_cumsum,
                     expert_tokens_before_capacity, (int)blocks, (int)expert_num, (int)count_or_cumsum_flag);
  hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)blocks), dim3(1024), (size_t)16 * expert_num * sizeof(int), s, expert_idx,
                     block_hist, expert_base, expanded_row_idx, n, (int)expert_num);
  if (quant_dtype == MSCO_DT_NONE) {
    hipLaunchKernelGGL(route_scatter_kernel, dim3((unsigned)((num_rows + 3) / 4)), dim3(256), 0, s, static_cast<const unsigned char *>(x),
                       expanded_row_idx, static_cast<unsigned char *>(expanded_x), (long long)num_rows, (long long)hidden * elem_bytes,
                       (int)k);
  } else {
    const dim3 grid((unsigned)((num_rows + 3) / 4)), block(256);
    if (quant_dtype == MSCO_DT_BF16) {
      hipLaunchKernelGGL(route_scatter_quant_kernel<true>, grid, block, 0, s, static_cast<const unsigned short *>(x),
                         expanded_row_idx, static_cast<signed char *>(expanded_x), expanded_scale, (long long)num_rows,
                         (long long)hidden, (int)k);
    } else {
      hipLaunchKernelGGL(route_scatter_quant_kernel<false>, grid, block, 0, s, static_cast<const unsigned short *>(x),
                         expanded_row_idx, static_cast<signed char *>(expanded_x), expanded_scale, (long long)num_rows,
                         (long long)hidden, (int)k);
    }
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
