// MoE routing (stable counting sort of (token, k) entries by expert + activation gather) and weighted
// un-permutation for gfx950.  Both are HBM-bound row copies around a small integer problem:
//
//   init_routing   1. per block of 1024 entries: histogram of the expert ids (LDS atomics)
//                  2. one workgroup: per expert, exclusive scan over the blocks, then over the experts;
//                     writes the count / cumulative-count output
//                  3. per block, one wavefront walks its entries 64 at a time in flat order and ranks
//                     them among equal expert ids with ballots, which keeps the sort stable
//                  4. one workgroup per output row copies x[token] with 16-byte loads and stores
//   unpermute      one workgroup per token: 16 bytes of every selected row per lane, the running sum kept
//                  in the element type and rounded exactly where the golden rounds it
#include "msco_moe.h"

#include <hip/hip_runtime.h>

#include "gmm_common.h"

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

__global__ void __launch_bounds__(64) route_rank_kernel(const int *expert_idx, const int *block_first, int *expanded_row_idx,
                                                        int *sorted_src, long long n, int expert_num) {
  __shared__ int next[kMaxExperts];
  const int lane = threadIdx.x;
  for (int e = lane; e < expert_num; e += 64) next[e] = block_first[(long long)blockIdx.x * expert_num + e];
  __syncthreads();
  const long long first = (long long)blockIdx.x * kRouteBlock;
  for (int c = 0; c < kRouteBlock / 64; ++c) {
    const long long i = first + c * 64 + lane;
    const bool live = i < n;
    const int e = live ? clamp_expert(expert_idx[i], expert_num) : -1;
    unsigned long long todo = __ballot(live);
    int dest = 0;
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const int e0 = __shfl(e, leader);
      const unsigned long long same = __ballot(e == e0) & todo;
      if (e == e0 && live) dest = next[e0] + __popcll(same & ((1ull << lane) - 1ull));
      __syncthreads();                                   // one wavefront: orders the LDS read above and the update below
      if (lane == leader) next[e0] += __popcll(same);
      __syncthreads();
      todo &= ~same;
    }
    if (live) {
      expanded_row_idx[i] = dest;
      sorted_src[dest] = (int)i;
    }
  }
}

__global__ void __launch_bounds__(256) route_gather_kernel(const unsigned char *x, const int *sorted_src, unsigned char *expanded_x,
                                                           long long row_bytes, int k) {
  const long long j = blockIdx.x;
  const long long token = sorted_src[j] / k;
  const uint4 *src = reinterpret_cast<const uint4 *>(x + token * row_bytes);
  uint4 *dst = reinterpret_cast<uint4 *>(expanded_x + j * row_bytes);
  for (long long v = threadIdx.x; v < row_bytes / 16; v += 256) dst[v] = src[v];
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

template <bool BF16>
__global__ void __launch_bounds__(256) unpermute_kernel(const unsigned short *permuted, const int *sorted_indices,
                                                        const unsigned short *probs, unsigned short *out, int top_k,
                                                        long long hidden) {
  const long long token = blockIdx.x;
  for (long long h0 = (long long)threadIdx.x * 8; h0 < hidden; h0 += 256 * 8) {
    unsigned short acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0;
    for (int kk = 0; kk < top_k; ++kk) {
      const long long row = sorted_indices[token * top_k + kk];
      const float p = from_elem<BF16>(probs[token * top_k + kk]);
      const uint4 q = *reinterpret_cast<const uint4 *>(permuted + row * hidden + h0);
      const unsigned w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const unsigned short v = (unsigned short)(w[j >> 1] >> (16 * (j & 1)));
        // product rounded to the element type, then the running sum rounded to it: two float32 operations,
        // kept apart (no fused multiply-add) because the golden rounds in between
        float prod = p * from_elem<BF16>(v);
        asm volatile("" : "+v"(prod));
        const float prod_r = from_elem<BF16>(to_elem<BF16>(prod));
        float sum = from_elem<BF16>(acc[j]) + prod_r;
        asm volatile("" : "+v"(sum));
        acc[j] = to_elem<BF16>(sum);
      }
    }
    uint4 o;
    o.x = acc[0] | ((unsigned)acc[1] << 16); o.y = acc[2] | ((unsigned)acc[3] << 16);
    o.z = acc[4] | ((unsigned)acc[5] << 16); o.w = acc[6] | ((unsigned)acc[7] << 16);
    *reinterpret_cast<uint4 *>(out + token * hidden + h0) = o;
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

int msco_moe_init_routing_v2(const void *x, const int32_t *expert_idx, void *expanded_x, int32_t *expanded_row_idx,
                             int32_t *expert_tokens_count_or_cumsum, int32_t *expert_tokens_before_capacity,
                             void *workspace, size_t workspace_bytes, int64_t num_rows, int64_t hidden, int64_t k,
                             int64_t expert_num, int32_t elem_bytes, int32_t count_or_cumsum_flag, void *stream) {
  using namespace msco;
  if (num_rows < 0 || hidden <= 0 || k <= 0 || expert_num <= 0 || expert_num > kMaxExperts) return MSCO_ERR_SHAPE;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) return MSCO_ERR_UNSUPPORTED;
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
  if (count_or_cumsum_flag != 0 && expert_tokens_count_or_cumsum == nullptr) return MSCO_ERR_INVALID_ARG;
  if (workspace == nullptr || workspace_bytes < msco_moe_init_routing_v2_workspace_bytes(num_rows, k, expert_num))
    return MSCO_ERR_WORKSPACE;
  const long long blocks = route_blocks(n);
  int *block_hist = static_cast<int *>(workspace);
  int *sorted_src = block_hist + blocks * expert_num;
  hipLaunchKernelGGL(route_hist_kernel, dim3((unsigned)blocks), dim3(256), 0, s, expert_idx, block_hist, n, (int)expert_num);
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, block_hist, expert_tokens_count_or_cumsum,
                     expert_tokens_before_capacity, (int)blocks, (int)expert_num, (int)count_or_cumsum_flag);
  hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)blocks), dim3(64), 0, s, expert_idx, block_hist, expanded_row_idx,
                     sorted_src, n, (int)expert_num);
  hipLaunchKernelGGL(route_gather_kernel, dim3((unsigned)n), dim3(256), 0, s, static_cast<const unsigned char *>(x), sorted_src,
                     static_cast<unsigned char *>(expanded_x), (long long)hidden * elem_bytes, (int)k);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
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
  if (dtype == MSCO_DT_BF16)
    hipLaunchKernelGGL(unpermute_kernel<true>, dim3((unsigned)num_tokens), dim3(256), 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);
  else
    hipLaunchKernelGGL(unpermute_kernel<false>, dim3((unsigned)num_tokens), dim3(256), 0, s, pt, sorted_indices, pr, o, (int)top_k, (long long)hidden);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

}  // extern "C"
