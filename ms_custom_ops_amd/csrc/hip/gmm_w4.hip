// Grouped A8W4 matmul for gfx950: int8 activations x int4 weights (two per byte, [E, N, K/2], K contiguous), float32
// scales per (expert, K group, column), per-token activation scales, float16 out.
//
//   out[m, n] = x_scale[m] * sum_g w_scale[e, g, n] * sum_{k in g} x[m, k] * w[e, n, k]        (e = the group of row m)
//
// (tests/st/test_grouped_matmul_w4.py:100-113; ops/c_api/grouped_matmul_w4/grouped_matmul_w4.cc:50-88.)  The
// reference's workloads route 5 .. 32 rows to 256 experts: almost every group is empty or holds one row, so this is a
// batch of matrix-vector products bound by the bytes of the weights of the experts that were hit.  Hence no MFMA:
//   * one workgroup per (group that holds rows, 16 or more columns): the grid has min(E, M) group slots and a workgroup
//     finds the group of its slot's rank with ballots over group_list; a short K lets several columns share a wavefront's lanes;
//   * the group's rows (four at a time) sit in LDS, de-interleaved into even-k and odd-k bytes so that they line up
//     with the low and the high nibbles of a weight word;
//   * a wavefront owns four columns and requests all their weights at once (one memory round trip; they stay in
//     registers for every block of rows), lane L holding the 16-byte pieces L, L + 64, ... of a column (32
//     consecutive k, always inside one K group): nibbles are multiplied as u ^ 8 in [0, 15] with v_dot4_i32_i8 and
//     8 * sum(x) of the piece is subtracted (u ^ 8 = s + 8 for the signed nibble s); the int32 sum of a piece is
//     exact, is scaled by its K group's float32 scale and added up in float32; lanes are reduced with shuffles.
#include "gmm_common.h"
#include "gmm_kernels.h"
#include "msco_gmm.h"

namespace msco {
namespace {

constexpr int W4_ROWS = 4;           // rows of a group held in LDS at a time (k bytes each: small, so that many workgroups fit a CU)
constexpr int W4_WAVE_COLS = 4;      // columns per lane segment of a wavefront, all in registers at once
constexpr int W4_MAX_K = 8192;
constexpr int W4_LANE_PIECES = W4_MAX_K / 32 / 64;   // 16-byte pieces of a column per lane

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__global__ void __launch_bounds__(256) gmm_a8w4_kernel(const int8_t *x, const unsigned char *w, const int *group_list,
                                                       const float *x_scale, const float *w_scale, unsigned short *out, int m,
                                                       int k, int n, int e, int group_size) {
  extern __shared__ __align__(16) int xs[];   // min(W4_ROWS, m) rows: [row][piece of 32 k]: 4 words of even-k bytes, then 4 of odd-k bytes
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // blockIdx.y counts the groups that hold rows (at most min(e, m) of them): find the one with that rank, 64 groups
  // per round of ballots, and leave if there are fewer
  int grp = -1, g_start = 0, g_end = 0;
  for (int g0 = 0, seen = 0, carry = 0; g0 < e && grp < 0; g0 += 256) {
    int lo[4], hi[4];   // four rounds' worth of boundaries requested together: one memory round trip per 256 groups
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int g = g0 + 64 * u + lane;
      hi[u] = g < e ? min(max(group_list[g], 0), m) : 0;
    }
    // row end of a group = running maximum of the list clamped into [0, m] (a list that is not monotonic can then
    // never make two groups overlap); `carry` is the end of the last group of the round before
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      hi[u] = max(carry, wave_scan_max(hi[u], lane));
      const int prev = __shfl_up(hi[u], 1);
      lo[u] = lane == 0 ? carry : prev;
      carry = wave_bcast(hi[u], 63);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      unsigned long long holds = __ballot(hi[u] > lo[u]);
      const int here = __popcll(holds);
      if (grp < 0 && seen + here > (int)blockIdx.y) {
        for (int skip = (int)blockIdx.y - seen; skip > 0; --skip) holds &= holds - 1;
        const int src = __ffsll((long long)holds) - 1;
        grp = g0 + 64 * u + src;
        g_start = __shfl(lo[u], src);
        g_end = __shfl(hi[u], src);
      }
      seen += here;
    }
  }
  if (grp < 0) return;
  const int pieces = k / 32;
  // a short K leaves lanes over: lanes_per_col lanes share a column, the wavefront works on 64 / lanes_per_col columns side by side
  int lanes_per_col = 64;
  while (lanes_per_col / 2 >= pieces) lanes_per_col /= 2;
  const int side = 64 / lanes_per_col;
  const int pl = lane % lanes_per_col, sub = lane / lanes_per_col;
  const int k_groups = k / group_size;
  const int pieces_per_group = group_size / 32;
  const unsigned char *wg = w + (long long)grp * n * (k / 2);
  const float *sg = w_scale + (long long)grp * k_groups * n;
  const int col0 = (blockIdx.x * 4 + wave) * W4_WAVE_COLS * side + sub;   // this lane's columns: col0 + c * side

  // this wavefront's columns: every piece and its scale requested at once (one memory round trip), nibbles as u ^ 8
  uint4 wv[W4_WAVE_COLS][W4_LANE_PIECES];
  float sc[W4_WAVE_COLS][W4_LANE_PIECES];
#pragma unroll
  for (int c = 0; c < W4_WAVE_COLS; ++c)
#pragma unroll
    for (int i = 0; i < W4_LANE_PIECES; ++i) {
      const int p = pl + lanes_per_col * i, col = col0 + c * side;
      const bool live = p < pieces && col < n;
      wv[c][i] = live ? *(reinterpret_cast<const uint4 *>(wg + (long long)col * (k / 2)) + p) : make_uint4(0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u);
      sc[c][i] = live ? sg[(long long)(p / pieces_per_group) * n + col] : 0.f;
    }

  for (int r0 = g_start; r0 < g_end; r0 += W4_ROWS) {
    const int rows = min(W4_ROWS, g_end - r0);
    __syncthreads();   // the previous block of rows is no longer read
    for (int idx = threadIdx.x; idx < rows * pieces * 2; idx += 256) {
      // 16 bytes (k0 .. k15 of a half piece) -> two words of even-k bytes and two of odd-k bytes
      const int r = idx / (pieces * 2), h = idx - r * pieces * 2;
      const uint4 v = *reinterpret_cast<const uint4 *>(x + (long long)(r0 + r) * k + h * 16);
      const unsigned e0 = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u), o0 = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);
      const unsigned e1 = __builtin_amdgcn_perm(v.w, v.z, 0x06040200u), o1 = __builtin_amdgcn_perm(v.w, v.z, 0x07050301u);
      int *dst = xs + (r * pieces + (h >> 1)) * 8 + (h & 1) * 2;
      dst[0] = (int)e0; dst[1] = (int)e1; dst[4] = (int)o0; dst[5] = (int)o1;
    }
    __syncthreads();
    for (int r = 0; r < rows; ++r) {
      float acc[W4_WAVE_COLS];
#pragma unroll
      for (int c = 0; c < W4_WAVE_COLS; ++c) acc[c] = 0.f;
#pragma unroll
      for (int i = 0; i < W4_LANE_PIECES; ++i) {
        const int p = pl + lanes_per_col * i;
        if (p < pieces) {
          const int4 xe = *reinterpret_cast<const int4 *>(xs + (r * pieces + p) * 8);
          const int4 xo = *reinterpret_cast<const int4 *>(xs + (r * pieces + p) * 8 + 4);
          int sx = 0;
          sx = dot4(xe.x, 0x01010101, sx); sx = dot4(xo.x, 0x01010101, sx); sx = dot4(xe.y, 0x01010101, sx);
          sx = dot4(xo.y, 0x01010101, sx); sx = dot4(xe.z, 0x01010101, sx); sx = dot4(xo.z, 0x01010101, sx);
          sx = dot4(xe.w, 0x01010101, sx); sx = dot4(xo.w, 0x01010101, sx);
#pragma unroll
          for (int c = 0; c < W4_WAVE_COLS; ++c) {
            const unsigned t[4] = {wv[c][i].x ^ 0x88888888u, wv[c][i].y ^ 0x88888888u, wv[c][i].z ^ 0x88888888u, wv[c][i].w ^ 0x88888888u};
            const int xev[4] = {xe.x, xe.y, xe.z, xe.w}, xov[4] = {xo.x, xo.y, xo.z, xo.w};
            int d = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              d = dot4(xev[j], (int)(t[j] & 0x0F0F0F0Fu), d);           // k = 8 j + 0, 2, 4, 6
              d = dot4(xov[j], (int)((t[j] >> 4) & 0x0F0F0F0Fu), d);    // k = 8 j + 1, 3, 5, 7
            }
            acc[c] += (float)(d - 8 * sx) * sc[c][i];
          }
        }
      }
      const float xsr = x_scale[r0 + r];
#pragma unroll
      for (int c = 0; c < W4_WAVE_COLS; ++c) {
        float v = acc[c];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
          if (o < lanes_per_col) v += __shfl_xor(v, o);   // wave-uniform
        if (pl == 0 && col0 + c * side < n) out[(long long)(r0 + r) * n + col0 + c * side] = f32_to_f16_rne(v * xsr);
      }
    }
  }
}

}  // namespace
}  // namespace msco

extern "C" int msco_gmm_a8w4(const int8_t *x, const void *weight, const int32_t *group_list, const float *x_scale,
                             const float *weight_scale, void *out, int64_t m, int64_t k, int64_t n, int64_t e,
                             int64_t group_size, void *stream) {
  using namespace msco;
  if (m < 0 || k <= 0 || n <= 0 || e <= 0 || group_size <= 0) return MSCO_ERR_SHAPE;
  if (k % 32 != 0 || group_size % 32 != 0 || k % group_size != 0) return MSCO_ERR_SHAPE;
  if (k > W4_MAX_K || e > 65535 || m > INT32_MAX || n > INT32_MAX) return MSCO_ERR_UNSUPPORTED;
  if (m == 0) return MSCO_OK;
  if (x == nullptr || weight == nullptr || group_list == nullptr || x_scale == nullptr || weight_scale == nullptr || out == nullptr)
    return MSCO_ERR_INVALID_ARG;
  int lanes_per_col = 64;
  while (lanes_per_col / 2 >= k / 32) lanes_per_col /= 2;
  const long long wg_cols = 4ll * W4_WAVE_COLS * (64 / lanes_per_col);
  const dim3 grid((unsigned)((n + wg_cols - 1) / wg_cols), (unsigned)(e < m ? e : m));
  const size_t lds = (size_t)(m < W4_ROWS ? m : W4_ROWS) * (size_t)k;
  hipLaunchKernelGGL(gmm_a8w4_kernel, grid, dim3(256), lds, static_cast<hipStream_t>(stream), x,
                     static_cast<const unsigned char *>(weight), group_list, x_scale, weight_scale,
                     static_cast<unsigned short *>(out), (int)m, (int)k, (int)n, (int)e, (int)group_size);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}
