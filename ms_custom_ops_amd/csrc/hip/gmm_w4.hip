// Grouped A8W4 matmul for gfx950: int8 activations x int4 weights (two per byte, [E, N, K/2], K contiguous), float32
// scales per (expert, K group, column), per-token activation scales, float16 out.
//
//   out[m, n] = x_scale[m] * sum_g w_scale[e, g, n] * sum_{k in g} x[m, k] * w[e, n, k]        (e = the group of row m)
//
// (tests/st/test_grouped_matmul_w4.py:100-113; ops/c_api/grouped_matmul_w4/grouped_matmul_w4.cc:50-88.)  The
// reference's workloads route 5 .. 32 rows to 256 experts: almost every group is empty or holds one row, so this is a
// batch of matrix-vector products bound by the bytes of the weights of the experts that were hit.  Hence no MFMA:
//   * one workgroup per (group, 16 columns); a workgroup whose group is empty leaves at once;
//   * the group's rows (eight at a time) sit in LDS, de-interleaved into even-k and odd-k bytes so that they line up
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

constexpr int W4_ROWS = 8;           // rows of a group held in LDS at a time
constexpr int W4_WAVE_COLS = 4;      // columns per wavefront, all in registers at once
constexpr int W4_COLS = 4 * W4_WAVE_COLS;   // columns per workgroup
constexpr int W4_MAX_K = 8192;
constexpr int W4_LANE_PIECES = W4_MAX_K / 32 / 64;   // 16-byte pieces of a column per lane

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__global__ void __launch_bounds__(256) gmm_a8w4_kernel(const int8_t *x, const unsigned char *w, const int *group_list,
                                                       const float *x_scale, const float *w_scale, unsigned short *out, int m,
                                                       int k, int n, int e, int group_size) {
  __shared__ __align__(16) int xs[W4_ROWS * W4_MAX_K / 4];   // [row][piece of 32 k]: 4 words of even-k bytes, then 4 of odd-k bytes
  const int grp = blockIdx.y;
  const int g_start = grp == 0 ? 0 : min(max(group_list[grp - 1], 0), m);
  const int g_end = min(max(group_list[grp], g_start), m);
  if (g_end <= g_start) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pieces = k / 32;
  const int k_groups = k / group_size;
  const int pieces_per_group = group_size / 32;
  const unsigned char *wg = w + (long long)grp * n * (k / 2);
  const float *sg = w_scale + (long long)grp * k_groups * n;
  const int col0 = blockIdx.x * W4_COLS + wave * W4_WAVE_COLS;

  // this wavefront's columns: every piece and its scale requested at once (one memory round trip), nibbles as u ^ 8
  uint4 wv[W4_WAVE_COLS][W4_LANE_PIECES];
  float sc[W4_WAVE_COLS][W4_LANE_PIECES];
#pragma unroll
  for (int c = 0; c < W4_WAVE_COLS; ++c)
#pragma unroll
    for (int i = 0; i < W4_LANE_PIECES; ++i) {
      const int p = lane + 64 * i, col = col0 + c;
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
        const int p = lane + 64 * i;
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
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
        if (lane == 0 && col0 + c < n) out[(long long)(r0 + r) * n + col0 + c] = f32_to_f16_rne(v * xsr);
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
  const dim3 grid((unsigned)((n + W4_COLS - 1) / W4_COLS), (unsigned)e);
  hipLaunchKernelGGL(gmm_a8w4_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), x,
                     static_cast<const unsigned char *>(weight), group_list, x_scale, weight_scale,
                     static_cast<unsigned short *>(out), (int)m, (int)k, (int)n, (int)e, (int)group_size);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}
