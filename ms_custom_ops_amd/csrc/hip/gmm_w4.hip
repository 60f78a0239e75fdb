// Grouped A8W4 matmul for gfx950: int8 activations x int4 weights (two per byte, [E, N, K/2], K contiguous), float32
// scales per (expert, K group, column), per-token activation scales, float16 out.
//
//   out[m, n] = x_scale[m] * sum_g w_scale[e, g, n] * sum_{k in g} x[m, k] * w[e, n, k]        (e = the group of row m)
//
// (tests/st/test_grouped_matmul_w4.py:100-113; ops/c_api/grouped_matmul_w4/grouped_matmul_w4.cc:50-88.)  The
// reference's workloads route 5 .. 32 rows to 256 experts: almost every group is empty or holds one row, so this is a
// batch of matrix-vector products bound by the bytes of the weights of the experts that were hit.  Hence no MFMA:
//   * one workgroup per (group, 64 columns); a workgroup whose group is empty leaves at once;
//   * the group's rows (eight at a time) sit in LDS, de-interleaved into even-k and odd-k bytes so that they line up
//     with the low and the high nibbles of a weight word;
//   * a wavefront walks one column at a time, lane L taking the 16-byte pieces L, L + 64, ... of the column (32
//     consecutive k, always inside one K group): nibbles are multiplied as u ^ 8 in [0, 15] with v_dot4_i32_i8 and
//     8 * sum(x) of the piece is subtracted (u ^ 8 = s + 8 for the signed nibble s); the int32 sum of a piece is
//     exact, is scaled by its K group's float32 scale and added up in float32; lanes are reduced with shuffles.
#include "gmm_common.h"
#include "gmm_kernels.h"
#include "msco_gmm.h"

namespace msco {
namespace {

constexpr int W4_ROWS = 8;           // rows of a group held in LDS at a time
constexpr int W4_COLS = 64;          // columns per workgroup (16 per wavefront)
constexpr int W4_MAX_K = 8192;

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
    for (int c = 0; c < W4_COLS / 4; ++c) {
      const int col = blockIdx.x * W4_COLS + wave * (W4_COLS / 4) + c;
      if (col >= n) break;   // wave-uniform
      float acc[W4_ROWS];
#pragma unroll
      for (int r = 0; r < W4_ROWS; ++r) acc[r] = 0.f;
      const uint4 *wc = reinterpret_cast<const uint4 *>(wg + (long long)col * (k / 2));
      for (int p = lane; p < pieces; p += 64) {
        const uint4 wv = *(wc + p);
        const float s = sg[(long long)(p / pieces_per_group) * n + col];
        const unsigned t[4] = {wv.x ^ 0x88888888u, wv.y ^ 0x88888888u, wv.z ^ 0x88888888u, wv.w ^ 0x88888888u};
        int lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lo[i] = (int)(t[i] & 0x0F0F0F0Fu);           // k = 8 i + 0, 2, 4, 6
          hi[i] = (int)((t[i] >> 4) & 0x0F0F0F0Fu);    // k = 8 i + 1, 3, 5, 7
        }
#pragma unroll
        for (int r = 0; r < W4_ROWS; ++r) {
          if (r < rows) {   // wave-uniform
            const int4 xe = *reinterpret_cast<const int4 *>(xs + (r * pieces + p) * 8);
            const int4 xo = *reinterpret_cast<const int4 *>(xs + (r * pieces + p) * 8 + 4);
            int d = 0, sx = 0;
            d = dot4(xe.x, lo[0], d); d = dot4(xo.x, hi[0], d); d = dot4(xe.y, lo[1], d); d = dot4(xo.y, hi[1], d);
            d = dot4(xe.z, lo[2], d); d = dot4(xo.z, hi[2], d); d = dot4(xe.w, lo[3], d); d = dot4(xo.w, hi[3], d);
            sx = dot4(xe.x, 0x01010101, sx); sx = dot4(xo.x, 0x01010101, sx); sx = dot4(xe.y, 0x01010101, sx);
            sx = dot4(xo.y, 0x01010101, sx); sx = dot4(xe.z, 0x01010101, sx); sx = dot4(xo.z, 0x01010101, sx);
            sx = dot4(xe.w, 0x01010101, sx); sx = dot4(xo.w, 0x01010101, sx);
            acc[r] += (float)(d - 8 * sx) * s;
          }
        }
      }
#pragma unroll
      for (int r = 0; r < W4_ROWS; ++r) {
        if (r < rows) {
          float v = acc[r];
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
          if (lane == 0) out[(long long)(r0 + r) * n + col] = f32_to_f16_rne(v * x_scale[r0 + r]);
        }
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
