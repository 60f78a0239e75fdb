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
#ifndef MSCO_W4_WAVE_COLS
#define MSCO_W4_WAVE_COLS 4
#endif
constexpr int W4_WAVE_COLS = MSCO_W4_WAVE_COLS;      // columns per lane segment of a wavefront, all in registers at once
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
  const __amdgpu_buffer_rsrc_t rs_list = buffer_over(group_list, 4ll * e);
  for (int g0 = 0, seen = 0, carry = 0; g0 < e && grp < 0; g0 += 256) {
    // four rounds' worth of boundaries requested together: one memory round trip per 256 groups.  Through a buffer
    // descriptor over the list (entries past its end read as 0): a load under `g < e ? ... : 0` is a branch, and the
    // compiler waits for every such load (vmcnt(0)) where its value meets the 0 of the other path.
    int lo[4], hi[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) hi[u] = __builtin_amdgcn_raw_buffer_load_b32(rs_list, 4u * (unsigned)(g0 + 64 * u + lane), 0, 0);
#pragma unroll
    for (int u = 0; u < 4; ++u) hi[u] = min(max(hi[u], 0), m);
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
  const int wg_cols = 4 * W4_WAVE_COLS * side;          // columns of this workgroup
  const int col_base = blockIdx.x * wg_cols;
  const int col0 = col_base + wave * W4_WAVE_COLS * side + sub;   // this lane's columns: col0 + c * side

  // this wavefront's columns: every piece and its scale requested at once (one memory round trip), nibbles as u ^ 8.
  // Branch-free, through buffer descriptors over this workgroup's columns of the group's weights and scales: what a
  // lane has no use for (a piece past K, a column past N) is asked at an offset beyond the descriptor and reads as 0.
  const int cols_here = min(wg_cols, n - col_base);
  const __amdgpu_buffer_rsrc_t rs_w = buffer_over(wg + (long long)col_base * (k / 2), (long long)cols_here * (k / 2));
  const __amdgpu_buffer_rsrc_t rs_s = buffer_over(sg + col_base, 4ll * ((long long)(k_groups - 1) * n + cols_here));
  // (Staging the scales through LDS with coalesced requests measured slower, 12.4 against 11.4 us: the per-lane form
  // below repeats cache lines, but it needs no barrier between the scales and the first dot product.)
  uint4 wv[W4_WAVE_COLS][W4_LANE_PIECES];
  float sc[W4_WAVE_COLS][W4_LANE_PIECES];
#pragma unroll
  for (int c = 0; c < W4_WAVE_COLS; ++c)
#pragma unroll
    for (int i = 0; i < W4_LANE_PIECES; ++i) {
      const int p = pl + lanes_per_col * i, cl = col0 + c * side - col_base;   // column inside the workgroup
      const bool live = p < pieces && cl < cols_here;
      const v4i raw = __builtin_amdgcn_raw_buffer_load_b128(rs_w, live ? (unsigned)(cl * (k / 2) + p * 16) : 0xFFFFFFF0u, 0, 0);
      wv[c][i] = make_uint4((unsigned)raw[0], (unsigned)raw[1], (unsigned)raw[2], (unsigned)raw[3]);
      sc[c][i] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(
          rs_s, live ? 4u * (unsigned)((p / pieces_per_group) * n + cl) : 0xFFFFFFFCu, 0, 0));
    }

  // A block of up to W4_ROWS rows of the group is rows * k consecutive bytes of x: thread t holds the 16-byte pieces
  // t, t + 256, ... of them (requested through a descriptor over just these bytes, so nothing branches), together with
  // the rows' activation scales.  The first block is requested right behind the weights -- loads return in order, so
  // it costs no round trip of its own -- and before anything waits for the weights.
  constexpr int W4_X_VECS = W4_ROWS * (W4_MAX_K / 16) / 256;   // 16-byte pieces of a block per thread
  uint4 xr[W4_X_VECS];
  float xsr[W4_ROWS];
  const __amdgpu_buffer_rsrc_t rs_xs = buffer_over(x_scale, 4ll * m);
  auto request_rows = [&](int r0, int rows) {
    const __amdgpu_buffer_rsrc_t rs_x = buffer_over(x + (long long)r0 * k, (long long)rows * k);
#pragma unroll
    for (int u = 0; u < W4_X_VECS; ++u) {
      const v4i raw = __builtin_amdgcn_raw_buffer_load_b128(rs_x, 16u * (unsigned)(threadIdx.x + 256 * u), 0, 0);
      xr[u] = make_uint4((unsigned)raw[0], (unsigned)raw[1], (unsigned)raw[2], (unsigned)raw[3]);
    }
#pragma unroll
    for (int r = 0; r < W4_ROWS; ++r)
      xsr[r] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rs_xs, r < rows ? 4u * (unsigned)(r0 + r) : 0xFFFFFFFCu, 0, 0));
  };
  request_rows(g_start, min(W4_ROWS, g_end - g_start));

  for (int r0 = g_start; r0 < g_end; r0 += W4_ROWS) {
    const int rows = min(W4_ROWS, g_end - r0);
    if (r0 != g_start) request_rows(r0, rows);
    __syncthreads();   // the previous block of rows is no longer read
#pragma unroll
    for (int u = 0; u < W4_X_VECS; ++u) {
      // 16 bytes (k0 .. k15 of a half piece) -> two words of even-k bytes and two of odd-k bytes
      const int idx = threadIdx.x + 256 * u;
      if (idx < rows * pieces * 2) {
        const uint4 v = xr[u];
        const int r = idx / (pieces * 2), h = idx - r * pieces * 2;
        const unsigned e0 = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u), o0 = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);
        const unsigned e1 = __builtin_amdgcn_perm(v.w, v.z, 0x06040200u), o1 = __builtin_amdgcn_perm(v.w, v.z, 0x07050301u);
        int *dst = xs + (r * pieces + (h >> 1)) * 8 + (h & 1) * 2;
        dst[0] = (int)e0; dst[1] = (int)e1; dst[4] = (int)o0; dst[5] = (int)o1;
      }
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
      float xs_r = xsr[0];   // (selected, not indexed: the array stays in registers)
#pragma unroll
      for (int q = 1; q < W4_ROWS; ++q) xs_r = r == q ? xsr[q] : xs_r;
#pragma unroll
      for (int c = 0; c < W4_WAVE_COLS; ++c) {
        float v = acc[c];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
          if (o < lanes_per_col) v += __shfl_xor(v, o);   // wave-uniform
        if (pl == 0 && col0 + c * side < n) out[(long long)(r0 + r) * n + col0 + c * side] = f32_to_f16_rne(v * xs_r);
      }
    }
  }
}

// 4-bit values widened to int8: 16 source bytes (32 nibbles) -> 32 bytes per thread, low nibble first, sign extended
__global__ void __launch_bounds__(256) unpack_int4_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, long long pieces,
                                                          const unsigned char *src_tail, signed char *dst_tail, int tail_bytes) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  auto widen = [](unsigned w, unsigned &lo, unsigned &hi) {
    // bytes b0 b1 b2 b3 of w -> lo = {b0.lo, b0.hi, b1.lo, b1.hi}, hi = {b2.lo, b2.hi, b3.lo, b3.hi}, each nibble sign extended
    const unsigned even = w & 0x0F0F0F0Fu, odd = (w >> 4) & 0x0F0F0F0Fu;
    const unsigned l = __builtin_amdgcn_perm(odd, even, 0x05010400u);   // e0 o0 e1 o1
    const unsigned h = __builtin_amdgcn_perm(odd, even, 0x07030602u);   // e2 o2 e3 o3
    // sign extension of a 4-bit value held in a byte: (v ^ 8) - 8, per byte without carries between bytes
    lo = ((l ^ 0x08080808u) | 0x80808080u) - 0x08080808u;
    lo ^= 0x80808080u;
    hi = ((h ^ 0x08080808u) | 0x80808080u) - 0x08080808u;
    hi ^= 0x80808080u;
  };
  if (i < pieces) {
    const uint4 v = src[i];
    uint4 a, b;
    widen(v.x, a.x, a.y); widen(v.y, a.z, a.w); widen(v.z, b.x, b.y); widen(v.w, b.z, b.w);
    dst[2 * i] = a;
    dst[2 * i + 1] = b;
  }
  if (i < tail_bytes) {   // the last bytes of a source whose size is not a multiple of 16
    const unsigned char t = src_tail[i];
    const int lo = t & 15, hi = t >> 4;
    dst_tail[2 * i] = (signed char)(lo >= 8 ? lo - 16 : lo);
    dst_tail[2 * i + 1] = (signed char)(hi >= 8 ? hi - 16 : hi);
  }
}

}  // namespace
}  // namespace msco

extern "C" int msco_unpack_int4(const void *src, void *dst, int64_t src_bytes, void *stream) {
  using namespace msco;
  if (src_bytes < 0) return MSCO_ERR_SHAPE;
  if (src_bytes == 0) return MSCO_OK;
  if (src == nullptr || dst == nullptr) return MSCO_ERR_INVALID_ARG;
  if ((reinterpret_cast<uintptr_t>(src) & 15) != 0 || (reinterpret_cast<uintptr_t>(dst) & 15) != 0) return MSCO_ERR_INVALID_ARG;
  const long long pieces = src_bytes / 16;
  const int tail = (int)(src_bytes % 16);
  const long long threads = pieces > tail ? pieces : tail;
  if ((threads + 255) / 256 > 0x7FFFFFFFll) return MSCO_ERR_SHAPE;
  const unsigned char *s8 = static_cast<const unsigned char *>(src);
  hipLaunchKernelGGL(unpack_int4_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), pieces, s8 + pieces * 16,
                     static_cast<signed char *>(dst) + pieces * 32, tail);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

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
