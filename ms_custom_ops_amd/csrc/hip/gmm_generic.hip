// Shape-agnostic fallback kernels: one output element per thread, any K and N.
// They exist so that shapes outside the MFMA kernels' alignment rules (K % 16, N % 16) still run on
// the device; they are also the on-device cross-check used by the tests for the fast kernels.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

// Locate the group of row m by walking group_list.  Returns -1 when m lies past the last boundary.
__device__ __forceinline__ int group_of_row(const GmmParams &p, int m) {
  int prev = 0;
  for (int g = 0; g < p.e; ++g) {
    const int end = group_end(p, g, prev);
    if (m < end) return g;
    prev = end;
  }
  return -1;
}

// byte offset of w[k][n] inside one group's weights; LAYOUT 0 [K,N], 1 [N,K], 2 packed (1 KiB blocks of 16 columns x
// 64 K bytes: byte 16 l + i of block (n / 16, k / 64) holds k % 64 = 16 (l / 16) + i, n % 16 = l % 16)
template <int LAYOUT>
__device__ __forceinline__ long long weight_offset(const GmmParams &p, int k, int n) {
  if (LAYOUT == 0) return (long long)k * p.n + n;
  if (LAYOUT == 1) return (long long)n * p.k + k;
  const long long k_blocks = (p.k + 63) / 64;
  const int kk = k & 63;
  return ((long long)(n >> 4) * k_blocks + (k >> 6)) * 1024 + ((kk >> 4) * 16 + (n & 15)) * 16 + (kk & 15);
}
template <int LAYOUT>
__device__ __forceinline__ long long weight_group_bytes(const GmmParams &p) {
  if (LAYOUT == 2) return (long long)((p.n + 15) / 16) * ((p.k + 63) / 64) * 1024;
  return (long long)p.k * p.n;
}

template <int LAYOUT>
__global__ void __launch_bounds__(256) gmm_w8a8_generic_kernel(const GmmParams p) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)p.m * p.n) return;
  const int m = (int)(idx / p.n), n = (int)(idx % p.n);
  const int g = group_of_row(p, m);
  if (g < 0) {  // rows past the last boundary are defined as zero
    store_out(p, idx, 0, 0.0f);
    return;
  }
  const int8_t *x = reinterpret_cast<const int8_t *>(p.x) + (long long)m * p.k;
  const int8_t *w = p.w + (long long)g * weight_group_bytes<LAYOUT>(p);
  int acc = 0;
  for (int k = 0; k < p.k; ++k) acc += (int)x[k] * (int)w[weight_offset<LAYOUT>(p, k, n)];
  acc += load_bias(p, g, n);
  const float f = dequant(acc, load_scale(p, g, n), p.per_token ? p.per_token[m] : 1.0f);
  store_out(p, idx, acc, f);
}

__device__ __forceinline__ float load_half_like(const void *ptr, long long i, int dtype) {
  const unsigned short b = reinterpret_cast<const unsigned short *>(ptr)[i];
  return dtype == DT_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}

// out[m,n] = s[g,n] * (sum_k x[m,k] * w[g,k,n] + o[g,n] * sum_k x[m,k]), float32 accumulation.
template <int LAYOUT>
__global__ void __launch_bounds__(256) gmm_a16w8_generic_kernel(const GmmParams p) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)p.m * p.n) return;
  const int m = (int)(idx / p.n), n = (int)(idx % p.n);
  const int g = group_of_row(p, m);
  unsigned short *out = reinterpret_cast<unsigned short *>(p.out);
  if (g < 0) {
    out[idx] = 0;
    return;
  }
  const int8_t *w = p.w + (long long)g * weight_group_bytes<LAYOUT>(p);
  float acc = 0.0f, xsum = 0.0f;
  for (int k = 0; k < p.k; ++k) {
    const float xv = load_half_like(p.x, (long long)m * p.k + k, p.x_dtype);
    acc = fmaf(xv, (float)w[weight_offset<LAYOUT>(p, k, n)], acc);
    xsum += xv;
  }
  const float s = p.aq_scale ? load_half_like(p.aq_scale, (long long)g * p.n + n, p.x_dtype) : 1.0f;
  const float o = p.aq_offset ? load_half_like(p.aq_offset, (long long)g * p.n + n, p.x_dtype) : 0.0f;
  const float f = (acc + o * xsum) * s;
  out[idx] = half_out(p, f);
}

// Batched 2-D transpose through a padded LDS tile: src [batch, rows, cols] -> dst [batch, cols, rows].
template <typename T>
__global__ void __launch_bounds__(256) transpose_2d_kernel(const T *src, T *dst, long long rows, long long cols) {
  __shared__ T tile[32][33];
  const long long b = blockIdx.z;
  const T *s = src + b * rows * cols;
  T *d = dst + b * rows * cols;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const long long c0 = (long long)blockIdx.x * 32, r0 = (long long)blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8) {
    if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = s[(r0 + i) * cols + c0 + tx];
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    if (c0 + i < cols && r0 + tx < rows) d[(c0 + i) * rows + r0 + tx] = tile[tx][i];
  }
}

hipError_t launch_transpose_2d(const void *src, void *dst, long long batch, long long rows, long long cols,
                               int elem_bytes, hipStream_t stream) {
  if (batch == 0 || rows == 0 || cols == 0) return hipSuccess;
  const dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32), (unsigned)batch);
  if (elem_bytes == 1) {
    hipLaunchKernelGGL(transpose_2d_kernel<unsigned char>, grid, dim3(256), 0, stream,
                       static_cast<const unsigned char *>(src), static_cast<unsigned char *>(dst), rows, cols);
  } else if (elem_bytes == 2) {
    hipLaunchKernelGGL(transpose_2d_kernel<unsigned short>, grid, dim3(256), 0, stream,
                       static_cast<const unsigned short *>(src), static_cast<unsigned short *>(dst), rows, cols);
  } else if (elem_bytes == 4) {
    hipLaunchKernelGGL(transpose_2d_kernel<unsigned>, grid, dim3(256), 0, stream, static_cast<const unsigned *>(src),
                       static_cast<unsigned *>(dst), rows, cols);
  } else {
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_generic_w8a8(const GmmParams &p, int layout, hipStream_t stream) {
  const long long total = (long long)p.m * p.n;
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (layout == 2) {
    hipLaunchKernelGGL(gmm_w8a8_generic_kernel<2>, dim3(grid), dim3(256), 0, stream, p);
  } else if (layout == 1) {
    hipLaunchKernelGGL(gmm_w8a8_generic_kernel<1>, dim3(grid), dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_w8a8_generic_kernel<0>, dim3(grid), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_generic_a16w8(const GmmParams &p, int layout, hipStream_t stream) {
  const long long total = (long long)p.m * p.n;
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (layout == 2) {
    hipLaunchKernelGGL(gmm_a16w8_generic_kernel<2>, dim3(grid), dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_a16w8_generic_kernel<0>, dim3(grid), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace msco
