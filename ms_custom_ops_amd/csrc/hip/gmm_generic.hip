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

template <bool NK>
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
  const int8_t *w = p.w + (long long)g * p.k * p.n;
  int acc = 0;
  if (NK) {
    const int8_t *wr = w + (long long)n * p.k;
    for (int k = 0; k < p.k; ++k) acc += (int)x[k] * (int)wr[k];
  } else {
    for (int k = 0; k < p.k; ++k) acc += (int)x[k] * (int)w[(long long)k * p.n + n];
  }
  acc += load_bias(p, g, n);
  const float f = dequant(acc, load_scale(p, g, n), p.per_token ? p.per_token[m] : 1.0f);
  store_out(p, idx, acc, f);
}

__device__ __forceinline__ float load_half_like(const void *ptr, long long i, int dtype) {
  const unsigned short b = reinterpret_cast<const unsigned short *>(ptr)[i];
  return dtype == DT_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}

// out[m,n] = s[g,n] * (sum_k x[m,k] * w[g,k,n] + o[g,n] * sum_k x[m,k]), float32 accumulation.
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
  const int8_t *w = p.w + (long long)g * p.k * p.n;
  float acc = 0.0f, xsum = 0.0f;
  for (int k = 0; k < p.k; ++k) {
    const float xv = load_half_like(p.x, (long long)m * p.k + k, p.x_dtype);
    acc = fmaf(xv, (float)w[(long long)k * p.n + n], acc);
    xsum += xv;
  }
  const float s = p.aq_scale ? load_half_like(p.aq_scale, (long long)g * p.n + n, p.x_dtype) : 1.0f;
  const float o = p.aq_offset ? load_half_like(p.aq_offset, (long long)g * p.n + n, p.x_dtype) : 0.0f;
  const float f = (acc + o * xsum) * s;
  out[idx] = (p.out_dtype == DT_BF16) ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
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

hipError_t launch_generic_w8a8(const GmmParams &p, bool nk, hipStream_t stream) {
  const long long total = (long long)p.m * p.n;
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (nk) {
    hipLaunchKernelGGL(gmm_w8a8_generic_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL(gmm_w8a8_generic_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_generic_a16w8(const GmmParams &p, hipStream_t stream) {
  const long long total = (long long)p.m * p.n;
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(gmm_a16w8_generic_kernel, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace msco
