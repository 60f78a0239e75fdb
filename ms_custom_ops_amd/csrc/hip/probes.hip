// Measurement aids, built into a library of their own (nothing here enters the operators).
//
// 1. What the matrix pipe of this chip sustains on a given operand distribution with no memory traffic.
// 256 workgroups (one per compute unit) of four wavefronts (one per SIMD) each run `iters` rounds of the 16
// v_mfma_i32_32x32x32_i8 of a 128 x 128 wave tile (four weight fragments x four activation fragments, the order the
// persistent tile kernel issues them in) on operand fragments read once from `operands` (8 fragments of 16 bytes per
// thread: 32 KiB that every workgroup reads alike).  The clock the chip sustains depends on what the operands are:
// uniformly random int8 toggles far more logic than zeros, so the same loop runs at different rates.  The benchmark
// times it with events.
//
// 2. What one launch that does nothing but read a buffer front to back costs: the floor under every decode kernel of
// the same weight size.  Each workgroup reads one contiguous share of the buffer, its four wavefronts taking
// neighbouring 1 KiB pieces (16 bytes per lane), eight loads in flight per wavefront, non-temporal loads: the access
// pattern of the packed-layout decode kernels.
#include "gmm_common.h"
#include "msco_probes.h"

namespace msco {
namespace {

__global__ void __launch_bounds__(256, 1) probe_mfma_kernel(const v4i *operands, int *sink, int iters) {
  v4i wf[4], xf[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wf[j] = operands[threadIdx.x + 256 * j];
    xf[j] = operands[threadIdx.x + 256 * (4 + j)];
  }
  v16i acc[4][4];
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[f][i][r] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[f][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[f], xf[i], acc[f][i], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  int s = 0;
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[f][i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;   // keeps the loop alive
}


constexpr int kReadDepth = 8;
__global__ void __launch_bounds__(256) probe_read_kernel(const unsigned char *src, long long bytes, int *sink) {
  // share of this workgroup, in 4 KiB steps (one 1 KiB piece per wavefront)
  const long long steps = bytes / 4096;
  const long long per_wg = (steps + gridDim.x - 1) / gridDim.x;
  const long long first = (long long)blockIdx.x * per_wg;
  const long long last = first + per_wg < steps ? first + per_wg : steps;
  const __amdgpu_buffer_rsrc_t rs = buffer_over(src + first * 4096, (last - first) * 4096);
  const unsigned lane_off = threadIdx.x * 16;   // wave w, lane l: byte 1024 w + 16 l of a step
  const long long n = last - first;
  v4i ring[kReadDepth];
  v4i acc = v4i{0, 0, 0, 0};
#pragma unroll
  for (int d = 0; d < kReadDepth; ++d)
    ring[d] = __builtin_amdgcn_raw_buffer_load_b128(rs, d < n ? lane_off : kBufferOob, d * 4096, kStreamAux);
  for (long long i = 0; i < n; i += kReadDepth) {
#pragma unroll
    for (int d = 0; d < kReadDepth; ++d) {
      acc ^= ring[d];
      const long long nxt = i + kReadDepth + d;
      ring[d] = __builtin_amdgcn_raw_buffer_load_b128(rs, nxt < n ? lane_off : kBufferOob, (int)(nxt * 4096), kStreamAux);
    }
  }
  sink[blockIdx.x * 256 + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

}  // namespace
}  // namespace msco

extern "C" int msco_probe_mfma(const void *operands, void *sink, int32_t iters, void *stream) {
  if (operands == nullptr || sink == nullptr || iters < 0) return MSCO_ERR_INVALID_ARG;
  hipLaunchKernelGGL(msco::probe_mfma_kernel, dim3(MSCO_PROBE_MFMA_WORKGROUPS), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const msco::v4i *>(operands), static_cast<int *>(sink), iters);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

extern "C" int msco_probe_read(const void *src, size_t bytes, void *sink, int32_t workgroups, void *stream) {
  if (src == nullptr || sink == nullptr || workgroups <= 0 || workgroups > 65535) return MSCO_ERR_INVALID_ARG;
  if (bytes / (size_t)workgroups >= ((size_t)1 << 31)) return MSCO_ERR_SHAPE;   // a share is addressed with 32-bit offsets
  hipLaunchKernelGGL(msco::probe_read_kernel, dim3((unsigned)workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const unsigned char *>(src), (long long)bytes, static_cast<int *>(sink));
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}
