// Measurement aid: what the matrix pipe of this chip sustains on a given operand distribution with no memory traffic.
// 256 workgroups (one per compute unit) of four wavefronts (one per SIMD) each run `iters` rounds of the 16
// v_mfma_i32_32x32x32_i8 of a 128 x 128 wave tile (four weight fragments x four activation fragments, the order the
// persistent tile kernel issues them in) on operand fragments read once from `operands` (8 fragments of 16 bytes per
// thread: 32 KiB that every workgroup reads alike).  The clock the chip sustains depends on what the operands are:
// uniformly random int8 toggles far more logic than zeros, so the same loop runs at different rates.  The benchmark
// times it with events; nothing here enters the operators.
#include "gmm_common.h"
#include "msco_gmm.h"

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

}  // namespace
}  // namespace msco

extern "C" int msco_probe_mfma(const void *operands, void *sink, int32_t iters, void *stream) {
  if (operands == nullptr || sink == nullptr || iters < 0) return MSCO_ERR_INVALID_ARG;
  hipLaunchKernelGGL(msco::probe_mfma_kernel, dim3(MSCO_PROBE_MFMA_WORKGROUPS), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const msco::v4i *>(operands), static_cast<int *>(sink), iters);
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}
