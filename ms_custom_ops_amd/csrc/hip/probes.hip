// Measurement aids, built into a library of their own (nothing here enters the operators).
//
// 1. What the matrix pipe sustains, and what a wavefront that is alone on its SIMD can issue between MFMAs.  256
// workgroups (one per compute unit) of four wavefronts (one per SIMD) run rounds of 64 v_mfma_i32_16x16x64_i8 (or 32
// v_mfma_i32_32x32x32_i8: the same multiply-adds) on operand fragments read once from `operands` (8 fragments of 16 bytes
// per thread: 32 KiB that every workgroup reads alike).  Pattern 0 (12) is the bare loop: the clock the chip sustains
// depends on what the operands are -- uniformly random int8 toggles far more logic than zeros -- and on the
// instruction shape.  The other patterns weave memory operations in at fixed places -- LDS fragment reads, LDS writes of
// 16, 8 or 4 bytes per lane, 16-byte buffer loads -- in the proportions of the persistent tile kernels' K loop (per 64
// MFMAs: 16 reads, 8 x 16 bytes written, 8 loads); nothing ever waits for a result, so a round's duration in core
// clocks is what issuing that pattern costs.  Everything is assembly: the order is the one written here.
//
// 2. What one launch that does nothing but read a buffer front to back costs: the floor under every decode kernel of
// the same weight size.  Each workgroup reads one contiguous share of the buffer, its four wavefronts taking
// neighbouring 1 KiB pieces (16 bytes per lane), eight loads in flight per wavefront, non-temporal loads: the access
// pattern of the packed-layout decode kernels.
#include "gmm_common.h"
#include "msco_probes.h"

#include <type_traits>

namespace msco {
namespace {

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

// MF: 0 16 x 16 x 64 (64 per round), 1 32 x 32 x 32 (32 per round, behind every second slot).  Per round of 64 slots: RD
// ds_read_b128 in the slots n % (64 / RD) == 1; WR LDS writes of WB bytes per lane in the slots n % (64 / WR) == WP; LD
// buffer loads in the slots n % (64 / LD) == LP.
constexpr int kIssueRoundsPerPass = 8;
template <int MF, int RD, int WB, int WR, int WP, int LD, int LP>
__global__ void __launch_bounds__(256, 1) probe_issue_kernel(const v4i *operands, int *sink, int iters, long long *clocks) {
  __shared__ __align__(16) unsigned char lds[65536];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v4i wf[8], xf[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    wf[j] = operands[threadIdx.x + 256 * (j % 4)];
    xf[j] = operands[threadIdx.x + 256 * (4 + j % 4)];
  }
  for (int j = threadIdx.x; j < 65536 / 4; j += 256) reinterpret_cast<int *>(lds)[j] = 0;
  __syncthreads();
  // (from here on the compiler must not count outstanding loads: its own waits would stall the loop)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    asm volatile("" : "+v"(wf[j]));
    asm volatile("" : "+v"(xf[j]));
  }
  constexpr int NB = MF == 0 ? 8 : 4;
  typename std::conditional<MF == 0, v4i, v16i>::type acc[NB][NB];
#pragma unroll
  for (int f = 0; f < NB; ++f)
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int r = 0; r < (MF == 0 ? 4 : 16); ++r) acc[f][i][r] = 0;
  const unsigned laddr = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)lds + wave * 1024 + lane * 16;
  const unsigned goff = threadIdx.x * 16;
  const __amdgpu_buffer_rsrc_t rsrc = buffer_over(operands, MSCO_PROBE_MFMA_OPERAND_BYTES);
  v4i r0 = wf[0], r1 = wf[1], r2 = xf[0], r3 = xf[1];
  const v4i w16 = wf[2];
  typedef int v2i_t __attribute__((ext_vector_type(2)));
  const v2i_t w8 = v2i_t{wf[3].x, wf[3].y};
  const int w4 = wf[3].z;
  const int passes = iters / kIssueRoundsPerPass;
  int last = passes - 1;   // (laundered: known to be the last pass, it would be peeled off and the copies move with it)
  asm volatile("" : "+s"(last));
  const long long c0 = __builtin_readcyclecounter(), t0 = wall_clock64();
  for (int it = 0; it < passes; ++it) {
#pragma unroll
    for (int slot = 0; slot < 64 * kIssueRoundsPerPass; ++slot) {
      const int n = slot % 64;
      if constexpr (MF == 1) {
        if (n % 2 == 0)
          asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(acc[(n / 8) % 4][(n / 2) % 4]) : "v"(wf[(n / 8) % 4]), "v"(xf[(n / 2) % 4]));
      } else {
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc[n / 8][n % 8]) : "v"(wf[n / 8]), "v"(xf[n % 8]));
      }
      if (RD > 0 && n % (64 / (RD > 0 ? RD : 1)) == 1) {
        if (n % 4 == 1) asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(r0) : "v"(laddr));
        else asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(r1) : "v"(laddr));
      }
      if (WR > 0 && n % (64 / (WR > 0 ? WR : 1)) == WP) {
        if (WB == 16) asm volatile("ds_write_b128 %0, %1 offset:32768" ::"v"(laddr), "v"(w16));
        if (WB == 8) asm volatile("ds_write_b64 %0, %1 offset:32768" ::"v"(laddr), "v"(w8));
        if (WB == 4) asm volatile("ds_write_b32 %0, %1 offset:32768" ::"v"(laddr), "v"(w4));
      }
      if (LD > 0 && n % (64 / (LD > 0 ? LD : 1)) == LP) {
        if (n % 16 < 8) asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(r2) : "v"(goff), "s"(rsrc));
        else asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(r3) : "v"(goff), "s"(rsrc));
      }
    }
    // (the compiler does not know that the statements above are MFMAs and copies accumulators right behind the loop: the
    // wait states between the last MFMA and the first read of its result stand here, inside the last pass; the test
    // costs 48 clocks of issue, hence several rounds per pass)
    if (it == last) asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15");
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  const long long c1 = __builtin_readcyclecounter(), t1 = wall_clock64();
  asm volatile("" ::"v"(r0), "v"(r1), "v"(r2), "v"(r3));   // (what the woven-in loads brought is of no interest)
  int s = 0;
#pragma unroll
  for (int f = 0; f < NB; ++f)
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int r = 0; r < (MF == 0 ? 4 : 16); ++r) s += acc[f][i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;   // keeps the loop alive
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = c1 - c0;   // core clocks
    clocks[1] = t1 - t0;   // 100 MHz ticks
  }
}

}  // namespace
}  // namespace msco

extern "C" int msco_probe_mfma_issue(const void *operands, void *sink, void *clocks, int32_t pattern, int32_t iters, void *stream) {
  if (operands == nullptr || sink == nullptr || clocks == nullptr || iters < 0 || iters % msco::kIssueRoundsPerPass != 0) return MSCO_ERR_INVALID_ARG;
  const auto st = static_cast<hipStream_t>(stream);
  const auto *ops = static_cast<const msco::v4i *>(operands);
  int *snk = static_cast<int *>(sink);
  long long *clk = static_cast<long long *>(clocks);
#define MSCO_ISSUE(MF, RD, WB, WR, WP, LD, LP)                                                                                     \
  hipLaunchKernelGGL((msco::probe_issue_kernel<MF, RD, WB, WR, WP, LD, LP>), dim3(MSCO_PROBE_MFMA_WORKGROUPS), dim3(256), 0, st, ops, snk, \
                     iters, clk);                                                                                                  \
  break
  switch (pattern) {   // (the table of include/msco_probes.h)
    case 0: MSCO_ISSUE(0, 0, 0, 0, 0, 0, 0);
    case 1: MSCO_ISSUE(0, 16, 0, 0, 0, 0, 0);
    case 2: MSCO_ISSUE(0, 16, 0, 0, 0, 8, 3);
    case 3: MSCO_ISSUE(0, 0, 16, 8, 0, 0, 0);
    case 4: MSCO_ISSUE(0, 0, 8, 16, 0, 0, 0);
    case 5: MSCO_ISSUE(0, 0, 4, 32, 0, 0, 0);
    case 6: MSCO_ISSUE(0, 16, 16, 8, 0, 8, 3);
    case 7: MSCO_ISSUE(0, 16, 16, 8, 2, 8, 3);
    case 8: MSCO_ISSUE(0, 16, 8, 16, 0, 8, 3);
    case 9: MSCO_ISSUE(0, 16, 8, 16, 1, 8, 3);
    case 10: MSCO_ISSUE(0, 16, 8, 16, 0, 8, 0);
    case 11: MSCO_ISSUE(0, 16, 4, 32, 0, 8, 3);
    case 12: MSCO_ISSUE(1, 0, 0, 0, 0, 0, 0);
    case 13: MSCO_ISSUE(1, 16, 16, 8, 0, 8, 3);
    case 14: MSCO_ISSUE(1, 16, 8, 16, 2, 8, 3);
    default: return MSCO_ERR_INVALID_ARG;
  }
#undef MSCO_ISSUE
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

extern "C" int msco_probe_read(const void *src, size_t bytes, void *sink, int32_t workgroups, void *stream) {
  if (src == nullptr || sink == nullptr || workgroups <= 0 || workgroups > 65535) return MSCO_ERR_INVALID_ARG;
  if (bytes / (size_t)workgroups >= ((size_t)1 << 31)) return MSCO_ERR_SHAPE;   // a share is addressed with 32-bit offsets
  hipLaunchKernelGGL(msco::probe_read_kernel, dim3((unsigned)workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const unsigned char *>(src), (long long)bytes, static_cast<int *>(sink));
  return hipGetLastError() == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}
