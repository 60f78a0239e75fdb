// Shared device-side definitions for the gfx950 grouped quantized matmul kernels.
#ifndef MSCO_GMM_COMMON_H_
#define MSCO_GMM_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include <type_traits>
#include <utility>

namespace msco {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// dtype codes shared with include/msco_gmm.h (msco_dtype)
enum : int { DT_NONE = 0, DT_I8 = 1, DT_I32 = 2, DT_I64 = 3, DT_U64 = 4, DT_F16 = 5, DT_BF16 = 6, DT_F32 = 7 };

constexpr int kNumXcd = 8;        // MI355X: 8 accelerator complex dies, workgroups are dealt round-robin
constexpr int kSkinnyRows = 16;   // rows one MFMA covers in the skinny kernels
constexpr int kSkinnyCols = 256;  // output columns one skinny workgroup owns

// Kernel argument block.  Plain pointers and sizes only.
struct GmmParams {
  const void *x;            // [M,K] int8 or bf16/f16
  const int8_t *w;          // [E,K,N] or [E,N,K]
  const int32_t *bias;      // [E,N] or [N] or null
  const void *scale;        // [E,N] / [N] / [1] in scale_dtype, or null
  const void *group_list;   // [E] int32/int64 or null
  const float *per_token;   // [M] or null
  const void *aq_scale;     // [E,N] bf16/f16 (W8A16)
  const void *aq_offset;    // [E,N] bf16/f16 or null
  void *out;                // [M,N]
  int32_t *partial;         // split-K partial tiles (workspace)
  unsigned *counters;       // split-K arrival counters (handle-owned, self-resetting)
  int m, k, n, e;
  int gl_dtype;             // DT_NONE / DT_I32 / DT_I64
  int gl_type;              // 0 cumulative ends, 1 counts
  int scale_dtype;          // DT_NONE / DT_F32 / DT_BF16 / DT_I64 / DT_U64
  int scale_per_group;      // scale & bias carry a row per group
  int scale_is_scalar;      // scale has a single element
  int out_dtype;            // DT_BF16 / DT_F16 / DT_I32
  int x_dtype;              // DT_I8 / DT_BF16 / DT_F16
  int split_k;              // number of K splits across workgroups (skinny kernels)
  int n_strips;             // ceil(N / kSkinnyCols)
  int max_chunks;           // ceil(M / kSkinnyRows): 16-row chunks a group can have (skinny W8A8 kernel)
  int strip_groups;         // packed-layout kernels: 16-column groups per strip (1..16); n_strips counts these strips
  int act_type;             // ACT_*: activation on the float32 result before the output cast (never with int32 output)
  int x_via_lds;            // packed-layout W8A8 decode kernel: stage the chunk's x rows through LDS (pays from about 8 rows per chunk)
  int wide_k_slabs;         // small tile kernels on K-major weights: 128-byte K slabs (planned when the workgroups run in one round)
  int w_nontemporal;        // small tile kernels on packed weights: non-temporal weight loads (a large weight stream that at most two m-tiles read)
  int rows_lo, rows_hi;     // tile kernels: only groups with rows_lo < rows <= rows_hi are worked on (a launch pair splits the groups by size)
};

// ---- group_list --------------------------------------------------------------------------------
// Row end of group g given the previous end; the result is clamped into [prev, M] so a malformed
// list can never produce an out-of-range row.
__device__ __forceinline__ int group_end(const GmmParams &p, int g, int prev) {
  long long v;
  if (p.gl_dtype == DT_I64) {
    v = reinterpret_cast<const long long *>(p.group_list)[g];
  } else if (p.gl_dtype == DT_I32) {
    v = reinterpret_cast<const int *>(p.group_list)[g];
  } else {
    v = (long long)(p.m / p.e) * (g + 1);  // dense / batched: equal groups
  }
  long long end = (p.gl_type == 1 && p.gl_dtype != DT_NONE) ? (long long)prev + v : v;
  if (end < prev) end = prev;
  if (end > p.m) end = p.m;
  return (int)end;
}

// ---- wave-parallel walk of group_list (tile scheduler) --------------------------------------------
// Row ends of up to 64 groups at once: lane l handles group g0 + l.  The sequential rule of
// group_end() has closed forms, so a wave computes it with prefix scans instead of E dependent loads:
//   cumulative ends: end_g = min(max(carry, v_0..v_g), M)            (prefix maximum)
//   counts:          end_g = min(carry + max(v_0,0) + .. + max(v_g,0), M)   (saturating prefix sum)
__device__ __forceinline__ int wave_scan_max(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int t = __shfl_up(v, d);
    if (lane >= d) v = max(v, t);
  }
  return v;
}
__device__ __forceinline__ int wave_scan_add_sat(int v, int lane, int cap) {   // operands in [0, cap], cap < 2^30
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int t = __shfl_up(v, d);
    if (lane >= d) v = min(v + t, cap);
  }
  return v;
}
__device__ __forceinline__ int wave_scan_add(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int t = __shfl_up(v, d);
    if (lane >= d) v += t;
  }
  return v;
}
__device__ __forceinline__ int wave_bcast(int v, int src_lane) {
  return __builtin_amdgcn_readfirstlane(__shfl(v, src_lane));
}

// Lane l receives [start, end) of group g0 + l (empty for lanes past E); `carry` is the row end of
// group g0 - 1 on entry and of the chunk's last group on exit.  Requires M < 2^30 for counts.
__device__ __forceinline__ void group_rows_chunk(const GmmParams &p, int g0, int lane, int &carry, int &start, int &end) {
  const int g = g0 + lane;
  const bool valid = g < p.e;
  long long v = 0;
  if (valid) {
    if (p.gl_dtype == DT_I64) v = reinterpret_cast<const long long *>(p.group_list)[g];
    else if (p.gl_dtype == DT_I32) v = reinterpret_cast<const int *>(p.group_list)[g];
    else v = (long long)(p.m / p.e) * (g + 1);
  }
  const int c = (int)(v < 0 ? 0 : (v > p.m ? p.m : v));   // clamping the operands first changes neither closed form
  int e_l;
  if (p.gl_type == 1 && p.gl_dtype != DT_NONE) e_l = min(carry + wave_scan_add_sat(valid ? c : 0, lane, p.m), p.m);
  else e_l = max(carry, wave_scan_max(valid ? c : 0, lane));
  const int prev = __shfl_up(e_l, 1);
  start = lane == 0 ? carry : prev;
  end = e_l;
  carry = wave_bcast(e_l, 63);
}

// [start, end) of group `grp`, wave-uniform, by the wave-parallel walk above: one round of loads per 64 groups instead
// of grp + 1 dependent ones.  Every lane of the wave must call it (the scans use cross-lane moves).
__device__ __forceinline__ void group_range(const GmmParams &p, int grp, int lane, int &g_start, int &g_end) {
  int carry = 0, start = 0, end = 0;
  int g0 = 0;
  for (;; g0 += 64) {
    group_rows_chunk(p, g0, lane, carry, start, end);
    if (grp < g0 + 64) break;
  }
  g_start = wave_bcast(start, grp - g0);
  g_end = wave_bcast(end, grp - g0);
}

// Dispatch slot -> (group, chunk of rows_per_chunk rows) for the decode kernels: the grid's y extent enumerates only the
// chunks that hold rows, group after group, so that many experts with few rows cost no empty workgroups.  Returns false
// for a slot past the last chunk.  The number of chunks is at most min(E, M) + M / rows_per_chunk for any group_list
// (every group with rows has at most one partial chunk), which is what the launchers size grid.y by.  Every lane of the
// wave must call it; grp, mc and the row range come back wave-uniform.
__device__ __forceinline__ bool chunk_of_slot(const GmmParams &p, int slot, int rows_per_chunk, int lane, int &grp, int &mc,
                                              int &g_start, int &g_end) {
  int carry = 0, seen = 0;
  for (int g0 = 0; g0 < p.e; g0 += 64) {
    int s0, e0;
    group_rows_chunk(p, g0, lane, carry, s0, e0);
    const int chunks = (e0 - s0 + rows_per_chunk - 1) / rows_per_chunk;   // 0 for empty groups and for lanes past E
    const int upto = seen + wave_scan_add(chunks, lane);                  // chunks up to and including this lane's group
    const unsigned long long beyond = __ballot(upto > slot);               // `upto` is non-decreasing
    if (beyond != 0) {
      const int first = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(beyond));
      grp = g0 + first;
      mc = slot - (wave_bcast(upto, first) - wave_bcast(chunks, first));
      g_start = wave_bcast(s0, first);
      g_end = wave_bcast(e0, first);
      return true;
    }
    seen = wave_bcast(upto, 63);
  }
  return false;
}

// ---- number formats ----------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short b) { return __uint_as_float((unsigned)b << 16); }

// float32 -> bfloat16, round to nearest even (NaN stays quiet NaN).
__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (unsigned short)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}

// Two float32 -> packed bfloat16 (lo in bits 0..15) with the hardware's round-to-nearest-even
// conversion (v_cvt_pk_bf16_f32).
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  const v2f v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, v2bf));
}

__device__ __forceinline__ unsigned short f32_to_f16_rne(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32, IEEE round to nearest even
  return __builtin_bit_cast(unsigned short, h);
}

__device__ __forceinline__ float f16_bits_to_f32(unsigned short b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

// Dequant scale of column n for group g.  int64/uint64 scales carry float32 bits in the low word.
__device__ __forceinline__ float load_scale(const GmmParams &p, int g, int n) {
  if (p.scale_dtype == DT_NONE) return 1.0f;
  long long idx = p.scale_is_scalar ? 0 : ((p.scale_per_group ? (long long)g * p.n : 0) + n);
  if (p.scale_dtype == DT_F32) return reinterpret_cast<const float *>(p.scale)[idx];
  if (p.scale_dtype == DT_BF16) return bf16_bits_to_f32(reinterpret_cast<const unsigned short *>(p.scale)[idx]);
  return __uint_as_float(reinterpret_cast<const unsigned *>(p.scale)[2 * idx]);
}

__device__ __forceinline__ int load_bias(const GmmParams &p, int g, int n) {
  if (p.bias == nullptr) return 0;
  return p.bias[(p.scale_per_group ? (long long)g * p.n : 0) + n];
}

// Epilogue of one element in the reference golden's operation order:
// float32(acc + bias) * scale[n] * per_token[m], each product rounded to float32.
__device__ __forceinline__ float dequant(int acc_plus_bias, float scale, float per_token) {
  float f = (float)acc_plus_bias;
  f = f * scale;
  f = f * per_token;
  return f;
}

// Activation on the dequantised value (msco_act in include/msco_gmm.h).  The three smooth ones are v * sigmoid(t(v));
// written as v / (1 + exp(-t)) there is no cancellation anywhere on the real line (exp(-t) = inf gives -0 for very
// negative v, where the true value underflows).  Fast exponential and reciprocal: a few float32 ulps, far below the
// rounding of the 16-bit output.
enum : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU_TANH = 2, ACT_GELU_ERF = 3, ACT_FAST_GELU = 4, ACT_SILU = 5 };
__device__ __forceinline__ float activate(float v, int act) {
  if (act == ACT_RELU) return v < 0.0f ? 0.0f : v;
  float t = v;
  if (act == ACT_FAST_GELU) t = 1.702f * v;
  if (act == ACT_GELU_TANH) t = 1.5957691216057308f * (v + 0.044715f * v * v * v);
  return __fdividef(v, 1.0f + __expf(-t));
}

// float32 result -> 16-bit output pattern (bf16 or f16 as the plan says), activation first
__device__ __forceinline__ unsigned short half_out(const GmmParams &p, float f) {
  if (p.act_type != ACT_NONE) f = activate(f, p.act_type);
  return p.out_dtype == DT_BF16 ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
}

__device__ __forceinline__ void store_out(const GmmParams &p, long long idx, int acc_plus_bias, float f) {
  if (p.act_type != ACT_NONE) f = activate(f, p.act_type);
  if (p.out_dtype == DT_BF16) {
    reinterpret_cast<unsigned short *>(p.out)[idx] = f32_to_bf16_rne(f);
  } else if (p.out_dtype == DT_F16) {
    reinterpret_cast<unsigned short *>(p.out)[idx] = f32_to_f16_rne(f);
  } else {
    reinterpret_cast<int *>(p.out)[idx] = acc_plus_bias;
  }
}

// ---- buffer descriptors ---------------------------------------------------------------------------
// Raw buffer over [base, base + bytes): loads whose *vector* offset is at or beyond `bytes` return 0
// (the scalar offset is not range-checked), so tails are masked by setting bit 31 of the vector offset.
constexpr unsigned kBufferOob = 0x80000000u;
// Cache policy of buffer loads that stream data which is read once (decode weights): the non-temporal bit.  Measured
// on MI355X: a 470 MB weight stream runs at 6.7 TB/s with it and 5.7 TB/s without.  Only for loads whose instruction
// covers whole 128-byte lines: the [N,K] decode walk (64-byte pieces per instruction) gets slower with it.
#ifndef MSCO_STREAM_AUX
#define MSCO_STREAM_AUX 2
#endif
constexpr int kStreamAux = MSCO_STREAM_AUX;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_over(const void *base, long long bytes) {
  const unsigned n = bytes > 0x7FFFFFFFll ? 0x7FFFFFFFu : (unsigned)(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

// ---- split-K hand-off ------------------------------------------------------------------------------
// Called by every thread of a workgroup after it has written its share of a partial tile with agent-scope stores
// and before one thread bumps the tile's arrival counter.  A workgroup-scope release fence does not wait for the
// outstanding vector stores of the other wavefronts, so every wavefront drains its own stores (vmcnt == 0: each
// store has been acknowledged at the scope its cache bits name) before it enters the barrier; the thread that
// bumps the counter behind the barrier therefore does so after all the workgroup's partials are visible to the agent.
__device__ __forceinline__ void publish_partials_and_sync() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
}

// ---- byte shuffles -----------------------------------------------------------------------------
// v_perm_b32: result byte i = byte sel[i] of the 8-byte value {hi:lo} (0..3 -> lo, 4..7 -> hi).
__device__ __forceinline__ unsigned perm(unsigned hi, unsigned lo, unsigned sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// 4x4 byte transpose: r[i] holds 4 column bytes of row i; c[j] receives the 4 row bytes of column j.
__device__ __forceinline__ void transpose4x4(unsigned r0, unsigned r1, unsigned r2, unsigned r3, unsigned &c0,
                                             unsigned &c1, unsigned &c2, unsigned &c3) {
  const unsigned lo01 = perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
  const unsigned hi01 = perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
  const unsigned lo23 = perm(r3, r2, 0x05010400u);
  const unsigned hi23 = perm(r3, r2, 0x07030602u);
  c0 = perm(lo23, lo01, 0x05040100u);
  c1 = perm(lo23, lo01, 0x07060302u);
  c2 = perm(hi23, hi01, 0x05040100u);
  c3 = perm(hi23, hi01, 0x07060302u);
}

// f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N - 1>), in order
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

}  // namespace msco
#endif  // MSCO_GMM_COMMON_H_
