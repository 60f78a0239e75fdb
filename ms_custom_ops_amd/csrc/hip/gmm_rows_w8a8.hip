// Grouped W8A8 on packed weights for groups of a few dozen to a few hundred rows (gfx950): the weights of a group are
// streamed from memory exactly once, straight into MFMA operands, while the group's x rows pass through LDS.
//
// Between decode (x fits in registers, the launch is a weight stream) and prefill (256 x 256 tiles, the launch is MFMA
// work) lies the serving range: a group holds 32 .. 256 rows, its weights are still read once or twice in all, and what
// a launch costs is the weight stream plus whatever the kernel wastes around it.  Square tiles waste twice there: a tile
// of 256 rows multiplies the padding of a 130-row group, and a launch of 1.75 tiles per CU takes two rounds.  This kernel
// keeps the weight stream of the decode kernels and makes the row count a run-time quantity:
//
//   * workgroup (4 waves) = one chunk of at most 16 RBMAX rows of one group x one strip of 256 columns x all of K;
//     wave w owns column groups 4 w .. 4 w + 3 of the strip.  In the packed layout a 1 KiB block IS the second operand of
//     v_mfma_i32_16x16x64_i8 (16 columns x 64 K bytes), so weights go memory -> registers -> MFMA, eight K blocks (32 KiB
//     per wave) in flight, non-temporal, each byte requested by exactly one wave of the launch.
//   * the chunk's x rows come in slabs of 128 K bytes per row through a double-buffered LDS stage (one barrier per
//     slab); every wave reads its first operands from there, one 16 x 64 fragment per four MFMAs.  Rows are 128 bytes
//     apart and the 16-byte pieces of row r sit at piece ^ ((r >> 1) & 7), so that the 16 rows of a fragment read and
//     the two rows of a staging write fall into 16 different bank groups.
//   * the K loop exists once per number of live 16-row blocks RB (1 .. RBMAX): accumulators are registers and a group of
//     130 rows costs the MFMAs of 144, not of 256.
//   * three forms: chunks of up to 128 rows (accumulators in VGPRs, two workgroups per CU, 4 or 8 K blocks of weights
//     in flight per wave), of up to 160 rows (160 accumulators in VGPRs leave room for two K blocks in flight; the second
//     workgroup of the CU covers the wait) and of up to 256 rows (256 accumulation registers, one wave per SIMD);
//   * epilogue as everywhere: float32(acc + bias) * scale[n] * per_token[m], activation, 16-bit output, staged through
//     LDS 16 rows at a time for whole-row stores.
#include "gmm_common.h"
#include "gmm_kernels.h"

namespace msco {

namespace {
constexpr int XR_WAVES = 4;
constexpr int XR_THREADS = XR_WAVES * 64;
constexpr int XR_COLS = 256;       // columns per strip at most
constexpr int XR_CG = 4;           // column groups per wave
constexpr int XR_SLAB = 128;       // K bytes per row and LDS stage: two blocks of the packed layout
constexpr int XR_AHEAD = 3;        // x fragments requested from LDS ahead of their MFMAs
constexpr int XR_OUT_PITCH = XR_COLS + 4;   // float32 elements per staged output row

template <int RBMAX>
struct XrShape {
  static constexpr int kRows = 16 * RBMAX;
  static constexpr int kStage = kRows * XR_SLAB;   // bytes of one x stage
  static constexpr int kOutStage = 16 * XR_OUT_PITCH * 4;   // bytes of one staged block of 16 output rows (float32)
  static constexpr int kStages = 2 * kStage > 2 * kOutStage ? 2 * kStage : 2 * kOutStage;   // the output staging reuses the x stages
  static constexpr size_t kLds = (size_t)kStages + (size_t)kRows * 4;   // two stages + the chunk's per-token scales
};
}  // namespace

// acc += a x b with the accumulator tied to one block of accumulation registers (256-row chunks: one wave per SIMD,
// 256 accumulation registers).  Left to the register allocator, the accumulator blocks of that form change places
// between the unrolled slabs of the K loop: two to three v_accvgpr_mov / read / write per MFMA (8 experts x 128 / 192 / 256
// rows, K = 4096, N = 14336: 107.6 / 132 / 222 us against 104.2 / 125 / 195 us pinned).  Declared to touch memory, the
// statement also keeps the LDS reads and memory requests around it in the order they are written in.
__device__ __forceinline__ void mfma_pinned(v4i &acc, const v4i &a, const v4i &b) {
  asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b) : "memory");
}

template <int RBMAX, int RB>
__device__ __forceinline__ void rows_run(const GmmParams &p, unsigned char *smem, int grp, int m0, int chunk_rows, int strip) {
  using S = XrShape<RBMAX>;
  // K blocks of weights in flight per wave (a multiple of 4: stages alternate inside a round of DEPTH / 2 slabs): eight
  // while few rows are multiplied and a slab passes in less than a memory round trip, four where the accumulators and
  // the x staging registers leave room for no more
  // (the 160-row form keeps 160 accumulators in VGPRs beside a second workgroup on the CU: two K blocks is all the room
  // left, and the other workgroup's MFMAs are what covers the wait for them)
  constexpr int DEPTH = RBMAX == 10 ? 2 : 2 * RB <= RBMAX ? 8 : 4;
  constexpr int ROUND = DEPTH >= 4 ? DEPTH / 2 : 2;   // steps per trip round the loop (an even number: stages alternate)
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, h = lane >> 4;
  const int col_groups = (p.n + 15) / 16, k_blocks = (p.k + 63) / 64;
  const long long group_bytes = (long long)col_groups * k_blocks * 1024;
  const __amdgpu_buffer_rsrc_t rx = buffer_over(p.x, (long long)p.m * p.k);   // planned only below 2^31
  // a strip holds p.strip_groups column groups (at most 16: the launch picks the width that fills whole rounds of
  // workgroups); wave w owns those of 4 w .. 4 w + 3 that exist
  const int cg0 = strip * p.strip_groups + wave * XR_CG;   // the wave's first column group
  const int n0 = strip * p.strip_groups * 16;
  const int strip_cols = min(p.strip_groups * 16, p.n - n0);
  float *s_pt = reinterpret_cast<float *>(smem + S::kStages);

  // ---- weights: one descriptor per column group of the wave, over exactly that group's K blocks (nothing for a column
  // group past N), so that the range check masks blocks past K without a compare; block kb, 16 bytes per lane
  __amdgpu_buffer_rsrc_t rw[XR_CG];
#pragma unroll
  for (int cg = 0; cg < XR_CG; ++cg)
    rw[cg] = buffer_over(p.w + (long long)grp * group_bytes + (long long)(cg0 + cg) * k_blocks * 1024,
                         (wave * XR_CG + cg < p.strip_groups && cg0 + cg < col_groups) ? (long long)k_blocks * 1024 : 0);
  const unsigned lane_off = (unsigned)lane * 16;
  auto wload = [&](int kb, int cg) {
    return __builtin_amdgcn_raw_buffer_load_b128(rw[cg], (unsigned)kb * 1024u + lane_off, 0, kStreamAux);
  };

  // ---- x staging: thread -> (row tid / 8 + 32 pass, 16-byte piece tid % 8) of a slab.  Rows past the chunk read the rows
  // that follow in memory (or zeros past the end of x): their products are never stored.  K bytes past K meet zero weights.
  constexpr int XP = (RB + 1) / 2;
  const int xrow = tid >> 3, xpiece = tid & 7;
  const unsigned x_voff = (unsigned)(m0 + xrow) * (unsigned)p.k + (unsigned)xpiece * 16u;
  const unsigned x_pass = 32u * (unsigned)p.k;
  unsigned char *xw = smem + xrow * XR_SLAB + ((xpiece ^ ((xrow >> 1) & 7)) << 4);
  // A slab's rows are requested XD slabs before they are written to their stage (register set slab % XD): one slab of
  // weights passes in less than the round trip of an x request while few rows are multiplied, two where registers allow
  constexpr int XD = (RBMAX != 10 && (2 * RB <= RBMAX || (RBMAX == 16 && RB <= 12))) ? 2 : 1;
  v4i xs[XD][XP];
  auto xload = [&](int slab, auto set_c) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int u = 0; u < XP; ++u)   // (the K offset in the range-checked part of the address: a slab past K in the last row reads zeros)
      xs[SET][u] = __builtin_amdgcn_raw_buffer_load_b128(rx, x_voff + (unsigned)u * x_pass + (unsigned)slab * XR_SLAB, 0, 0);
  };
  auto xstore = [&](int stage, auto set_c) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int u = 0; u < XP; ++u) *reinterpret_cast<v4i *>(xw + stage * S::kStage + u * 32 * XR_SLAB) = xs[SET][u];
  };

  // ---- fragment reads: lane (c16, h) holds K bytes 16 h .. 16 h + 15 of block kbs of row 16 rb + c16
  const int swz = (c16 >> 1) & 7;
  const unsigned char *xr0 = smem + c16 * XR_SLAB + ((h ^ swz) << 4);
  const unsigned char *xr1 = smem + c16 * XR_SLAB + (((4 + h) ^ swz) << 4);

  v4i acc[XR_CG][RB];
#pragma unroll
  for (int cg = 0; cg < XR_CG; ++cg)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[cg][rb] = v4i{0, 0, 0, 0};

  // epilogue operands of the lane's four columns, requested long before they are needed and not looked at before the
  // epilogue (the scale as raw bits, whatever its type: converting it here would wait for the loads in flight)
  int ep_bias[XR_CG];
  unsigned ep_scale_bits[XR_CG];
#pragma unroll
  for (int cg = 0; cg < XR_CG; ++cg) {
    const int n = n0 + 16 * (wave * XR_CG + cg) + c16;
    const bool live = 16 * (wave * XR_CG + cg) < strip_cols;
    ep_bias[cg] = (live && p.bias != nullptr) ? p.bias[(p.scale_per_group ? (long long)grp * p.n : 0) + n] : 0;
    ep_scale_bits[cg] = 0x3F800000u;   // 1.0f
    if (live && p.out_dtype != DT_I32 && p.scale_dtype != DT_NONE) {
      const long long idx = p.scale_is_scalar ? 0 : ((p.scale_per_group ? (long long)grp * p.n : 0) + n);
      if (p.scale_dtype == DT_BF16) ep_scale_bits[cg] = reinterpret_cast<const unsigned short *>(p.scale)[idx];
      else if (p.scale_dtype == DT_F32) ep_scale_bits[cg] = reinterpret_cast<const unsigned *>(p.scale)[idx];
      else ep_scale_bits[cg] = reinterpret_cast<const unsigned *>(p.scale)[2 * idx];   // int64 / uint64: float32 bits in the low word
    }
  }
  if (tid < S::kRows) s_pt[tid] = (p.per_token && tid < chunk_rows) ? p.per_token[m0 + tid] : 1.0f;

  // Prologue = the memory operations of the DEPTH / 2 steps in front of slab 0, in the loop's own order (the x request, a
  // step's two weight blocks, the staging write): the wait counts in front of the loop's MFMAs and staging writes are
  // computed over both ways into the loop, and a prologue in another order would shorten them to its own.  x requests
  // for slabs in front of slab 0 ask for slab 0 and are overwritten.
  v4i ring[DEPTH][XR_CG];
  __builtin_amdgcn_sched_barrier(0);
  static_for<DEPTH / 2>([&](auto j_c) {
    constexpr int SLAB = decltype(j_c)::value - DEPTH / 2, J = SLAB + ROUND, ST = J & 1;   // the last steps of a round
    xload(SLAB + XD > 0 ? SLAB + XD : 0, std::integral_constant<int, XD == 2 ? ST : 0>{});
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kbs = 0; kbs < 2; ++kbs)
#pragma unroll
      for (int cg = 0; cg < XR_CG; ++cg) ring[(2 * J + kbs) % DEPTH][cg] = wload(2 * SLAB + kbs + DEPTH, cg);
    if constexpr (SLAB == -1) xstore(0, std::integral_constant<int, XD == 2 ? (ST ^ 1) : 0>{});
    __builtin_amdgcn_sched_barrier(0);
  });

  // slab s = ROUND i + J: stage J % 2, K blocks 2 s and 2 s + 1 in ring slots (2 J) % DEPTH and (2 J + 1) % DEPTH.  The 2 RB fragment
  // reads of a slab run XR_AHEAD fragments ahead of the MFMAs that use them.
  auto step = [&](int s, auto j_c) {
    constexpr int J = decltype(j_c)::value, ST = J & 1;
    __syncthreads();   // slab s is in its stage; every wave is done with the other stage (slab s - 1)
    // The x rows of slab s + XD are requested in front of this step's weight blocks and go to their stage at the end of
    // step s + XD - 1: memory operations complete in order, so a staging write waits for everything requested before
    // its rows -- requested behind the weight blocks, it would wait for those too and no more than XD slabs of weights
    // would ever be in flight.
    xload(s + XD, std::integral_constant<int, XD == 2 ? ST : 0>{});
    auto frag = [&](int i) {   // fragment i of the slab: block i / RB, rows 16 (i % RB) ..
      return *reinterpret_cast<const v4i *>((i >= RB ? xr1 : xr0) + ST * S::kStage + (i % RB) * 16 * XR_SLAB);
    };
    v4i fq[XR_AHEAD + 1];
#pragma unroll
    for (int i = 0; i < XR_AHEAD; ++i) fq[i] = frag(i < 2 * RB ? i : 0);
    static_for<2 * RB>([&](auto i_c) {
      constexpr int I = decltype(i_c)::value, KBS = I / RB, R = I % RB;
      if constexpr (I + XR_AHEAD < 2 * RB) fq[(I + XR_AHEAD) % (XR_AHEAD + 1)] = frag(I + XR_AHEAD);
#pragma unroll
      for (int cg = 0; cg < XR_CG; ++cg) {
        if constexpr (RBMAX == 16) mfma_pinned(acc[cg][R], fq[I % (XR_AHEAD + 1)], ring[(2 * J + KBS) % DEPTH][cg]);
        else acc[cg][R] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fq[I % (XR_AHEAD + 1)], ring[(2 * J + KBS) % DEPTH][cg], acc[cg][R], 0, 0, 0);
      }
      if constexpr (R == RB - 1) {
#pragma unroll
        for (int cg = 0; cg < XR_CG; ++cg) ring[(2 * J + KBS) % DEPTH][cg] = wload(2 * s + KBS + DEPTH, cg);
      }
    });
    xstore(ST ^ 1, std::integral_constant<int, XD == 2 ? (ST ^ 1) : 0>{});   // slab s + 1 to its stage
    // the order the instructions of this slab are issued in: x requests, fragment reads XR_AHEAD ahead of their four
    // MFMAs, a K block's four weight requests behind its last MFMA, staging writes at the end (0x008 MFMA, 0x020 memory
    // read, 0x100 LDS read, 0x200 LDS write).  (The pinned MFMAs of the 256-row form keep the written order by themselves.)
    if constexpr (RBMAX != 16) {
    __builtin_amdgcn_sched_group_barrier(0x020, XP, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, XR_AHEAD < 2 * RB ? XR_AHEAD : 2 * RB, 0);
    static_for<2 * RB>([&](auto i_c) {
      constexpr int I = decltype(i_c)::value;
      __builtin_amdgcn_sched_group_barrier(0x008, XR_CG, 0);
      if constexpr (I + XR_AHEAD < 2 * RB) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (I % RB == RB - 1) __builtin_amdgcn_sched_group_barrier(0x020, XR_CG, 0);
    });
    __builtin_amdgcn_sched_group_barrier(0x200, XP, 0);
    }
  };
  const int slabs = (k_blocks + 1) / 2;
  for (int s = 0; s < slabs; s += ROUND) {
    // (whole rounds only, without a branch inside: slabs past K multiply masked weight blocks, zeros; a skipped step
    // would be one more way round the loop for the wait counts to allow for)
    static_for<ROUND>([&](auto j_c) { step(s + decltype(j_c)::value, j_c); });
  }

  // ---- epilogue: acc[cg][rb][r] = row 16 rb + 4 h + r, column 16 (4 wave + cg) + c16 of the tile -------------------------
  if (p.out_dtype == DT_I32) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int cg = 0; cg < XR_CG; ++cg) {
        const int n = n0 + 16 * (wave * XR_CG + cg) + c16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = 16 * rb + 4 * h + r;
          if (row < chunk_rows && 16 * (wave * XR_CG + cg) < strip_cols) reinterpret_cast<int *>(p.out)[(long long)(m0 + row) * p.n + n] = acc[cg][rb][r] + ep_bias[cg];
        }
      }
    return;
  }
  float ep_scale[XR_CG];
#pragma unroll
  for (int cg = 0; cg < XR_CG; ++cg)
    ep_scale[cg] = __uint_as_float((p.scale_dtype == DT_BF16 && p.out_dtype != DT_I32) ? ep_scale_bits[cg] << 16 : ep_scale_bits[cg]);
  __syncthreads();   // every wave is done with the x stages: they become two float32 stages of 16 output rows
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float(*tile_out)[XR_OUT_PITCH] = reinterpret_cast<float(*)[XR_OUT_PITCH]>(smem + (rb & 1) * S::kOutStage);
    const v4f pt = *reinterpret_cast<const v4f *>(s_pt + 16 * rb + 4 * h);
#pragma unroll
    for (int cg = 0; cg < XR_CG; ++cg) {
      const int cl = 16 * (wave * XR_CG + cg) + c16;
#pragma unroll
      for (int r = 0; r < 4; ++r) tile_out[4 * h + r][cl] = dequant(acc[cg][rb][r] + ep_bias[cg], ep_scale[cg], pt[r]);
    }
    __syncthreads();   // (also orders this block's reads before the writes of block rb + 2 into the same stage)
    // whole-row stores: 16 rows x 32 pieces of 8 columns, two pieces per thread; activation and the 16-bit cast here
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int item = tid + XR_THREADS * u;
      const int row = item >> 5, c8 = (item & 31) * 8;
      const int n = n0 + c8;
      if (16 * rb + row < chunk_rows && c8 < strip_cols) {   // N % 16 == 0: 8 columns all inside or all outside
        const v4f lo = *reinterpret_cast<const v4f *>(&tile_out[row][c8]);
        const v4f hi = *reinterpret_cast<const v4f *>(&tile_out[row][c8 + 4]);
        float f[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if (p.act_type != ACT_NONE) {
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = activate(f[j], p.act_type);
        }
        uint4 q;
        if (p.out_dtype == DT_BF16) {
          q = uint4{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        } else {
          q = uint4{(unsigned)f32_to_f16_rne(f[0]) | ((unsigned)f32_to_f16_rne(f[1]) << 16), (unsigned)f32_to_f16_rne(f[2]) | ((unsigned)f32_to_f16_rne(f[3]) << 16),
                    (unsigned)f32_to_f16_rne(f[4]) | ((unsigned)f32_to_f16_rne(f[5]) << 16), (unsigned)f32_to_f16_rne(f[6]) | ((unsigned)f32_to_f16_rne(f[7]) << 16)};
        }
        *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned short *>(p.out) + (long long)(m0 + 16 * rb + row) * p.n + n) = q;
      }
    }
  }
}

template <int RBMAX>
__global__ void __launch_bounds__(XR_THREADS, RBMAX <= 10 ? 2 : 1) gmm_w8a8_rows_kernel(const GmmParams p) {
  extern __shared__ __align__(16) unsigned char xr_smem[];
  const int lane = threadIdx.x & 63;
  // (grid.y enumerates the chunks that hold rows, group after group: a slot past the last one has nothing to do)
  int grp, mc, g_start, g_end;
  if (!chunk_of_slot(p, (int)blockIdx.y, 16 * RBMAX, lane, grp, mc, g_start, g_end)) return;
  const int m0 = g_start + mc * 16 * RBMAX;
  const int chunk_rows = min(16 * RBMAX, g_end - m0);
  const int rb = (chunk_rows + 15) / 16;
  const int strip = blockIdx.x;
  // one copy of the K loop per number of live 32-row block pairs
  bool done = false;
  // (the 160-row form is for groups that just miss 128 rows: it has copies for 6, 8 and 10 blocks only)
  static_for<(RBMAX == 10 ? 3 : RBMAX / 2)>([&](auto i_c) {
    constexpr int RB = RBMAX == 10 ? 2 * decltype(i_c)::value + 6 : 2 * decltype(i_c)::value + 2;
    if (!done && rb <= RB) {
      rows_run<RBMAX, RB>(p, xr_smem, grp, m0, chunk_rows, strip);
      done = true;
    }
  });
}

template <int RBMAX>
static hipError_t rows_launch(const GmmParams &p, hipStream_t stream) {
  auto kern = gmm_w8a8_rows_kernel<RBMAX>;
  constexpr size_t lds = XrShape<RBMAX>::kLds;
  static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race between first launches repeats it at worst
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  if (p.strip_groups < 1 || p.strip_groups > XR_COLS / 16) return hipErrorInvalidValue;
  const int col_groups = (p.n + 15) / 16;
  const dim3 grid((unsigned)((col_groups + p.strip_groups - 1) / p.strip_groups), chunk_slots(p, 16 * RBMAX), 1);
  if (grid.y > 65535u) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kern, grid, dim3(XR_THREADS), lds, stream, p);
  return hipGetLastError();
}

// rbmax = 16-row blocks per chunk (16); packed weights, K % 16 == 0, N % 16 == 0, M K and one group's weights below 2^31 bytes
hipError_t launch_rows_w8a8(const GmmParams &p, int rbmax, hipStream_t stream) {
  if (p.m == 0) return hipSuccess;
  if (p.k % 16 != 0 || p.n % 16 != 0) return hipErrorInvalidValue;
  if (rbmax == 8) return rows_launch<8>(p, stream);
  if (rbmax == 10) return rows_launch<10>(p, stream);
  if (rbmax == 16) return rows_launch<16>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace msco
