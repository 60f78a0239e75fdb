// Host-side declarations of the kernel launchers (one translation unit per kernel family).
#ifndef MSCO_GMM_KERNELS_H_
#define MSCO_GMM_KERNELS_H_

#include <hip/hip_runtime.h>
#include "gmm_common.h"

namespace msco {

enum TileCfg : int {
  TILE_256x256 = 0, TILE_128x128 = 1, TILE_64x128 = 2, TILE_128x256 = 3,
  TILE_256x256_W4 = 4,   // persistent, four wavefronts with 128 x 128 accumulators each: gmm_tile4m_w8a8.hip (16 x 16 x 64 MFMAs)
  TILE_256x256_W4_MFMA32 = 5,   // the same on 32 x 32 x 32 MFMAs: gmm_tile4_w8a8.hip (never planned; kept to be measured against)
  TILE_ROWS256 = 6,   // packed weights only: chunks of up to 256 rows x strips of 256 columns, x through LDS, weights straight into MFMA operands: gmm_rows_w8a8.hip
  TILE_ROWS128 = 7,   // the same with chunks of up to 128 rows and two workgroups per CU
  TILE_ROWS160 = 8,   // ... of up to 160 rows, two workgroups per CU, two K blocks of weights in flight
  TILE_CFG_COUNT = 9
};

// MFMA tile kernel for W8A8 (prefill shapes).  nk: weights stored [E,N,K]; packed: the packed layout (nk is ignored).
hipError_t launch_tile_w8a8(const GmmParams &p, int tile_cfg, bool nk, bool packed, hipStream_t stream);
const char *tile_cfg_name(int tile_cfg);
hipError_t launch_tile4m_w8a8(const GmmParams &p, int layout, hipStream_t stream);  // layout 0 [E,N,K], 1 packed, 2 [E,K,N] (N % 16 == 0)
hipError_t launch_tile4_w8a8(const GmmParams &p, int layout, hipStream_t stream);   // layout 0 [E,N,K], 1 packed, 2 [E,K,N] (N % 16 == 0)
void tile_cfg_dims(int tile_cfg, int *bm, int *bn);
// packed weights, several groups of a few dozen to a few hundred rows: chunks of 16 rbmax rows (rbmax = 8, 10 or 16), see gmm_rows_w8a8.hip
hipError_t launch_rows_w8a8(const GmmParams &p, int rbmax, hipStream_t stream);
// K split across workgroups (p.split_k > 1; four-wave tile shapes only): partial tiles and arrival counters
size_t tile_count_bound(int tile_cfg, int64_t m, int64_t n, int64_t e);
size_t tile_workspace_bytes(int tile_cfg, int64_t m, int64_t n, int64_t e, int split_k);

// grid.y of the decode kernels: an upper bound, for any group_list, of the number of chunks of rows_per_chunk rows that
// hold rows (see chunk_of_slot in gmm_common.h)
inline unsigned chunk_slots(const GmmParams &p, int rows_per_chunk) {
  const long long per_group = ((long long)p.m + rows_per_chunk - 1) / rows_per_chunk;
  const long long all = (long long)p.e * (per_group > 1 ? per_group : 1);
  const long long held = (p.m < p.e ? p.m : p.e) + p.m / rows_per_chunk;
  const long long slots = all < held ? all : held;
  return (unsigned)(slots > 1 ? slots : 1);
}

// Skinny (decode) kernels: one workgroup streams a 128-column weight strip of one group over a K
// range; waves split K and reduce through LDS, workgroups split K and reduce through the workspace.
// wide16: the 16-wave / 128-column-strip variant for small weight sets, else 4 waves / 256-column strips
hipError_t launch_skinny_w8a8(const GmmParams &p, bool nk, bool wide16, hipStream_t stream);
hipError_t launch_skinny_a16w8(const GmmParams &p, hipStream_t stream);
size_t skinny_workspace_bytes(int64_t m, int64_t n, int64_t e, int split_k, int cols);
size_t skinny_counter_count(int64_t m, int64_t n, int64_t e, int cols);
size_t a16w8_workspace_bytes(int64_t m, int64_t n, int64_t e, int split_k);

// Decode kernels for weights in the packed layout (gmm_stream.hip): 4 waves, strips of up to 256 columns, K slices of
// at most 128 blocks of 64 bytes (split_k chosen accordingly); workspace and counters as for the 4-wave skinny kernel.
hipError_t launch_stream_w8a8(const GmmParams &p, hipStream_t stream);
hipError_t launch_stream_a16w8(const GmmParams &p, hipStream_t stream);   // K slices of at most 64 blocks
// more than 16 rows per group on packed weights: chunks of 16 tch rows (tch = 2, 4, 8), strips of 64 columns
hipError_t launch_streamm_w8a8(const GmmParams &p, int tch, hipStream_t stream);
hipError_t launch_streamm_a16w8(const GmmParams &p, int tch, bool packed, hipStream_t stream);   // weight-only, 32 / 64 / 128 rows per chunk (tch = 2, 4, 8), packed or [E,K,N] weights, no K split
size_t streamm_tile_bytes(int tch);   // workspace bytes of one (chunk, strip, K slice) partial tile
size_t rows32_a16w8_slice_bytes(int strip_groups);   // workspace bytes of one (chunk, strip, K slice) partial tile of the 128-row weight-only kernel
size_t stream_a16w8_tile_bytes();   // workspace bytes of one (strip, K slice) partial tile of the weight-only kernel
int stream_blocks_per_wave(int64_t k, int split_k);
size_t packed_weight_bytes(int64_t k, int64_t n);   // bytes of one group's weights in the packed layout
hipError_t launch_pack_weight(const void *src, void *dst, long long e, long long k, long long n, bool src_nk,
                              hipStream_t stream);

// Shape-agnostic fallback kernels (one output element per thread), any K / N.
// layout: 0 [E,K,N], 1 [E,N,K], 2 packed
hipError_t launch_generic_w8a8(const GmmParams &p, int layout, hipStream_t stream);
hipError_t launch_generic_a16w8(const GmmParams &p, int layout, hipStream_t stream);

// Batched 2-D transpose, src [batch, rows, cols] -> dst [batch, cols, rows].
hipError_t launch_transpose_2d(const void *src, void *dst, long long batch, long long rows, long long cols,
                               int elem_bytes, hipStream_t stream);

}  // namespace msco
#endif  // MSCO_GMM_KERNELS_H_
