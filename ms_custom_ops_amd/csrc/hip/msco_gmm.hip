// C ABI of the gfx950 grouped quantized matmul backend (see include/msco_gmm.h).
// Host side only: argument checking, kernel-family choice from shapes (never from tensor values),
// workspace sizing and the launches.
#include "msco_gmm.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "gmm_kernels.h"

namespace {

using namespace msco;

enum Family : int { FAM_NONE = 0, FAM_TILE = 1, FAM_SKINNY = 2, FAM_GENERIC = 3 };

// values of msco_gmm_desc::kernel_override
enum Override : int {
  OV_AUTO = 0, OV_TILE_256 = 1, OV_TILE_128 = 2, OV_TILE_64 = 3, OV_SKINNY = 4, OV_GENERIC = 5,
  OV_TILE_256_W4 = 6,  // persistent four-wave 256 x 256 kernel
  OV_TILE_128x256 = 7,  // four waves side by side, 128 x 256
  OV_TILE_256_W4_MFMA32 = 8,  // the persistent kernel's 32 x 32 x 32 form (never planned)
  OV_ROWS128 = 9,  // packed weights: chunks of up to 128 rows through LDS, weights straight into MFMA operands (other layouts: 128 x 256 tiles)
  OV_ROWS256 = 10,  // the same with chunks of up to 256 rows (other layouts: the persistent kernel)
  OV_ROWS160 = 11   // ... of up to 160 rows (other layouts: the persistent kernel)
};

constexpr int64_t kSkinnyMaxRows = 64;   // total rows up to which the weight-streaming kernel is planned
constexpr int64_t kSkinnyMaxChunkSlots = 1024;   // (group, 16-row chunk) slots up to which many small groups take the decode kernels
constexpr int kTargetWorkgroups = 512;  // skinny kernels with a K split: aim for this many workgroups (2 per CU)
constexpr int kMaxSplitK = 8;             // keeps the last arriver's reduction to two rounds of loads
constexpr int kDefaultCUs = 256;   // MI355X; the plan uses the count the device reports
constexpr int kTileTargetWorkgroups = 256;   // tile kernels with a K split: aim for this many workgroups (one per CU)
constexpr int kTileSplitMaxTiles = 128;      // ... and only split below this many tiles (measured: beyond it the partial-tile exchange costs more than it hides)
constexpr size_t kTileSplitMaxWorkspace = (size_t)128 << 20;   // bytes of split-K partial tiles a plan may ask the caller for
constexpr int kTileMinSlabs = 4;               // 64-byte K slabs every slice keeps at least

int env_int(const char *name, int fallback) {
  const char *v = std::getenv(name);
  return (v && *v) ? std::atoi(v) : fallback;
}

// MSCO_PRINT_PLAN (the counterpart of the reference's INTERNAL_PRINT_TILING) is read from the environment once per
// process, at the first plan; planning itself reads no environment.  The other fields override plan constants for
// tuning sweeps and exist only in a library built with -DMSCO_TUNING_SWITCHES (build.py --tuning): the shipped
// library has no such switches.
struct Tuning {
  int print_plan, tile_cfg, tile_target_wgs, tile_split_k, stream_max_slots, skinny_wide16, stream_min_wgs, stream_groups,
      skinny_target_wgs, skinny_split_k, tile_wide_k, stream_tch, two_level;
};
const Tuning &tuning() {
#ifdef MSCO_TUNING_SWITCHES
  static const Tuning t = {env_int("MSCO_PRINT_PLAN", 0),        env_int("MSCO_TILE_CFG", -1),
                           env_int("MSCO_TILE_TARGET_WGS", 0),   env_int("MSCO_TILE_SPLIT_K", 0),
                           env_int("MSCO_STREAM_MAX_SLOTS", 0),  env_int("MSCO_SKINNY_WIDE16", -1),
                           env_int("MSCO_STREAM_MIN_WGS", 0),    env_int("MSCO_STREAM_GROUPS", 0),
                           env_int("MSCO_SKINNY_TARGET_WGS", 0), env_int("MSCO_SKINNY_SPLIT_K", 0),
                           env_int("MSCO_TILE_WIDE_K", -1),      env_int("MSCO_STREAM_TCH", 0),
                           env_int("MSCO_TWO_LEVEL", 1)};
#else
  static const Tuning t = {env_int("MSCO_PRINT_PLAN", 0), -1, 0, 0, 0, -1, 0, 0, 0, 0, -1, 0, 1};
#endif
  return t;
}
int or_default(int v, int fallback) { return v > 0 ? v : fallback; }

}  // namespace

struct msco_gmm_op {
  msco_gmm_desc desc{};
  bool planned = false;
  int64_t m = 0, k = 0, n = 0, e = 0;
  int family = FAM_NONE;
  int tile_cfg = 0;
  int split_k = 1;
  int max_chunks = 1;
  int skinny_wide16 = 0;
  int skinny_cols = kSkinnyCols;
  int n_strips = 0;
  int strip_groups = 16;
  int stream_tch = 1;        // packed and, weight-only, [E,K,N] weights: 16-row fragments per chunk (1: the 16-row streaming kernels, 2/4/8: the multi-row ones)
  int wide_k_slabs = 0;      // small tile kernels on K-major weights: 128-byte K slabs
  int w_nontemporal = 0;     // small tile kernels on packed weights: non-temporal weight loads
  int small_group_rows = 0;  // > 0: the persistent kernel takes the groups with more rows, a second launch of 64 x 128 tiles the others
  size_t workspace_bytes = 0;
  unsigned *counters = nullptr;
  size_t counters_cap = 0;
  int num_cus = kDefaultCUs;   // compute units of the device that was current at create time
  std::string info;
  std::mutex mu;
};

namespace {

bool is_w8a8(const msco_gmm_desc &d) { return d.x_dtype == MSCO_DT_I8; }
bool is_a16w8(const msco_gmm_desc &d) { return d.x_dtype == MSCO_DT_BF16 || d.x_dtype == MSCO_DT_F16; }
bool is_packed(const msco_gmm_desc &d) { return d.weight_layout == MSCO_WL_PACKED; }
// 0 [E,K,N], 1 [E,N,K], 2 packed
int layout_of(const msco_gmm_desc &d) { return is_packed(d) ? 2 : (d.transpose_b ? 1 : 0); }

int check_desc(const msco_gmm_desc &d) {
  if (d.abi_version != MSCO_GMM_ABI_VERSION) return MSCO_ERR_INVALID_ARG;
  if (d.weight_dtype != MSCO_DT_I8) return MSCO_ERR_UNSUPPORTED;
  if (d.group_list_dtype != MSCO_DT_NONE && d.group_list_dtype != MSCO_DT_I32 && d.group_list_dtype != MSCO_DT_I64)
    return MSCO_ERR_UNSUPPORTED;
  if (d.group_list_type != 0 && d.group_list_type != 1) return MSCO_ERR_INVALID_ARG;
  if (d.kernel_override < OV_AUTO || d.kernel_override > OV_ROWS160) return MSCO_ERR_INVALID_ARG;
  if (d.weight_layout != MSCO_WL_ROW_MAJOR && d.weight_layout != MSCO_WL_PACKED) return MSCO_ERR_INVALID_ARG;
  if (d.force_split_k < 0) return MSCO_ERR_INVALID_ARG;
  if (d.act_type < MSCO_ACT_NONE || d.act_type > MSCO_ACT_SILU) return MSCO_ERR_INVALID_ARG;
  if (d.act_type == MSCO_ACT_GELU_ERF) return MSCO_ERR_UNSUPPORTED;
  if (d.act_type != MSCO_ACT_NONE && d.out_dtype == MSCO_DT_I32) return MSCO_ERR_UNSUPPORTED;
  if (is_w8a8(d)) {
    if (d.out_dtype != MSCO_DT_BF16 && d.out_dtype != MSCO_DT_F16 && d.out_dtype != MSCO_DT_I32)
      return MSCO_ERR_UNSUPPORTED;
    if (d.bias_dtype != MSCO_DT_NONE && d.bias_dtype != MSCO_DT_I32) return MSCO_ERR_UNSUPPORTED;
    if (d.scale_dtype != MSCO_DT_NONE && d.scale_dtype != MSCO_DT_F32 && d.scale_dtype != MSCO_DT_BF16 &&
        d.scale_dtype != MSCO_DT_I64 && d.scale_dtype != MSCO_DT_U64)
      return MSCO_ERR_UNSUPPORTED;
    if (d.per_token_dtype != MSCO_DT_NONE && d.per_token_dtype != MSCO_DT_F32) return MSCO_ERR_UNSUPPORTED;
    if (d.antiquant_dtype != MSCO_DT_NONE) return MSCO_ERR_UNSUPPORTED;
    return MSCO_OK;
  }
  if (is_a16w8(d)) {
    if (d.out_dtype != d.x_dtype) return MSCO_ERR_UNSUPPORTED;       // weight-only output keeps x's dtype
    if (d.antiquant_dtype != d.x_dtype) return MSCO_ERR_UNSUPPORTED; // scale / offset share x's dtype
    if (d.transpose_b && d.weight_layout == MSCO_WL_ROW_MAJOR) return MSCO_ERR_UNSUPPORTED;
    if (d.bias_dtype != MSCO_DT_NONE || d.scale_dtype != MSCO_DT_NONE || d.per_token_dtype != MSCO_DT_NONE)
      return MSCO_ERR_UNSUPPORTED;
    return MSCO_OK;
  }
  return MSCO_ERR_UNSUPPORTED;
}

void choose_plan(msco_gmm_op *op) {
  const msco_gmm_desc &d = op->desc;
  const int num_cus = op->num_cus;
  const int64_t m = op->m, k = op->k, n = op->n, e = op->e;
  const bool aligned = (k % 16 == 0) && (n % 16 == 0) && k >= 16 && n >= 16;
  op->split_k = 1;
  op->max_chunks = 1;
  op->skinny_wide16 = 0;
  op->skinny_cols = kSkinnyCols;
  op->n_strips = (int)((n + kSkinnyCols - 1) / kSkinnyCols);
  op->workspace_bytes = 0;
  op->tile_cfg = TILE_256x256;
  op->wide_k_slabs = 0;
  op->w_nontemporal = 0;
  op->small_group_rows = 0;

  int family;
  // All three W8A8 weight layouts follow the same tile rules: packed weights are K-contiguous per column like [E,N,K],
  // and [E,K,N] weights run the same LDS-direct tile kernels (transpose reads turn them on the way out of LDS; rows of
  // whole 16-column chunks, which the alignment rule guarantees).  Only the decode kernels are per layout.
  // (a group that overflows its 16-row chunk streams its weights twice, so 1.5 x the average has to fit; beyond that
  // the 64 x 128 tile kernel with non-temporal weight loads is the better streamer -- 128 rows over 8 experts, 470 MB
  // of weights: 76 us against 82 us for the 32-row streaming kernel and 105 us for 16-row chunks; row-major [E,N,K]:
  // 111 us against 140 us)
  // row-major [E,N,K] weights at decode sizes: a column's K bytes are contiguous and the columns are K bytes apart, which
  // suits the 64 x 128 tile's LDS-direct loads better than the decode kernel's 64-byte row pieces (K = 4096, N = 11008,
  // 1 / 16 rows: 15.8 / 15.9 us against 16.8 / 17.7 us; 32 rows over 8 experts, N = 14336: 103 against 115 us)
  // (a few rows over hundreds of experts are the decode kernel's again -- 40 rows over 256 experts, K = 512, N = 7168: 41 us
  // against 95 us -- but not a thousand rows over them: K = 2048, N = 7168: 635 against 595 us, K = 7168, N = 4096: 1467
  // against 1244 us)
  const bool nk_rows = is_w8a8(d) && d.transpose_b != 0 && !is_packed(d) && !(e > 32 && m <= kSkinnyMaxRows);
  const int64_t avg_rows = (m + (e > 0 ? e : 1) - 1) / (e > 0 ? e : 1);
  // (the decode kernels' grid enumerates the chunks that hold rows -- at most min(E, M) + M / 16 of them -- so experts
  // without rows cost nothing)
  const bool many_small_groups = e > 1 && avg_rows + avg_rows / 2 <= kSkinnyRows &&
                                 std::min<int64_t>(m, e) + m / kSkinnyRows <= kSkinnyMaxChunkSlots;
  if (!aligned) {
    family = FAM_GENERIC;
  } else if (is_a16w8(d)) {
    family = FAM_SKINNY;  // the weight-only path is a decode path; large M re-streams weights per 16 rows
  } else if (((m <= kSkinnyMaxRows && !(e == 1 && m > kSkinnyRows)) || many_small_groups) && !nk_rows) {
    // decode: few rows in total, or groups of about one 16-row chunk each (the weights stream once per chunk).  The
    // grid enumerates every (group, chunk) a malformed-to-the-limit group_list could fill; beyond a thousand slots
    // the empty workgroups cost more than the tile kernel's partial tiles.  A single group of more than one 16-row
    // chunk takes the small tile kernel with a K split instead (measured on packed weights, K = 4096, N = 11008:
    // 32 / 48 / 64 rows 17.1 / 17.5 / 18.0 us against 18.7 / 24.4 / 26.3 us of the multi-row streaming kernel, which
    // stays for several groups of a few dozen rows each; [E,K,N] weights, same shape, 17 / 32 / 64 rows: 16.5 / 16.9 /
    // 18.3 us).
    family = FAM_SKINNY;
  } else {
    family = FAM_TILE;
    // tile shape from shapes only: average rows per group and how many tiles fill 256 CUs
    const int64_t rows_per_group = m / (e > 0 ? e : 1);
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    // several groups, a few dozen to a few hundred rows each: the launch is bound by the weight
    // stream (every group's matrix is read once per m-tile of the group), so the m-tile should hold a whole group --
    // real routings are uneven, hence 1.5 x the average -- as long as there are tiles for most CUs.  Measured (E = 8,
    // K = 4096, N = 14336, packed; 64 x 128 / 128 x 128 / 256 x 256 tiles): 64 rows per group 112 / 97 / 100 us, 128 rows per
    // group 162 / 150 / 109 us (136 us with 128 x 256), 32 rows per group 87.5 us with the first.
    auto group_tiles = [&](int bm, int bn) { return e * ((rows_per_group + bm - 1) / bm) * ((n + bn - 1) / bn); };
    const int64_t cover = rows_per_group + rows_per_group / 2;
    const int64_t busy = (num_cus > 0 ? num_cus : kTileTargetWorkgroups) * 3 / 4;
    // (the persistent four-wave kernel: at least four 128-byte K slabs per tile, a group table that fits in LDS)
    const bool w4_ok = k >= 512 && e <= 1024;
    // (128-row m-tiles while every group fits one: 8 experts, 72 .. 112 rows per group on average, the largest group 80 ..
    // 126 rows: 84 - 92 us with 128 x 256 tiles against 100 - 109 us with 256 x 256; at 120 rows on average the largest
    // group has 131, streams its weights twice and the launch takes 126 against 113 us -- so the 256-row tile takes
    // over at 1.5 x the average = 174 rows, not at 128; at 112 rows on average, the largest group 126, [E,K,N] weights:
    // 104 us with 128 x 256 tiles against 116 us)
    // Packed weights, several groups of up to about 150 rows each and enough columns that 256-column strips give every CU
    // a workgroup: the row-chunk kernels stream a group's weights once, straight into MFMA operands, and multiply only
    // the 16-row blocks that hold rows.  Measured, 8 experts, K = 4096, N = 14336 (470 MB of weights; a launch that only
    // reads them takes 72 us), rows per group 16 / 32 / 64 / 96 / 112: 72.8 / 75.8 / 79.2 / 83.8 / 85.9 us with 128-row
    // chunks against 76.5 / 79.6 / 82.4 / 89.1 / 111.0 us for the tiles picked below.  A group that overflows its chunk
    // takes a second workgroup that streams its weights again (128 rows on average, half of the groups above 128: 131 us),
    // hence 160-row chunks from 116 rows on average (still two workgroups per CU, with room for two K blocks of weights
    // in flight only): 120 / 128 / 136 / 144 rows per group 88.6 / 89.3 / 91.6 / 91.7 us against 100 / 103 / 103 / 105 us
    // with 256-row chunks (one workgroup per CU) and 110 - 112 us for the persistent kernel.  256-row chunks are left with
    // 147 .. 155 rows per group (152 rows, the largest group 164: 107.9 against 118 us); the persistent kernel wins beyond
    // (160 rows: 115 us either way; 192 rows: 125 against 115 us).  Few columns leave CUs idle: N = 1344, K = 5120: 41
    // against 24 us for 64 x 128 tiles with a K split.
    // (narrower strips for fewer columns do not pay: with one or two column groups per wave, strips of 6 / 3 column groups,
    // 8 experts, 1024 rows, K = 5120, N = 2688 / 1344: 55 / 40 us against 46 / 24 us for the 64 x 128 tiles)
    const bool rows_kernel_ok = is_packed(d) && e > 1 && k >= 1024 && ((n + 255) / 256) * std::min<int64_t>(e, m) >= num_cus;
    if (rows_kernel_ok && avg_rows <= 116) {
      op->tile_cfg = TILE_ROWS128;
    } else if (rows_kernel_ok && avg_rows <= 146) {
      op->tile_cfg = TILE_ROWS160;
    } else if (rows_kernel_ok && avg_rows <= 155) {
      op->tile_cfg = TILE_ROWS256;
    } else if (e > 1 && w4_ok && cover > 174 && cover <= 384 && group_tiles(256, 256) >= busy) {
      op->tile_cfg = TILE_256x256_W4;
    } else if (e > 1 && cover > 64 && cover <= 192 && group_tiles(128, 128) >= busy) {
      // (128 x 256 tiles re-read x half as often: 64 / 96 rows per group 93 / 99 us against 100 / 111 us)
      op->tile_cfg = group_tiles(128, 256) >= busy ? TILE_128x256 : TILE_128x128;
    } else if (e == 1 && w4_ok && tiles(256, 256) >= busy * 2 / 3 && tiles(128, 256) > busy * 4 / 3) {
      // one group, a few hundred to a thousand rows: the persistent kernel already on half of the CUs
      // when 128 x 256 tiles would no longer run in one round (N = 11008: M = 768 / 1024: 47 / 52 us against 63 / 68 us
      // with 128 x 128 tiles) ...
      op->tile_cfg = TILE_256x256_W4;
    } else if (e == 1 && tiles(128, 256) >= busy * 4 / 5 && tiles(128, 256) <= busy * 4 / 3) {
      // ... and 128 x 256 tiles while they do and fill most of the chip (M = 448 .. 640: 40 - 42 us against 45 - 47 us;
      // M = 384, 129 tiles: 41 us against 35 us with 128 x 128)
      op->tile_cfg = TILE_128x256;
    } else if (rows_per_group >= 192 && tiles(256, 256) >= 256) {
      op->tile_cfg = w4_ok ? TILE_256x256_W4 : TILE_256x256;
    } else if (rows_per_group >= 96 && tiles(128, 128) >= 256) {
      op->tile_cfg = TILE_128x128;
    } else if (tiles(128, 128) >= 512) {
      op->tile_cfg = TILE_128x128;
    } else if (rows_per_group >= 192 && tiles(128, 128) > kTileSplitMaxTiles) {
      // a few hundred rows: 128 x 128 tiles on at least half of the CUs beat twice as many 64 x 128
      // tiles (measured: M = 256, N = 11008: 32 us against 44 us); with fewer tiles the K split of the small tile wins
      op->tile_cfg = TILE_128x128;
    } else {
      op->tile_cfg = TILE_64x128;
    }
  }
  switch (d.kernel_override) {
    case OV_TILE_256: family = FAM_TILE; op->tile_cfg = TILE_256x256; break;
    case OV_TILE_256_W4: family = FAM_TILE; op->tile_cfg = TILE_256x256_W4; break;
    case OV_TILE_256_W4_MFMA32: family = FAM_TILE; op->tile_cfg = TILE_256x256_W4_MFMA32; break;
    case OV_TILE_128: family = FAM_TILE; op->tile_cfg = TILE_128x128; break;
    case OV_TILE_128x256: family = FAM_TILE; op->tile_cfg = TILE_128x256; break;
    case OV_TILE_64: family = FAM_TILE; op->tile_cfg = TILE_64x128; break;
    case OV_ROWS128: family = FAM_TILE; op->tile_cfg = is_packed(d) ? TILE_ROWS128 : TILE_128x256; break;
    case OV_ROWS256: family = FAM_TILE; op->tile_cfg = is_packed(d) ? TILE_ROWS256 : TILE_256x256_W4; break;
    case OV_ROWS160: family = FAM_TILE; op->tile_cfg = is_packed(d) ? TILE_ROWS160 : TILE_256x256_W4; break;
    case OV_SKINNY: family = FAM_SKINNY; break;
    case OV_GENERIC: family = FAM_GENERIC; break;
    default: break;
  }
  // (what the persistent kernel cannot take runs the eight-wave kernel of the same tile shape; the plan says so)
  if (family == FAM_TILE && (op->tile_cfg == TILE_256x256_W4 || op->tile_cfg == TILE_256x256_W4_MFMA32) && !(k >= 512 && e <= 1024))
    op->tile_cfg = TILE_256x256;
  // the MFMA kernels address x and one group's weights through 32-bit buffer offsets
  const bool fits32 = (is_packed(d) ? (int64_t)packed_weight_bytes(k, n) : k * n) < ((int64_t)1 << 31) &&
                      m * k < ((int64_t)1 << 31);
  if ((family == FAM_TILE || family == FAM_SKINNY) && !(aligned && fits32)) family = FAM_GENERIC;
  if (family == FAM_TILE && !is_w8a8(d)) family = FAM_SKINNY;
  if (family == FAM_TILE) {
    const int forced = tuning().tile_cfg;
    if (forced >= 0 && forced < TILE_CFG_COUNT && d.kernel_override == OV_AUTO) op->tile_cfg = forced;
    if ((op->tile_cfg == TILE_ROWS256 || op->tile_cfg == TILE_ROWS160) && !is_packed(d)) op->tile_cfg = TILE_256x256_W4;
    if (op->tile_cfg == TILE_ROWS128 && !is_packed(d)) op->tile_cfg = TILE_128x256;
    // Few tiles (M of a few hundred rows): split K across workgroups until about kTileTargetWorkgroups of them
    // stream operands; every slice keeps at least kTileMinSlabs 64-byte K slabs.  Small tile shapes only.
    if (op->tile_cfg == TILE_128x128 || op->tile_cfg == TILE_64x128) {
      int bm, bn;
      tile_cfg_dims(op->tile_cfg, &bm, &bn);
      // tiles the launch is expected to have: every group that holds rows has at least one m-tile
      const int64_t groups_with_rows = std::min<int64_t>(e, m);
      const int64_t t = std::max<int64_t>((m + bm - 1) / bm, groups_with_rows) * ((n + bn - 1) / bn);
      // t tiles x s slices run in ceil(t s / CUs) rounds (the operand ring takes most of a CU's LDS: one workgroup per
      // CU).  In units of one 64-byte K slab of a tile (0.2 us): a round costs its slabs plus 10 (prologue, epilogue),
      // a split adds 8 per slice for 64 x 128 tiles and 12 for 128 x 128 (its partial tile out and in, one round trip of
      // the last arriver), less 2.  The cheapest s wins, the smaller one on a tie.  Fitted to M = 128, K = N = 4096
      // (64 tiles; s = 1 / 2 / 3 / 4 / 6: 18.7 / 15.2 / 14.5 / 15.3 / 21.3 us) and M = 64, K = 4096, N = 11008 (86 tiles;
      // s = 1 / 2 / 3: 20.9 / 18.0 / 24.3 us, the third slice starting a second round).
      const int cus = or_default(tuning().tile_target_wgs, num_cus > 0 ? num_cus : kTileTargetWorkgroups);
      const int cap = (int)std::max<int64_t>(1, ((k + 63) / 64) / kTileMinSlabs);
      auto split_cost = [&](int sl) {
        const int64_t slabs = ((k + 63) / 64 + sl - 1) / sl;
        const int64_t rounds = (t * sl + cus - 1) / cus;
        const int64_t exchange = sl > 1 ? (int64_t)(4 + bm * bn / 2048) * sl - 2 : 0;
        return rounds * (slabs + 10 + exchange);
      };
      int want = 1;
      if (t <= kTileSplitMaxTiles) {
        for (int sl = 2; sl <= std::min(kMaxSplitK, cap); ++sl)
          if (split_cost(sl) < split_cost(want)) want = sl;
      }
      const int forced_split = d.force_split_k > 0 ? d.force_split_k : tuning().tile_split_k;
      if (forced_split > 0) want = std::min(forced_split, cap);
      // the partial tiles of a K split are sized for the worst group_list (one partial m-tile per group): with many
      // groups that bound dwarfs the problem, so the split is halved until the workspace fits under the cap
      while (want > 1 && tile_workspace_bytes(op->tile_cfg, m, n, e, want) > kTileSplitMaxWorkspace) want /= 2;
      op->split_k = want;
      op->workspace_bytes = tile_workspace_bytes(op->tile_cfg, m, n, e, op->split_k);
      // 128-byte K slabs (a 4-stage ring of them takes most of a CU's LDS: one workgroup per CU) when the workgroups
      // run in one round; more tiles than CUs keep 64-byte slabs and two workgroups per CU (M = 512, N = 11008: 344
      // tiles, 46.8 us against 50.1 us)
      op->wide_k_slabs = t * want <= (num_cus > 0 ? num_cus : kTileTargetWorkgroups);
      if (tuning().tile_wide_k >= 0) op->wide_k_slabs = tuning().tile_wide_k != 0;
    }
    if (op->tile_cfg == TILE_128x128 || op->tile_cfg == TILE_64x128 || op->tile_cfg == TILE_128x256) {
      // Non-temporal weight loads: a weight stream of tens of megabytes that at most two m-tiles read should not push x
      // out of the caches (E = 8 x 32 rows, 470 MB: 87.7 -> 79.4 us; M = 128, 45 MB: 20.8 -> 19.6 us); three m-tiles
      // re-read it from the cache and lose badly without it there (M = 384: 35 -> 47 us), and a weight set the caches
      // hold anyway gains nothing (M = 128, 16.8 MB: 13.8 -> 14.4 us).
      int bm, bn;
      tile_cfg_dims(op->tile_cfg, &bm, &bn);
      const int64_t group_rows = e > 1 ? (m / e) + (m / e) / 2 : m;
      // ([E,K,N] rows: a wave instruction brings whole lines too; 470 MB over 8 experts, 64 / 128 rows in all: 94 -> 84 us
      // and 97 -> 87 us; on 45 MB it loses a little -- 32 rows 16.9 -> 17.3 us -- so the bar is higher there)
      const int64_t nt_bytes = is_packed(d) ? ((int64_t)32 << 20) : ((int64_t)64 << 20);
      op->w_nontemporal = (is_packed(d) || d.transpose_b == 0) && e * k * n >= nt_bytes && (group_rows + bm - 1) / bm <= 2;
    }
    if (op->tile_cfg == TILE_128x256 && tuning().tile_wide_k >= 0) op->wide_k_slabs = tuning().tile_wide_k != 0;   // (measured slower with 128-byte slabs: 99 against 93 us)
  }
  if (family == FAM_TILE && (op->tile_cfg == TILE_ROWS256 || op->tile_cfg == TILE_ROWS128 || op->tile_cfg == TILE_ROWS160)) {
    // Row-chunk kernel: every workgroup streams a strip of up to 16 column groups over all of K plus its chunk's x rows,
    // and the workgroups that share a CU share its operand path.  The strip is as wide as makes the bytes a CU moves
    // least: ceil(workgroups / CUs) x (strip bytes + x bytes of a chunk), one chunk per group expected.  8 experts x 14336
    // columns on 256 CUs: 448 workgroups of 16 column groups cost two per CU as 512 of 14 do (c3_t64 82.2 -> 72.8 us).
    const int64_t cus = num_cus > 0 ? num_cus : kDefaultCUs;
    const int64_t col_groups = (n + 15) / 16, chunks = std::max<int64_t>(1, std::min<int64_t>(e, m));
    const int64_t chunk_rows = op->tile_cfg == TILE_ROWS128 ? 128 : op->tile_cfg == TILE_ROWS160 ? 160 : 256;
    const int64_t x_bytes = std::min<int64_t>(avg_rows, chunk_rows) * k;
    int best = 16;
    int64_t best_cost = INT64_MAX;
    for (int sg = 16; sg >= 10; --sg) {
      const int64_t wgs = ((col_groups + sg - 1) / sg) * chunks;
      const int64_t cost = ((wgs + cus - 1) / cus) * ((int64_t)sg * 16 * k + x_bytes);
      if (cost < best_cost) { best_cost = cost; best = sg; }
    }
    op->strip_groups = best;
    const int forced_groups = tuning().stream_groups;
    if (forced_groups >= 1 && forced_groups <= 16) op->strip_groups = forced_groups;
    op->n_strips = (int)((col_groups + op->strip_groups - 1) / op->strip_groups);
  }
  // Many experts with uneven loads (a skewed routing): every group of a few rows costs the persistent kernel a whole
  // 256-row m-tile per n-tile.  The groups of at most 64 rows go to a second launch of 64 x 128 tiles instead, which
  // streams their weights once with non-temporal loads.  On the skewed 64-expert workload (49152 rows, K = 2048, N = 2816;
  // 29 groups of at most 64 rows) the persistent kernel's tiles go from 10.2 to 8.9 per workgroup and the pair of launches
  // measures 336 against 348 us on packed weights and 340 against 352 us on [E,K,N]; on [E,N,K] weights (64-byte row
  // pieces, no non-temporal loads) 347 against 350, not worth a launch.  Which groups are small only the device knows;
  // with few experts the second launch would mostly find none.
  if (family == FAM_TILE && op->tile_cfg == TILE_256x256_W4 && (is_packed(d) || d.transpose_b == 0) && e >= 16 &&
      (d.kernel_override == OV_AUTO || d.kernel_override == OV_TILE_256_W4) && tuning().two_level != 0)
    op->small_group_rows = 64;
  op->stream_tch = 1;
  if (family == FAM_SKINNY && is_packed(d) && is_w8a8(d)) {
    // rows a group is expected to hold (shapes only): 16-row chunks up to 16 rows, else chunks of 32 / 64 / 128 rows
    // (several groups: 1.5 x the average, real routings are uneven and a group that overflows its chunk streams its
    // weights twice -- 128 rows over 8 experts: 90.5 us with 32-row chunks against 105 us with 16-row chunks)
    const int64_t avg = (m + e - 1) / e;
    const int64_t rows = e == 1 ? m : avg + avg / 2;
    op->stream_tch = rows <= 16 ? 1 : rows <= 32 ? 2 : rows <= 64 ? 4 : 8;
    // fewer, larger chunks when there would be more chunks than the grid should enumerate
    while (op->stream_tch < 8 && std::min<int64_t>(m, e) + m / (16 * op->stream_tch) > or_default(tuning().stream_max_slots, (int)kSkinnyMaxChunkSlots))
      op->stream_tch = op->stream_tch == 1 ? 2 : op->stream_tch * 2;
    if (tuning().stream_tch == 1 || tuning().stream_tch == 2 || tuning().stream_tch == 4 || tuning().stream_tch == 8) op->stream_tch = tuning().stream_tch;
  } else if (family == FAM_SKINNY && is_a16w8(d) && (is_packed(d) || (d.transpose_b == 0 && n % 16 == 0))) {
    // weight-only on packed or [E,K,N] weights: chunks of 32, 64 or 128 rows by the same estimate; larger groups stream
    // their weights once per chunk (8 experts, K = 4096, N = 14336, 128 / 512 / 2048 rows: 111 / 334 / 1307 us with
    // 16-row chunks)
    const int64_t avg = (m + e - 1) / e;
    const int64_t rows = e == 1 ? m : avg + avg / 2;
    op->stream_tch = rows <= 16 ? 1 : rows <= 32 ? 2 : rows <= 64 ? 4 : 8;
    while (op->stream_tch < 8 && std::min<int64_t>(m, e) + m / (16 * op->stream_tch) > or_default(tuning().stream_max_slots, (int)kSkinnyMaxChunkSlots))
      op->stream_tch *= 2;
    // One group whose column strips do not fill the chip: the multi-row kernels walk all of K in every workgroup (only
    // the 128-row form has a K split, below), and for few rows the 16-row kernels with their K split are faster
    // although they stream the weights once per 16 rows (K = 4096, N = 11008, 32 / 64 rows: packed 24 / 41 us against
    // 49 / 51; [E,K,N] 32 us against 39 at 32 rows -- its 33 to 64 rows go on to the 128-row form, 39 us against 48).
    if (e == 1 && (n + 127) / 128 < num_cus && m <= (is_packed(d) ? 64 : 32)) op->stream_tch = 1;
    if (tuning().stream_tch == 1 || tuning().stream_tch == 2 || tuning().stream_tch == 4 || tuning().stream_tch == 8)
      op->stream_tch = tuning().stream_tch;
  }
  if (family == FAM_SKINNY) {
    // grid.y enumerates (group, chunk of 16 * stream_tch rows)
    const int64_t chunk_rows = (int64_t)kSkinnyRows * op->stream_tch;
    op->max_chunks = (int)((m + chunk_rows - 1) / chunk_rows);
    if (op->max_chunks < 1) op->max_chunks = 1;
    if (e * op->max_chunks > 65535) family = FAM_GENERIC;
  }
  if (family == FAM_SKINNY) {
    // Only shapes enter: the number of (group, chunk) pairs that can hold rows is estimated from M and E.
    const int64_t active = std::max<int64_t>(
      1, std::min<int64_t>(e * op->max_chunks, std::min<int64_t>(m, e) + m / (kSkinnyRows * op->stream_tch)));
    const int64_t tiles128 = ((n + 127) / 128) * active;
    int wide16 = is_w8a8(d) && tiles128 <= num_cus && !is_packed(d);
    const int forced_variant = tuning().skinny_wide16;
    if (forced_variant >= 0 && is_w8a8(d)) wide16 = forced_variant != 0;
    op->skinny_wide16 = wide16;
    int want, cap;
    if (op->stream_tch > 1 && !is_w8a8(d)) {
      // multi-row weight-only kernels: strips of 16 column groups (256 columns) when they still give every CU two
      // workgroups, else of 8; every workgroup walks all of K (one exception below).
      const int64_t col_groups = (n + 15) / 16;
      op->strip_groups = ((col_groups + 15) / 16) * active >= 2 * (int64_t)num_cus ? 16 : 8;
      op->n_strips = (int)((col_groups + op->strip_groups - 1) / op->strip_groups);
      op->skinny_cols = op->strip_groups * 16;
      want = cap = 1;
      // One group whose strips leave most CUs idle: 128-row chunks with a K split (slices of at least 8 blocks) up to
      // about two workgroups per CU.  K = 4096, N = 11008, 128 / 256 / 512 rows without it: 59 / 61 / 83 us.
      const int64_t base = (int64_t)op->n_strips * active, k_blocks = (k + 63) / 64;
      if (e == 1 && base < num_cus && tuning().stream_tch == 0) {
        op->stream_tch = 8;
        op->max_chunks = (int)((m + 127) / 128);
        want = (int)std::min<int64_t>(kTargetWorkgroups / std::max<int64_t>((int64_t)op->n_strips * op->max_chunks, 1), kMaxSplitK);
        cap = std::max<int>(1, (int)(k_blocks / 8));
      }
    } else if (is_packed(d) && op->stream_tch > 1) {
      // multi-row kernel: strips of four column groups, K split until about two workgroups per CU stream operands
      const int64_t col_groups = (n + 15) / 16, k_blocks = (k + 63) / 64;
      op->strip_groups = 4;
      op->n_strips = (int)((col_groups + 3) / 4);
      op->skinny_cols = 64;
      const int64_t base = (int64_t)op->n_strips * active;
      want = (int)(kTargetWorkgroups / std::max<int64_t>(base, 1));
      cap = std::max<int>(1, (int)(k_blocks / 16));      // a slice keeps at least 16 blocks
      want = std::max(1, std::min(std::min(want, kMaxSplitK), cap));
    } else if (is_packed(d)) {
      // Packed weights: strips as wide as still give every CU a workgroup without splitting K (a slice holds at
      // most 128 blocks of 64 bytes), then a K split up to about two workgroups per CU.
      const int64_t col_groups = (n + 15) / 16, k_blocks = (k + 63) / 64;
      const int slice_blocks = is_w8a8(d) ? 128 : 64;
      const int floor_split = (int)((k_blocks + slice_blocks - 1) / slice_blocks);
      int groups = 16;
      const int min_wgs = or_default(tuning().stream_min_wgs, num_cus);
      while (groups > 1 && ((col_groups + groups - 1) / groups) * active * floor_split < min_wgs) groups /= 2;
      const int forced_groups = tuning().stream_groups;
      if (forced_groups >= 1 && forced_groups <= 16) groups = forced_groups;
      op->strip_groups = groups;
      op->n_strips = (int)((col_groups + groups - 1) / groups);
      op->skinny_cols = groups * 16;
      const int64_t base = (int64_t)op->n_strips * active;
      want = (int)(kTargetWorkgroups / std::max<int64_t>(base, 1));
      cap = std::max<int>(1, (int)(k_blocks / 16));      // a slice keeps at least 16 blocks
      want = std::max(floor_split, std::min(std::min(want, kMaxSplitK), cap));
      cap = kMaxSplitK * 64;
    } else if (wide16) {
      // at most one 16-wave workgroup per CU, every wave keeps at least one block
      want = (int)(num_cus / std::max<int64_t>(tiles128, 1));
      cap = std::max<int>(1, (int)(d.transpose_b ? (k + 63) / 64 : (k + 31) / 32) / 16);
      want = std::min(want, 8);
    } else {
      // K is split across workgroups until about kTargetWorkgroups of them stream weights
      const int64_t base = (int64_t)op->n_strips * active;
      const int target = or_default(tuning().skinny_target_wgs, 2 * num_cus);
      want = (int)((target + base / 2) / base);
      cap = std::max<int>(1, (int)(d.transpose_b ? (k + 63) / 64 : (k + 31) / 32) / 4);
      want = std::min(want, kMaxSplitK);
    }
    want = std::max(1, std::min(want, cap));
    const int forced = d.force_split_k > 0 ? d.force_split_k : tuning().skinny_split_k;
    if (forced > 0) want = std::min(forced, cap);
    if (is_packed(d) && op->stream_tch == 1) {   // also under a forced split
      const int slice_blocks = is_w8a8(d) ? 128 : 64;
      want = std::max(want, (int)(((k + 63) / 64 + slice_blocks - 1) / slice_blocks));
    }
    if (op->stream_tch > 1 && !is_w8a8(d) && !(e == 1 && op->stream_tch == 8)) want = 1;   // the multi-row weight-only kernels walk all of K, but for one group in 128-row chunks
    op->split_k = want;
    if (!is_packed(d) && !(op->stream_tch > 1 && !is_w8a8(d))) op->skinny_cols = wide16 ? 128 : kSkinnyCols;
    if (op->stream_tch > 1 && !is_w8a8(d)) {
      op->workspace_bytes = op->split_k > 1 ? (size_t)e * op->max_chunks * op->n_strips * op->split_k * rows32_a16w8_slice_bytes(op->strip_groups) : 0;
    } else if (is_packed(d)) {
      // the packed-layout kernels keep a full 16 x 256 partial tile per (strip, K slice) whatever the strip's width
      const size_t tile_bytes = !is_w8a8(d)           ? stream_a16w8_tile_bytes()
                                : op->stream_tch > 1 ? streamm_tile_bytes(op->stream_tch)
                                                     : (size_t)kSkinnyRows * kSkinnyCols * 4;
      const size_t tiles = op->stream_tch > 1 ? (size_t)e * op->max_chunks * op->n_strips
                                              : skinny_counter_count(m, n, e, op->skinny_cols);
      op->workspace_bytes = op->split_k > 1 ? tiles * (size_t)op->split_k * tile_bytes : 0;
    } else {
      op->workspace_bytes = is_w8a8(d) ? skinny_workspace_bytes(m, n, e, op->split_k, op->skinny_cols)
                                       : a16w8_workspace_bytes(m, n, e, op->split_k);
    }
  }
  op->family = family;

  char buf[320];
  const char *fam = family == FAM_TILE ? "tile" : family == FAM_SKINNY ? "skinny" : "generic";
  std::snprintf(buf, sizeof(buf),
                "msco_gmm plan: kernel=%s%s%s%s layout=%s m=%lld k=%lld n=%lld e=%lld split_k=%d strips=%d "
                "workspace=%zu%s",
                is_w8a8(d) ? "w8a8_" : "a16w8_", (family == FAM_SKINNY && is_packed(d)) ? (op->stream_tch > 1 ? "stream_rows" : "stream")
                : (family == FAM_SKINNY && op->stream_tch > 1)    ? "skinny_rows" : fam,
                family == FAM_TILE ? (std::string("_") + tile_cfg_name(op->tile_cfg)).c_str() : "",
                (family == FAM_SKINNY && op->skinny_wide16) ? "_16w" : "",
                is_packed(d) ? "packed" : d.transpose_b ? "[E,N,K]" : "[E,K,N]", (long long)m, (long long)k, (long long)n, (long long)e,
                op->split_k, op->n_strips, op->workspace_bytes,
                op->small_group_rows > 0 ? (" small_groups=" + std::to_string(op->small_group_rows) + ":tile_64x128").c_str() : "");
  op->info = buf;
}

}  // namespace

extern "C" {

int msco_gmm_abi_version(void) { return MSCO_GMM_ABI_VERSION; }

const char *msco_status_string(int status) {
  switch (status) {
    case MSCO_OK: return "ok";
    case MSCO_ERR_INVALID_ARG: return "invalid argument";
    case MSCO_ERR_UNSUPPORTED: return "unsupported dtype or layout";
    case MSCO_ERR_SHAPE: return "shape rule violated";
    case MSCO_ERR_NOT_PLANNED: return "launch before plan";
    case MSCO_ERR_WORKSPACE: return "workspace missing or too small";
    case MSCO_ERR_DEVICE: return "HIP runtime error";
    default: return "unknown status";
  }
}

int msco_gmm_create(const msco_gmm_desc *desc, msco_gmm_handle *out_handle) {
  if (desc == nullptr || out_handle == nullptr) return MSCO_ERR_INVALID_ARG;
  const int rc = check_desc(*desc);
  if (rc != MSCO_OK) return rc;
  msco_gmm_op *op = new (std::nothrow) msco_gmm_op();
  if (op == nullptr) return MSCO_ERR_DEVICE;
  op->desc = *desc;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
      cus > 0) {
    op->num_cus = cus;
  } else {
    (void)hipGetLastError();   // no device yet: planning falls back to the MI355X count, launch reports the error
  }
  *out_handle = op;
  return MSCO_OK;
}

int msco_gmm_plan(msco_gmm_handle h, int64_t m, int64_t k, int64_t n, int64_t e, size_t *workspace_bytes) {
  if (h == nullptr) return MSCO_ERR_INVALID_ARG;
  if (m < 0 || k <= 0 || n <= 0 || e <= 0) return MSCO_ERR_SHAPE;
  if (m > INT32_MAX || k > INT32_MAX || n > INT32_MAX || e > 65535 || m * n > ((int64_t)1 << 40)) return MSCO_ERR_SHAPE;
  if (h->desc.group_list_dtype == MSCO_DT_NONE && m % e != 0) return MSCO_ERR_SHAPE;
  std::lock_guard<std::mutex> lock(h->mu);
  h->m = m; h->k = k; h->n = n; h->e = e;
  choose_plan(h);
  if ((h->family == FAM_SKINNY || h->family == FAM_TILE) && h->split_k > 1) {
    const size_t need = h->family == FAM_TILE ? tile_count_bound(h->tile_cfg, m, n, e)
                                              : skinny_counter_count(m, n, e, h->skinny_cols);
    if (need > h->counters_cap) {
      if (h->counters) (void)hipFree(h->counters);
      h->counters = nullptr;
      h->counters_cap = 0;
      if (hipMalloc(reinterpret_cast<void **>(&h->counters), need * sizeof(unsigned)) != hipSuccess) {
        (void)hipGetLastError();
        return MSCO_ERR_DEVICE;
      }
      if (hipMemset(h->counters, 0, need * sizeof(unsigned)) != hipSuccess) {
        (void)hipGetLastError();
        return MSCO_ERR_DEVICE;
      }
      h->counters_cap = need;
    } else if (h->counters != nullptr) {
      // the counters reset themselves at the end of a launch; one that was abandoned half-way (a failed launch, a
      // destroyed stream) may have left tickets behind, so a new plan starts from zero again
      if (hipMemset(h->counters, 0, h->counters_cap * sizeof(unsigned)) != hipSuccess) {
        (void)hipGetLastError();
        return MSCO_ERR_DEVICE;
      }
    }
  }
  h->planned = true;
  if (workspace_bytes) *workspace_bytes = h->workspace_bytes;
  if (tuning().print_plan) std::fprintf(stderr, "%s\n", h->info.c_str());
  return MSCO_OK;
}

int msco_gmm_plan_info(msco_gmm_handle h, char *buf, size_t buf_len) {
  if (h == nullptr) return -1;
  std::lock_guard<std::mutex> lock(h->mu);
  if (buf && buf_len) {
    std::strncpy(buf, h->info.c_str(), buf_len - 1);
    buf[buf_len - 1] = '\0';
  }
  return (int)h->info.size();
}

int msco_gmm_launch(msco_gmm_handle h, const void *const *inputs, void *out, void *workspace, size_t workspace_bytes,
                    void *stream) {
  if (h == nullptr || inputs == nullptr) return MSCO_ERR_INVALID_ARG;
  if (!h->planned) return MSCO_ERR_NOT_PLANNED;
  const msco_gmm_desc &d = h->desc;
  if (h->m == 0) return MSCO_OK;
  if (out == nullptr || inputs[MSCO_IN_X] == nullptr || inputs[MSCO_IN_WEIGHT] == nullptr) return MSCO_ERR_INVALID_ARG;
  // a present dtype needs a pointer, an absent one must not get one
  auto need = [&](int slot, int dtype) { return (dtype != MSCO_DT_NONE) == (inputs[slot] != nullptr); };
  if (!need(MSCO_IN_BIAS, d.bias_dtype) || !need(MSCO_IN_SCALE, d.scale_dtype) ||
      !need(MSCO_IN_GROUP_LIST, d.group_list_dtype) || !need(MSCO_IN_PER_TOKEN_SCALE, d.per_token_dtype) ||
      !need(MSCO_IN_ANTIQUANT_SCALE, d.antiquant_dtype))
    return MSCO_ERR_INVALID_ARG;
  if ((d.has_antiquant_offset != 0) != (inputs[MSCO_IN_ANTIQUANT_OFFSET] != nullptr)) return MSCO_ERR_INVALID_ARG;
  if (h->workspace_bytes > 0 && (workspace == nullptr || workspace_bytes < h->workspace_bytes))
    return MSCO_ERR_WORKSPACE;

  GmmParams p{};
  p.x = inputs[MSCO_IN_X];
  p.w = static_cast<const int8_t *>(inputs[MSCO_IN_WEIGHT]);
  p.bias = static_cast<const int32_t *>(inputs[MSCO_IN_BIAS]);
  p.scale = inputs[MSCO_IN_SCALE];
  p.group_list = inputs[MSCO_IN_GROUP_LIST];
  p.per_token = static_cast<const float *>(inputs[MSCO_IN_PER_TOKEN_SCALE]);
  p.aq_scale = inputs[MSCO_IN_ANTIQUANT_SCALE];
  p.aq_offset = inputs[MSCO_IN_ANTIQUANT_OFFSET];
  p.out = out;
  p.partial = static_cast<int32_t *>(workspace);
  p.counters = h->counters;
  p.m = (int)h->m; p.k = (int)h->k; p.n = (int)h->n; p.e = (int)h->e;
  p.gl_dtype = d.group_list_dtype;
  p.gl_type = d.group_list_type;
  p.scale_dtype = d.scale_dtype;
  p.scale_per_group = d.scale_per_group;
  p.scale_is_scalar = d.scale_is_scalar;
  p.out_dtype = d.out_dtype;
  p.x_dtype = d.x_dtype;
  p.split_k = h->split_k;
  p.n_strips = h->n_strips;
  p.max_chunks = h->max_chunks;
  p.strip_groups = h->strip_groups;
  p.act_type = d.act_type;
  // rows a 16-row chunk is expected to hold (shapes only): measured on the dense 45 MB decode, 16 rows 13.1 -> 12.35 us with
  // the x rows staged through LDS, one row 11.85 -> 12.2 us, four rows per chunk (8 experts x 32 rows) 70.1 -> 70.4 us
  p.x_via_lds = (h->e > 0 ? (h->m + h->e - 1) / h->e : h->m) >= 8;
  p.wide_k_slabs = h->wide_k_slabs;
  p.w_nontemporal = h->w_nontemporal;
  p.rows_lo = 0;
  p.rows_hi = 0x7FFFFFFF;

  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t err = hipSuccess;
  const bool nk = d.transpose_b != 0;
  const int layout = layout_of(d);
  if (is_w8a8(d)) {
    if (h->family == FAM_TILE && h->small_group_rows > 0) {
      GmmParams big = p, small = p;
      big.rows_lo = h->small_group_rows;
      small.rows_hi = h->small_group_rows;
      small.split_k = 1;
      small.wide_k_slabs = 0;              // (128-byte slabs measured slower here: 340 against 336 us)
      small.w_nontemporal = layout == 2 || !nk;   // each small group's weights are read by one m-tile (packed, [E,K,N])
      err = launch_tile_w8a8(big, h->tile_cfg, nk, layout == 2, s);
      if (err == hipSuccess) err = launch_tile_w8a8(small, TILE_64x128, nk, layout == 2, s);
    } else if (h->family == FAM_TILE) err = launch_tile_w8a8(p, h->tile_cfg, nk, layout == 2, s);
    else if (h->family == FAM_SKINNY && layout == 2) err = h->stream_tch > 1 ? launch_streamm_w8a8(p, h->stream_tch, s) : launch_stream_w8a8(p, s);
    else if (h->family == FAM_SKINNY) err = launch_skinny_w8a8(p, nk, h->skinny_wide16 != 0, s);
    else err = launch_generic_w8a8(p, layout, s);
  } else {
    if (h->family == FAM_SKINNY && h->stream_tch > 1) err = launch_streamm_a16w8(p, h->stream_tch, layout == 2, s);
    else if (h->family == FAM_SKINNY && layout == 2) err = launch_stream_a16w8(p, s);
    else if (h->family == FAM_SKINNY) err = launch_skinny_a16w8(p, s);
    else err = launch_generic_a16w8(p, layout, s);
  }
  return err == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

// ---- launch without a caller workspace ----------------------------------------------------------------------------
// The split-K partial tiles go to a fixed device array instead of a caller buffer.  Host code never passes the array's
// name to a kernel or a runtime call (on the host it is a stand-in, not a device address): the address on each device
// is looked up once with hipGetSymbolAddress, with that device current, and kept.
namespace {
static __device__ __align__(256) unsigned char scratch[MSCO_GMM_STATIC_WORKSPACE_BYTES];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};

// the current device's copy of `scratch`; nullptr (and *status set) on failure
void *scratch_of_current_device(int *status) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    *status = MSCO_ERR_DEVICE;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      *status = MSCO_ERR_DEVICE;
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

int msco_gmm_launch_static(msco_gmm_handle h, const void *const *inputs, void *out, void *stream) {
  if (h == nullptr || inputs == nullptr) return MSCO_ERR_INVALID_ARG;
  if (!h->planned) return MSCO_ERR_NOT_PLANNED;
  if (h->workspace_bytes > (size_t)MSCO_GMM_STATIC_WORKSPACE_BYTES) {
    std::fprintf(stderr, "msco_gmm_launch_static: the plan needs %zu bytes of workspace, the static one holds %zu\n",
                 h->workspace_bytes, (size_t)MSCO_GMM_STATIC_WORKSPACE_BYTES);
    return MSCO_ERR_WORKSPACE;
  }
  int status = MSCO_OK;
  void *ws = scratch_of_current_device(&status);
  if (ws == nullptr) return status;
  // nothing in the array has to start at zero: every K slice writes its whole partial tile before it takes a ticket,
  // and the tickets live in the handle
  return msco_gmm_launch(h, inputs, out, ws, (size_t)MSCO_GMM_STATIC_WORKSPACE_BYTES, stream);
}

int msco_transpose_2d(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int32_t elem_bytes,
                      void *stream) {
  if (batch < 0 || rows < 0 || cols < 0 || batch > 65535) return MSCO_ERR_SHAPE;
  if (batch * rows * cols == 0) return MSCO_OK;
  if (src == nullptr || dst == nullptr) return MSCO_ERR_INVALID_ARG;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) return MSCO_ERR_UNSUPPORTED;
  const hipError_t err =
    launch_transpose_2d(src, dst, batch, rows, cols, elem_bytes, static_cast<hipStream_t>(stream));
  return err == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

size_t msco_packed_weight_bytes(int64_t k, int64_t n) {
  if (k <= 0 || n <= 0) return 0;
  return packed_weight_bytes(k, n);
}

int msco_pack_weight(const void *src, void *dst, int64_t e, int64_t k, int64_t n, int32_t src_transposed, void *stream) {
  if (e < 0 || k < 0 || n < 0 || k > INT32_MAX || n > INT32_MAX) return MSCO_ERR_SHAPE;
  if (e * k * n == 0) return MSCO_OK;
  if (src == nullptr || dst == nullptr) return MSCO_ERR_INVALID_ARG;
  if ((e * (int64_t)(packed_weight_bytes(k, n) / 16) + 255) / 256 > 0x7FFFFFFFll) return MSCO_ERR_SHAPE;
  const hipError_t err = launch_pack_weight(src, dst, e, k, n, src_transposed != 0, static_cast<hipStream_t>(stream));
  return err == hipSuccess ? MSCO_OK : MSCO_ERR_DEVICE;
}

int msco_gmm_destroy(msco_gmm_handle h) {
  if (h == nullptr) return MSCO_ERR_INVALID_ARG;
  if (h->counters) (void)hipFree(h->counters);
  delete h;
  return MSCO_OK;
}

}  // extern "C"
