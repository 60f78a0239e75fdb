"""GPU parity of the HIP backend against the CPU oracle, through the C ABI (ctypes).

Bar: int32 accumulators bit-exact; bf16 output within 1 bf16 ulp of the oracle
(|err| <= 2**-7 * |ref|) -- in practice bit-exact too, which is asserted as well because the
epilogue performs the same float32 operations in the same order."""
import json
import os

import numpy as np
import pytest

from ms_custom_ops_amd import cabi, workloads
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FAMILIES = [("generic", cabi.OV_GENERIC), ("skinny", cabi.OV_SKINNY), ("tile64", cabi.OV_TILE_64),
            ("tile128", cabi.OV_TILE_128), ("tile256", cabi.OV_TILE_256), ("tile256_w4", cabi.OV_TILE_256_W4),
            ("tile256_w4_mfma32", cabi.OV_TILE_256_W4_MFMA32)]


def _inputs(seed, m, k, n, e):
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    return rng, x, w, bias, scale, pt


def _check(x, w, gl, bias, scale, pt, *, transpose_b, override, group_list_type=0, gl_dtype=np.int64):
    from gpu_utils import run_w8a8
    starts, ends = O.group_bounds(gl, group_list_type)
    last = int(ends[-1])
    ref_acc = O.grouped_matmul_w8a8(x, w, gl, bias, group_list_type=group_list_type, out_dtype="i32")
    ref_bits = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, group_list_type=group_list_type)
    acc, info = run_w8a8(x, w, gl, bias, out="i32", transpose_b=transpose_b, override=override,
                         group_list_type=group_list_type, gl_dtype=gl_dtype, launches=2)
    assert np.array_equal(acc[:last], ref_acc[:last]), info
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=transpose_b, override=override,
                          group_list_type=group_list_type, gl_dtype=gl_dtype, launches=2)
    rel, bad = O.bf16_ulp_check(bits[:last], ref_bits[:last])
    assert bad == 0, (info, rel)                                  # the stated tolerance: 1 bf16 ulp
    assert np.array_equal(bits[:last], ref_bits[:last]), info     # and in fact bit-exact
    return info


@pytest.mark.parametrize("family,override", FAMILIES)
@pytest.mark.parametrize("transpose_b", [False, True])
def test_ragged_groups_with_empty_groups(device, family, override, transpose_b):
    rng, x, w, bias, scale, pt = _inputs(1, 333, 256, 384, 8)
    gl = [5, 5, 40, 100, 100, 230, 300, 333]   # two empty groups, ragged sizes
    _check(x, w, gl, bias, scale, pt, transpose_b=transpose_b, override=override)


@pytest.mark.parametrize("family,override", FAMILIES[1:])
@pytest.mark.parametrize("transpose_b", [False, True])
def test_k_and_n_tails_single_group_int32_list(device, family, override, transpose_b):
    # K = 160 is not a multiple of the 128-byte slab, N = 272 is not a multiple of any tile width
    rng, x, w, bias, scale, pt = _inputs(2, 300, 160, 272, 1)
    _check(x, w, [300], bias, scale, pt, transpose_b=transpose_b, override=override, gl_dtype=np.int32)


@pytest.mark.parametrize("transpose_b", [False, True])
def test_unaligned_shapes_take_the_generic_kernel(device, transpose_b):
    rng, x, w, bias, scale, pt = _inputs(3, 37, 100, 24, 2)   # K % 16 != 0, N % 16 != 0
    info = _check(x, w, [10, 37], bias, scale, pt, transpose_b=transpose_b, override=cabi.OV_AUTO)
    assert "generic" in info


@pytest.mark.parametrize("m,e,gl", [(16, 1, [16]), (1, 1, [1]), (12, 8, [0, 3, 3, 4, 9, 9, 12, 12])])
@pytest.mark.parametrize("transpose_b", [False, True])
def test_decode_shapes_use_split_k_and_stay_exact(device, m, e, gl, transpose_b):
    rng, x, w, bias, scale, pt = _inputs(4, m, 4096, 1024, e)
    info = _check(x, w, gl, bias, scale, pt, transpose_b=transpose_b, override=cabi.OV_AUTO)
    # either the K reduction is split across workgroups, or there are enough strips x groups for the
    # 16-wave workgroups that keep it inside one workgroup
    # ([E,N,K] weights take the 64 x 128 tile with its own K split at these sizes)
    assert ("skinny" in info or (transpose_b and "tile_64x128" in info)) and ("split_k=1 " not in info or "16w64c" in info)


def test_counts_and_last_boundary_below_m(device):
    rng, x, w, bias, scale, pt = _inputs(5, 200, 128, 256, 8)
    counts = [10, 0, 30, 20, 0, 50, 40, 25]   # sums to 175 < 200: rows 175.. are not part of any group
    for _, ov in FAMILIES:
        _check(x, w, counts, bias, scale, pt, transpose_b=False, override=ov, group_list_type=1)


def test_malformed_group_list_is_clamped_not_faulting(device):
    from gpu_utils import run_w8a8
    rng, x, w, bias, scale, pt = _inputs(6, 64, 128, 128, 4)
    bad = [10, 5, 1000, 64]   # decreasing and beyond M: clamped into [previous end, M] on the device
    good = [10, 10, 64, 64]
    for _, ov in FAMILIES:
        a, _ = run_w8a8(x, w, bad, bias, out="i32", override=ov)
        b, _ = run_w8a8(x, w, good, bias, out="i32", override=ov)
        assert np.array_equal(a, b)


@pytest.mark.parametrize("name", ["c1", "c2_m1", "c2_m16", "c2_m256", "c3", "c4"])
@pytest.mark.parametrize("transpose_b", [False, True])
def test_scaled_down_workloads_match_committed_digests(device, name, transpose_b):
    """The five configurations at 1/4 scale: regenerate the seeded inputs, prove they are the inputs the
    fixture was made from, and compare the GPU result with the oracle (bit-exact) and its digest."""
    import hashlib
    from gpu_utils import run_w8a8
    dig = json.load(open(os.path.join(GOLDEN, "digests.json")))[f"{name}/4"]
    wl = workloads.make(name, scale_down=4)
    sha = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
    assert sha(wl.x) == dig["x"] and sha(wl.w) == dig["w"] and wl.group_list.tolist() == dig["group_list"]
    if name == "c4":
        assert dig["empty_groups"] > 0 and dig["max_over_mean"] > 2.0
    acc, info = run_w8a8(wl.x, wl.w, wl.group_list, None, out="i32", transpose_b=transpose_b)
    assert sha(acc) == dig["acc"], info
    bits, info = run_w8a8(wl.x, wl.w, wl.group_list, wl.bias, wl.scale, wl.per_token, transpose_b=transpose_b)
    assert sha(bits) == dig["bf16"], info
    assert np.array_equal(bits, O.grouped_matmul_w8a8(wl.x, wl.w, wl.group_list, wl.bias, wl.scale, wl.per_token))


def test_committed_tiny_known_answer(device):
    from gpu_utils import run_w8a8
    k = np.load(os.path.join(GOLDEN, "kat_tiny.npz"))
    for _, ov in FAMILIES:
        for tb in (False, True):
            acc, _ = run_w8a8(k["x"], k["w"], k["group_list"], k["bias"], out="i32", override=ov, transpose_b=tb)
            assert np.array_equal(acc, k["acc_plus_bias"])
            bits, _ = run_w8a8(k["x"], k["w"], k["group_list"], k["bias"], k["scale"], k["per_token"], override=ov,
                               transpose_b=tb)
            assert np.array_equal(bits, k["bf16_bits"])
            f16, _ = run_w8a8(k["x"], k["w"], k["group_list"], k["bias"], k["scale"], k["per_token"], out="f16",
                              override=ov, transpose_b=tb)
            assert np.array_equal(f16, k["f16_bits"])


def test_scale_wire_formats_int64_bf16_scalar_and_shared_rows(device):
    from gpu_utils import run_w8a8
    rng, x, w, bias, scale, pt = _inputs(7, 96, 128, 128, 4)
    gl = [20, 50, 50, 96]
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    got, _ = run_w8a8(x, w, gl, bias, O.encode_scale_int64(scale), pt, scale_dtype=cabi.DT_I64)
    assert np.array_equal(got, ref)
    sb = O.f32_to_bf16_bits(scale)
    ref_b = O.grouped_matmul_w8a8(x, w, gl, bias, O.bf16_bits_to_f32(sb), pt)
    got, _ = run_w8a8(x, w, gl, bias, sb, pt, scale_dtype=cabi.DT_BF16)
    assert np.array_equal(got, ref_b)
    # one [N] row shared by all groups, and a single scalar
    ref_s = O.grouped_matmul_w8a8(x, w, gl, np.tile(bias[:1], (4, 1)), np.tile(scale[:1], (4, 1)), pt)
    got, _ = run_w8a8(x, w, gl, bias[0], scale[0], pt, scale_per_group=0)
    assert np.array_equal(got, ref_s)
    ref_1 = O.grouped_matmul_w8a8(x, w, gl, None, np.full((4, 128), scale[0, 0], np.float32), pt)
    got, _ = run_w8a8(x, w, gl, None, scale[0, :1], pt, scale_per_group=0, scale_is_scalar=1)
    assert np.array_equal(got, ref_1)


def test_dense_equal_groups_without_group_list(device):
    from gpu_utils import run_w8a8
    rng, x, w, bias, scale, pt = _inputs(8, 4 * 48, 128, 128, 4)
    ref = O.grouped_matmul_w8a8(x, w, [48, 96, 144, 192], None, scale, None)
    for _, ov in FAMILIES:
        got, _ = run_w8a8(x, w, None, None, scale, None, override=ov)
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("transpose_b", [False, True])
def test_few_tiles_split_k_across_workgroups(device, transpose_b):
    # 2 x 8 tiles of 64 x 128: the plan splits K across workgroups; partial tiles meet in the workspace
    rng, x, w, bias, scale, pt = _inputs(23, 100, 2064, 1024, 2)
    info = _check(x, w, [37, 100], bias, scale, pt, transpose_b=transpose_b, override=cabi.OV_AUTO)
    assert "tile_64x128" in info and "split_k=1 " not in info


# ------------------------------------------------------------- persistent four-wave tile kernel
W4 = cabi.OV_TILE_256_W4
# both forms of the persistent kernel: 16 x 16 x 64 MFMAs (what the plan takes) and 32 x 32 x 32
W4_FORMS = pytest.mark.parametrize("W4", [cabi.OV_TILE_256_W4, cabi.OV_TILE_256_W4_MFMA32], ids=["mfma16", "mfma32"])


@W4_FORMS
def test_w4_ragged_groups_k_tail_and_odd_slab_count(device, W4):
    # K = 1296: ten full 128-byte slabs and a 16-byte tail, an odd slab count (padded with a slab of
    # zeros); N = 400 leaves a partial n-tile; groups: empty, 1 row, exactly 256, 257, a few hundred
    rng, x, w, bias, scale, pt = _inputs(20, 1100, 1296, 400, 8)
    gl = [0, 1, 257, 257, 514, 600, 1099, 1100]
    info = _check(x, w, gl, bias, scale, pt, transpose_b=True, override=W4)
    assert "256x256x128_w4" in info


@W4_FORMS
def test_w4_workgroups_walk_several_tiles(device, W4):
    # 18 m-tiles x 16 n-tiles = 288 tiles for at most 256 persistent workgroups: some walk two tiles,
    # so the operand stream crosses a tile boundary, also into a tile of another group
    rng, x, w, bias, scale, pt = _inputs(21, 4200, 640, 4096, 3)
    info = _check(x, w, [1500, 1501, 4200], bias, scale, pt, transpose_b=True, override=W4)
    assert "256x256x128_w4" in info


@W4_FORMS
def test_w4_scale_wire_formats_f16_out_and_absent_operands(device, W4):
    from gpu_utils import run_w8a8
    rng, x, w, bias, scale, pt = _inputs(22, 700, 512, 528, 4)
    gl = [100, 300, 300, 700]
    kw = dict(transpose_b=True, override=W4)
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    got, info = run_w8a8(x, w, gl, bias, O.encode_scale_int64(scale), pt, scale_dtype=cabi.DT_I64, **kw)
    assert "256x256x128_w4" in info and np.array_equal(got, ref)
    sb = O.f32_to_bf16_bits(scale)
    got, _ = run_w8a8(x, w, gl, bias, sb, pt, scale_dtype=cabi.DT_BF16, **kw)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, bias, O.bf16_bits_to_f32(sb), pt))
    # one [N] row shared by all groups; a single scalar; no bias; no per-token scale
    got, _ = run_w8a8(x, w, gl, bias[0], scale[0], pt, scale_per_group=0, **kw)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, np.tile(bias[:1], (4, 1)), np.tile(scale[:1], (4, 1)), pt))
    got, _ = run_w8a8(x, w, gl, None, scale[0, :1], None, scale_per_group=0, scale_is_scalar=1, **kw)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, None, np.full((4, 528), scale[0, 0], np.float32), None))
    got, _ = run_w8a8(x, w, gl, bias, scale, pt, out="f16", **kw)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, out_dtype="f16").view(np.uint16))
    # counts instead of cumulative ends, int32 list, rows past the last boundary stay untouched
    counts = [100, 0, 250, 300]
    _check(x, w, counts, bias, scale, pt, transpose_b=True, override=W4, group_list_type=1, gl_dtype=np.int32)


# ------------------------------------------------------------------------------- weight-only path
def _a16w8_bound(k):
    return k


@pytest.mark.parametrize("override", [cabi.OV_AUTO, cabi.OV_GENERIC])
def test_weight_only_known_answer_fixture(device, override):
    """Tolerance (floating point): |out - exact| <= 2**-7 * |exact| + 1e-5 * sum_k |x (w+o) s| --
    one bf16 ulp for the final rounding plus float32 accumulation noise relative to the magnitude of
    the summed terms (the sums cancel, so a purely relative bound is not meaningful)."""
    from gpu_utils import run_a16w8
    k = np.load(os.path.join(GOLDEN, "kat_a16w8.npz"))
    bits, info = run_a16w8(k["x_bf16"], k["w"], k["scale_bf16"], k["offset_bf16"], k["ends"], override=override)
    last = int(k["ends"][-1])
    got = O.bf16_bits_to_f32(bits[:last]).astype(np.float64)
    exact, mag = k["expected_f64"][:last], k["abs_sum_f64"][:last]
    assert (np.abs(got - exact) <= 2.0 ** -7 * np.abs(exact) + 1e-5 * mag).all(), info


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_weight_only_scaled_c5_and_constant_scale_case(device, dtype):
    from gpu_utils import run_a16w8
    wl = workloads.make("c5", scale_down=4)
    if dtype == "bf16":
        x, s, o = wl.x, wl.scale, wl.offset
        xf, sf, of = (O.bf16_bits_to_f32(v) for v in (x, s, o))
        to_f = O.bf16_bits_to_f32
    else:
        xf = O.bf16_bits_to_f32(wl.x).astype(np.float16).astype(np.float32)
        sf = O.bf16_bits_to_f32(wl.scale).astype(np.float16).astype(np.float32)
        of = O.bf16_bits_to_f32(wl.offset).astype(np.float16).astype(np.float32)
        x, s, o = (v.astype(np.float16).view(np.uint16) for v in (xf, sf, of))
        to_f = lambda b: b.view(np.float16).astype(np.float32)
    exact = O.a16w8_grouped_f64(xf, wl.w, sf, of, wl.group_list)
    starts, ends = O.group_bounds(wl.group_list)
    mag = np.zeros_like(exact)
    for g in range(wl.e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(wl.w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    bits, info = run_a16w8(x, wl.w, s, o, wl.group_list, dtype=dtype)
    got = to_f(bits).astype(np.float64)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (np.abs(got - exact) <= ulp * np.abs(exact) + 1e-5 * mag).all(), info
    assert "skinny" in info


@pytest.mark.parametrize("m", [40, 300])
@pytest.mark.parametrize("layout", ["kn", "nk", "packed"])
def test_hundreds_of_experts_few_rows_decode_kernels_enumerate_only_chunks_with_rows(device, m, layout):
    """256 experts, 40 and 300 rows (the reference's DeepSeek-shaped cases, tests/st/test_grouped_matmul.py:190-204, at a
    small K and N): most experts hold no row, some hold more than one 16-row chunk.  The decode kernels' grid counts
    chunks that hold rows, not experts; every layout stays bit-exact, for cumulative and for count lists."""
    from gpu_utils import run_w8a8
    e, k, n = 256, 128, 272
    rng, x, w, bias, scale, pt = _inputs(40 + m, m, k, n, e)
    counts = np.zeros(e, dtype=np.int64)
    hit = rng.choice(e, size=m // 5, replace=False)
    if m > 40:
        counts[hit[0]] = 37                          # one expert with several 16-row chunks
    for _ in range(m - 5 - int(counts.sum())):       # (five rows stay behind the last boundary)
        counts[hit[rng.integers(1, len(hit))]] += 1
    ends = np.cumsum(counts)
    last = int(ends[-1])
    assert last == m - 5 and (counts == 0).sum() > e // 2 and (m == 40 or counts.max() > 32)
    ref = O.grouped_matmul_w8a8(x, w, ends, bias, scale, pt)
    ref_acc = O.grouped_matmul_w8a8(x, w, ends, bias, out_dtype="i32")
    for gl, gl_type in ((ends, 0), (counts, 1)):
        bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=layout == "nk", packed=layout == "packed",
                              group_list_type=gl_type, launches=2)
        # ([E,N,K] weights beyond 64 rows stay with the small tile kernel, whose tiles are cut per group as well)
        assert ("skinny" in info or "stream" in info or (layout == "nk" and m > 64 and "tile_64x128" in info)), info
        assert np.array_equal(bits[:last], ref[:last]), info
        assert (bits[last:] == 0x7FC0).all(), info     # rows past the last boundary are not written
        acc, info = run_w8a8(x, w, gl, bias, out="i32", transpose_b=layout == "nk", packed=layout == "packed",
                             group_list_type=gl_type)
        assert np.array_equal(acc[:last], ref_acc[:last]), info


@pytest.mark.parametrize("layout", ["kn", "nk", "packed"])
def test_groups_of_about_a_hundred_rows_take_128_row_tiles_and_the_forced_128x256_family_agrees(device, layout):
    """Eight groups of 70 .. 126 rows (the MoE layer at a few hundred tokens): the plan gives them 128-row m-tiles while
    1.5 x the average group stays within 174 rows, and 256-row tiles beyond; both are bit-exact, and so is the 128 x 256
    family when it is forced (kernel_override 7) on groups that spill into a second m-tile."""
    from gpu_utils import run_w8a8
    e, k, n = 8, 512, 6144
    for counts, want in (([96, 70, 126, 101, 88, 113, 90, 84], "128x256"), ([120, 131, 96, 150, 118, 109, 140, 96], "256x256")):
        m = sum(counts) + 3                       # (three rows stay behind the last boundary)
        rng, x, w, bias, scale, pt = _inputs(m, m, k, n, e)
        ends = np.cumsum(counts)
        last = int(ends[-1])
        ref = O.grouped_matmul_w8a8(x, w, ends, bias, scale, pt)
        for override in (0, cabi.OV_TILE_128x256):
            bits, info = run_w8a8(x, w, ends, bias, scale, pt, out="bf16", transpose_b=layout == "nk", packed=layout == "packed",
                                  override=override, launches=2)
            assert ("128x256" if override else want) in info, info
            assert np.array_equal(bits[:last], ref[:last]), info
            assert (bits[last:] == 0x7FC0).all(), info
