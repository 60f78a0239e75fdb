"""The row-chunk kernels for packed weights (kernel_override 9: chunks of up to 128 rows, 10: of up to 256 rows, 11: of up to 160 rows; several groups of a few dozen to a few hundred rows): the
group's x rows pass through LDS, the weights go from memory straight into MFMA operands.  GPU parity against the CPU
oracle through the C ABI; bar: int32 accumulators and 16-bit outputs bit-exact."""
import numpy as np
import pytest

from ms_custom_ops_amd import cabi
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(seed, m, k, n, e):
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    return x, w, bias, scale, pt


BOTH = [cabi.OV_ROWS128, cabi.OV_ROWS256, cabi.OV_ROWS160]
NAME = {cabi.OV_ROWS128: "_rows128", cabi.OV_ROWS256: "_rows256", cabi.OV_ROWS160: "_rows160"}


def _check(x, w, gl, bias, scale, pt, *, override, group_list_type=0, src_transposed=False):
    from gpu_utils import run_w8a8
    _, ends = O.group_bounds(gl, group_list_type)
    last = int(ends[-1])
    ref_acc = O.grouped_matmul_w8a8(x, w, gl, bias, group_list_type=group_list_type, out_dtype="i32")
    ref_bits = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, group_list_type=group_list_type)
    acc, info = run_w8a8(x, w, gl, bias, out="i32", override=override, packed=True, transpose_b=src_transposed,
                         group_list_type=group_list_type, launches=2)
    assert NAME[override] in info and "layout=packed" in info, info
    assert np.array_equal(acc[:last], ref_acc[:last]), info
    assert (acc[last:] == -7777).all(), info                       # rows past the last boundary stay untouched
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", override=override, packed=True,
                          transpose_b=src_transposed, group_list_type=group_list_type, launches=2)
    assert np.array_equal(bits[:last], ref_bits[:last]), info
    assert (bits[last:] == 0x7FC0).all(), info
    return info


@pytest.mark.parametrize("override", BOTH)
@pytest.mark.parametrize("m,k,n,e,gl", [
    (32, 128, 256, 1, [32]),                                    # one chunk, one slab, one strip
    (300, 640, 272, 2, [100, 300]),                             # a strip with one live column group; an odd number of slabs
    (700, 576, 528, 4, [100, 300, 300, 700]),                   # an odd number of 64-byte K blocks, an empty group, a group of two chunks
    (1500, 720, 1040, 8, [0, 40, 300, 300, 900, 1210, 1480, 1490]),   # K not a multiple of 64, ragged and empty groups
    (530, 4096, 512, 5, [1, 18, 19, 275, 530]),                 # 1, 17, 1, 256 and 255 rows: every block count edge
    (257, 192, 256, 1, [257]),                                  # a second chunk of one row
    (20, 80, 48, 2, [7, 20]),                                   # K of one and a quarter blocks, three column groups
])
def test_rows_kernel_is_bit_exact(device, m, k, n, e, gl, override):
    x, w, bias, scale, pt = _inputs(41, m, k, n, e)
    _check(x, w, gl, bias, scale, pt, override=override)


@pytest.mark.parametrize("override", BOTH)
@pytest.mark.parametrize("rows", [1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 159, 161, 191, 193, 223, 225, 255, 256])
def test_rows_kernel_every_block_count(device, rows, override):
    # two groups of `rows` rows and of 40: each number of live 16-row blocks has a K loop of its own (with 128-row
    # chunks the larger groups take two chunks)
    x, w, bias, scale, pt = _inputs(1000 + rows, rows + 40, 448, 304, 2)
    _check(x, w, [rows, rows + 40], bias, scale, pt, override=override)


@pytest.mark.parametrize("override", BOTH)
def test_rows_kernel_counts_list_and_rows_past_the_last_boundary(device, override):
    x, w, bias, scale, pt = _inputs(43, 400, 512, 768, 4)
    _check(x, w, [90, 0, 130, 150], bias, scale, pt, group_list_type=1, override=override)   # 370 of 400 rows


@pytest.mark.parametrize("override", BOTH)
@pytest.mark.parametrize("n", [3584, 3600, 2240, 208])
def test_rows_kernel_strip_widths(device, n, override):
    # the strip width follows the column count and the CU count (10 .. 16 column groups): wide N with and without a tail
    x, w, bias, scale, pt = _inputs(47 + n, 230, 256, n, 2)
    _check(x, w, [100, 230], bias, scale, pt, override=override)


def test_rows_kernel_from_transposed_source(device):
    x, w, bias, scale, pt = _inputs(44, 200, 320, 336, 3)
    _check(x, w, [70, 130, 200], bias, scale, pt, src_transposed=True, override=cabi.OV_ROWS128)


@pytest.mark.parametrize("override", BOTH)
@pytest.mark.parametrize("out,scale_dtype,act", [("f16", cabi.DT_F32, 0), ("bf16", cabi.DT_BF16, 0), ("bf16", cabi.DT_I64, 0),
                                                 ("bf16", cabi.DT_F32, cabi.ACT_SILU), ("f16", cabi.DT_F32, cabi.ACT_RELU),
                                                 ("bf16", cabi.DT_F32, cabi.ACT_FAST_GELU), ("bf16", cabi.DT_F32, cabi.ACT_GELU_TANH)])
def test_rows_kernel_output_types_scale_types_and_activations(device, out, scale_dtype, act, override):
    # whatever the 64 x 128 tile kernel writes for the same problem (itself checked against the oracle elsewhere)
    from gpu_utils import run_w8a8
    x, w, bias, scale, pt = _inputs(45, 260, 384, 528, 3)
    gl = [100, 101, 260]
    sc = scale
    if scale_dtype == cabi.DT_BF16:
        sc = O.f32_to_bf16_bits(scale)
    elif scale_dtype == cabi.DT_I64:
        sc = O.encode_scale_int64(scale)
    kw = dict(out=out, scale_dtype=scale_dtype, packed=True, act_type=act, launches=2)
    got, info = run_w8a8(x, w, gl, bias, sc, pt, override=override, **kw)
    assert "_rows" in info, info
    want, info2 = run_w8a8(x, w, gl, bias, sc, pt, override=cabi.OV_TILE_64, **kw)
    assert "64x128" in info2, info2
    assert np.array_equal(got, want), (info, info2)


def test_rows_kernel_without_bias_scale_or_per_token(device):
    from gpu_utils import run_w8a8
    x, w, bias, scale, pt = _inputs(46, 150, 256, 320, 2)
    gl = [60, 150]
    got, info = run_w8a8(x, w, gl, None, scale, None, override=cabi.OV_ROWS256, packed=True)
    assert "_rows" in info, info
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, None, scale, None))
    got, info = run_w8a8(x, w, gl, None, scale[0], pt, override=cabi.OV_ROWS256, packed=True, scale_per_group=0)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, None, np.broadcast_to(scale[0], scale.shape), pt))


@pytest.mark.parametrize("seed,per_group,want", [(0, 40, "rows128"), (1, 100, "rows128"), (2, 112, "rows128"), (3, 126, "rows160"), (4, 144, "rows160"), (5, 152, "rows256")])
def test_the_plan_picks_the_rows_kernels_for_several_groups_of_up_to_about_130_rows(device, seed, per_group, want):
    # eight groups, enough columns that 256-column strips give every CU a workgroup: 128-row chunks up to 116 rows per group
    # on average, 160-row chunks up to 146, 256-row chunks up to 155; uneven groups (some spill into a second chunk), three rows behind the last boundary
    from gpu_utils import run_w8a8
    rng = np.random.default_rng(7000 + seed)
    e, k, n = 8, 1024, 8192
    counts = np.maximum(1, rng.normal(per_group, per_group * 0.12, e).astype(np.int64))
    counts[-1] += per_group * e - counts.sum()          # the average is exact
    m = int(counts.sum()) + 3
    gl = np.cumsum(counts)
    x, w, bias, scale, pt = _inputs(300 + seed, m, k, n, e)
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", packed=True, launches=2)
    assert want in info and "layout=packed" in info, info
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    last = int(gl[-1])
    assert np.array_equal(bits[:last], ref[:last]), info
    assert (bits[last:] == 0x7FC0).all(), info



@pytest.mark.parametrize("seed", range(16))
def test_rows_kernels_random_shapes(device, seed):
    # a seeded sweep: one to seventeen groups, a handful to three hundred rows per group (several chunks per group for the
    # smaller forms), K with and without 64-byte tails, N from one column group to 225; every form against the oracle
    from gpu_utils import run_w8a8
    rng = np.random.default_rng(9000 + seed)
    e = int(rng.choice([1, 2, 3, 5, 8, 17]))
    per = int(rng.choice([3, 20, 60, 100, 128, 140, 170, 260, 300]))
    m = max(1, int(per * e * rng.uniform(0.6, 1.3)))
    k = int(rng.integers(1, 20)) * 64 + int(rng.choice([0, 0, 16, 32, 48]))
    n = int(rng.choice([16, 48, 224, 256, 272, 1008, 2240, 3600]))
    cuts = np.sort(rng.integers(0, m + 1, e - 1)) if e > 1 else np.array([], dtype=np.int64)
    gl = np.maximum.accumulate(np.concatenate([cuts, [m - int(rng.choice([0, 0, 5]))]]).astype(np.int64).clip(0))
    x, w, bias, scale, pt = _inputs(9000 + seed, m, k, n, e)
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    last = int(gl[-1])
    for override in BOTH:
        bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", packed=True, override=override, launches=2)
        assert NAME[override] in info, info
        assert np.array_equal(bits[:last], ref[:last]), (m, k, n, e, gl.tolist(), info)
        assert (bits[last:] == 0x7FC0).all(), info
