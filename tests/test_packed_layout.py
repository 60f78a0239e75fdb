"""The packed weight layout: the device-side packing against the layout's numpy restatement, and GPU parity of the kernels
that read it (the streaming decode kernel, the generic kernel for everything else) against the CPU oracle, through the
C ABI.  Bar as for the row-major layouts: int32 accumulators and bf16 outputs bit-exact."""
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


def _check(x, w, gl, bias, scale, pt, *, src_transposed=False, override=cabi.OV_AUTO, group_list_type=0, split=0):
    from gpu_utils import run_w8a8
    _, ends = O.group_bounds(gl, group_list_type)
    last = int(ends[-1])
    ref_acc = O.grouped_matmul_w8a8(x, w, gl, bias, group_list_type=group_list_type, out_dtype="i32")
    ref_bits = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, group_list_type=group_list_type)
    acc, info = run_w8a8(x, w, gl, bias, out="i32", transpose_b=src_transposed, override=override, packed=True,
                         group_list_type=group_list_type, launches=2, force_split_k=split)
    assert np.array_equal(acc[:last], ref_acc[:last]), info
    assert (acc[last:] == -7777).all(), info                       # rows past the last boundary stay untouched
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=src_transposed, override=override, packed=True,
                          group_list_type=group_list_type, launches=2, force_split_k=split)
    assert np.array_equal(bits[:last], ref_bits[:last]), info
    return info


@pytest.mark.parametrize("e,k,n,src_transposed", [(1, 64, 16, False), (3, 200, 40, False), (2, 4096, 272, True),
                                                  (8, 130, 1000, True)])
def test_device_packing_matches_the_layout_definition(device, e, k, n, src_transposed):
    import torch
    from gpu_utils import pack_on_device, to_dev
    w = np.random.default_rng(7).integers(-128, 128, (e, k, n), dtype=np.int8)
    src = np.ascontiguousarray(w.transpose(0, 2, 1)) if src_transposed else w
    got = pack_on_device(to_dev(src), e, k, n, src_transposed)
    torch.cuda.synchronize()
    assert cabi.packed_weight_bytes(k, n) == ((n + 15) // 16) * ((k + 63) // 64) * 1024
    assert np.array_equal(got.cpu().numpy().reshape(e, -1), O.pack_weights(w))


@pytest.mark.parametrize("m,k,n,e,gl", [
    (16, 4096, 512, 1, [16]),                                   # one strip walk per column group pair, no K split
    (13, 1024, 272, 2, [5, 13]),                                # N tail inside the last strip, short K
    (40, 2048, 1040, 4, [0, 17, 17, 40]),                       # empty groups, a group of two 16-row chunks
    (16, 4096 + 64 * 5, 256, 1, [16]),                          # K blocks not a multiple of the four waves
    (33, 720, 48, 3, [16, 16, 33]),                             # K not a multiple of 64: zero-padded last block
    (16, 11008, 4096, 1, [16]),                                 # K beyond one slice: split across workgroups
    (16, 64, 16, 1, [16]),                                      # a single block
    (20, 4096, 3584, 8, [2, 4, 4, 9, 12, 15, 18, 20]),          # MoE decode shape (quarter width), full-width strips
    (9, 8192, 512, 2, [4, 9]),                                  # 32 blocks per wave
])
def test_streaming_decode_kernel_is_bit_exact(device, m, k, n, e, gl):
    x, w, bias, scale, pt = _inputs(11, m, k, n, e)
    info = _check(x, w, gl, bias, scale, pt)
    assert "w8a8_stream" in info and "layout=packed" in info


@pytest.mark.parametrize("split", [2, 3, 8])
def test_streaming_decode_with_forced_k_split(device, split):
    x, w, bias, scale, pt = _inputs(12, 21, 2048, 528, 2)
    info = _check(x, w, [10, 21], bias, scale, pt, src_transposed=True, split=split)
    assert f"split_k={split} " in info


def test_counts_and_rows_past_the_last_boundary(device):
    x, w, bias, scale, pt = _inputs(13, 48, 1024, 256, 4)
    _check(x, w, [10, 0, 20, 5], bias, scale, pt, group_list_type=1)    # 35 of 48 rows belong to a group


@pytest.mark.parametrize("m,k,n,e,gl", [
    (32, 1024, 128, 1, [32]),                                   # two 16-row fragments per chunk
    (17, 512, 80, 1, [17]),                                     # one row into the second fragment, N tail
    (64, 2048, 272, 1, [64]),                                   # four fragments, K split across workgroups
    (128, 4096, 256, 1, [128]),                                 # eight fragments (the dense 128-row configuration's M and K)
    (300, 720, 144, 2, [100, 300]),                             # chunks of 128 rows, K not a multiple of 64
    (500, 512, 64, 8, [0, 40, 40, 200, 210, 350, 480, 490]),    # ragged groups, empty groups, rows past the last boundary
    (1000, 256, 1040, 4, [250, 500, 750, 1000]),                # several chunks per group, 17 strips
    (60, 1024, 160, 3, [25, 25, 60]),                           # a few dozen rows in several groups: planned by itself
])
def test_multi_row_streaming_kernel_is_bit_exact(device, m, k, n, e, gl):
    """Planned by itself for up to 64 rows in several groups; forced here for the other cases (one group of more than
    16 rows, or more rows, go to the tile kernels)."""
    x, w, bias, scale, pt = _inputs(16, m, k, n, e)
    auto = m <= 64 and e > 1
    info = _check(x, w, gl, bias, scale, pt, src_transposed=(e == 8), override=cabi.OV_AUTO if auto else cabi.OV_SKINNY)
    assert "w8a8_stream_rows" in info and "layout=packed" in info


def test_groups_of_about_a_hundred_rows_take_128_row_tiles_over_256_columns(device):
    # several groups whose 1.5-fold average size fits a 128-row m-tile, enough columns for three quarters of the CUs: one
    # group longer than the tile (140 rows: two m-tiles), one short (40), a tail of 60
    x, w, bias, scale, pt = _inputs(27, 320, 1024, 12288, 4)
    info = _check(x, w, [40, 180, 260, 320], bias, scale, pt)
    assert "w8a8_tile_128x256" in info and "layout=packed" in info, info


@pytest.mark.parametrize("m,k,n", [(17, 512, 80), (32, 4096, 1408), (48, 1024, 128), (64, 2048, 272)])
def test_one_group_of_17_to_64_rows_takes_the_small_tile_with_a_k_split(device, m, k, n):
    x, w, bias, scale, pt = _inputs(26, m, k, n, 1)
    info = _check(x, w, [m], bias, scale, pt)
    assert "w8a8_tile_64x128" in info and "layout=packed" in info, info


@pytest.mark.parametrize("family,override", [("64x128", cabi.OV_TILE_64), ("128x128", cabi.OV_TILE_128), ("256x256x64", cabi.OV_TILE_256)])
@pytest.mark.parametrize("m,k,n,e,gl,split", [
    (333, 256, 384, 8, [5, 5, 40, 100, 100, 230, 300, 333], 0),     # ragged and empty groups
    (300, 160, 272, 1, [300], 0),                                   # K and N tails
    (128, 2048, 512, 1, [128], 0),                                  # few tiles: K split across workgroups
    (200, 720, 144, 2, [90, 200], 2),                               # forced K split, K not a multiple of 64
])
def test_eight_wave_and_small_tile_kernels_on_packed_weights(device, family, override, m, k, n, e, gl, split):
    x, w, bias, scale, pt = _inputs(19, m, k, n, e)
    info = _check(x, w, gl, bias, scale, pt, override=override, split=split)
    assert f"tile_{family}" in info and "layout=packed" in info


def test_a_few_hundred_rows_on_packed_weights_take_the_small_tiles(device):
    x, w, bias, scale, pt = _inputs(20, 256, 1024, 4096, 1)
    info = _check(x, w, [256], bias, scale, pt)
    assert "w8a8_tile_" in info and "layout=packed" in info


@pytest.mark.parametrize("m,k,n,e,gl", [
    (256, 512, 256, 1, [256]),                                  # one tile, four slabs
    (300, 640, 272, 2, [100, 300]),                             # partial tiles, N tail inside a column group pair
    (700, 576, 528, 4, [100, 300, 300, 700]),                   # odd number of 64-byte K blocks: the last slab is half empty
    (2048, 1024, 768, 3, [1, 1030, 2048]),                      # workgroups walk several tiles
    (1500, 720, 1040, 8, [0, 40, 300, 300, 900, 1210, 1480, 1490]),   # K not a multiple of 64, ragged and empty groups
])
def test_persistent_tile_kernel_on_packed_weights_is_bit_exact(device, m, k, n, e, gl):
    x, w, bias, scale, pt = _inputs(17, m, k, n, e)
    info = _check(x, w, gl, bias, scale, pt, override=cabi.OV_TILE_256_W4)
    assert "tile_256x256x128_w4" in info and "layout=packed" in info


def test_prefill_sized_problems_on_packed_weights_take_the_tile_kernel(device):
    from gpu_utils import run_w8a8
    x, w, bias, scale, pt = _inputs(18, 4096, 512, 4096, 8)
    gl = [500, 1000, 1600, 2000, 2600, 3000, 3500, 4096]
    got, info = run_w8a8(x, w, gl, None, scale, pt, packed=True)
    assert "tile_256x256x128_w4" in info and "layout=packed" in info
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, None, scale, pt))


def test_forced_generic_kernel_on_packed_weights(device):
    x, w, bias, scale, pt = _inputs(14, 64, 512, 256, 2)
    info = _check(x, w, [30, 64], bias, scale, pt, override=cabi.OV_GENERIC)
    assert "generic" in info and "layout=packed" in info


def test_wire_formats_on_packed_weights(device):
    """bf16 scale, int64-encoded scale, a single shared scale row, fp16 output."""
    from gpu_utils import run_w8a8
    x, w, bias, scale, pt = _inputs(15, 16, 1024, 256, 2)
    gl = [7, 16]
    sb = O.f32_to_bf16_bits(scale)
    got, _ = run_w8a8(x, w, gl, None, sb, pt, out="bf16", scale_dtype=cabi.DT_BF16, packed=True)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, None, O.bf16_bits_to_f32(sb), pt))
    got, _ = run_w8a8(x, w, gl, bias, O.encode_scale_int64(scale), pt, out="bf16", scale_dtype=cabi.DT_I64, packed=True)
    assert np.array_equal(got, O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt))
    got, _ = run_w8a8(x, w, gl, bias[0], scale[0], pt, out="f16", scale_per_group=0, packed=True)
    ref = O.grouped_matmul_w8a8(x, w, gl, np.tile(bias[:1], (2, 1)), np.tile(scale[:1], (2, 1)), pt, out_dtype="f16")
    assert np.array_equal(got, ref.view(np.uint16))


# ------------------------------------------------------------------------------- weight-only path on packed weights
def _weight_only_case(seed, m, k, n, e, gl, dtype):
    rng = np.random.default_rng(seed)
    half = np.float16 if dtype == "f16" else None
    def to_bits(a):
        return a.astype(np.float16).view(np.uint16) if half else O.f32_to_bf16_bits(a.astype(np.float32))
    def to_f(b):
        return b.view(np.float16).astype(np.float32) if half else O.bf16_bits_to_f32(b)
    x = to_bits(rng.standard_normal((m, k)))
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    s = to_bits(rng.uniform(1e-3, 1e-2, (e, n)))
    o = to_bits(rng.integers(-8, 9, (e, n)).astype(np.float32))
    xf, sf, of = to_f(x), to_f(s), to_f(o)
    exact = O.a16w8_grouped_f64(xf, w, sf, of, gl)
    starts, ends = O.group_bounds(gl)
    mag = np.zeros_like(exact)
    for g in range(e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    return x, w, s, o, exact, mag, to_f, int(ends[-1])


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("m,k,n,e,gl", [
    (32, 1024, 3584, 8, [3, 7, 7, 12, 20, 25, 30, 32]),     # the weight-only decode configuration at quarter size
    (16, 4096, 272, 1, [16]),                               # 16 blocks per wave, N tail
    (40, 720, 48, 2, [17, 40]),                             # K not a multiple of 64, groups of two chunks
    (9, 8192 + 320, 256, 2, [4, 9]),                        # K beyond one slice: split across workgroups
])
def test_weight_only_streaming_kernel_within_tolerance(device, dtype, m, k, n, e, gl):
    """Tolerance (floating point, as for the row-major weight-only kernel): |out - exact| <= ulp * |exact| +
    1e-5 * sum_k |x (w + o) s|, ulp = 2**-7 (bf16) or 2**-10 (f16), against the float64 value of the reference's
    a16w8 golden (tests/st/test_grouped_matmul_v4_cops.py:166-174)."""
    from gpu_utils import run_a16w8
    x, w, s, o, exact, mag, to_f, last = _weight_only_case(21, m, k, n, e, gl, dtype)
    bits, info = run_a16w8(x, w, s, o, gl, dtype=dtype, packed=True)
    assert "a16w8_stream" in info and "layout=packed" in info
    got = to_f(bits).astype(np.float64)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (np.abs(got[:last] - exact[:last]) <= ulp * np.abs(exact[:last]) + 1e-5 * mag[:last]).all(), info
    # and the same inputs through the row-major kernel agree to the same bound (two float32 summation orders)
    bits_rm, _ = run_a16w8(x, w, s, o, gl, dtype=dtype)
    assert (np.abs(to_f(bits_rm).astype(np.float64)[:last] - got[:last]) <= 2 * ulp * np.abs(exact[:last]) + 2e-5 * mag[:last]).all()


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("m,k,n,e,gl", [
    (150, 1024 + 64, 272, 3, [70, 70, 150]),                # chunks of 64 rows: 64 + 6 rows, an empty group, 64 + 16; N tail
    (80, 2048, 128, 2, [64, 80]),                           # one full chunk of 64 rows and a quarter of one
    (33, 512 + 16, 64, 2, [20, 33]),                        # chunks of 32 rows, K not a multiple of 64
    (300, 4096, 512, 4, [10, 100, 100, 300]),               # chunks of 128 rows: groups of 10, 90, 0 and 200 (128 + 72) rows
    (260, 1024 + 48, 400, 2, [129, 260]),                   # 128 + 1 and 128 + 3 rows, K and N tails
    (1200, 320, 8192, 8, [100, 250, 400, 550, 700, 850, 1000, 1200]),   # chunks of 128 rows, strips of 256 columns
])
def test_weight_only_multi_row_streaming_kernel_within_tolerance(device, dtype, m, k, n, e, gl):
    """More than 16 rows per group on packed weights: chunks of 32, 64 or 128 rows share one pass over the group's weights
    (128-row chunks on 32 x 32 x 16 MFMAs, the packed blocks through LDS).
    Same tolerance as the 16-row kernel, against the float64 value of the reference's a16w8 golden."""
    from gpu_utils import run_a16w8
    x, w, s, o, exact, mag, to_f, last = _weight_only_case(23, m, k, n, e, gl, dtype)
    bits, info = run_a16w8(x, w, s, o, gl, dtype=dtype, packed=True)
    assert "a16w8_stream_rows" in info and "layout=packed" in info and "split_k=1 " in info, info
    got = to_f(bits).astype(np.float64)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (np.abs(got[:last] - exact[:last]) <= ulp * np.abs(exact[:last]) + 1e-5 * mag[:last]).all(), info
    assert (bits[last:] == 0x7FC0).all()   # rows past the last boundary keep the fill value
    # and the same inputs through the row-major kernel agree to the same bound (two float32 summation orders)
    bits_rm, _ = run_a16w8(x, w, s, o, gl, dtype=dtype)
    assert (np.abs(to_f(bits_rm).astype(np.float64)[:last] - got[:last]) <= 2 * ulp * np.abs(exact[:last]) + 2e-5 * mag[:last]).all()


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("m,k,n,e,gl", [
    (150, 1024 + 64, 272, 3, [70, 70, 150]),                # chunks of 64 rows: 64 + 6 rows, an empty group, 64 + 16; N tail
    (80, 2048, 128, 2, [64, 80]),                           # one full chunk of 64 rows and a quarter of one
    (33, 512 + 16, 64, 2, [20, 33]),                        # chunks of 32 rows, K not a multiple of 64
    (300, 4096, 512, 4, [10, 100, 100, 300]),               # chunks of 128 rows: groups of 10, 90, 0 and 200 (128 + 72) rows
    (160, 256, 14336, 8, [20, 40, 60, 80, 100, 120, 140, 160]),   # chunks of 32 rows, wide N: strips of 256 columns
    (260, 1024 + 48, 400, 2, [129, 260]),                   # chunks of 128 rows: 128 + 1 and 128 + 3 rows, K and N tails
    (700, 512, 4096, 2, [300, 700]),                        # chunks of 128 rows, strips of 128 columns
    (320, 256, 14336, 8, [40, 80, 120, 160, 200, 240, 280, 320]),       # chunks of 64 rows, strips of 256 columns
    (1200, 320, 8192, 8, [100, 250, 400, 550, 700, 850, 1000, 1200]),   # chunks of 128 rows, strips of 256 columns
])
def test_weight_only_multi_row_kernel_on_row_major_weights(device, dtype, m, k, n, e, gl):
    """The same on [E,K,N] weights as stored: the strip's weight slab goes through LDS and transpose reads turn it into
    MFMA operands (16 x 16 x 32 on 32-row chunks, 32 x 32 x 16 on 64- and 128-row chunks).  Tolerance as above; the
    packed layout's kernel agrees to the same bound."""
    from gpu_utils import run_a16w8
    x, w, s, o, exact, mag, to_f, last = _weight_only_case(24, m, k, n, e, gl, dtype)
    bits, info = run_a16w8(x, w, s, o, gl, dtype=dtype)
    assert "a16w8_skinny_rows" in info and "layout=[E,K,N]" in info and "split_k=1 " in info, info
    got = to_f(bits).astype(np.float64)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (np.abs(got[:last] - exact[:last]) <= ulp * np.abs(exact[:last]) + 1e-5 * mag[:last]).all(), info
    assert (bits[last:] == 0x7FC0).all()   # rows past the last boundary keep the fill value
    bits_p, _ = run_a16w8(x, w, s, o, gl, dtype=dtype, packed=True)   # the packed layout's kernel: another summation order
    assert (np.abs(to_f(bits_p).astype(np.float64)[:last] - got[:last]) <= 2 * ulp * np.abs(exact[:last]) + 2e-5 * mag[:last]).all()


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("m,k,n,last", [
    (128, 4096, 1024, 128),          # one full 128-row chunk, 8 strips: K in 8 slices
    (200, 1024 + 64, 400, 190),      # two chunks (128 + 62 rows), K and N tails, 17 blocks in slices of 9 and 8
    (70, 512 + 16, 2048, 70),        # 9 blocks: one slice
    (300, 8192, 256, 300),           # three chunks (the last with two live row fragments), 128 blocks in 8 slices
])
def test_weight_only_one_group_k_split(device, dtype, packed, m, k, n, last):
    """One group of more than 64 rows whose column strips leave most CUs idle: 128-row chunks with a K split, partial
    accumulators and row sums through the workspace, added in slice order by the last arriver.  Same tolerance against
    the float64 golden; a second launch on the same inputs gives the same bits (one summation order, counters back at zero)."""
    from gpu_utils import run_a16w8
    x, w, s, o, exact, mag, to_f, last_row = _weight_only_case(31, m, k, n, 1, [last], dtype)
    bits, info = run_a16w8(x, w, s, o, [last], dtype=dtype, packed=packed)
    assert ("a16w8_stream_rows" if packed else "a16w8_skinny_rows") in info, info
    if k >= 1024:
        assert "split_k=1 " not in info, info
    got = to_f(bits).astype(np.float64)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (np.abs(got[:last_row] - exact[:last_row]) <= ulp * np.abs(exact[:last_row]) + 1e-5 * mag[:last_row]).all(), info
    assert (bits[last_row:] == 0x7FC0).all()
    bits2, _ = run_a16w8(x, w, s, o, [last], dtype=dtype, packed=packed)
    assert (bits2 == bits).all()


@pytest.mark.parametrize("seed", range(10))
def test_weight_only_rows_kernels_random_shapes(device, seed):
    # a seeded sweep over the shapes of the multi-row weight-only kernels: K with odd and even block counts and 16..48-byte
    # tails, N from one column group to several strips with tails, ragged group lists with empty groups and sizes on both
    # sides of the 32 / 64 / 128-row chunks; packed weights and [E,K,N], both 16-bit types, against the float64 golden
    from gpu_utils import run_a16w8
    rng = np.random.default_rng(9000 + seed)
    k = int(rng.integers(1, 20)) * 64 + int(rng.choice([0, 0, 16, 32, 48]))
    n = int(rng.integers(1, 40)) * 16
    e = int(rng.choice([1, 2, 3, 5, 8]))
    m = int(rng.integers(17 * e, 140 * e))
    cuts = np.sort(rng.integers(0, m + 1, e - 1)) if e > 1 else np.array([], dtype=np.int64)
    gl = [int(v) for v in cuts] + [m - int(rng.choice([0, 0, 5]))]
    gl = [int(v) for v in np.maximum.accumulate(gl)]
    dtype = "bf16" if seed % 2 == 0 else "f16"
    x, w, s, o, exact, mag, to_f, last = _weight_only_case(100 + seed, m, k, n, e, gl, dtype)
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    for packed in (True, False):
        bits, info = run_a16w8(x, w, s, o, gl, dtype=dtype, packed=packed)
        if not (e == 1 and m <= 64):   # (one small group goes back to the 16-row kernels and their K split)
            assert ("a16w8_stream_rows" if packed else "a16w8_skinny_rows") in info, info
        got = to_f(bits).astype(np.float64)
        assert (np.abs(got[:last] - exact[:last]) <= ulp * np.abs(exact[:last]) + 1e-5 * mag[:last]).all(), info
        assert (bits[last:] == 0x7FC0).all(), info


def test_weight_only_generic_kernel_on_packed_weights(device):
    from gpu_utils import run_a16w8
    x, w, s, o, exact, mag, to_f, last = _weight_only_case(22, 12, 200, 48, 2, [5, 12], "bf16")
    # K % 16 != 0 has no MFMA path: generic kernel, packed indexing
    bits, info = run_a16w8(x, w, s, o, [5, 12], packed=True)
    assert "generic" in info
    got = to_f(bits).astype(np.float64)
    assert (np.abs(got[:last] - exact[:last]) <= 2.0 ** -7 * np.abs(exact[:last]) + 1e-5 * mag[:last]).all(), info


@pytest.mark.parametrize("seed", range(12))
def test_persistent_tile_kernel_random_shapes_both_layouts(device, seed):
    # a seeded sweep over K (every slab count from 4 up, whole and with 16..112-byte tails, i.e. every mix of the
    # steady-state and the general K-loop body), N with and without a tail, group counts and ragged group lists with
    # empty groups, partial m-tiles of at most and more than 128 rows; packed weights and [E,N,K], bit for bit
    from gpu_utils import run_w8a8
    rng = np.random.default_rng(1000 + seed)
    k = int(rng.integers(4, 18)) * 128 + int(rng.choice([0, 0, 16, 48, 64, 112]))
    n = int(rng.integers(1, 5)) * 256 - int(rng.choice([0, 0, 16, 240]))
    e = int(rng.choice([1, 2, 3, 5, 8]))
    m = int(rng.integers(200, 1400))
    cuts = np.sort(rng.integers(0, m + 1, e - 1)) if e > 1 else np.array([], dtype=np.int64)
    gl = [int(v) for v in cuts] + [m - int(rng.choice([0, 0, 7]))]
    gl = list(np.maximum.accumulate(gl))
    x, w, bias, scale, pt = _inputs(seed, m, k, n, e)
    info = _check(x, w, gl, bias, scale, pt, override=cabi.OV_TILE_256_W4)
    assert "tile_256x256x128_w4" in info and "layout=packed" in info, info
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=True, override=cabi.OV_TILE_256_W4, launches=2)   # stores [E,N,K]
    assert "tile_256x256x128_w4" in info, info
    assert np.array_equal(bits[:gl[-1]], ref[:gl[-1]]), info
    # [E,K,N] as stored: the same kernel turns the weights on their way out of LDS (N tails: chunks past N are killed)
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=False, override=cabi.OV_TILE_256_W4, launches=2)
    assert "tile_256x256x128_w4" in info and "layout=[E,K,N]" in info, info
    assert np.array_equal(bits[:gl[-1]], ref[:gl[-1]]), info
    acc, info = run_w8a8(x, w, gl, bias, out="i32", transpose_b=False, override=cabi.OV_TILE_256_W4, launches=2)
    assert np.array_equal(acc[:gl[-1]], O.grouped_matmul_w8a8(x, w, gl, bias, out_dtype="i32")[:gl[-1]]), info


@pytest.mark.parametrize("e,seed", [(16, 0), (24, 1), (40, 2)])
def test_many_uneven_groups_split_between_the_persistent_kernel_and_small_tiles(device, e, seed):
    # sixteen experts and more: the groups of at most 64 rows go to a second launch of 64 x 128 tiles, the others to the
    # persistent kernel (packed and [E,K,N] weights; [E,N,K] stays one launch); group sizes on both sides of the boundary
    from gpu_utils import run_w8a8
    rng = np.random.default_rng(7000 + seed)
    sizes = [0, 1, 63, 64, 65, 300, 64, 257] + [int(v) for v in rng.choice([0, 3, 17, 40, 64, 65, 100, 129, 420], e - 8)]
    sizes = [sizes[i] for i in rng.permutation(e)]
    gl = [int(v) for v in np.cumsum(sizes)]
    m, k, n = gl[-1] + 5, int(rng.choice([512, 640 + 48, 1024])), int(rng.choice([256, 512 - 16, 640]))
    x, w, bias, scale, pt = _inputs(seed, m, k, n, e)
    info = _check(x, w, gl, bias, scale, pt, override=cabi.OV_TILE_256_W4)
    assert "tile_256x256x128_w4" in info and "small_groups=64:tile_64x128" in info and "layout=packed" in info, info
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=True, override=cabi.OV_TILE_256_W4, launches=2)   # stores [E,N,K]
    assert "tile_256x256x128_w4" in info and "small_groups" not in info, info   # one launch on [E,N,K] weights
    assert np.array_equal(bits[:gl[-1]], ref[:gl[-1]]), info
    bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", transpose_b=False, override=cabi.OV_TILE_256_W4, launches=2)   # [E,K,N] as stored
    assert "tile_256x256x128_w4" in info and "small_groups=64:tile_64x128" in info and "layout=[E,K,N]" in info, info
    assert np.array_equal(bits[:gl[-1]], ref[:gl[-1]]), info
    assert (bits[gl[-1]:] == 0x7FC0).all()   # rows past the last boundary keep the fill value


@pytest.mark.parametrize("seed", range(24))
def test_whatever_the_plan_picks_is_bit_exact_on_every_layout(device, seed):
    # a seeded sweep over the shapes where the plan changes its mind: one group or several, a handful to several hundred
    # rows per group (16- and 32-row streaming chunks, 64 / 128 / 256-row tiles, K splits), K with and without 64- and
    # 128-byte tails, narrow and wide N; packed weights, [E,N,K] and [E,K,N], every one against the oracle bit for bit
    from gpu_utils import run_w8a8
    rng = np.random.default_rng(5000 + seed)
    wide = seed >= 16   # the last seeds: enough columns that several groups of 70 .. 260 rows get 128- and 256-row tiles
    e = int(rng.choice([4, 8])) if wide else int(rng.choice([1, 1, 2, 4, 8, 12]))
    per_group = int(rng.choice([70, 100, 150, 260])) if wide else int(rng.choice([6, 14, 20, 40, 70, 100, 150, 260]))
    m = max(1, int(per_group * e * rng.uniform(0.8, 1.2)))
    k = int(rng.integers(8, 12) if wide else rng.integers(2, 40)) * 64 + int(rng.choice([0, 0, 16, 32, 48]))
    n = int(rng.choice([6144, 12288 - 16])) if wide else int(rng.choice([48, 128, 272, 1024, 1408, 3072]))
    cuts = np.sort(rng.integers(0, m + 1, e - 1)) if e > 1 else np.array([], dtype=np.int64)
    gl = list(np.maximum.accumulate([int(v) for v in cuts] + [m - int(rng.choice([0, 0, 3]))]))
    x, w, bias, scale, pt = _inputs(100 + seed, m, k, n, e)
    ref = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt)
    infos = []
    for kwargs in ({"packed": True}, {"transpose_b": True}, {}):
        bits, info = run_w8a8(x, w, gl, bias, scale, pt, out="bf16", launches=2, **kwargs)
        infos.append(info)
        assert np.array_equal(bits[:gl[-1]], ref[:gl[-1]]), (m, k, n, e, gl, info)
