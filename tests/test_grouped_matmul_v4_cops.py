"""grouped_matmul_v4_cops through the Python entry -- the quantized cases of the reference's
tests/st/test_grouped_matmul_v4_cops.py (per-token, per-channel + bias, a16w8, counts vs cumulative
group_list, a last boundary below M, multi-output group_type -1), both execution modes."""
import os

import numpy as np
import pytest
import torch

import ms_custom_ops_amd as ms_custom_ops
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
MODES = [ms_custom_ops.GRAPH_MODE, ms_custom_ops.PYNATIVE_MODE]
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


@pytest.mark.parametrize("mode", MODES)
def test_v4_pertoken_constant_scales(device, mode):
    """scale = 10 (bf16), per-token = 10 -> 100 * acc (test_grouped_matmul_v4_cops.py:281-319)."""
    k = np.load(os.path.join(GOLDEN, "kat_const_scale.npz"))
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops(
            [_t(k["x"])], [_t(k["w"])], None, [_t(np.full((8, 128), 10, np.float32), torch.bfloat16)], None, None, None,
            [_t(np.full(32, 10, np.float32))], _t(k["counts"]), split_item=3, group_type=0, group_list_type=1)
    assert len(res) == 1 and res[0].dtype == torch.bfloat16 and res[0].shape == (32, 128)
    np.testing.assert_allclose(k["pertoken_expected"], res[0].float().cpu().numpy(), rtol=4e-3)   # reference's bar
    want = O.f32_to_bf16_bits(k["pertoken_expected"])
    assert np.array_equal(res[0].view(torch.int16).cpu().numpy().view(np.uint16), want)          # this build's bar


@pytest.mark.parametrize("mode", MODES)
def test_v4_perchannel_bias_constant_scales(device, mode):
    """scale = 10 (bf16), bias = 1 -> 10 * (acc + 1) (test_grouped_matmul_v4_cops.py:338-376)."""
    k = np.load(os.path.join(GOLDEN, "kat_const_scale.npz"))
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops(
            [_t(k["x"])], [_t(k["w"])], [_t(np.ones((8, 128), np.int32))],
            [_t(np.full((8, 128), 10, np.float32), torch.bfloat16)], None, None, None, None, _t(k["counts"]),
            split_item=3, group_type=0, group_list_type=1)
    np.testing.assert_allclose(k["perchannel_bias_expected"], res[0].float().cpu().numpy(), rtol=4e-3)
    assert np.array_equal(res[0].view(torch.int16).cpu().numpy().view(np.uint16),
                          O.f32_to_bf16_bits(k["perchannel_bias_expected"]))


@pytest.mark.parametrize("mode", MODES)
def test_v4_no_scale_returns_int32_accumulators(device, mode):
    k = np.load(os.path.join(GOLDEN, "kat_const_scale.npz"))
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops([_t(k["x"])], [_t(k["w"])], group_list=_t(k["counts"]),
                                                   split_item=3, group_type=0, group_list_type=1)
    assert res[0].dtype == torch.int32 and np.array_equal(res[0].cpu().numpy(), k["acc"])


@pytest.mark.parametrize("mode", MODES)
def test_v4_float32_scale_output_dtype_rules(device, mode):
    rng = np.random.default_rng(0)
    x = rng.integers(-127, 128, (96, 128), dtype=np.int8)
    w = rng.integers(-127, 128, (8, 128, 256), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, (8, 256)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, 96).astype(np.float32)
    gl = np.array([10, 10, 30, 41, 60, 77, 77, 96], dtype=np.int64)
    with ms_custom_ops.exec_mode(mode):
        f16 = ms_custom_ops.grouped_matmul_v4_cops([_t(x)], [_t(w)], None, [_t(s)], None, None, None, [_t(pt)], _t(gl),
                                                   split_item=3, group_type=0)[0]
        bf16 = ms_custom_ops.grouped_matmul_v4_cops([_t(x)], [_t(w)], None, [_t(s)], None, None, None, [_t(pt)],
                                                    _t(gl), split_item=3, group_type=0,
                                                    output_dtype=torch.bfloat16)[0]
    assert f16.dtype == torch.float16     # float32 scale -> float16 (reference rule)
    assert np.array_equal(f16.cpu().numpy().view(np.uint16),
                          O.grouped_matmul_w8a8(x, w, gl, None, s, pt, out_dtype="f16").view(np.uint16))
    assert bf16.dtype == torch.bfloat16   # explicit output_dtype (backend extension)
    assert np.array_equal(bf16.view(torch.int16).cpu().numpy().view(np.uint16),
                          O.grouped_matmul_w8a8(x, w, gl, None, s, pt))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_v4_a16w8_beyond_decode_sizes(device, mode, dtype):
    """The a16w8 form of the reference's test (test_grouped_matmul_v4_cops.py:139-192) at serving batch sizes: 300 rows
    over 4 experts (groups of 10, 90, 0 and 180 rows, the last boundary below M) through the operator in both modes --
    the [E,K,N] weights take the multi-row kernel (one pass over a group's weights per 64 rows)."""
    rng = np.random.default_rng(5)
    m, k, n, e = 300, 512, 256, 4
    ends = np.array([10, 100, 100, 280], dtype=np.int64)
    x = _t(rng.uniform(-4, 4, (m, k)).astype(np.float32), dtype)
    w = rng.integers(-127, 128, (e, k, n)).astype(np.int8)
    s = _t(rng.uniform(0.005, 0.02, (e, n)).astype(np.float32), dtype)
    o = _t(rng.integers(-8, 9, (e, n)).astype(np.float32), dtype)
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops([x], [_t(w)], None, None, None, [s], [o], None, _t(ends), None, None,
                                                   None, 3, 0, 0)
    assert res[0].dtype == dtype and res[0].shape == (m, n)
    xf, sf, of = x.float().cpu().numpy(), s.float().cpu().numpy(), o.float().cpu().numpy()
    last = int(ends[-1])
    exact = O.a16w8_grouped_f64(xf, w, sf, of, ends)[:last]
    mag = np.zeros_like(exact)
    starts = np.concatenate([[0], ends[:-1]])
    for g in range(e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    got = res[0][:last].float().cpu().numpy().astype(np.float64)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert (np.abs(got - exact) <= ulp * np.abs(exact) + 1e-5 * mag).all()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_v4_a16w8_last_boundary_below_m(device, mode, dtype):
    """a16w8 with scale 0.01 and offset 1, group_list [1,3,10,14,18,22,24,30] over 32 rows: only the first
    30 rows are defined (test_grouped_matmul_v4_cops.py:139-192)."""
    rng = np.random.default_rng(1)
    m, k, n, e = 32, 256, 128, 8
    ends = np.array([1, 3, 10, 14, 18, 22, 24, 30], dtype=np.int64)
    x = _t(rng.uniform(-128, 127, (m, k)).astype(np.float32), dtype)
    w = rng.uniform(-128, 127, (e, k, n)).astype(np.int8)
    s = _t(np.full((e, n), 0.01, np.float32), dtype)
    o = _t(np.full((e, n), 1, np.float32), dtype)
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops([x], [_t(w)], None, None, None, [s], [o], None, _t(ends), None, None,
                                                   None, 3, 0, 0)
    assert res[0].dtype == dtype and res[0].shape == (m, n)
    xf, sf, of = x.float().cpu().numpy(), s.float().cpu().numpy(), o.float().cpu().numpy()
    exact = O.a16w8_grouped_f64(xf, w, sf, of, ends)[:30]
    mag = np.zeros_like(exact)
    starts = np.concatenate([[0], ends[:-1]])
    for g in range(e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    got = res[0][:30].float().cpu().numpy().astype(np.float64)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    # floating-point tolerance: one output ulp plus float32 accumulation noise relative to sum |terms|
    assert (np.abs(got - exact) <= ulp * np.abs(exact) + 1e-5 * mag).all()
    big = np.abs(exact) > 0.05 * mag
    np.testing.assert_allclose(got[big], exact[big], rtol=1e-2 if dtype == torch.bfloat16 else 2e-3)


@pytest.mark.parametrize("mode", MODES)
def test_v4_multi_output_group_type_minus_one(device, mode):
    rng = np.random.default_rng(2)
    x0 = rng.integers(-127, 128, (2, 3, 16, 256), dtype=np.int8)
    x1 = rng.integers(-127, 128, (127, 96), dtype=np.int8)
    w0 = rng.integers(-127, 128, (256, 128), dtype=np.int8)
    w1 = rng.integers(-127, 128, (96, 64), dtype=np.int8)
    s0 = rng.uniform(1e-3, 1e-2, 128).astype(np.float32)
    s1 = rng.uniform(1e-3, 1e-2, 64).astype(np.float32)
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops([_t(x0), _t(x1)], [_t(w0), _t(w1)], None, [_t(s0), _t(s1)],
                                                   split_item=0, group_type=-1, output_dtype=torch.bfloat16)
    assert [tuple(r.shape) for r in res] == [(2, 3, 16, 128), (127, 64)]
    for r, x, w, s in ((res[0], x0, w0, s0), (res[1], x1, w1, s1)):
        ref = O.quant_batch_matmul_oracle(x.reshape(-1, x.shape[-1]), w, s).reshape(r.shape)
        assert np.array_equal(r.view(torch.int16).cpu().numpy().view(np.uint16), ref)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("weight_format", ["ND", "FRACTAL_NZ"])
def test_v4_fractal_nz(device, mode, weight_format):
    """The reference's test_ops_grouped_mamtul_v4_fractal_nz (test_grouped_matmul_v4_cops.py:486-520) on the quantized
    path: the weight goes through trans_data(ND_TO_FRACTAL_NZ) and the op is told weight_format="FRACTAL_NZ";
    group_type -1 with one [16, 256] x [256, 128] problem as there, and the grouped form (group_type 0)."""
    rng = np.random.default_rng(1)
    x0 = rng.integers(-127, 128, (16, 256), dtype=np.int8)
    w0 = rng.integers(-127, 128, (256, 128), dtype=np.int8)
    s0 = rng.uniform(1e-3, 1e-2, 128).astype(np.float32)
    prep = (lambda t: ms_custom_ops.trans_data(t, transdata_type=1)) if weight_format == "FRACTAL_NZ" else (lambda t: t)
    with ms_custom_ops.exec_mode(mode):
        res = ms_custom_ops.grouped_matmul_v4_cops([_t(x0)], [prep(_t(w0))], None, [_t(s0)], split_item=0, group_type=-1,
                                                   weight_format=weight_format, output_dtype=torch.bfloat16)
    assert tuple(res[0].shape) == (16, 128)
    assert np.array_equal(res[0].view(torch.int16).cpu().numpy().view(np.uint16), O.quant_batch_matmul_oracle(x0, w0, s0))

    x = rng.integers(-127, 128, (40, 320), dtype=np.int8)
    w = rng.integers(-127, 128, (8, 320, 272), dtype=np.int8)
    s = rng.uniform(1e-3, 1e-2, (8, 272)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, 40).astype(np.float32)
    gl = np.array([3, 3, 10, 17, 22, 30, 30, 40], dtype=np.int64)
    with ms_custom_ops.exec_mode(mode):
        out = ms_custom_ops.grouped_matmul_v4_cops([_t(x)], [prep(_t(w))], None, [_t(s)], None, None, None, [_t(pt)], _t(gl),
                                                   split_item=3, group_type=0, weight_format=weight_format,
                                                   output_dtype=torch.bfloat16)[0]
        acc = ms_custom_ops.grouped_matmul_v4_cops([_t(x)], [prep(_t(w))], group_list=_t(gl), split_item=3, group_type=0,
                                                   weight_format=weight_format)[0]
    ref_bits, ref_acc = O.grouped_matmul_w8a8(x, w, gl, None, s, pt, return_acc=True)
    assert np.array_equal(acc.cpu().numpy(), ref_acc)
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), ref_bits)
    # weight-only path on the same prepacked weights
    xb = _t(rng.standard_normal((40, 320)).astype(np.float32), torch.bfloat16)
    aq = _t(rng.uniform(1e-3, 1e-2, (8, 272)).astype(np.float32), torch.bfloat16)
    ao = _t(rng.integers(-8, 9, (8, 272)).astype(np.float32), torch.bfloat16)
    with ms_custom_ops.exec_mode(mode):
        wo = ms_custom_ops.grouped_matmul_v4_cops([xb], [prep(_t(w))], None, None, None, [aq], [ao], None, _t(gl),
                                                  split_item=3, group_type=0, weight_format=weight_format)[0]
    exact = O.a16w8_grouped_f64(xb.float().cpu().numpy(), w, aq.float().cpu().numpy(), ao.float().cpu().numpy(), gl)
    np.testing.assert_allclose(wo.float().cpu().numpy(), exact, rtol=2 ** -6, atol=0.05)


def test_v4_errors(device):
    x = torch.zeros(32, 64, dtype=torch.int8, device="cuda")
    w = torch.zeros(8, 64, 128, dtype=torch.int8, device="cuda")
    gl = torch.full((8,), 4, dtype=torch.int64, device="cuda")
    f = ms_custom_ops.grouped_matmul_v4_cops
    with pytest.raises(ValueError, match="weight_format 'FRACTAL_NZ' takes Int8 weights prepacked by trans_data"):
        f([x], [w], group_list=gl, split_item=3, group_type=0, weight_format="FRACTAL_NZ")
    with pytest.raises(RuntimeError, match="weight_format must be 'ND' or 'FRACTAL_NZ'"):
        f([x], [w], group_list=gl, split_item=3, group_type=0, weight_format="NC1HWC0")
    with pytest.raises(RuntimeError, match="quantized paths only"):
        f([x.bfloat16()], [w.bfloat16()], group_list=gl, split_item=3, group_type=0)
    with pytest.raises(ValueError, match="group_type 0 needs 'group_list'"):
        f([x], [w], split_item=3, group_type=0)
    with pytest.raises(ValueError, match="'group_list' must be Int64"):
        f([x], [w], group_list=gl.int(), split_item=3, group_type=0)
    with pytest.raises(ValueError, match="the scale only support"):
        f([x], [w], None, [torch.ones(8, 128, dtype=torch.float16, device="cuda")], group_list=gl, split_item=3,
          group_type=0)
    with pytest.raises(TypeError):
        f(x, [w], group_list=gl)


def test_graph_kernel_module_inits_once_resizes_on_new_shapes_and_reads_fresh_tensors(device):
    """The graph-mode life cycle of the reference (docs/ops_develop_guide.md:193-197): Init once per node, Resize only
    when shapes, dtypes or attributes change, Launch on the tensors of the call (not on those seen by Resize)."""
    rng = np.random.default_rng(21)
    stats = lambda: ms_custom_ops._C._graph_node_stats("grouped_matmul_v4_cops")
    def run(m, seed):
        r = np.random.default_rng(seed)
        x = r.integers(-127, 128, (m, 64), dtype=np.int8)
        w = r.integers(-127, 128, (8, 64, 128), dtype=np.int8)
        counts = np.full(8, m // 8, dtype=np.int64)
        with ms_custom_ops.exec_mode(ms_custom_ops.GRAPH_MODE):
            out = ms_custom_ops.grouped_matmul_v4_cops([_t(x)], [_t(w)], group_list=_t(counts), split_item=3, group_type=0,
                                                       group_list_type=1)[0]
        assert np.array_equal(out.cpu().numpy(), O.grouped_matmul_w8a8(x, w, counts, group_list_type=1, out_dtype="i32"))
    run(32, 1)
    inits0, resizes0, launches0 = stats()
    run(32, 2)          # same signature, other tensors (other device addresses, other values)
    run(32, 3)
    assert stats() == (inits0, resizes0, launches0 + 2)
    run(64, 4)          # new shape: planned again, same kernel module
    assert stats() == (inits0, resizes0 + 1, launches0 + 3)
    assert inits0 == 1


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("output_dtype", [torch.float16, torch.bfloat16, None])
def test_v4_a8w4_reference_case(device, mode, output_dtype):
    """The reference's A8W4 case (tests/st/test_grouped_matmul_v4_cops.py:429-485): int8 x, qint4x2 weight [e, k, n / 2]
    (two nibbles per byte along n), uint64-encoded per-channel scale [e, 1, n], per-token scale [m, 1], float32 bias
    (the reference kernel's compensation term, not part of the expected value), counts list; same seed, shapes and
    tolerance; output float16 / bfloat16 (bfloat16 when output_dtype is not given).  This build's bar on top: the
    output is one rounding of the oracle's exact float32 value, bit for bit."""
    np.random.seed(1)
    e, m, k, n = 8, 32, 256, 128
    x_np = np.random.randint(-5, 5, size=(m, k)).astype(np.int8)
    w_np = np.random.randint(-5, 5, size=(e, k, n)).astype(np.int8)
    w_int4_np = O.pack_int4(w_np)
    assert w_int4_np.shape == (e, k, n // 2)
    scale_np = np.random.normal(0, 0.01, size=(e, 1, n)).astype(np.float32)
    scale_u64 = O.encode_scale_uint64(scale_np)
    bias_np = 8 * (w_np.astype(np.float32) * scale_np).sum(axis=1)
    pertoken_np = np.random.normal(0, 0.01, (m, 1)).astype(np.float32)
    counts = np.array([1, 2, 7, 4, 4, 4, 2, 8], dtype=np.int64)
    expect = O.golden_v4_a8w4(x_np, w_np, scale_u64, pertoken_np, counts)
    # (torch moves uint64 only as raw bytes on some builds: the bits travel as int64 and are viewed back)
    scale_t = torch.from_numpy(scale_u64.view(np.int64)).cuda().view(torch.uint64)
    with ms_custom_ops.exec_mode(mode):
        for _ in range(2):   # the second call reuses the graph-mode module and its extra workspace slice
            out = ms_custom_ops.grouped_matmul_v4_cops(
                [_t(x_np)], [ms_custom_ops.as_qint4x2(_t(w_int4_np))], bias=[_t(bias_np)], scale=[scale_t],
                per_token_scale=[_t(pertoken_np)], group_list=_t(counts), split_item=3, group_type=0, group_list_type=1,
                output_dtype=output_dtype)[0]
            assert out.shape == (m, n) and out.dtype == (output_dtype or torch.bfloat16)
            cnt = expect.shape[0]
            np.testing.assert_allclose(expect, out[:cnt].float().cpu().numpy(), rtol=5e-3, atol=5e-3)   # the reference's bar
            if out.dtype == torch.float16:
                assert np.array_equal(out.cpu().numpy().view(np.uint16), O.f32_to_f16(expect).view(np.uint16))
            else:
                assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), O.f32_to_bf16_bits(expect))


def test_v4_a8w4_full_nibble_range_ragged_groups_and_rules(device):
    """Every 4-bit value (-8 .. 7), int8 x over its whole range, empty groups, a K that is not a multiple of 64 and a
    byte count that is not a multiple of 16 per row; then the argument rules."""
    rng = np.random.default_rng(11)
    e, m, k, n = 8, 50, 96, 48
    x = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-8, 8, (e, k, n), dtype=np.int8)
    assert w.min() == -8 and w.max() == 7
    scale = rng.uniform(1e-3, 1e-2, (e, 1, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, (m, 1)).astype(np.float32)
    counts = np.array([0, 9, 0, 17, 1, 0, 20, 3], dtype=np.int64)
    expect = O.golden_v4_a8w4(x, w, O.encode_scale_uint64(scale), pt, counts)
    scale_t = torch.from_numpy(O.encode_scale_uint64(scale).view(np.int64)).cuda().view(torch.uint64)
    f = ms_custom_ops.grouped_matmul_v4_cops
    wq = ms_custom_ops.as_qint4x2(_t(O.pack_int4(w)))
    for mode in MODES:
        with ms_custom_ops.exec_mode(mode):
            out = f([_t(x)], [wq], scale=[scale_t], per_token_scale=[_t(pt)], group_list=_t(counts), split_item=3,
                    group_type=0, group_list_type=1, output_dtype=torch.float16)[0]
        assert np.array_equal(out.cpu().numpy().view(np.uint16), O.f32_to_f16(expect).view(np.uint16))
    # cumulative list (group_list_type 0) gives the same rows
    out = f([_t(x)], [wq], scale=[scale_t], per_token_scale=[_t(pt)], group_list=_t(np.cumsum(counts)), split_item=3,
            group_type=0, group_list_type=0)[0]
    assert out.dtype == torch.bfloat16
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), O.f32_to_bf16_bits(expect))
    with pytest.raises(ValueError, match="the output type must be in"):
        f([_t(x)], [wq], scale=[scale_t], group_list=_t(counts), split_item=3, group_type=0, group_list_type=1,
          output_dtype=torch.float32)
    with pytest.raises(ValueError, match="'scale' must be given"):
        f([_t(x)], [wq], group_list=_t(counts), split_item=3, group_type=0, group_list_type=1)
    with pytest.raises(ValueError, match="'bias' must be Float32"):
        f([_t(x)], [wq], bias=[_t(np.zeros((e, n), np.int32))], scale=[scale_t], group_list=_t(counts), split_item=3,
          group_type=0, group_list_type=1)
    with pytest.raises(RuntimeError, match="int4 weights are implemented for"):
        f([_t(x)], [ms_custom_ops.as_qint4x2(_t(O.pack_int4(w[0])))], scale=[scale_t[0]], group_type=-1)
    with pytest.raises(TypeError, match="carried by an int8 or uint8"):
        ms_custom_ops.as_qint4x2(_t(x).int())


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_v4_a16w4_reference_case(device, mode, dtype):
    """The reference's A16W4 case (tests/st/test_grouped_matmul_v4_cops.py:197-262): float16 x in [-128, 127), qint4x2
    weight [e, k, n / 2] holding values 0 / 1 (two nibbles per byte along n, low nibble first), antiquant scale 0.01 and
    offset 1 in x's dtype, cumulative group_list whose last boundary (30) lies below the 32 rows; same shapes, data
    distribution and tolerance (rtol = atol = 1e-3 against the numpy golden on its float16 case).  This build's bar on
    top, for both 16-bit types: one output ulp of the float64 value plus float32 accumulation noise."""
    np.random.seed(3)
    m, k, n, e = 32, 256, 128, 8
    ends = np.array([1, 3, 10, 14, 18, 22, 24, 30], dtype=np.int64)
    x_np = np.random.uniform(-128, 127, size=[m, k]).astype(np.float16)
    w_np = (np.random.uniform(0, 2, size=[e, k, n]).astype(np.int8)) & 0xF
    s_np = np.full([e, n], 0.01).astype(np.float16)
    o_np = np.full([e, n], 1).astype(np.float16)
    w_int4 = O.pack_int4(w_np)
    assert w_int4.shape == (e, k, n // 2)
    x, s, o = _t(x_np.astype(np.float32), dtype), _t(s_np.astype(np.float32), dtype), _t(o_np.astype(np.float32), dtype)
    with ms_custom_ops.exec_mode(mode):
        for _ in range(2):   # the second call reuses the graph-mode module and its staging slice
            res = ms_custom_ops.grouped_matmul_v4_cops([x], [ms_custom_ops.as_qint4x2(_t(w_int4))], None, None, None, [s], [o],
                                                       None, _t(ends), None, None, None, 3, 0, 0)
            assert res[0].dtype == dtype and res[0].shape == (m, n)
            got = res[0][:30].float().cpu().numpy().astype(np.float64)
            if dtype == torch.float16:   # the reference's comparison, on its own golden
                expect = O.golden_v4_a16w4(x_np, w_np, s_np, o_np, ends)
                np.testing.assert_allclose(expect.astype(np.float64), got, rtol=1e-3, atol=1e-3)
            xf, sf, of = x.float().cpu().numpy(), s.float().cpu().numpy(), o.float().cpu().numpy()
            exact = O.a16w8_grouped_f64(xf, w_np, sf, of, ends)[:30]
            mag = np.zeros_like(exact)
            starts = np.concatenate([[0], ends[:-1]])
            for g in range(e):
                a, b = int(starts[g]), int(ends[g])
                mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(w_np[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
            ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
            assert (np.abs(got - exact) <= ulp * np.abs(exact) + 1e-5 * mag).all()


def test_v4_a16w4_signed_nibbles_ragged_groups_equal_the_a16w8_path(device):
    """Every 4-bit value (-8 .. 7), empty groups, rows behind the last boundary: the A16W4 result is bit for bit the a16w8
    result on the same values given as int8 (the nibbles are widened, then the same kernels run), in both modes."""
    rng = np.random.default_rng(12)
    e, m, k, n = 8, 70, 192, 96
    w = rng.integers(-8, 8, (e, k, n), dtype=np.int8)
    assert w.min() == -8 and w.max() == 7
    counts = np.array([0, 9, 0, 27, 1, 0, 20, 6], dtype=np.int64)
    for dtype in (torch.bfloat16, torch.float16):
        x = _t(rng.uniform(-2, 2, (m, k)).astype(np.float32), dtype)
        s = _t(rng.uniform(0.005, 0.02, (e, n)).astype(np.float32), dtype)
        o = _t(rng.integers(-3, 4, (e, n)).astype(np.float32), dtype)
        f = ms_custom_ops.grouped_matmul_v4_cops
        ref = f([x], [_t(w)], None, None, None, [s], [o], None, _t(counts), None, None, None, 3, 0, 1)[0]
        for mode in MODES:
            with ms_custom_ops.exec_mode(mode):
                out = f([x], [ms_custom_ops.as_qint4x2(_t(O.pack_int4(w)))], None, None, None, [s], [o], None, _t(counts), None,
                        None, None, 3, 0, 1)[0]
            last = int(counts.sum())
            assert torch.equal(out[:last].view(torch.int16), ref[:last].view(torch.int16))
    with pytest.raises(ValueError, match="needs 'antiquant_scale'"):
        f([x], [ms_custom_ops.as_qint4x2(_t(O.pack_int4(w)))], group_list=_t(counts), split_item=3, group_type=0, group_list_type=1)


def test_widen_qint4x2_once_then_the_int8_paths(device):
    """Weights widened at load time give the same bits as the op's per-call widening, for A8W4 and for A16W4."""
    rng = np.random.default_rng(13)
    e, m, k, n = 4, 40, 128, 64
    w = rng.integers(-8, 8, (e, k, n), dtype=np.int8)
    packed = _t(O.pack_int4(w))
    wide = ms_custom_ops.widen_qint4x2(ms_custom_ops.as_qint4x2(packed))
    assert wide.dtype == torch.int8 and tuple(wide.shape) == (e, k, n) and np.array_equal(wide.cpu().numpy(), w)
    assert torch.equal(ms_custom_ops.widen_qint4x2(packed.view(torch.uint8)), wide)
    counts = _t(np.array([7, 0, 20, 13], dtype=np.int64))
    f = ms_custom_ops.grouped_matmul_v4_cops
    x8 = _t(rng.integers(-128, 128, (m, k), dtype=np.int8))
    scale = rng.uniform(1e-3, 1e-2, (e, 1, n)).astype(np.float32)
    pt = _t(rng.uniform(1e-3, 1e-2, (m, 1)).astype(np.float32))
    su = torch.from_numpy(O.encode_scale_uint64(scale).view(np.int64)).cuda().view(torch.uint64)
    a = f([x8], [ms_custom_ops.as_qint4x2(packed)], scale=[su], per_token_scale=[pt], group_list=counts, split_item=3, group_type=0,
          group_list_type=1, output_dtype=torch.bfloat16)[0]
    b = f([x8], [wide], scale=[_t(scale.reshape(e, n))], per_token_scale=[pt.reshape(m)], group_list=counts, split_item=3,
          group_type=0, group_list_type=1, output_dtype=torch.bfloat16)[0]
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    x16 = _t(rng.uniform(-2, 2, (m, k)).astype(np.float32), torch.float16)
    s16, o16 = _t(np.full((e, n), 0.01, np.float32), torch.float16), _t(np.full((e, n), 1, np.float32), torch.float16)
    a = f([x16], [ms_custom_ops.as_qint4x2(packed)], None, None, None, [s16], [o16], None, counts, None, None, None, 3, 0, 1)[0]
    b = f([x16], [wide], None, None, None, [s16], [o16], None, counts, None, None, None, 3, 0, 1)[0]
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ms_custom_ops.widen_qint4x2(packed.cpu())


def test_unpack_int4_through_the_c_abi(device):
    """msco_unpack_int4 against the oracle's unpack, sizes that end inside a 16-byte piece included."""
    from ms_custom_ops_amd import cabi
    rng = np.random.default_rng(2)
    for nbytes in (1, 15, 16, 17, 4096 + 5, 1 << 20):
        src = rng.integers(0, 256, nbytes, dtype=np.uint8)
        t = torch.from_numpy(src).cuda()
        dst = torch.full((2 * nbytes + 16,), 99, dtype=torch.int8, device="cuda")
        cabi.unpack_int4(t.data_ptr(), dst.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        got = dst.cpu().numpy()
        assert np.array_equal(got[:2 * nbytes], O.unpack_int4(src)) and (got[2 * nbytes:] == 99).all()
