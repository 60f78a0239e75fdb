"""grouped_matmul through the Python entry, in both execution modes -- the cases of the reference's
tests/st/test_grouped_matmul.py (shapes, optional inputs, scale wire formats), checked against the
CPU oracle at this build's bar (int32 bit-exact, output bit-exact / within 1 ulp) and against the
reference's own count-based bar."""
import numpy as np
import pytest
import torch

import ms_custom_ops_amd as ms_custom_ops
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
MODES = [ms_custom_ops.GRAPH_MODE, ms_custom_ops.PYNATIVE_MODE]


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def custom_grouped_matmul(m, k, n, e, trans_b=True, with_bias=True, with_pertoken_scale=False, scale_dtype="float32",
                          out_dtype=None, seed=0, prepack=False):
    """Same input recipe as the reference's custom_grouped_matmul (test_grouped_matmul.py:85-159)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-20, 20, size=[m, k]).astype(np.int8)
    w = rng.uniform(-20, 20, size=[e, k, n]).astype(np.int8)
    b = rng.integers(-10, 10, (e, n)).astype(np.int32) if with_bias else None
    s = (rng.random((e, n)) / 1000).astype(np.float32)
    ps = rng.random(m).astype(np.float32) if with_pertoken_scale else None
    gl = O.random_group_list(m, e, rng).astype(np.int32)

    w_dev = np.transpose(w, (0, 2, 1)) if trans_b else w
    if prepack:
        # the reference's flow (weight to the device's blocked format first, test_grouped_matmul.py:131-133): the packed
        # tensor carries its own layout, so the op is then called with transpose_b = False
        weight = ms_custom_ops.trans_data(_t(w_dev), transdata_type=1, transposed=trans_b)
        assert tuple(weight.shape) == (e, n // 16, (k + 63) // 64, 1024)
        back = ms_custom_ops.trans_data(weight, transdata_type=0, nd_shape=(e, k, n), transposed=trans_b)
        assert torch.equal(back, _t(w_dev))
        trans_b = False
    else:
        weight = _t(w_dev)
    scale = _t(s) if scale_dtype == "float32" else _t(O.encode_scale_int64(s))
    out = ms_custom_ops.grouped_matmul(_t(x), weight, _t(gl), _t(b), scale, _t(ps), None, False, trans_b,
                                       output_dtype=out_dtype)
    assert out.shape == (m, n)
    if out_dtype is None:
        assert out.dtype == torch.float16   # the reference's output type
        ref = O.grouped_matmul_w8a8(x, w, gl, b, s, ps, out_dtype="f16")
        assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))
        gold = O.golden_grouped_w8a8(x, w, gl, b, s, ps, out="f16")
        assert O.count_compare(out.float().cpu().numpy(), gold.astype(np.float32), 0.004)   # reference's bar
    else:
        assert out.dtype == torch.bfloat16
        ref = O.grouped_matmul_w8a8(x, w, gl, b, s, ps)
        got = out.view(torch.int16).cpu().numpy().view(np.uint16)
        rel, bad = O.bf16_ulp_check(got, ref)
        assert bad == 0 and np.array_equal(got, ref)


@pytest.mark.parametrize("m", [32, 1000])
@pytest.mark.parametrize("with_pertoken_scale", [True, False])
@pytest.mark.parametrize("exec_mode", MODES)
def test_gmm_v4_with_scale(device, m, with_pertoken_scale, exec_mode):
    with ms_custom_ops.exec_mode(exec_mode):
        custom_grouped_matmul(m, 64, 128, 8, with_pertoken_scale=with_pertoken_scale)
        custom_grouped_matmul(m, 64, 128, 8, with_pertoken_scale=with_pertoken_scale, out_dtype=torch.bfloat16)


@pytest.mark.parametrize("inputs_shape", [[40, 512, 7168], [1024, 2048, 7168], [1024, 7168, 4096]])
def test_gmm_v4_with_scale_ds(device, inputs_shape):
    with ms_custom_ops.exec_mode(ms_custom_ops.GRAPH_MODE):
        custom_grouped_matmul(*inputs_shape, 256, with_pertoken_scale=True, out_dtype=torch.bfloat16)


@pytest.mark.parametrize("input_shape", [[32, 32, 64, 8], [1000, 256, 512, 16]])
@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("with_bias", [False, True])
def test_gmm_quant_int64_scale(device, input_shape, exec_mode, with_bias):
    with ms_custom_ops.exec_mode(exec_mode):
        custom_grouped_matmul(*input_shape, with_bias=with_bias, scale_dtype="int64")


@pytest.mark.parametrize("trans_b", [False, True])
def test_gmm_real_moe_shape(device, trans_b):
    custom_grouped_matmul(1024, 5120, 2688, 8, trans_b=trans_b, with_pertoken_scale=True, out_dtype=torch.bfloat16)
    custom_grouped_matmul(1024, 5120, 1344, 8, trans_b=trans_b, with_pertoken_scale=True, out_dtype=torch.bfloat16)


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("shape", [[40, 64, 128, 8], [1000, 512, 256, 8]])
def test_gmm_transpose_a(device, exec_mode, shape):
    """transpose_a=True: x arrives [K, M] (the reference passes the flag down to its kernel,
    ops/c_api/grouped_matmul/grouped_matmul.cc:73-74,216-218); same result as the [M, K] call, bit for bit, twice in a
    row (the graph-mode module keeps its extra workspace slice across calls) and with a second shape."""
    m, k, n, e = shape
    rng = np.random.default_rng(m)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    s = (rng.random((e, n)) / 1000).astype(np.float32)
    ps = rng.random(m).astype(np.float32)
    b = rng.integers(-10, 10, (e, n)).astype(np.int32)
    gl = O.random_group_list(m, e, rng).astype(np.int32)
    ref = O.grouped_matmul_w8a8(x, w, gl, b, s, ps)
    xt = _t(x.T)   # [K, M], contiguous
    with ms_custom_ops.exec_mode(exec_mode):
        for _ in range(2):
            out = ms_custom_ops.grouped_matmul(xt, _t(w), _t(gl), _t(b), _t(s), _t(ps), None, True, False,
                                               output_dtype=torch.bfloat16)
            assert out.shape == (m, n)
            assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), ref)
        with pytest.raises(RuntimeError, match="must have the same dimension of 'k'"):
            ms_custom_ops.grouped_matmul(_t(x), _t(w), _t(gl), _t(b), _t(s), _t(ps), None, True, False)


def test_gmm_errors(device):
    x = torch.zeros(32, 64, dtype=torch.int8, device="cuda")
    w = torch.zeros(8, 64, 128, dtype=torch.int8, device="cuda")
    gl = torch.full((8,), 32, dtype=torch.int32, device="cuda")
    s = torch.ones(8, 128, device="cuda")
    with pytest.raises(RuntimeError, match="input 'group_list' must be int32"):
        ms_custom_ops.grouped_matmul(x, w, gl.long(), None, s)
    with pytest.raises(RuntimeError, match="quantized int8 path only"):
        ms_custom_ops.grouped_matmul(x.half(), w.half(), gl)
    with pytest.raises(RuntimeError, match="needs the dequant 'scale'"):
        ms_custom_ops.grouped_matmul(x, w, gl)
    with pytest.raises(RuntimeError, match="x_format must be 0"):
        ms_custom_ops.grouped_matmul(x, w, gl, None, s, x_format=1)
    with pytest.raises(RuntimeError, match="is not contiguous"):
        ms_custom_ops.grouped_matmul(x, w.transpose(1, 2), gl, None, s, transpose_b=True)
    with pytest.raises(RuntimeError, match=r"'scale' must have shape \[E, N\]"):
        ms_custom_ops.grouped_matmul(x, w, gl, None, s[:, :64].contiguous())


def test_plan_cache_hits_on_repeated_shapes(device):
    ms_custom_ops._C._plan_cache_clear()
    h0, m0, _ = ms_custom_ops.plan_cache_stats()
    for _ in range(3):
        custom_grouped_matmul(64, 64, 128, 8, seed=3)
    h1, m1, size = ms_custom_ops.plan_cache_stats()
    assert m1 - m0 == 1 and h1 - h0 == 2 and size >= 1


@pytest.mark.parametrize("m", [24, 1000])
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("exec_mode", MODES)
def test_gmm_on_weights_prepacked_by_trans_data(device, m, trans_b, exec_mode):
    """trans_data(ND_TO_FRACTAL_NZ) then grouped_matmul, as the reference's callers do (test_grouped_matmul.py:131-147):
    decode-sized M takes the streaming kernels, larger M the tile kernels; both bit-exact."""
    with ms_custom_ops.exec_mode(exec_mode):
        custom_grouped_matmul(m, 192, 128, 8, trans_b=trans_b, with_pertoken_scale=True, prepack=True)
        custom_grouped_matmul(m, 192, 128, 8, trans_b=trans_b, out_dtype=torch.bfloat16, prepack=True)


def test_trans_data_rules(device):
    w = torch.zeros(8, 64, 40, dtype=torch.int8, device="cuda")
    with pytest.raises(ValueError, match="N dimension must be aligned to 16"):
        ms_custom_ops.trans_data(w, 1)
    with pytest.raises(ValueError, match="transdata_type must be 0"):
        ms_custom_ops.trans_data(w, 2)
    with pytest.raises(ValueError, match="FRACTAL_NZ_TO_ND takes a tensor made by"):
        ms_custom_ops.trans_data(w, 0)
    f = torch.zeros(8, 64, 48, dtype=torch.float16, device="cuda")
    assert ms_custom_ops.trans_data(f, 1) is f                      # only int8 weights have a blocked form
    packed = ms_custom_ops.trans_data(torch.zeros(8, 64, 48, dtype=torch.int8, device="cuda"), 1)
    x = torch.zeros(4, 64, dtype=torch.int8, device="cuda")
    gl = torch.full((8,), 4, dtype=torch.int32, device="cuda")
    s = torch.ones(8, 48, device="cuda")
    with pytest.raises(RuntimeError, match="'transpose_b' must be false"):
        ms_custom_ops.grouped_matmul(x, packed, gl, None, s, None, None, False, True)
    with pytest.raises(RuntimeError, match="same dimension of 'k'"):
        ms_custom_ops.grouped_matmul(torch.zeros(4, 128, dtype=torch.int8, device="cuda"), packed, gl, None, s)
