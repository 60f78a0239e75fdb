"""quant_batch_matmul through the Python entry -- the cases of the reference's
tests/st/test_quant_batch_matmul.py (basic bf16 / int32, batched, per-token, both transposes, int64
scale), both execution modes, plus the Llama-7B FFN linear sweep at reduced size."""
import numpy as np
import pytest
import torch

import ms_custom_ops_amd as ms_custom_ops
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
MODES = [ms_custom_ops.GRAPH_MODE, ms_custom_ops.PYNATIVE_MODE]


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.int32])
def test_custom_quant_batch_matmul_basic(device, exec_mode, dtype):
    rng = np.random.default_rng(0)
    m, k, n = 128, 256, 128
    x1 = rng.integers(-5, 5, (m, k)).astype(np.int8)
    x2 = rng.integers(-5, 5, (k, n)).astype(np.int8)
    scale = np.ones([1]).astype(np.float32)
    expected = np.matmul(x1.astype(np.int32), x2.astype(np.int32)) * scale
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), output_dtype=dtype)
    assert out.dtype == dtype
    assert np.allclose(expected, out.float().cpu().numpy(), 0.01)                 # reference's bar
    if dtype == torch.int32:
        assert np.array_equal(out.cpu().numpy(), x1.astype(np.int32) @ x2.astype(np.int32))
    else:
        assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale))


@pytest.mark.parametrize("exec_mode", MODES)
def test_custom_quant_batch_matmul_bfp16_nz(device, exec_mode):
    """The reference's test_custom_quant_batch_matmul_bfp16_nz (tests/st/test_quant_batch_matmul.py:86-118): x2 goes
    through trans_data(ND_TO_FRACTAL_NZ) and the op is told x2_format="FRACTAL_NZ"; batched, then one shared x2 and a
    decode-sized x1."""
    rng = np.random.default_rng(5)
    batch, m, k, n = 2, 128, 256, 128
    x1 = rng.integers(-5, 5, (batch, m, k)).astype(np.int8)
    x2 = rng.integers(-5, 5, (batch, k, n)).astype(np.int8)
    scale = np.ones([n]).astype(np.float32)
    expected = np.matmul(x1.astype(np.int32), x2.astype(np.int32)) * scale
    with ms_custom_ops.exec_mode(exec_mode):
        x2_nz = ms_custom_ops.trans_data(_t(x2), transdata_type=1)
        out = ms_custom_ops.quant_batch_matmul(_t(x1), x2_nz, _t(scale), x2_format="FRACTAL_NZ", output_dtype=torch.bfloat16)
    assert tuple(x2_nz.shape) == (batch, n // 16, k // 64, 1024) and out.shape == (batch, m, n)
    assert np.allclose(expected, out.float().cpu().numpy(), 0.01)                 # reference's bar
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale))
    # one x2 for every batch of x1, 16 rows each: the streaming decode kernel on packed weights
    x1d = rng.integers(-127, 128, (3, 16, 320)).astype(np.int8)
    w = rng.integers(-127, 128, (320, 272)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, 272).astype(np.float32)
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1d), ms_custom_ops.trans_data(_t(w), 1), _t(sc), x2_format="FRACTAL_NZ",
                                               output_dtype=torch.bfloat16)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1d.reshape(-1, 320), w, sc).reshape(3, 16, 272))


def test_default_output_dtype_is_float16(device):
    x1 = torch.ones(16, 32, dtype=torch.int8, device="cuda")
    x2 = torch.ones(32, 16, dtype=torch.int8, device="cuda")
    out = ms_custom_ops.quant_batch_matmul(x1, x2, torch.ones(1, device="cuda"))
    assert out.dtype == torch.float16 and (out == 32).all()


@pytest.mark.parametrize("exec_mode", MODES)
def test_custom_quant_batch_matmul_batched(device, exec_mode):
    rng = np.random.default_rng(1)
    batch, m, k, n = 2, 128, 256, 128
    x1 = rng.integers(-5, 5, (batch, m, k)).astype(np.int8)
    x2 = rng.integers(-5, 5, (batch, k, n)).astype(np.int8)
    scale = rng.uniform(0.5, 1.5, n).astype(np.float32)
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), output_dtype=torch.bfloat16)
    assert out.shape == (batch, m, n)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale))


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_custom_quant_batch_matmul_pertoken(device, exec_mode, dtype):
    rng = np.random.default_rng(2)
    m, k, n = 64, 512, 128
    x1 = rng.integers(-5, 5, (m, k)).astype(np.int8)
    x2 = rng.integers(-5, 5, (k, n)).astype(np.int8)
    scale = np.ones([n]).astype(np.float32)
    pts = rng.standard_normal(m).astype(np.float32)
    expected = np.matmul(x1.astype(np.int32), x2.astype(np.int32)) * scale * pts.reshape(-1, 1)
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), pertoken_scale=_t(pts), output_dtype=dtype)
    assert np.allclose(expected, out.float().cpu().numpy(), 0.01, atol=1e-2)
    name = "bf16" if dtype == torch.bfloat16 else "f16"
    ref = O.quant_batch_matmul_oracle(x1, x2, scale, None, pts, out_dtype=name)
    assert np.array_equal(_bits(out), ref.view(np.uint16))


@pytest.mark.parametrize("exec_mode", MODES)
def test_custom_quant_batch_matmul_with_transpose(device, exec_mode):
    rng = np.random.default_rng(3)
    batch, m, k, n = 8, 32, 64, 512
    x1 = rng.integers(-5, 5, (batch, k, m)).astype(np.int8)
    x2 = rng.integers(-5, 5, (batch, n, k)).astype(np.int8)
    scale = rng.standard_normal(1).astype(np.float32)
    expected = np.matmul(x1.astype(np.int32).transpose(0, 2, 1), x2.astype(np.int32).transpose(0, 2, 1)) * scale
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), transpose_x1=True, transpose_x2=True,
                                               output_dtype=torch.bfloat16)
    assert out.shape == (batch, m, n)
    assert np.allclose(expected, out.float().cpu().numpy(), 0.01)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale, transpose_x1=True, transpose_x2=True))


@pytest.mark.parametrize("exec_mode", MODES)
def test_custom_quant_batch_matmul_with_scale_int64(device, exec_mode):
    rng = np.random.default_rng(4)
    batch, m, k, n = 8, 16, 256, 96
    x1 = rng.integers(-5, 5, (batch, m, k)).astype(np.int8)
    x2 = rng.integers(-5, 5, (batch, k, n)).astype(np.int8)
    scale = rng.standard_normal(n).astype(np.float32)
    scale_i64 = O.encode_scale_int64_qbmm(scale)
    expected = np.matmul(x1.astype(np.int32), x2.astype(np.int32)) * scale
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale_i64), output_dtype=torch.float16)
    assert np.allclose(expected, out.float().cpu().numpy(), 0.01, atol=1e-2)
    ref = O.quant_batch_matmul_oracle(x1, x2, O.decode_scale_int64(scale_i64), out_dtype="f16")
    assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_broadcast_batches_and_pertoken_with_batches(device):
    rng = np.random.default_rng(5)
    x1 = rng.integers(-127, 128, (3, 1, 16, 64), dtype=np.int8)
    x2 = rng.integers(-127, 128, (5, 64, 32), dtype=np.int8)
    scale = rng.uniform(1e-3, 1e-2, 32).astype(np.float32)
    pts = rng.uniform(1e-3, 1e-2, 16).astype(np.float32)
    bias = rng.integers(-1000, 1001, 32).astype(np.int32)
    out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), None, _t(bias), _t(pts),
                                           output_dtype=torch.bfloat16)
    assert out.shape == (3, 5, 16, 32)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale, bias, pts))
    x2d = rng.integers(-127, 128, (64, 32), dtype=np.int8)      # 2-D x2 against batched x1
    out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2d), _t(scale), None, _t(bias), output_dtype=torch.bfloat16)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2d, scale, bias))


@pytest.mark.parametrize("m", [1, 16, 256, 2048])
def test_llama_ffn_linear_sweep_quarter_size(device, m):
    """Dense W8A8 linear sweep (K=4096, N=11008 at 1/4 size): decode rows take the split-K streaming
    kernel, prefill rows the MFMA tile kernel; every M is bit-exact."""
    rng = np.random.default_rng(10 + m)
    k, n = 1024, 2752
    x1 = rng.integers(-127, 128, (m, k), dtype=np.int8)
    x2 = rng.integers(-127, 128, (k, n), dtype=np.int8)
    scale = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    pts = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.integers(-1000, 1001, n).astype(np.int32)
    out = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), None, _t(bias), _t(pts),
                                           output_dtype=torch.bfloat16)
    assert np.array_equal(_bits(out), O.quant_batch_matmul_oracle(x1, x2, scale, bias, pts))
    acc = ms_custom_ops.quant_batch_matmul(_t(x1), _t(x2), _t(scale), None, _t(bias), output_dtype=torch.int32)
    assert np.array_equal(acc.cpu().numpy(), O.int32_matmul_exact(x1, x2) + bias)


def test_qbmm_errors(device):
    x1 = torch.zeros(16, 64, dtype=torch.int8, device="cuda")
    x2 = torch.zeros(64, 32, dtype=torch.int8, device="cuda")
    s = torch.ones(32, device="cuda")
    q = ms_custom_ops.quant_batch_matmul
    with pytest.raises(RuntimeError, match="'x2_format' is only support"):
        q(x1, x2, s, x2_format="NCHW")
    with pytest.raises(ValueError, match="'FRACTAL_NZ' takes an x2 prepacked by trans_data"):
        q(x1, x2, s, x2_format="FRACTAL_NZ")
    with pytest.raises(ValueError, match="'transpose_x2' must be false"):
        q(x1, ms_custom_ops.trans_data(x2, 1), s, transpose_x2=True, x2_format="FRACTAL_NZ")
    with pytest.raises(RuntimeError, match="'offset' is not implemented"):
        q(x1, x2, s, offset=s)
    with pytest.raises(RuntimeError, match="'output_dtype' must be"):
        q(x1, x2, s, output_dtype=torch.int8)
    with pytest.raises(RuntimeError, match="'scale' must have 1 or N"):
        q(x1, x2, torch.ones(5, device="cuda"))
    with pytest.raises(RuntimeError, match="must be int8"):
        q(x1.half(), x2, s)
