"""moe_init_routing_v2 and moe_token_unpermute through the Python entries -- the cases of the reference's
tests/st/test_custom_moe_init_routing_v2.py and tests/st/test_custom_moe_token_unpermute.py (same input
streams, both execution modes, the rejected arguments), checked bit for bit against the oracle."""
import numpy as np
import pytest
import torch

import ms_custom_ops_amd as ms_custom_ops
from oracle import moe_oracle as M

pytestmark = pytest.mark.gpu
MODES = [ms_custom_ops.GRAPH_MODE, ms_custom_ops.PYNATIVE_MODE]


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("num_rows,hidden,k,expert_num,flag", [(10, 2048, 8, 8, 1), (1001, 1024, 2, 64, 2), (64, 7168, 6, 256, 1)])
def test_moe_init_routing_v2(device, exec_mode, num_rows, hidden, k, expert_num, flag):
    np.random.seed(0)
    x = np.random.uniform(-1, 1, size=(num_rows, hidden)).astype(np.float16)
    expert_idx = np.random.randint(0, expert_num, size=(num_rows, k)).astype(np.int32)
    with ms_custom_ops.exec_mode(exec_mode):
        outs = ms_custom_ops.moe_init_routing_v2(_t(x), _t(expert_idx), 0, 0, expert_num, 0, flag, False)
    assert len(outs) == 4
    ref_x, ref_idx, ref_tok = M.moe_init_routing_v2(x, expert_idx, expert_num, flag)
    assert outs[0].dtype == torch.float16 and outs[0].shape == (num_rows * k, hidden)
    assert outs[1].dtype == torch.int32 and outs[2].shape == (expert_num,) and outs[3].shape == (expert_num,)
    np.testing.assert_allclose(outs[0].cpu().numpy(), ref_x, rtol=1e-3, atol=1e-3)      # reference's bar
    assert np.array_equal(outs[0].cpu().numpy().view(np.uint16), ref_x.view(np.uint16))
    assert np.array_equal(outs[1].cpu().numpy(), ref_idx)
    assert np.array_equal(outs[2].cpu().numpy(), ref_tok)


def test_moe_init_routing_v2_rejects_what_the_reference_rejects(device):
    x = torch.zeros(4, 1024, dtype=torch.float16, device="cuda")
    idx = torch.zeros(4, 2, dtype=torch.int32, device="cuda")
    for args, text in [((1, 0, 8, 0, 1, False), "active_num must be 0"), ((0, 2, 8, 0, 1, False), "expert_capacity must be 0"),
                       ((0, 0, 8, 1, 1, False), "drop_pad_mode must be 0"), ((0, 0, 300, 0, 1, False), "expert_num must be less than or equal to 256")]:
        with pytest.raises(ValueError, match=text):
            ms_custom_ops.moe_init_routing_v2(x, idx, *args)
    with pytest.raises(ValueError, match="multiple of 1024"):
        ms_custom_ops.moe_init_routing_v2(torch.zeros(4, 1000, dtype=torch.float16, device="cuda"), idx, 0, 0, 8, 0, 1, False)
    with pytest.raises(ValueError, match="rank of x must be 2"):
        ms_custom_ops.moe_init_routing_v2(x[0], idx, 0, 0, 8, 0, 1, False)


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("token_num", [1, 16, 1001])
@pytest.mark.parametrize("hidden", [7168, 2048])
def test_moe_token_unpermute(device, exec_mode, token_num, hidden):
    top_k = 8
    np.random.seed(token_num)
    permute_token = np.random.randn(token_num * top_k, hidden).astype(np.float16)
    sorted_idx = np.arange(token_num * top_k, dtype=np.int32)
    np.random.shuffle(sorted_idx)
    probs = np.random.randn(token_num, top_k).astype(np.float16)
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.moe_token_unpermute(_t(permute_token), _t(sorted_idx), _t(probs))
    expected = M.moe_token_unpermute(permute_token, sorted_idx, probs)
    assert out.dtype == torch.float16 and out.shape == (token_num, hidden)
    assert np.allclose(out.cpu().numpy(), expected, rtol=1e-3, atol=1e-3)               # reference's bar
    assert np.array_equal(out.cpu().numpy().view(np.uint16), expected.view(np.uint16))


@pytest.mark.parametrize("exec_mode", MODES)
def test_moe_token_unpermute_unsupported_arguments(device, exec_mode):
    def make(hidden, top_k=8, dtype=np.float16):
        return (_t(np.zeros((16 * top_k, hidden), dtype)), _t(np.arange(16 * top_k, dtype=np.int32)), _t(np.zeros((16, top_k), dtype)))
    with ms_custom_ops.exec_mode(exec_mode):
        with pytest.raises(RuntimeError, match="Tiling error"):                         # test_custom_moe_token_unpermute.py:100-103
            ms_custom_ops.moe_token_unpermute(*make(1024))
        with pytest.raises(RuntimeError, match="Tiling error"):
            ms_custom_ops.moe_token_unpermute(*make(7168, top_k=3))
        with pytest.raises(RuntimeError, match="float16"):
            ms_custom_ops.moe_token_unpermute(*make(7168, dtype=np.float32))
        with pytest.raises(RuntimeError, match="padded_mode"):
            ms_custom_ops.moe_token_unpermute(*make(7168), padded_mode=True)
        with pytest.raises(RuntimeError, match="padded_mode"):
            ms_custom_ops.moe_token_unpermute(*make(7168), restore_shape=(16, 7168))


@pytest.mark.parametrize("exec_mode", MODES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_moe_init_routing_quant_feeds_the_grouped_matmul(device, exec_mode, dtype):
    # routing + per-token int8 quantisation in one step, then the int8 grouped matmul on its three outputs: every
    # stage bit for bit what the goldens give (routing: test_custom_moe_init_routing_v2.py:38-65; quantisation:
    # test_grouped_matmul_w4.py:83-89; matmul: test_grouped_matmul_v4_cops.py:297-301)
    from oracle import gmm_oracle as O
    rows, hidden, k, e, n = 96, 1024, 2, 8, 256
    rng = np.random.default_rng(5)
    xt = torch.from_numpy(rng.uniform(-0.3, 0.3, (rows, hidden)).astype(np.float32)).to(dtype)
    vals = xt.to(torch.float32).numpy() if dtype == torch.bfloat16 else xt.numpy()
    idx = rng.integers(0, e, (rows, k)).astype(np.int32)
    with ms_custom_ops.exec_mode(exec_mode):
        q, scale, ridx, cum = ms_custom_ops.moe_init_routing_quant(xt.cuda(), _t(idx), e, 1)
    ref_rows, ref_idx, ref_cum = M.moe_init_routing_v2(vals, idx, e, 1)
    ref_q, ref_s = M.dyn_quant(ref_rows)
    assert q.dtype == torch.int8 and q.shape == (rows * k, hidden) and scale.dtype == torch.float32 and scale.shape == (rows * k,)
    assert np.array_equal(q.cpu().numpy(), ref_q) and np.array_equal(scale.cpu().numpy().view(np.uint32), ref_s.view(np.uint32))
    assert np.array_equal(ridx.cpu().numpy(), ref_idx) and np.array_equal(cum.cpu().numpy(), ref_cum)
    w = rng.integers(-127, 128, (e, hidden, n)).astype(np.int8)
    ws = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    with ms_custom_ops.exec_mode(exec_mode):
        out = ms_custom_ops.grouped_matmul_v4_cops([q], [_t(w)], None, [_t(ws)], None, None, None, [scale], cum.to(torch.int64),
                                                   None, None, None, split_item=3, group_type=0, group_list_type=0)[0]
    ref = O.grouped_matmul_w8a8(ref_q, w, ref_cum.astype(np.int64), None, ws, ref_s, out_dtype="f16")
    assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_moe_init_routing_quant_rejects_bad_arguments(device):
    idx = torch.zeros(4, 2, dtype=torch.int32, device="cuda")
    with pytest.raises(TypeError, match="Float16 or BFloat16"):
        ms_custom_ops.moe_init_routing_quant(torch.zeros(4, 64, dtype=torch.float32, device="cuda"), idx, 8)
    with pytest.raises(ValueError, match="multiple of 8"):
        ms_custom_ops.moe_init_routing_quant(torch.zeros(4, 60, dtype=torch.float16, device="cuda"), idx, 8)
    with pytest.raises(ValueError, match="expert_num must be in"):
        ms_custom_ops.moe_init_routing_quant(torch.zeros(4, 64, dtype=torch.float16, device="cuda"), idx, 0)
    with pytest.raises(ValueError, match="same number of rows"):
        ms_custom_ops.moe_init_routing_quant(torch.zeros(5, 64, dtype=torch.float16, device="cuda"), idx, 8)
