"""msco_gmm_launch_static -- the launch for callers that cannot allocate -- against msco_gmm_launch on the same inputs:
bit-exact outputs, on two calls in a row (the second on a smaller problem, so that stale contents of the library's
fixed workspace array from the first call would show), and its refusal of a plan whose workspace does not fit."""
import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi

pytestmark = pytest.mark.gpu


def _problem(seed, m, k, n, e, group_list, packed):
    from gpu_utils import to_dev, pack_on_device
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    tx, tw, ts, tp, tb = to_dev(x), to_dev(w), to_dev(scale), to_dev(pt), to_dev(bias)
    if packed:
        tw = pack_on_device(tw, e, k, n)
    tg = to_dev(np.asarray(group_list, dtype=np.int64))
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64, bias_dtype=cabi.DT_I32,
                    scale_dtype=cabi.DT_F32, per_token_dtype=cabi.DT_F32,
                    weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR)
    ws = op.plan(m, k, n, e)
    ins = [t.data_ptr() for t in (tx, tw, tb, ts, tg, tp)] + [None, None]
    keep = (tx, tw, ts, tp, tb, tg)
    return op, ws, ins, keep, (m, n)


def _both(op, ws, ins, shape):
    st = torch.cuda.current_stream().cuda_stream
    m, n = shape
    ref = torch.full((m, n), 0x7FC0, dtype=torch.int16, device="cuda:0")
    got = torch.full((m, n), 0x7FC0, dtype=torch.int16, device="cuda:0")
    tws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda:0")
    op.launch(ins, ref.data_ptr(), tws.data_ptr(), ws, st)
    op.launch_static(ins, got.data_ptr(), st)
    torch.cuda.synchronize()
    return ref.cpu().numpy(), got.cpu().numpy()


@pytest.mark.parametrize("packed", [True, False])
def test_static_workspace_launch_matches_the_workspace_launch_twice_in_a_row(packed):
    # a dense decode with a long K and then a smaller grouped decode: both plans split K across workgroups, so both
    # exchange partial tiles through the workspace
    first = _problem(1, 16, 8192, 1024, 1, [16], packed)
    second = _problem(2, 24, 4096, 512, 4, [5, 5, 17, 24], packed)
    for op, ws, ins, keep, shape in (first, second):
        assert 0 < ws <= cabi.STATIC_WORKSPACE_BYTES, op.plan_info()
        assert "split_k=1 " not in op.plan_info()
        ref, got = _both(op, ws, ins, shape)
        assert not (ref == 0x7FC0).all()
        assert np.array_equal(ref, got), op.plan_info()
    # a warm call takes no device memory: the free byte count of the device does not move across it
    op, ws, ins, keep, (m, n) = second
    got = torch.empty((m, n), dtype=torch.int16, device="cuda:0")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    op.launch_static(ins, got.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for op, *_ in (first, second):
        op.close()


def test_static_workspace_launch_refuses_a_plan_that_does_not_fit():
    # 128 x 128 tiles with a K split: the worst-case partial tiles (one more m-tile per group) exceed the fixed array
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_I32, group_list_dtype=cabi.DT_I64, kernel_override=cabi.OV_TILE_128,
                    force_split_k=8)
    ws = op.plan(128, 4096, 2048, 8)   # 144 tiles x 8 slices x 64 KiB = 72 MiB
    assert ws > cabi.STATIC_WORKSPACE_BYTES, op.plan_info()
    x = torch.zeros(8, dtype=torch.int8, device="cuda:0")
    with pytest.raises(cabi.BackendError) as err:
        op.launch_static([x.data_ptr(), x.data_ptr(), None, None, x.data_ptr()], x.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert err.value.status == 5   # MSCO_ERR_WORKSPACE
    op.close()
