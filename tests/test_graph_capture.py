"""msco_gmm_launch allocates nothing and never synchronises, so a launch can be recorded into a HIP graph: the graph is
replayed several times with eager work and synchronisations in between, and every replay is compared with the eager
result (bit-exact).  Covers the kernels with cross-workgroup state (K split: self-resetting arrival counters) and the
persistent tile kernel."""
import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", ["decode_split_k", "packed_decode", "packed_rows_split_k", "persistent_tile", "small_tile_split_k"])
def test_launch_is_graph_capturable_and_replays_match_eager(device, case):
    from gpu_utils import pack_on_device
    shapes = {"decode_split_k": (16, 4096, 1024, 1, False, False), "packed_decode": (20, 2048, 1024, 4, False, True),
              "packed_rows_split_k": (128, 4096, 256, 1, False, True), "persistent_tile": (2048, 512, 8192, 8, True, False),
              "small_tile_split_k": (128, 2048, 1024, 1, True, False)}
    m, k, n, e, nk, packed = shapes[case]
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    x = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (e, n, k) if nk else (e, k, n), dtype=torch.int8, device="cuda", generator=g)
    if packed:
        w = pack_on_device(w, e, k, n, nk)
    scale = torch.rand(e, n, device="cuda", generator=g) * 9e-3 + 1e-3
    pt = torch.rand(m, device="cuda", generator=g) * 9e-3 + 1e-3
    gl = torch.tensor([(m * (i + 1)) // e for i in range(e)], dtype=torch.int64, device="cuda")
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64, scale_dtype=cabi.DT_F32,
                    per_token_dtype=cabi.DT_F32, transpose_b=int(nk and not packed),
                    weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR)
    ws_bytes = op.plan(m, k, n, e)
    if "split_k" in case:
        assert "split_k=1 " not in op.plan_info(), op.plan_info()
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda")
    out = torch.empty((m, n), dtype=torch.int16, device="cuda")
    ins = [x.data_ptr(), w.data_ptr(), None, scale.data_ptr(), gl.data_ptr(), pt.data_ptr(), None, None]
    op.launch(ins, out.data_ptr(), ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = out.clone()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            op.launch(ins, out.data_ptr(), ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for replay in range(4):
        out.fill_(0x7FC0)                      # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), (case, replay, op.plan_info())
        # an eager launch between replays shares the handle's arrival counters with the graph's launches
        op.launch(ins, out.data_ptr(), ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), (case, replay, "eager after replay")
    op.close()


def test_moe_chain_is_graph_capturable(device):
    """Quantising routing -> int8 grouped matmul on its outputs -> un-permutation, recorded as one graph: none of the
    three allocates, clears memory with a memset node or synchronises, and the routing output feeds the matmul's
    group_list on the device.  Every replay must reproduce the eager result bit for bit."""
    rows, hidden, k, e, n = 256, 1024, 2, 8, 512
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    x = torch.randn((rows, hidden), dtype=torch.bfloat16, device="cuda", generator=g)
    idx = torch.argsort(torch.randn(rows, e, device="cuda", generator=g), dim=1)[:, :k].to(torch.int32).contiguous()
    w = torch.randint(-127, 128, (e, hidden, n), dtype=torch.int8, device="cuda", generator=g)
    wscale = torch.rand(e, n, device="cuda", generator=g) * 9e-3 + 1e-3
    probs = torch.rand((rows, k), dtype=torch.bfloat16, device="cuda", generator=g)
    xq = torch.empty((rows * k, hidden), dtype=torch.int8, device="cuda")
    xs = torch.empty(rows * k, dtype=torch.float32, device="cuda")
    ridx = torch.empty(rows * k, dtype=torch.int32, device="cuda")
    cum = torch.empty(e, dtype=torch.int32, device="cuda")
    y = torch.empty((rows * k, n), dtype=torch.int16, device="cuda")
    out = torch.empty((rows, n), dtype=torch.int16, device="cuda")
    rws_bytes = cabi.moe_init_routing_v2_workspace_bytes(rows, k, e)
    rws = torch.empty(max(rws_bytes, 1), dtype=torch.uint8, device="cuda")
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I32, scale_dtype=cabi.DT_F32,
                    per_token_dtype=cabi.DT_F32)
    ws_bytes = op.plan(rows * k, hidden, n, e)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda")

    def chain(stream):
        cabi.moe_init_routing_v2_quant(x.data_ptr(), idx.data_ptr(), xq.data_ptr(), xs.data_ptr(), ridx.data_ptr(), cum.data_ptr(), None,
                                       rws.data_ptr(), rws_bytes, rows, hidden, k, e, cabi.DT_BF16, 1, stream)
        op.launch([xq.data_ptr(), w.data_ptr(), None, wscale.data_ptr(), cum.data_ptr(), xs.data_ptr(), None, None], y.data_ptr(),
                  ws.data_ptr(), ws_bytes, stream)
        cabi.moe_token_unpermute(y.data_ptr(), ridx.data_ptr(), probs.data_ptr(), out.data_ptr(), rows, k, n, cabi.DT_BF16, stream)

    chain(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = out.clone()
    assert eager.ne(0).any()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            chain(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for replay in range(3):
        for t in (xq, y, out):
            t.fill_(0)                         # eager work between replays
        xs.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), replay
    op.close()
