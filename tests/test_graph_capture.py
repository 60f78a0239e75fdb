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
