"""Full BASELINE sizes on the GPU.  The oracle's answer for these sizes is committed as sha256
digests (tests/golden/digests.json, made by tests/golden/make_fixtures.py --full), so the GPU result
is compared bit for bit without running the oracle on the box; on top of that come
size-independent properties: the per-group column checksum identity
    sum_m acc[m, :] over a group == (sum_m x[m, :]) @ w[g]      (exact in int64 / float64)
linearity in x (negating x negates every accumulator), and agreement of both weight layouts."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi, workloads
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def _launch(tx, tw, tg, ts, tp, tb, m, k, n, e, out_dt, nk=False, override=0, packed=False):
    raw = out_dt == cabi.DT_I32
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=out_dt, group_list_dtype=cabi.DT_I64,
                    bias_dtype=cabi.DT_I32 if tb is not None else 0,
                    scale_dtype=0 if (raw or ts is None) else cabi.DT_F32,
                    per_token_dtype=0 if (raw or tp is None) else cabi.DT_F32, transpose_b=int(nk),
                    kernel_override=override, weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR)
    ws = op.plan(m, k, n, e)
    tws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda:0")
    out = torch.empty((m, n), dtype=torch.int32 if raw else torch.int16, device="cuda:0")
    ins = [tx.data_ptr(), tw.data_ptr(), tb.data_ptr() if tb is not None else None,
           None if (raw or ts is None) else ts.data_ptr(), tg.data_ptr(),
           None if (raw or tp is None) else tp.data_ptr(), None, None]
    op.launch(ins, out.data_ptr(), tws.data_ptr(), ws, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    info = op.plan_info()
    op.close()
    return out, info


@pytest.mark.parametrize("name", ["c1", "c2_m1", "c2_m16", "c2_m256", "c2_m2048", "c3", "c4"])
def test_full_size_workload_bit_exact_and_checksums(device, name):
    dig = json.load(open(os.path.join(GOLDEN, "digests.json")))[f"{name}/1"]
    wl = workloads.make(name)
    assert _sha(wl.x) == dig["x"] and _sha(wl.w) == dig["w"] and wl.group_list.tolist() == dig["group_list"]
    tx, tw = torch.from_numpy(wl.x).cuda(), torch.from_numpy(wl.w).cuda()
    tg = torch.from_numpy(wl.group_list).cuda()
    ts, tp = torch.from_numpy(wl.scale).cuda(), torch.from_numpy(wl.per_token).cuda()
    tb = None if wl.bias is None else torch.from_numpy(wl.bias).cuda()

    acc, info = _launch(tx, tw, tg, None, None, None, wl.m, wl.k, wl.n, wl.e, cabi.DT_I32)
    assert _sha(acc.cpu().numpy()) == dig["acc"], info                       # int32 accumulators, bit-exact
    # ([E,K,N] as stored: the prefill configurations run the persistent tile kernel through LDS transpose reads, a few
    # hundred rows the small tiles on the same path)
    assert "layout=[E,K,N]" in info and (("tile_256x256x128_w4" if wl.m >= 2048 else "skinny" if wl.m <= 16 else "tile_") in info), info
    bits, info = _launch(tx, tw, tg, ts, tp, tb, wl.m, wl.k, wl.n, wl.e, cabi.DT_BF16)
    assert _sha(bits.cpu().numpy().view(np.uint16)) == dig["bf16"], info     # bf16 output, bit-exact

    # checksum of checksums per group, exact in float64 (|values| < 2**53)
    starts, ends = O.group_bounds(wl.group_list)
    for g in range(wl.e):
        a, b = int(starts[g]), int(ends[g])
        if b <= a:
            continue
        col = acc[a:b].sum(dim=0, dtype=torch.int64).cpu().numpy()
        want = wl.x[a:b].astype(np.float64).sum(0) @ wl.w[g].astype(np.float64)
        assert np.array_equal(col.astype(np.float64), want), (name, g)

    # linearity: -x gives -acc
    neg, _ = _launch(-tx, tw, tg, None, None, None, wl.m, wl.k, wl.n, wl.e, cabi.DT_I32)
    assert torch.equal(neg, -acc)
    del neg

    # the [E,N,K] storage gives the same accumulators
    twt = tw.transpose(1, 2).contiguous()
    acc_nk, info = _launch(tx, twt, tg, None, None, None, wl.m, wl.k, wl.n, wl.e, cabi.DT_I32, nk=True)
    assert torch.equal(acc_nk, acc), info
    del acc_nk

    # ... and so does the packed layout: streaming kernels for the decode configurations, the small tile kernels for a
    # few hundred rows, the persistent tile kernel for the prefill ones
    from gpu_utils import pack_on_device
    twp = pack_on_device(twt, wl.e, wl.k, wl.n, True)
    del twt
    acc_p, info = _launch(tx, twp, tg, None, None, None, wl.m, wl.k, wl.n, wl.e, cabi.DT_I32, packed=True)
    assert ("tile_256x256x128_w4" if wl.m >= 2048 else "stream" if wl.m <= 64 else "tile_") in info and "layout=packed" in info, info
    assert torch.equal(acc_p, acc), info
    del acc_p
    bits_p, info = _launch(tx, twp, tg, ts, tp, tb, wl.m, wl.k, wl.n, wl.e, cabi.DT_BF16, packed=True)
    assert _sha(bits_p.cpu().numpy().view(np.uint16)) == dig["bf16"], info


def test_full_size_c5_weight_only_against_sampled_exact_rows(device):
    """C5 at full size: every row is checked against the float64 oracle (32 rows are cheap)."""
    from gpu_utils import run_a16w8
    wl = workloads.make("c5")
    xf, sf, of = (O.bf16_bits_to_f32(v) for v in (wl.x, wl.scale, wl.offset))
    exact = O.a16w8_grouped_f64(xf, wl.w, sf, of, wl.group_list)
    starts, ends = O.group_bounds(wl.group_list)
    mag = np.zeros_like(exact)
    for g in range(wl.e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(wl.w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    for packed in (False, True):
        bits, info = run_a16w8(wl.x, wl.w, wl.scale, wl.offset, wl.group_list, packed=packed)
        got = O.bf16_bits_to_f32(bits).astype(np.float64)
        assert (np.abs(got - exact) <= 2.0 ** -7 * np.abs(exact) + 1e-5 * mag).all(), info
        assert ("a16w8_stream" in info) == packed


def test_full_size_w8a8_moe_decode_both_layouts(device):
    """c3's weights at decode time (32 rows over 8 experts) at full size: row-major and packed weights against the
    oracle, bit-exact (the oracle needs 32 x 4096 x 14336 multiply-adds: cheap)."""
    from gpu_utils import run_w8a8
    wl = workloads.make("c3_decode")
    ref_bits, ref_acc = O.grouped_matmul_w8a8(wl.x, wl.w, wl.group_list, None, wl.scale, wl.per_token, return_acc=True)
    for packed in (False, True):
        acc, info = run_w8a8(wl.x, wl.w, wl.group_list, out="i32", packed=packed)
        assert np.array_equal(acc, ref_acc), info
        bits, info = run_w8a8(wl.x, wl.w, wl.group_list, None, wl.scale, wl.per_token, packed=packed)
        assert np.array_equal(bits, ref_bits), info
        assert ("w8a8_stream" in info) == packed
