"""grouped_matmul_w4 (int8 activations x int4 weights with K-group scales): GPU parity against the restated golden of
tests/st/test_grouped_matmul_w4.py:78-139, through the C ABI and through the Python entry.

Bar: the reference's own comparator (custom_compare, tests/st/st_utils.py:23-49: relative error above 0.004 on at
most 0.4 % of the elements of the float16 output) against the golden, and, tighter, every element within one
float16 rounding (2^-10 relative + a float32 summation allowance) of the exact integer form evaluated in float64."""
import random

import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu


def _case(seed, m, k, n, e, g, group_list=None):
    rng = np.random.default_rng(seed)
    x_fp = rng.uniform(-0.3, 0.3, (m, k)).astype(np.float16)                     # reference distributions (:99-101)
    from oracle import moe_oracle as M
    x, xs = M.dyn_quant(x_fp)
    wq, ws = O.quant_int4_groups(rng.uniform(-0.3, 0.3, (e, k, n)).astype(np.float16), g)
    wp = np.ascontiguousarray(O.pack_int4(wq.transpose(0, 2, 1)))
    if group_list is None:                                                        # generate_random_numbers (:64-71)
        random.seed(seed)
        group_list = sorted(random.choices(range(1, m + 1), k=e - 1) + [m])
    return x, xs, wp, ws.reshape(e, k // g, n), np.asarray(group_list, dtype=np.int32)


def _run(x, xs, wp, ws, gl, g):
    dev = "cuda:0"
    m, k = x.shape
    e, n = wp.shape[0], wp.shape[1]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    tx, txs, tw, tws, tgl = t(x), t(xs), t(wp), t(ws), t(gl)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=dev)
    cabi.gmm_a8w4(tx.data_ptr(), tw.data_ptr(), tgl.data_ptr(), txs.data_ptr(), tws.data_ptr(), out.data_ptr(), m, k, n, e, g,
                  torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _check(out, x, xs, wp, ws, gl, g):
    rows = int(gl[-1])
    gold = O.golden_grouped_a8w4(x, wp, gl, xs, ws, g)[:rows]
    exact = O.grouped_a8w4_f64(x, wp, gl, xs, ws, g)[:rows]
    got = out[:rows].astype(np.float64)
    assert np.isfinite(got).all()
    assert O.count_compare(out[:rows].astype(np.float32), gold, 0.004)              # the reference's bar for float16
    err = np.abs(got - exact)
    assert np.all(err <= np.abs(exact) * (2.0 ** -10 + 1e-5) + 1e-7)             # one float16 rounding of the exact value
    assert np.isnan(out[rows:].astype(np.float32)).all()                          # rows past the last boundary are not written


@pytest.mark.parametrize("m,k,n,e,g", [(17, 7168, 256, 256, 256),       # the reference's level-0 shape (:151)
                                      (32, 512, 7168, 256, 256)])       # a level-1 shape (:166)
def test_a8w4_reference_cases(m, k, n, e, g):
    case = _case(m + k, m, k, n, e, g)
    _check(_run(*case, g), *case, g)


@pytest.mark.parametrize("m,k,n,e,g,gl", [
    (40, 256, 48, 4, 32, [0, 19, 19, 40]),          # more than eight rows in a group (several row blocks), empty groups, N tail
    (3, 64, 16, 2, 64, [3, 3]),                      # one K group, everything in the first expert
    (12, 8192, 80, 3, 128, [1, 2, 9]),               # the longest K, last boundary below m
])
def test_a8w4_ragged_groups_row_blocks_and_tails(m, k, n, e, g, gl):
    case = _case(7, m, k, n, e, g, gl)
    _check(_run(*case, g), *case, g)


@pytest.mark.parametrize("seed", range(10))
def test_a8w4_random_small_shapes(seed):
    # a seeded sweep: K from 32 to 1024 (1 to 32 pieces of 32 per column: every lane-sharing factor), K groups of 32 to
    # 256, any N, 1 to 40 experts with empty ones, up to 60 rows (groups of more than four rows take several row blocks)
    rng = np.random.default_rng(500 + seed)
    g = int(rng.choice([32, 64, 128, 256]))
    k = g * int(rng.integers(1, 1024 // g + 1))
    n = int(rng.integers(1, 90))
    e = int(rng.integers(1, 41))
    m = int(rng.integers(1, 61))
    gl = sorted(int(v) for v in rng.integers(0, m + 1, e - 1)) + [m - int(rng.choice([0, 0, 1])) if m > 1 else m]
    gl = [int(v) for v in np.maximum.accumulate(gl)]
    case = _case(seed, m, k, n, e, g, gl)
    _check(_run(*case, g), *case, g)


def test_a8w4_rejects_bad_shapes():
    with pytest.raises(RuntimeError):
        cabi.gmm_a8w4(1, 1, 1, 1, 1, 1, 4, 100, 16, 2, 32)        # k not a multiple of 32
    with pytest.raises(RuntimeError):
        cabi.gmm_a8w4(1, 1, 1, 1, 1, 1, 4, 256, 16, 2, 96)        # k not a multiple of the group size
    with pytest.raises(RuntimeError):
        cabi.gmm_a8w4(1, 1, 1, 1, 1, 1, 4, 16384, 16, 2, 256)     # k beyond the supported range


# ------------------------------------------------------------------------------- the Python entry, both modes
@pytest.mark.parametrize("exec_mode", ["graph", "pynative"])
@pytest.mark.parametrize("batch_size", [5, 17])
def test_gmm_w4_swft_0(exec_mode, batch_size):
    # the reference's level-0 case (tests/st/test_grouped_matmul_w4.py:146-158): m in {5, 17}, k = 7168, n = 256, 256 experts,
    # with the bias the reference op requires (8 * column sums of the dequantised weight, :103-106)
    import ms_custom_ops_amd as ms_custom_ops
    e, k, n, g = 256, 7168, 256, 256
    x, xs, wp, ws, gl = _case(batch_size, batch_size, k, n, e, g)
    w_deq = (O.unpack_int4(wp).transpose(0, 2, 1).reshape(e, k // g, g, n).astype(np.float32) * ws.reshape(e, k // g, 1, n)).reshape(e, k, n)
    bias = np.matmul(np.ones((e, 1, k), dtype=np.float16) * 8, w_deq).astype(np.float32).reshape(e, n)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    mode = ms_custom_ops.GRAPH_MODE if exec_mode == "graph" else ms_custom_ops.PYNATIVE_MODE
    with ms_custom_ops.exec_mode(mode):
        out = ms_custom_ops.grouped_matmul_w4(t(x), t(wp.view(np.int8)), t(gl), t(bias), t(xs), t(ws))
    assert out.dtype == torch.float16 and out.shape == (batch_size, n)
    expect = O.golden_grouped_a8w4(x, wp, gl, xs, ws, g)
    assert O.count_compare(out.cpu().numpy().astype(np.float32), expect, 0.004)


def test_gmm_w4_rejects_what_the_reference_rejects():
    import ms_custom_ops_amd as ms_custom_ops
    z = lambda shape, dt: torch.zeros(shape, dtype=dt, device="cuda")
    x, w, gl = z((4, 64), torch.int8), z((2, 16, 32), torch.uint8), z((2,), torch.int32)
    b, xs, ws = z((2, 16), torch.float32), z((4,), torch.float32), z((2, 2, 16), torch.float32)
    with pytest.raises(RuntimeError, match="input 'x' must be 2D"):
        ms_custom_ops.grouped_matmul_w4(x[0], w, gl, b, xs, ws)
    with pytest.raises(RuntimeError, match="must have the same dimension of 'k'"):
        ms_custom_ops.grouped_matmul_w4(z((4, 96), torch.int8), w, gl, b, xs, ws)
    with pytest.raises(RuntimeError, match="input 'x' must be int8"):
        ms_custom_ops.grouped_matmul_w4(z((4, 64), torch.float16), w, gl, b, xs, ws)
    with pytest.raises(RuntimeError, match="input 'bias' must be float32"):
        ms_custom_ops.grouped_matmul_w4(x, w, gl, z((2, 16), torch.float16), xs, ws)
    with pytest.raises(RuntimeError, match="input 'group_list' must be int32"):
        ms_custom_ops.grouped_matmul_w4(x, w, z((2,), torch.int64), b, xs, ws)
    with pytest.raises(ValueError, match="weight_scale must be"):
        ms_custom_ops.grouped_matmul_w4(x, w, gl, b, xs, z((2, 2, 8), torch.float32))
    assert ms_custom_ops.grouped_matmul_w4(x, w, gl, b, xs, ws).shape == (4, 16)


def test_a8w4_malformed_group_list_is_clamped_like_the_other_kernels():
    # a list that is not monotonic or runs past m: the row end of a group is the running maximum clamped into [0, m],
    # so groups never overlap and the result is that of the repaired list
    m, k, n, e, g = 12, 256, 48, 4, 64
    bad = [5, 3, 8, 100]
    good = [5, 5, 8, 12]
    case_bad = _case(11, m, k, n, e, g, bad)
    case_good = _case(11, m, k, n, e, g, good)
    a = _run(*case_bad, g)
    b = _run(*case_good, g)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    _check(b, *case_good, g)
