"""moe_init_routing_v2 and moe_token_unpermute: oracle pins (CPU) and GPU parity through the C ABI.

The oracle restates the reference goldens (tests/st/test_custom_moe_init_routing_v2.py:33-93,
tests/st/test_custom_moe_token_unpermute.py:37-47).  Bar on the GPU: integer outputs and gathered rows
bit-exact; the un-permutation bit-exact too, because the kernel rounds where the golden rounds (the
reference's own tolerance is rtol = atol = 1e-3)."""
import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi
from oracle import moe_oracle as M


# ----------------------------------------------------------------------------------- oracle pins (CPU)
def _f32_nearest_even(fr):
    """The float32 nearest to a Fraction (ties to even), by integer arithmetic only."""
    from fractions import Fraction
    if fr == 0:
        return 0.0
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2 ** 24:
        fr /= 2
        e += 1
    while fr < 2 ** 23:
        fr *= 2
        e -= 1
    m = fr.numerator // fr.denominator
    rest = fr - m
    if rest > Fraction(1, 2) or (rest == Fraction(1, 2) and m % 2 == 1):
        m += 1
    return sign * float(m) * 2.0 ** e                       # exact in a double


def _dyn_quant_by_loops(rows):
    """test_grouped_matmul_w4.py:83-89 element by element: both divisions exactly, rounded to float32 once each; then
    half-to-even to an integer."""
    from fractions import Fraction
    q = np.zeros(rows.shape, dtype=np.int8)
    scale = np.zeros(rows.shape[0], dtype=np.float32)
    for r in range(rows.shape[0]):
        vals = [Fraction(float(v)) for v in rows[r]]
        s = _f32_nearest_even(max(abs(v) for v in vals) / 127)
        scale[r] = s
        for h, v in enumerate(vals):
            d = Fraction(_f32_nearest_even(v / Fraction(s)))
            lo = d.numerator // d.denominator                # floor
            frac = d - lo
            q[r, h] = lo + (1 if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and lo % 2 == 1) else 0)
    return q, scale


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_dyn_quant_oracle_against_exact_loops_and_what_the_formula_fixes(kind):
    rng = np.random.default_rng(11)
    if kind == "f16":
        x = rng.uniform(-0.3, 0.3, (6, 40)).astype(np.float16)               # the reference test's distribution (:99)
        x[1] *= 100
    else:
        x = M.bf16_bits_to_f32((rng.standard_normal((6, 40)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    x[2, 5] = 0
    x[3] = np.abs(x[3]).max() * np.sign(x[3]) * np.where(np.arange(40) % 2 == 0, 0.5, 1.0)   # ties: half of the maximum -> 63.5
    q, s = M.dyn_quant(x)
    q2, s2 = _dyn_quant_by_loops(x.astype(np.float32))
    assert np.array_equal(s.view(np.uint32), s2.view(np.uint32)) and np.array_equal(q, q2)
    x32 = x.astype(np.float32)
    amax = np.abs(x32).max(axis=1)
    assert np.array_equal(np.abs(q).max(axis=1), np.full(6, 127))            # the row maximum maps to +-127
    assert np.all(np.sign(q[np.arange(6), np.abs(x32).argmax(axis=1)]) == np.sign(x32[np.arange(6), np.abs(x32).argmax(axis=1)]))
    assert np.allclose(s * 127, amax, rtol=2e-7)                              # scale * 127 gives the maximum back
    assert np.all(np.abs(x32.astype(np.float64) - q.astype(np.float64) * s[:, None]) <= s[:, None] * 0.5000001)
    assert set(np.unique(q[3])) <= {-127, -64, 64, 127}                       # 63.5 goes to the even neighbour
    qz, sz = M.dyn_quant(np.zeros((2, 8), dtype=np.float16))                  # rows of zeros: scale 0, zeros
    assert not qz.any() and not sz.any()


def test_routing_oracle_tiny_case_by_hand():
    # 3 tokens, k = 2, 3 experts: flat expert ids [2, 0, 1, 2, 0, 0]; stable order of flat positions: 1, 4, 5 | 2 | 0, 3
    x = np.arange(12, dtype=np.float16).reshape(3, 4)
    ex, idx, tok = M.moe_init_routing_v2(x, np.array([[2, 0], [1, 2], [0, 0]], dtype=np.int32), 3, 1)
    assert idx.tolist() == [4, 0, 3, 5, 1, 2]
    assert np.array_equal(ex, x[[0, 2, 2, 1, 0, 1]])
    assert tok.tolist() == [3, 4, 6]
    assert M.moe_init_routing_v2(x, np.array([[2, 0], [1, 2], [0, 0]], dtype=np.int32), 3, 2)[2].tolist() == [3, 1, 2]


@pytest.mark.parametrize("n_rows,k,e", [(1, 1, 1), (17, 2, 8), (130, 6, 64), (64, 8, 256)])
def test_routing_oracle_against_independent_sort_and_invariants(n_rows, k, e):
    rng = np.random.default_rng(n_rows)
    x = rng.uniform(-1, 1, (n_rows, 16)).astype(np.float16)
    idx = rng.integers(0, e, (n_rows, k)).astype(np.int32)
    ex, ridx, cum = M.moe_init_routing_v2(x, idx, e, 1)
    ex2, ridx2, counts = M.moe_init_routing_v2_by_loops(x, idx, e)
    assert np.array_equal(ex, ex2) and np.array_equal(ridx, ridx2) and np.array_equal(cum, np.cumsum(counts))
    assert sorted(ridx.tolist()) == list(range(n_rows * k))                       # a permutation
    flat = idx.reshape(-1)
    dest_expert = np.empty(n_rows * k, dtype=np.int64)
    dest_expert[ridx] = flat
    assert np.all(np.diff(dest_expert) >= 0)                                      # rows end up sorted by expert
    for e_id in range(e):                                                         # stable inside every expert
        pos = np.nonzero(flat == e_id)[0]
        assert np.all(np.diff(ridx[pos]) > 0)
    assert np.array_equal(ex[ridx], np.repeat(x, k, axis=0))                      # every entry got its token's row
    assert cum[-1] == n_rows * k


def test_unpermute_oracle_against_scalar_loops_and_closed_forms():
    rng = np.random.default_rng(3)
    t, k, h = 9, 4, 32
    pt = rng.standard_normal((t * k, h)).astype(np.float16)
    pr = rng.standard_normal((t, k)).astype(np.float16)
    si = rng.permutation(t * k).astype(np.int32)
    got = M.moe_token_unpermute(pt, si, pr)
    # scalar loops with an independent half implementation (torch): round the product, then the running sum
    ref = torch.zeros(t, h, dtype=torch.float16)
    tp, tr = torch.from_numpy(pt), torch.from_numpy(pr)
    for i in range(t):
        for kk in range(k):
            prod = (tr[i, kk].float() * tp[int(si[i * k + kk])].float()).half()
            ref[i] = (ref[i].float() + prod.float()).half()
    assert np.array_equal(got.view(np.uint16), ref.numpy().view(np.uint16))
    # K = 1 with probability one is a plain gather; all-ones data sums to K exactly
    assert np.array_equal(M.moe_token_unpermute(pt[:t], si[:t] % t, np.ones((t, 1), np.float16)), pt[:t][si[:t] % t])
    ones = M.moe_token_unpermute(np.ones((t * k, h), np.float16), si, np.ones((t, k), np.float16))
    assert np.all(ones == k)
    # bfloat16 variant against torch's bfloat16 arithmetic
    pb = torch.randn(t * k, h).bfloat16()
    rb = torch.randn(t, k).bfloat16()
    ref_b = torch.zeros(t, h, dtype=torch.bfloat16)
    for i in range(t):
        for kk in range(k):
            prod = (rb[i, kk].float() * pb[int(si[i * k + kk])].float()).bfloat16()
            ref_b[i] = (ref_b[i].float() + prod.float()).bfloat16()
    got_b = M.moe_token_unpermute_bf16(pb.view(torch.int16).numpy().view(np.uint16), si, rb.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(got_b, ref_b.view(torch.int16).numpy().view(np.uint16))


def test_c_abi_exports_the_moe_entry_points_and_rejects_bad_shapes():
    lib = cabi.load()
    for name in ("msco_moe_init_routing_v2_workspace_bytes", "msco_moe_init_routing_v2", "msco_moe_token_unpermute"):
        assert hasattr(lib, name)
    assert cabi.moe_init_routing_v2_workspace_bytes(4096, 2, 8) == (8 + 1) * 8 * 4    # (blocks of 1024 entries + 1) x experts ints
    # argument checks happen before anything touches a device
    with pytest.raises(cabi.BackendError):
        cabi.moe_token_unpermute(1, 1, 1, 1, 4, 8, 1001, cabi.DT_F16)        # hidden not a multiple of 8
    with pytest.raises(cabi.BackendError):
        cabi.moe_init_routing_v2(1, 1, 1, 1, 1, None, 1, 1 << 20, 4, 1024, 2, 2000, 2, 1)   # more than 1024 experts


# ----------------------------------------------------------------------------------- GPU parity
def _route_gpu(x, idx, e, flag):
    n_rows, h = x.shape
    k = idx.shape[1]
    dev = "cuda:0"
    view = {1: np.int8, 2: np.int16, 4: np.int32}[x.dtype.itemsize]
    tx = torch.from_numpy(np.ascontiguousarray(x).view(view)).to(dev)
    ti = torch.from_numpy(idx).to(dev)
    ex = torch.full((n_rows * k, h), 77, dtype=tx.dtype, device=dev)
    ridx = torch.full((n_rows * k,), -5, dtype=torch.int32, device=dev)
    tok = torch.full((e,), -5, dtype=torch.int32, device=dev)
    cap = torch.full((e,), -5, dtype=torch.int32, device=dev)
    wsb = cabi.moe_init_routing_v2_workspace_bytes(n_rows, k, e)
    ws = torch.empty(max(wsb, 1), dtype=torch.uint8, device=dev)
    for _ in range(2):   # twice: nothing may depend on what the previous call left in the workspace
        cabi.moe_init_routing_v2(tx.data_ptr(), ti.data_ptr(), ex.data_ptr(), ridx.data_ptr(), tok.data_ptr(), cap.data_ptr(),
                                 ws.data_ptr(), wsb, n_rows, h, k, e, x.dtype.itemsize, flag, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return ex.cpu().numpy().view(x.dtype), ridx.cpu().numpy(), tok.cpu().numpy(), cap.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("n_rows,h,k,e,flag", [(1, 1024, 1, 1, 1), (10, 2048, 8, 8, 1), (1001, 1024, 2, 8, 2),
                                              (513, 1024, 6, 64, 1), (300, 7168, 4, 256, 1),
                                              (40, 256, 8, 1024, 1),       # the most experts (one copy of the count tables)
                                              (2048, 64, 8, 8, 1),         # 16384 entries: the largest single-launch problem
                                              (3000, 256, 6, 64, 2),       # 18000 entries: histogram, scan, ranking and row launches
                                              (17000, 32, 1, 128, 1),      # 17 blocks of 1024 entries
                                              (8192, 64, 6, 64, 1),        # 48 blocks in 16 runs of 3 per expert
                                              (25000, 16, 2, 1024, 1),     # the most experts: one run of 49 blocks per expert
                                              (20000, 16, 3, 3, 2),        # 341 runs for 59 blocks: most runs are empty
                                              (70000, 8, 1, 1, 1),         # one expert
                                              (9000, 2064, 2, 7, 1)])      # rows of more than one pass (8 KiB) of the row movement
def test_init_routing_matches_the_golden(n_rows, h, k, e, flag):
    np.random.seed(0)                                                             # the reference test's stream (:102-104)
    x = np.random.uniform(-1, 1, size=(n_rows, h)).astype(np.float16)
    idx = np.random.randint(0, e, size=(n_rows, k)).astype(np.int32)
    ex, ridx, tok, cap = _route_gpu(x, idx, e, flag)
    ref_x, ref_idx, ref_tok = M.moe_init_routing_v2(x, idx, e, flag)
    assert np.array_equal(ridx, ref_idx)
    assert np.array_equal(tok, ref_tok)
    assert np.array_equal(ex.view(np.uint16), ref_x.view(np.uint16))
    assert np.all(cap == 0)


@pytest.mark.gpu
def test_init_routing_skewed_experts_int8_rows_and_mixtral_shape():
    # Zipf-skewed expert popularity with empty experts, int8 activations (the quantised input of the grouped matmul)
    rng = np.random.default_rng(5)
    e, k, n_rows, h = 64, 6, 2048, 2048
    pop = 1.0 / np.arange(1, e + 1) ** 1.2
    idx = np.stack([rng.choice(e, size=k, replace=False, p=pop / pop.sum()) for _ in range(n_rows)]).astype(np.int32)
    idx[idx == 63] = 0                                                            # expert 63 stays empty
    x = rng.integers(-127, 128, (n_rows, h), dtype=np.int8)
    ex, ridx, tok, _ = _route_gpu(x, idx, e, 1)
    ref_x, ref_idx, ref_tok = M.moe_init_routing_v2(x, idx, e, 1)
    assert np.array_equal(ridx, ref_idx) and np.array_equal(tok, ref_tok) and np.array_equal(ex, ref_x)
    assert tok[-1] == tok[-2] == n_rows * k
    # the routing of the headline matmul workload: 4096 tokens, top-2 of 8 experts
    idx = np.argsort(-rng.standard_normal((4096, 8)), axis=1)[:, :2].astype(np.int32)
    x = rng.integers(-127, 128, (4096, 4096), dtype=np.int8)
    ex, ridx, tok, _ = _route_gpu(x, idx, 8, 1)
    ref_x, ref_idx, ref_tok = M.moe_init_routing_v2(x, idx, 8, 1)
    assert np.array_equal(ridx, ref_idx) and np.array_equal(tok, ref_tok) and np.array_equal(ex, ref_x)


def _unpermute_gpu(pt_bits, si, pr_bits, dtype):
    dev = "cuda:0"
    t, k = pr_bits.shape
    h = pt_bits.shape[1]
    tp = torch.from_numpy(pt_bits.view(np.int16)).to(dev)
    ts = torch.from_numpy(si).to(dev)
    tr = torch.from_numpy(pr_bits.view(np.int16)).to(dev)
    out = torch.full((t, h), 0x7FC0, dtype=torch.int16, device=dev)
    cabi.moe_token_unpermute(tp.data_ptr(), ts.data_ptr(), tr.data_ptr(), out.data_ptr(), t, k, h, dtype,
                             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("token_num", [1, 16, 1001])
@pytest.mark.parametrize("hidden", [7168, 2048])
@pytest.mark.parametrize("top_k", [8, 2])
def test_token_unpermute_matches_the_golden(token_num, hidden, top_k):
    np.random.seed(token_num + hidden)
    pt = np.random.randn(token_num * top_k, hidden).astype(np.float16)            # inputs as the reference test draws them (:66-70)
    si = np.arange(token_num * top_k, dtype=np.int32)
    np.random.shuffle(si)
    pr = np.random.randn(token_num, top_k).astype(np.float16)
    got = _unpermute_gpu(pt.view(np.uint16), si, pr.view(np.uint16), cabi.DT_F16)
    ref = M.moe_token_unpermute(pt, si, pr)
    assert np.allclose(got.view(np.float16), ref, rtol=1e-3, atol=1e-3)           # the reference's tolerance
    assert np.array_equal(got, ref.view(np.uint16))                               # and bit-exact


@pytest.mark.gpu
@pytest.mark.parametrize("token_num,hidden,top_k,bf16", [(1030, 7168, 8, False), (1500, 10240, 4, True), (1024, 2048, 2, False),
                                                        (1100, 1032, 3, True), (1200, 40960, 1, False)])
def test_token_unpermute_with_many_tokens(token_num, hidden, top_k, bf16):
    # 1024 tokens and more: a workgroup takes four 2048-element pieces of the row together (3.5 pieces at 7168, a second
    # workgroup with one piece at 10240, a run-time top_k, a row longer than the 16 workgroups of a token cover in one pass)
    rng = np.random.default_rng(token_num)
    si = rng.permutation(token_num * top_k).astype(np.int32)
    if bf16:
        pt = (rng.standard_normal((token_num * top_k, hidden)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        pr = (rng.standard_normal((token_num, top_k)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        assert np.array_equal(_unpermute_gpu(pt, si, pr, cabi.DT_BF16), M.moe_token_unpermute_bf16(pt, si, pr))
    else:
        pt = rng.standard_normal((token_num * top_k, hidden)).astype(np.float16)
        pr = rng.standard_normal((token_num, top_k)).astype(np.float16)
        got = _unpermute_gpu(pt.view(np.uint16), si, pr.view(np.uint16), cabi.DT_F16)
        assert np.array_equal(got, M.moe_token_unpermute(pt, si, pr).view(np.uint16))


@pytest.mark.gpu
def test_token_unpermute_bf16_and_round_trip_with_routing():
    rng = np.random.default_rng(11)
    t, k, h = 257, 4, 1024
    pt = (rng.standard_normal((t * k, h)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    pr = (rng.standard_normal((t, k)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    si = rng.permutation(t * k).astype(np.int32)
    got = _unpermute_gpu(pt, si, pr, cabi.DT_BF16)
    assert np.array_equal(got, M.moe_token_unpermute_bf16(pt, si, pr))
    # routing followed by un-permutation with weights 1, 0, 0, 0 returns every token's own row
    x = rng.standard_normal((t, h)).astype(np.float16)
    idx = rng.integers(0, 8, (t, k)).astype(np.int32)
    ex, ridx, _, _ = _route_gpu(x, idx, 8, 1)
    probs = np.zeros((t, k), np.float16)
    probs[:, 0] = 1
    back = _unpermute_gpu(ex.view(np.uint16), ridx, probs.view(np.uint16), cabi.DT_F16)
    assert np.array_equal(back, x.view(np.uint16))


def _route_quant_gpu(x_bits, bf16, idx, e, flag):
    n_rows, h = x_bits.shape
    k = idx.shape[1]
    dev = "cuda:0"
    tx = torch.from_numpy(x_bits.view(np.int16)).to(dev)
    ti = torch.from_numpy(idx).to(dev)
    ex = torch.full((n_rows * k, h), 77, dtype=torch.int8, device=dev)
    sc = torch.full((n_rows * k,), -1.0, dtype=torch.float32, device=dev)
    ridx = torch.full((n_rows * k,), -5, dtype=torch.int32, device=dev)
    tok = torch.full((e,), -5, dtype=torch.int32, device=dev)
    wsb = cabi.moe_init_routing_v2_workspace_bytes(n_rows, k, e)
    ws = torch.empty(max(wsb, 1), dtype=torch.uint8, device=dev)
    for _ in range(2):
        cabi.moe_init_routing_v2_quant(tx.data_ptr(), ti.data_ptr(), ex.data_ptr(), sc.data_ptr(), ridx.data_ptr(), tok.data_ptr(),
                                       None, ws.data_ptr(), wsb, n_rows, h, k, e, cabi.DT_BF16 if bf16 else cabi.DT_F16, flag,
                                       torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return ex.cpu().numpy(), sc.cpu().numpy(), ridx.cpu().numpy(), tok.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("n_rows,h,k,e,bf16", [(1, 8, 1, 1, False), (37, 1024, 2, 8, False), (300, 4096, 2, 8, True),
                                              (64, 7168, 6, 64, False), (20, 10240, 3, 4, True), (9, 8200, 2, 3, False),
                                              (2100, 512, 8, 8, True),     # 16800 entries: the separate launches
                                              (2100, 8200, 8, 8, False),   # ... with rows longer than a lane keeps in registers
                                              (16500, 64, 1, 8, True), (33, 4104, 1, 5, False)])   # one entry per token
def test_routing_with_dynamic_quantisation_is_bit_exact(n_rows, h, k, e, bf16):
    # the routing golden followed by the activation quantisation of the reference's int8-activation test
    # (tests/st/test_grouped_matmul_w4.py:83-89,99), row by row; int8 rows and float32 scales bit for bit
    rng = np.random.default_rng(n_rows + h)
    x32 = rng.uniform(-0.3, 0.3, (n_rows, h)).astype(np.float32)
    x32[::7] *= 37.0
    if n_rows > 5:
        x32[3] = 0.0                                                               # a row of zeros
        x32[4, 1:] = 0.0                                                           # a single non-zero element
        x32[5] = np.where(np.arange(h) % 3 == 0, 2.0, np.where(np.arange(h) % 3 == 1, -1.0, 0.0078125))   # 63.5: exact ties
    if bf16:
        bits = (x32.view(np.uint32) >> 16).astype(np.uint16)
        vals = M.bf16_bits_to_f32(bits)
    else:
        vals = x32.astype(np.float16)
        bits = vals.view(np.uint16)
    idx = rng.integers(0, e, (n_rows, k)).astype(np.int32)
    ex, sc, ridx, tok = _route_quant_gpu(np.ascontiguousarray(bits), bf16, idx, e, 1)
    ref_rows, ref_idx, ref_tok = M.moe_init_routing_v2(vals, idx, e, 1)
    ref_q, ref_s = M.dyn_quant(ref_rows)
    assert np.array_equal(ridx, ref_idx) and np.array_equal(tok, ref_tok)
    assert np.array_equal(sc.view(np.uint32), ref_s.view(np.uint32))
    assert np.array_equal(ex, ref_q)


@pytest.mark.gpu
def test_routing_with_dynamic_quantisation_rejects_what_it_cannot_take():
    with pytest.raises(RuntimeError):                                               # float32 activations
        cabi.moe_init_routing_v2_quant(1, 1, 1, 1, 1, None, None, 1, 0, 4, 64, 2, 8, cabi.DT_F32, 1)
    with pytest.raises(RuntimeError):                                               # hidden not a multiple of 8
        cabi.moe_init_routing_v2_quant(1, 1, 1, 1, 1, None, None, 1, 0, 4, 60, 2, 8, cabi.DT_F16, 1)
