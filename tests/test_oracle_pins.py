"""Pins for the CPU oracle: every function is checked against something other than itself --
brute force, closed forms, an independent C implementation, torch's casts, the reference's
constant-scale known answers -- chosen so that a dropped term, a wrong index or a transposed operand
fails at least one test."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import gmm_oracle as O


# ---------------------------------------------------------------- bf16 / f16 casts
def test_bf16_rne_hand_computed_ties():
    cases = {
        0x3F800000: 0x3F80,  # 1.0
        0x3F808000: 0x3F80,  # 1 + 2^-8: tie, even mantissa stays
        0x3F818000: 0x3F82,  # 1 + 3*2^-8: tie, odd mantissa rounds up
        0x3F808001: 0x3F81,  # just above the tie
        0x3F807FFF: 0x3F80,  # just below the tie
        0xBF818000: 0xBF82,  # sign does not matter
        0x7F7FFFFF: 0x7F80,  # largest float rounds to +inf
        0x00000000: 0x0000,
        0x80000000: 0x8000,
        0x7F800000: 0x7F80,  # inf
        0x00008000: 0x0000,  # subnormal tie to even
        0x00018000: 0x0002,
    }
    bits = np.array(list(cases.keys()), dtype=np.uint32)
    got = O.f32_to_bf16_bits(bits.view(np.float32))
    assert got.tolist() == list(cases.values())
    for b, want in cases.items():
        assert c_oracle.f32_to_bf16(float(np.array([b], dtype=np.uint32).view(np.float32)[0])) == want


def test_bf16_rne_matches_torch_cast():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000),
        rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, 3.4e38], dtype=np.float32),
    ]).astype(np.float32)
    vals = vals[~np.isnan(vals)]
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(vals), want)
    assert np.isnan(O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.array([np.nan], dtype=np.float32))))[0]


def test_bf16_roundtrip_is_identity_on_bf16_values():
    bits = np.arange(0, 0x7F80, dtype=np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(O.bf16_bits_to_f32(bits)), bits)


def test_f16_cast_matches_torch():
    rng = np.random.default_rng(1)
    v = (rng.standard_normal(100000) * 100).astype(np.float32)
    assert np.array_equal(O.f32_to_f16(v).view(np.uint16),
                          torch.from_numpy(v).to(torch.float16).view(torch.int16).numpy().view(np.uint16))


# ---------------------------------------------------------------- exact accumulators
@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (3, 5, 2), (4, 33, 7), (2, 64, 3)])
def test_exact_matmul_equals_bruteforce(m, k, n):
    rng = np.random.default_rng(m * 100 + k)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    assert np.array_equal(O.int32_matmul_exact(a, b), O.int32_matmul_bruteforce(a, b))


def test_exact_matmul_closed_forms():
    k = 4096
    ones = np.ones((3, k), dtype=np.int8)
    w = np.ones((k, 5), dtype=np.int8)
    assert (O.int32_matmul_exact(ones, w) == k).all()
    # saturated inputs: the largest magnitude a K=4096 int8 dot product can reach
    a = np.full((2, k), -127, dtype=np.int8)
    b = np.full((k, 2), 127, dtype=np.int8)
    assert (O.int32_matmul_exact(a, b) == -127 * 127 * k).all()
    # identity weights return x itself; a shifted identity catches transposed operands
    x = np.random.default_rng(2).integers(-127, 128, (7, 64), dtype=np.int8)
    eye = np.eye(64, dtype=np.int8)
    assert np.array_equal(O.int32_matmul_exact(x, eye), x.astype(np.int32))
    shift = np.roll(eye, 1, axis=1)  # shift[k, (k+1) % 64] = 1
    assert np.array_equal(O.int32_matmul_exact(x, shift), np.roll(x.astype(np.int32), 1, axis=1))


def test_exact_matmul_vs_int64_and_float64_and_chunking():
    rng = np.random.default_rng(3)
    a = rng.integers(-127, 128, (37, 5000), dtype=np.int8)   # K > chunk, not a multiple of it
    b = rng.integers(-127, 128, (5000, 29), dtype=np.int8)
    want = a.astype(np.int64) @ b.astype(np.int64)
    got = O.int32_matmul_exact(a, b)
    assert np.array_equal(got, want.astype(np.int32))
    assert np.array_equal(got, (a.astype(np.float64) @ b.astype(np.float64)).astype(np.int64).astype(np.int32))


def test_single_sgemm_golden_is_inexact_on_adversarial_data_but_exact_path_is_not():
    # all-max inputs push partial sums past 2**24, where one float32 dot loses integers; the chunked path must not
    k = 4096
    a = np.full((1, k), 127, dtype=np.int8)
    b = np.full((k, 1), 127, dtype=np.int8)
    b[-1, 0] = 126
    exact = O.int32_matmul_exact(a, b)[0, 0]
    assert exact == 127 * 127 * (k - 1) + 127 * 126


# ---------------------------------------------------------------- grouping
def test_group_bounds_cumulative_counts_and_empty_groups():
    s, e = O.group_bounds([0, 3, 3, 10], 0)
    assert s.tolist() == [0, 0, 3, 3] and e.tolist() == [0, 3, 3, 10]
    s2, e2 = O.group_bounds([0, 3, 0, 7], 1)
    assert s2.tolist() == s.tolist() and e2.tolist() == e.tolist()
    with pytest.raises(ValueError):
        O.group_bounds([5, 3], 0)


def _toy(rng, m=23, k=64, n=48, e=4):
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    return x, w


def test_grouped_acc_rows_use_only_their_groups_weights():
    rng = np.random.default_rng(4)
    x, w = _toy(rng)
    gl = [5, 5, 16, 23]  # group 1 empty
    acc = O.grouped_int32_acc(x, w, gl)
    for g, (s, t) in enumerate([(0, 5), (5, 5), (5, 16), (16, 23)]):
        assert np.array_equal(acc[s:t], O.int32_matmul_bruteforce(x[s:t], w[g]))
    # changing another group's weights leaves this group's rows alone
    w2 = w.copy()
    w2[0] = 0
    w2[1] = 7
    acc2 = O.grouped_int32_acc(x, w2, gl)
    assert np.array_equal(acc2[5:], acc[5:]) and (acc2[:5] == 0).all()
    # permuting rows inside a group permutes its outputs
    perm = np.arange(23)
    perm[5:16] = perm[5:16][::-1]
    assert np.array_equal(O.grouped_int32_acc(x[perm], w, gl), acc[perm])
    # E = 1 is the dense product; counts == cumulative; transposed storage == plain storage
    assert np.array_equal(O.grouped_int32_acc(x, w[:1], [23]), O.int32_matmul_exact(x, w[0]))
    assert np.array_equal(O.grouped_int32_acc(x, w, [5, 0, 11, 7], 1), acc)
    assert np.array_equal(O.grouped_int32_acc(x, np.ascontiguousarray(w.transpose(0, 2, 1)), gl, transpose_b=True), acc)
    # rows past the last boundary stay zero
    short = O.grouped_int32_acc(x, w, [5, 5, 16, 20])
    assert (short[20:] == 0).all() and np.array_equal(short[:20], acc[:20])


def test_numpy_and_c_oracles_agree_bit_for_bit():
    rng = np.random.default_rng(5)
    m, k, n, e = 150, 1088, 80, 8
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    gl = O.random_group_list(m, e, rng)
    bits, acc = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, return_acc=True)
    acc_b = O.grouped_matmul_w8a8(x, w, gl, bias, None, None, out_dtype="i32")
    c_acc, c_bits = c_oracle.gmm_w8a8(x, w, gl, bias, scale, pt)
    assert np.array_equal(c_acc, acc_b)
    assert np.array_equal(c_bits, bits)
    # transposed weights and counts in the C oracle too
    counts = np.diff(np.concatenate([[0], gl]))
    c_acc2, c_bits2 = c_oracle.gmm_w8a8(x, np.ascontiguousarray(w.transpose(0, 2, 1)), counts, bias, scale, pt,
                                        group_list_type=1, transpose_b=True)
    assert np.array_equal(c_acc2, acc_b) and np.array_equal(c_bits2, bits)


# ---------------------------------------------------------------- epilogue
def test_epilogue_reference_known_answers():
    rng = np.random.default_rng(6)
    x = rng.integers(-128, 128, (32, 256)).astype(np.int8)
    w = rng.integers(-128, 128, (8, 256, 128)).astype(np.int8)
    counts = np.array([1, 2, 7, 4, 4, 4, 2, 8])
    acc = O.grouped_int32_acc(x, w, counts, 1)
    # scale = 10, per-token = 10 -> 100 * acc (test_grouped_matmul_v4_cops.py:294-301)
    out = O.grouped_matmul_w8a8(x, w, counts, None, np.full((8, 128), 10, np.float32), np.full(32, 10, np.float32),
                                group_list_type=1, out_dtype="f32")
    assert np.array_equal(out, acc.astype(np.float32) * 100)
    # scale = 10, bias = 1 -> 10 * (acc + 1) (test_grouped_matmul_v4_cops.py:351-359)
    out = O.grouped_matmul_w8a8(x, w, counts, np.ones((8, 128), np.int32), np.full((8, 128), 10, np.float32), None,
                                group_list_type=1, out_dtype="f32")
    assert np.array_equal(out, (acc + 1).astype(np.float32) * 10)
    # scale = 1 and int32 output -> acc exactly (test_quant_batch_matmul.py:76-80)
    assert np.array_equal(O.quant_batch_matmul_oracle(x, w[0], np.ones(1, np.float32), out_dtype="i32"),
                          x.astype(np.int32) @ w[0].astype(np.int32))


def test_epilogue_operation_order_is_two_separate_float32_products():
    # values where (f*s)*p and f*(s*p) round differently in float32: the oracle must do the former
    acc = np.array([[16777217 // 3]], dtype=np.int32)
    s = np.array([0.1], dtype=np.float32)
    p = np.array([0.3], dtype=np.float32)
    want = np.float32(np.float32(np.float32(acc[0, 0]) * s[0]) * p[0])
    got = O.dequant_epilogue(acc, None, s, p, "f32")[0, 0]
    assert got == want
    # bias is added in int32 before the conversion to float
    big = np.array([[2 ** 24]], dtype=np.int32)
    assert O.dequant_epilogue(big, np.array([1], np.int32), None, None, "f32")[0, 0] == np.float32(2 ** 24 + 1)
    assert O.dequant_epilogue(big, np.array([1], np.int32), None, None, "i32")[0, 0] == 2 ** 24 + 1


def test_exact_path_agrees_with_literal_reference_goldens_under_their_tolerances():
    rng = np.random.default_rng(7)
    m, k, n, e = 64, 64, 128, 8
    x = rng.uniform(-20, 20, (m, k)).astype(np.int8)
    w = rng.uniform(-20, 20, (e, k, n)).astype(np.int8)
    bias = rng.integers(-10, 10, (e, n)).astype(np.int32)
    scale = (rng.random((e, n)) / 1000).astype(np.float32)
    pt = rng.random(m).astype(np.float32)
    gl = O.random_group_list(m, e, rng)
    gold = O.golden_grouped_w8a8(x, w, gl, bias, scale, pt, out="f16")
    mine = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, out_dtype="f16")
    assert np.array_equal(gold.view(np.uint16), mine.view(np.uint16))  # small sums: the golden's sgemm is exact
    assert O.count_compare(mine.astype(np.float32), gold.astype(np.float32), 0.004)
    # V4 float goldens (inexact by construction) at their rtol
    counts = np.array([1, 2, 7, 4, 4, 4, 2, 8]) * 2
    s10 = np.full((e, n), 10, np.float32)
    g1 = O.golden_v4_pertoken(x, w, s10, np.full(m, 10, np.float32), counts)
    o1 = O.grouped_matmul_w8a8(x, w, counts, None, s10, np.full(m, 10, np.float32), group_list_type=1, out_dtype="f32")
    np.testing.assert_allclose(g1, o1, rtol=4e-3)
    g2 = O.golden_v4_perchannel_bias(x, w, s10, np.ones((e, n), np.float32), counts)
    o2 = O.grouped_matmul_w8a8(x, w, counts, np.ones((e, n), np.int32), s10, None, group_list_type=1, out_dtype="f32")
    np.testing.assert_allclose(g2, o2, rtol=4e-3)


# ---------------------------------------------------------------- dense path
def test_quant_batch_matmul_oracle_batches_and_transposes():
    rng = np.random.default_rng(8)
    x1 = rng.integers(-5, 5, (8, 64, 32)).astype(np.int8)   # [batch, K, M]
    x2 = rng.integers(-5, 5, (8, 48, 64)).astype(np.int8)   # [batch, N, K]
    s = rng.standard_normal(1).astype(np.float32)
    want = np.matmul(x1.astype(np.int32).transpose(0, 2, 1), x2.astype(np.int32).transpose(0, 2, 1)) * s
    got = O.quant_batch_matmul_oracle(x1, x2, s, transpose_x1=True, transpose_x2=True, out_dtype="f32")
    np.testing.assert_allclose(got, want, rtol=1e-6)
    # broadcasting: 2-D x2 against batched x1
    y = O.quant_batch_matmul_oracle(x1.transpose(0, 2, 1), x2[0].T, np.ones(48, np.float32), out_dtype="i32")
    assert np.array_equal(y, np.matmul(x1.astype(np.int32).transpose(0, 2, 1), x2[0].astype(np.int32).T))


# ---------------------------------------------------------------- scale wire formats
def test_scale_wire_formats_round_trip():
    s = np.random.default_rng(9).uniform(1e-3, 1e-2, (4, 16)).astype(np.float32)
    enc = O.encode_scale_int64(s)
    assert enc.dtype == np.int64 and (enc >= 0).all() and (enc < 2 ** 32).all()
    assert np.array_equal(O.decode_scale_int64(enc), s)
    enc2 = O.encode_scale_int64_qbmm(s)
    assert ((enc2 >> 46) & 1 == 1).all()
    dec2 = O.decode_scale_int64(enc2)
    assert np.array_equal(dec2.view(np.uint32), s.view(np.uint32) & np.uint32(0xFFFFE000))
    np.testing.assert_allclose(dec2, s, rtol=2 ** -10)


# ---------------------------------------------------------------- weight-only
def test_a16w8_closed_forms_and_c_cross_check():
    rng = np.random.default_rng(10)
    m, k, n, e = 30, 256, 128, 8
    ends = [1, 3, 10, 14, 18, 22, 24, 30]
    x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32)))
    w = rng.integers(-128, 128, (e, k, n)).astype(np.int8)
    # constant scale 0.01 and offset 1 (test_grouped_matmul_v4_cops.py:156-157): out = 0.01 * x @ (w + 1)
    s = np.full((e, n), O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.float32(0.01))), np.float32)
    o = np.ones((e, n), np.float32)
    got = O.a16w8_grouped_f64(x, w, s, o, ends)
    starts = [0] + ends[:-1]
    for g, (a, b) in enumerate(zip(starts, ends)):
        want = (x[a:b].astype(np.float64) @ (w[g].astype(np.float64) + 1.0)) * np.float64(s[0, 0])
        np.testing.assert_allclose(got[a:b], want, rtol=1e-12, atol=1e-12)
    # zero weights: out = s * o * rowsum(x)
    z = O.a16w8_grouped_f64(x, np.zeros_like(w), s, 3 * o, ends)
    np.testing.assert_allclose(z[:30], (3.0 * x.astype(np.float64).sum(1) * np.float64(s[0, 0]))[:30, None] *
                               np.ones((1, n)), rtol=1e-12)
    # independent C implementation
    c = c_oracle.gmm_a16w8_f64(O.f32_to_bf16_bits(x), w, O.f32_to_bf16_bits(s), O.f32_to_bf16_bits(o), ends)
    np.testing.assert_allclose(c, got, rtol=1e-11, atol=1e-9)
    # the reference's own float golden agrees at its rtol on well-conditioned rows
    gold = O.golden_v4_a16w8(x.astype(np.float32), w, s, o, ends)
    big = np.abs(got[:30]) > 1.0
    np.testing.assert_allclose(gold[big], got[:30][big], rtol=1e-3)


def test_pack_weights_follows_the_layout_definition_byte_by_byte():
    """The packed weight layout is this backend's own (the reference's blocked format comes out of its closed trans_data
    kernel): the vectorised restatement is checked against a per-byte loop over the definition, padding included."""
    rng = np.random.default_rng(3)
    for e, k, n in [(1, 64, 16), (2, 70, 20), (1, 200, 33)]:
        w = rng.integers(-128, 128, (e, k, n), dtype=np.int8)
        packed = O.pack_weights(w)
        kb, ng = (k + 63) // 64, (n + 15) // 16
        assert packed.shape == (e, ng * kb * 1024)
        for g in range(e):
            for a in range(ng):
                for b in range(kb):
                    blk = packed[g, (a * kb + b) * 1024:(a * kb + b + 1) * 1024]
                    for l in range(64):
                        for i in range(16):
                            kk, nn = 64 * b + 16 * (l // 16) + i, 16 * a + (l % 16)
                            want = w[g, kk, nn] if (kk < k and nn < n) else 0
                            assert blk[16 * l + i] == want


# ------------------------------------------------------------------------------------------ A8W4
def test_int4_packing_by_hand_loops_and_round_trip():
    # -8 -> 0x8, -1 -> 0xF, 7 -> 0x7; even index in the low nibble (test_grouped_matmul_w4.py:115-118)
    assert O.pack_int4(np.array([-8, 7, -1, 0, 3, -4], dtype=np.int8)).tolist() == [0x78, 0x0F, 0xC3]
    rng = np.random.default_rng(0)
    w = rng.integers(-8, 8, (3, 5, 16)).astype(np.int8)
    p = O.pack_int4(w)
    assert p.shape == (3, 5, 8) and p.dtype == np.uint8
    for idx in np.ndindex(3, 5, 8):
        lo, hi = int(w[idx[0], idx[1], 2 * idx[2]]), int(w[idx[0], idx[1], 2 * idx[2] + 1])
        assert int(p[idx]) == ((hi & 0xF) << 4 | (lo & 0xF))
    assert np.array_equal(O.unpack_int4(p), w)


def test_a8w4_golden_against_integer_form_bruteforce_and_closed_forms():
    rng = np.random.default_rng(1)
    m, k, n, e, g = 9, 128, 16, 4, 32
    x = rng.integers(-127, 128, (m, k)).astype(np.int8)
    wq, ws = O.quant_int4_groups(rng.uniform(-0.3, 0.3, (e, k, n)).astype(np.float16), g)
    assert np.abs(wq).max() == 7 and ws.shape == (e, k // g, 1, n)
    wp = O.pack_int4(wq.transpose(0, 2, 1))                                   # [e, n, k/2], as the op takes it
    xs = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    gl = [2, 2, 7, 9]                                                         # one empty group
    gold = O.golden_grouped_a8w4(x, wp, gl, xs, ws, g)
    exact = O.grouped_a8w4_f64(x, wp, gl, xs, ws, g)
    assert np.allclose(gold, exact, rtol=2e-5, atol=1e-7)
    # brute force, one output at a time
    grp_of = [0, 0, 2, 2, 2, 2, 2, 3, 3]
    for (r, c) in [(0, 0), (3, 5), (8, 15)]:
        acc = 0.0
        for kk in range(k):
            acc += float(x[r, kk]) * float(wq[grp_of[r], kk, c]) * float(ws[grp_of[r], kk // g, 0, c])
        assert abs(acc * float(xs[r]) - exact[r, c]) <= 1e-9 * max(1.0, abs(exact[r, c]))
    # constant scales: plain integer matmul times the constants; ones: column sums
    ones = np.ones_like(ws)
    got = O.golden_grouped_a8w4(x, wp, gl, np.full(m, 2.0, np.float32), ones * 0.5, g)
    ref = np.concatenate([x[0:2].astype(np.int64) @ wq[0].astype(np.int64), x[2:7].astype(np.int64) @ wq[2].astype(np.int64),
                          x[7:9].astype(np.int64) @ wq[3].astype(np.int64)])
    assert np.array_equal(got, ref.astype(np.float32))


# ---------------------------------------------------------------- fused activation (no golden in the reference)
def test_activation_against_torch_other_formulations_and_identities():
    rng = np.random.default_rng(5)
    v = np.concatenate([rng.uniform(-60, 60, 4000), rng.uniform(-3, 3, 4000), [0.0, -0.0, 40.0, -40.0, 1e-6, -1e-6]]).astype(np.float32)
    t = torch.from_numpy(v).double()
    close = lambda a, b: np.allclose(a, b, rtol=1e-12, atol=1e-300)
    # library routines in float64
    assert np.array_equal(O.activation(v, O.ACT_NONE), v.astype(np.float64))
    assert np.array_equal(O.activation(v, O.ACT_RELU), torch.relu(t).numpy())
    assert close(O.activation(v, O.ACT_SILU), torch.nn.functional.silu(t).numpy())
    # (torch's tanh form cancels for very negative arguments where the sigmoid form does not: compare where it is accurate)
    mid = np.abs(v) < 4
    assert np.allclose(O.activation(v, O.ACT_GELU_TANH)[mid], torch.nn.functional.gelu(t, approximate="tanh").numpy()[mid], rtol=1e-9, atol=0)
    # the textbook tanh form against the sigmoid form used by the oracle
    x = v.astype(np.float64)
    tanh_form = 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))
    assert np.allclose(O.activation(v, O.ACT_GELU_TANH)[mid], tanh_form[mid], rtol=1e-9, atol=0)
    # CANN's published fast-gelu expression x / (1 + exp(-1.702 |x|)) * exp(0.851 (x - |x|)) is x * sigmoid(1.702 x)
    cann = x / (1.0 + np.exp(-1.702 * np.abs(x))) * np.exp(0.851 * (x - np.abs(x)))
    assert close(O.activation(v, O.ACT_FAST_GELU), cann)
    # identities and limits: x * sigmoid(t(x)) with an odd t gives f(x) - f(-x) = x; f(40) = 40 and f(-40) = -0 to double precision
    for act in (O.ACT_SILU, O.ACT_FAST_GELU, O.ACT_GELU_TANH):
        f = lambda a: O.activation(np.asarray(a, dtype=np.float32), act)
        assert np.allclose(f(v) - f(-v), x, rtol=1e-12, atol=1e-12)
        assert abs(f([40.0])[0] - 40.0) < 1e-12 and abs(f([-40.0])[0]) < 1e-12
        assert f([0.0])[0] == 0.0
    with pytest.raises(ValueError):
        O.activation(v, O.ACT_GELU_ERF)


# ---------------------------------------------------------------- the two helpers that only had shape checks
def test_quant_int4_groups_element_by_element_and_by_what_the_formula_fixes():
    """quant (tests/st/test_grouped_matmul_w4.py:91-97): per (expert, K group, column) scale = max|y| / 7 in float32 and
    q = round(y / scale) -- restated with scalar loops in exact rational arithmetic, plus the properties the formula
    fixes: the group's largest magnitude maps to +-7 with its sign, 7 * scale returns it, |y - q * scale| <= scale / 2."""
    from fractions import Fraction
    rng = np.random.default_rng(8)
    e, k, n, g = 2, 64, 5, 32
    y = rng.uniform(-0.3, 0.3, (e, k, n)).astype(np.float16)
    q, s = O.quant_int4_groups(y, g)
    assert q.shape == (e, k, n) and s.shape == (e, k // g, 1, n) and s.dtype == np.float32 and q.dtype == np.int8
    for ee in range(e):
        for kg in range(k // g):
            for c in range(n):
                col = [Fraction(float(v)) for v in y[ee, kg * g:(kg + 1) * g, c]]
                big = max(abs(v) for v in col)
                scale = np.float32(float(big)) / np.float32(7.0)          # the golden divides float32 by float32
                assert s[ee, kg, 0, c] == scale
                for j, v in enumerate(col):
                    quot = np.float32(np.float32(float(v)) / scale)       # float32 quotient, as numpy computes it
                    want = int(np.round(quot))                            # half to even
                    assert q[ee, kg * g + j, c] == want
                    assert abs(float(v) - want * float(scale)) <= float(scale) / 2 * (1 + 1e-6)
                top = int(np.argmax([abs(v) for v in col]))
                assert abs(int(q[ee, kg * g + top, c])) == 7 and np.sign(q[ee, kg * g + top, c]) == np.sign(float(col[top]))
                assert abs(7 * float(scale) - float(big)) <= 1e-6 * float(big)


def test_count_compare_counts_like_the_reference_comparator():
    """custom_compare (tests/st/st_utils.py:23-49): at most int(size * limit) elements may have a relative error above
    limit -- on hand-built cases either side of the count and of the error threshold."""
    expect = np.ones(1000, dtype=np.float32)
    out = expect.copy()
    assert O.count_compare(out, expect, 0.004)
    out[:4] = 1.0 + 0.0041                       # 4 elements just above the limit: int(1000 * 0.004) = 4 are allowed
    assert O.count_compare(out, expect, 0.004)
    out[4] = 1.0 + 0.0041                        # the fifth is one too many
    assert not O.count_compare(out, expect, 0.004)
    out[:5] = 1.0 + 0.0039                       # below the error threshold nothing counts
    assert O.count_compare(out, expect, 0.004)
    out[:] = 2.0                                 # bfloat16's limit: 0.03 of the elements, 0.03 relative
    assert not O.count_compare(out, expect, 0.03)
    out[:] = 1.0
    out[:30] = 1.05
    assert O.count_compare(out, expect, 0.03)
    out[30] = 1.05
    assert not O.count_compare(out, expect, 0.03)
    # relative to the expected value, sign and scale free
    assert O.count_compare(np.array([-100.3]), np.array([-100.0]), 0.004)
    assert not O.count_compare(np.array([-100.5] * 1000), np.array([-100.0] * 1000), 0.004)


def test_v4_a8w4_golden_against_exact_integers_a_scalar_loop_and_the_wire_formats():
    """golden_v4_a8w4 / encode_scale_uint64 (tests/st/test_grouped_matmul_v4_cops.py:453-476) pinned by what the formula
    fixes: the integer sums in exact Python integers, each of the two products rounded to float32 once; constant scales
    give the plain integer matmul; the exact-path oracle of the W8A8 op on the same values agrees bit for bit; nibble
    pairs along n by hand."""
    rng = np.random.default_rng(5)
    e, m, k, n = 4, 11, 48, 16
    counts = np.array([3, 0, 6, 2], dtype=np.int64)
    x = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-8, 8, (e, k, n), dtype=np.int8)
    scale = rng.normal(0, 0.01, (e, 1, n)).astype(np.float32)
    pt = rng.normal(0, 0.01, (m, 1)).astype(np.float32)
    su = O.encode_scale_uint64(scale)
    assert su.dtype == np.uint64 and su.shape == (e, 1, n) and (su >> np.uint64(32) == 0).all()
    assert np.array_equal((su & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.float32), scale)
    got = O.golden_v4_a8w4(x, w, su, pt, counts)
    assert got.dtype == np.float32 and got.shape == (m, n)
    ends = np.cumsum(counts)
    for row in range(m):
        g = int(np.searchsorted(ends, row, side="right"))
        for col in range(n):
            acc = sum(int(x[row, kk]) * int(w[g, kk, col]) for kk in range(k))
            want = np.float32(np.float32(np.float32(acc) * scale[g, 0, col]) * pt[row, 0])
            assert got[row, col] == want, (row, col)
    # the exact-path oracle of the int8 op on the same 4-bit values: same bits
    ref = O.grouped_matmul_w8a8(x, w, ends, None, scale.reshape(e, n), pt.reshape(m), out_dtype="f32")
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    # scale 1 and per-token 1: the integer matmul itself
    ones = O.golden_v4_a8w4(x, w, O.encode_scale_uint64(np.ones((e, 1, n), np.float32)), np.ones((m, 1), np.float32), counts)
    for g, (a, b) in enumerate(zip(np.concatenate([[0], ends[:-1]]), ends)):
        assert np.array_equal(ones[a:b], (x[a:b].astype(np.int64) @ w[g].astype(np.int64)).astype(np.float32))
    # the packing of the test (:458-460): flattened, element 2 i in the low nibble, 2 i + 1 in the high one = pairs along n
    wn = np.array([[[1, -1, 7, -8]]], dtype=np.int8)
    flat = wn.reshape(-1) & 0x000F
    literal = (flat[0::2] | (flat[1::2] << 4)).reshape(1, 1, 2)
    assert np.array_equal(literal.astype(np.uint8), np.array([[[0xF1, 0x87]]], dtype=np.uint8))
    assert np.array_equal(O.pack_int4(wn), literal.astype(np.uint8)) and np.array_equal(O.unpack_int4(O.pack_int4(w)), w)


def test_v4_a16w4_golden_against_the_reference_packing_loop_float64_and_the_closed_form_of_its_data():
    """golden_v4_a16w4 (tests/st/test_grouped_matmul_v4_cops.py:197-262): the nibble packing the reference's test writes
    out as a loop (:229-233) is what pack_int4 produces; the expected value is the a16w8 formula on the unpacked values,
    checked in float64 and, on the test's own data (weights in {0, 1}, scale 0.01, offset 1), against a closed form."""
    rng = np.random.default_rng(21)
    e, k, n, m = 3, 8, 6, 7
    w = rng.integers(-8, 8, (e, k, n)).astype(np.int8)
    flat = w.reshape(-1)
    by_loop = np.zeros(flat.size // 2, dtype=np.int8)
    for i in range(flat.size // 2):   # the reference's loop, values masked to their nibbles
        by_loop[i] = np.int8(np.uint8((int(flat[2 * i]) & 15) | ((int(flat[2 * i + 1]) & 15) << 4)))
    packed = O.pack_int4(w)
    assert packed.shape == (e, k, n // 2) and np.array_equal(packed.reshape(-1).view(np.int8), by_loop)
    assert np.array_equal(O.unpack_int4(packed), w)
    # the formula in float64 on the unpacked values
    ends = np.array([2, 2, 6], dtype=np.int64)          # an empty group, one row behind the last boundary
    x = rng.uniform(-4, 4, (m, k)).astype(np.float16)
    s = rng.uniform(0.01, 0.02, (e, n)).astype(np.float16)
    o = rng.integers(-2, 3, (e, n)).astype(np.float16)
    got = O.golden_v4_a16w4(x, O.unpack_int4(packed), s, o, ends)
    assert got.shape == (6, n) and got.dtype == np.float16
    starts = [0, 2, 2]
    for g in range(e):
        a, b = starts[g], int(ends[g])
        want = x[a:b].astype(np.float64) @ ((w[g].astype(np.float64) + o[g].astype(np.float64)) * s[g].astype(np.float64))
        np.testing.assert_allclose(got[a:b].astype(np.float64), want, rtol=2e-3, atol=2e-3)
    # the test's data: weights 0 / 1, scale 0.01, offset 1  ->  0.01 * (rowsum(x) + x @ w), exactly in float64
    w01 = rng.integers(0, 2, (e, k, n)).astype(np.int8)
    s01, o01 = np.full((e, n), 0.01, np.float16), np.full((e, n), 1, np.float16)
    got01 = O.a16w8_grouped_f64(x.astype(np.float32), O.unpack_int4(O.pack_int4(w01)), s01.astype(np.float32),
                                o01.astype(np.float32), ends)
    for g in range(e):
        a, b = starts[g], int(ends[g])
        xs = x[a:b].astype(np.float64)
        want = np.float64(np.float16(0.01)) * (xs.sum(1, keepdims=True) + xs @ w01[g].astype(np.float64))
        np.testing.assert_allclose(got01[a:b], want, rtol=1e-12, atol=1e-12)
