"""Activation fused into the epilogue (act_type of grouped_matmul_v4_cops).

PARITY UNPINNED BY THE REFERENCE: it forwards act_type to aclnnGroupedMatmulV4 untouched
(ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:96,112,363), names no values and holds no golden
(grouped_matmul_v4_cops_doc.md:26).  The values are CANN's GMMActType (1 relu, 2 gelu_tanh, 4 fast_gelu, 5 silu);
the oracle's functions are pinned by torch's routines, alternative formulations and identities
(tests/test_oracle_pins.py).

Bar: relu bit-exact (it is a select on the float32 value); the smooth functions within one 16-bit output ulp of
the float64 evaluation on the exact float32 dequantised value: |err| <= 2^-7 |ref| (bf16), 2^-10 |ref| + 2^-24 (f16)."""
import numpy as np
import pytest
import torch

import ms_custom_ops_amd as ms_custom_ops
from ms_custom_ops_amd import cabi
from oracle import gmm_oracle as O

pytestmark = pytest.mark.gpu
ACTS = [O.ACT_RELU, O.ACT_GELU_TANH, O.ACT_FAST_GELU, O.ACT_SILU]
# kernel family, weight storage (transpose_b, packed), shape (m, k, n, e, group_list)
RAGGED = (333, 256, 384, 8, [5, 5, 40, 100, 100, 230, 300, 333])
CASES = [
    ("generic", cabi.OV_GENERIC, False, False, RAGGED),
    ("skinny", cabi.OV_SKINNY, False, False, RAGGED),
    ("skinny_nk", cabi.OV_SKINNY, True, False, RAGGED),
    ("skinny_16w", cabi.OV_AUTO, False, False, (16, 512, 384, 1, [16])),
    ("stream", cabi.OV_AUTO, False, True, (24, 512, 384, 4, [5, 5, 17, 24])),
    ("stream_rows", cabi.OV_AUTO, False, True, (48, 512, 384, 2, [20, 48])),
    ("tile64", cabi.OV_TILE_64, True, False, RAGGED),
    ("tile128", cabi.OV_TILE_128, False, False, RAGGED),
    ("tile256", cabi.OV_TILE_256, False, False, RAGGED),
    ("tile256_w4", cabi.OV_TILE_256_W4, True, False, (700, 640, 512, 3, [300, 300, 700])),
    ("tile256_w4_packed", cabi.OV_TILE_256_W4, False, True, (700, 640, 512, 3, [300, 300, 700])),
    ("tile256_w4_mfma32", cabi.OV_TILE_256_W4_MFMA32, True, False, (700, 640, 512, 3, [300, 300, 700])),
    ("tile256_w4_mfma32_packed", cabi.OV_TILE_256_W4_MFMA32, False, True, (700, 640, 512, 3, [300, 300, 700])),
    ("tile256_w4_mfma32_kn", cabi.OV_TILE_256_W4_MFMA32, False, False, (700, 640 + 48, 512 - 16, 3, [300, 300, 700])),
    ("tile256_w4_kn", cabi.OV_TILE_256_W4, False, False, (700, 640 + 48, 512 - 16, 3, [300, 300, 700])),   # [E,K,N] through transpose reads, K and N tails
    # 128 x 256 tiles (several groups of about a hundred rows, enough columns to fill the chip with them)
    ("tile128x256", cabi.OV_AUTO, True, False, (800, 256, 6144, 8, [90, 200, 310, 400, 400, 530, 700, 800])),
    ("tile128x256_packed", cabi.OV_AUTO, False, True, (800, 256, 6144, 8, [90, 200, 310, 400, 400, 530, 700, 800])),
    # row chunks through LDS, weights straight into MFMA operands (packed weights): 128- and 256-row chunks
    ("rows128_packed", cabi.OV_ROWS128, False, True, RAGGED),
    ("rows256_packed", cabi.OV_ROWS256, False, True, RAGGED),
    ("rows160_packed", cabi.OV_ROWS160, False, True, RAGGED),
    # sixteen uneven groups: the persistent kernel takes the large ones, a second launch of 64 x 128 tiles the small ones
    ("two_launches_packed", cabi.OV_TILE_256_W4, False, True,
     (1200, 512, 512, 16, [300, 303, 303, 373, 437, 502, 503, 783, 783, 800, 830, 900, 964, 1100, 1101, 1200])),
    ("two_launches_kn", cabi.OV_TILE_256_W4, False, False,
     (1200, 512, 512, 16, [300, 303, 303, 373, 437, 502, 503, 783, 783, 800, 830, 900, 964, 1100, 1101, 1200])),
]
# what the plan of a case has to name, so that the case keeps reaching the code it is there for
PLAN_MUST_NAME = {"tile128x256": "128x256", "tile128x256_packed": "128x256", "two_launches_packed": "small_groups=64",
                  "two_launches_kn": "small_groups=64", "stream_rows": "stream_rows", "rows128_packed": "rows128", "rows256_packed": "rows256", "rows160_packed": "rows160"}


def _reference(x, w, gl, bias, scale, pt, act):
    pre = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, out_dtype="f32")   # exact float32 dequantised values
    return pre, O.activation(pre, act)


def _assert_close(got, ref64, out, info):
    got = got.astype(np.float64)
    if out == "bf16":
        ok = np.abs(got - ref64) <= 2.0 ** -7 * np.abs(ref64) + 1e-30
    else:
        ok = np.abs(got - ref64) <= 2.0 ** -10 * np.abs(ref64) + 2.0 ** -24
    assert ok.all(), (info, float(np.abs(got - ref64).max()))


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name,override,transpose_b,packed,shape", CASES, ids=[c[0] for c in CASES])
def test_fused_activation_every_kernel_family(name, override, transpose_b, packed, shape, act):
    from gpu_utils import run_w8a8
    m, k, n, e, gl = shape
    rng = np.random.default_rng(17)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    # scales large enough that the dequantised values spread over [-30, 30]: both tails and the bend of every function
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    last = gl[-1]
    pre, ref64 = _reference(x, w, gl, bias, scale, pt, act)
    assert (pre[:last] < -1).any() and (pre[:last] > 1).any() and (np.abs(pre[:last]) < 1).any()
    for out in ("bf16", "f16"):
        bits, info = run_w8a8(x, w, gl, bias, scale, pt, out=out, transpose_b=transpose_b, override=override, packed=packed,
                              act_type=act, launches=2)
        got = O.bf16_bits_to_f32(bits) if out == "bf16" else bits.view(np.float16).astype(np.float32)
        assert PLAN_MUST_NAME.get(name, "") in info, info
        if act == O.ACT_RELU:
            want = O.f32_to_bf16_bits(ref64.astype(np.float32)) if out == "bf16" else O.f32_to_f16(ref64.astype(np.float32)).view(np.uint16)
            assert np.array_equal(bits[:last], want[:last]), info
        else:
            _assert_close(got[:last], ref64[:last], out, info)


# weight-only shapes (m, k, e, group_list, what the plan must name): the 16-row decode kernels, the multi-row kernels
# with chunks of 32, 64 and 128 rows, and one group of 200 rows whose 128-row chunks split K across workgroups (the
# epilogue then runs in the last arriver)
A16_SHAPES = [
    (32, 512, 4, [7, 7, 20, 32], ""),
    (40, 512, 2, [20, 40], "_rows"),
    (48, 512, 2, [40, 48], "_rows"),
    (130, 512, 2, [100, 130], "_rows"),
    (200, 1024, 1, [200], "_rows"),
]


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("shape", A16_SHAPES, ids=[f"m{s[0]}e{s[2]}" for s in A16_SHAPES])
def test_fused_activation_weight_only(act, packed, shape):
    from gpu_utils import run_a16w8
    rng = np.random.default_rng(3)
    m, k, e, gl, must_name = shape
    n = 384
    xf = rng.standard_normal((m, k)).astype(np.float32)
    x_bits = O.f32_to_bf16_bits(xf)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    s_bits = O.f32_to_bf16_bits(rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32))
    o_bits = O.f32_to_bf16_bits(rng.integers(-8, 9, (e, n)).astype(np.float32))
    xv, sv, ov = (O.bf16_bits_to_f32(b) for b in (x_bits, s_bits, o_bits))
    exact = O.a16w8_grouped_f64(xv, w, sv, ov, gl)
    plain, info = run_a16w8(x_bits, w, s_bits, o_bits, gl, packed=packed)
    bits, info = run_a16w8(x_bits, w, s_bits, o_bits, gl, packed=packed, act_type=act)
    assert must_name in info and (m != 200 or "split_k=1 " not in info), info
    got = O.bf16_bits_to_f32(bits).astype(np.float64)
    # the matmul itself is floating point (tolerance 2^-7 |exact| + 1e-5 sum|terms|, as for the plain weight-only path);
    # the activations are 1.13-Lipschitz, so the same allowance carries through them, plus the output rounding
    mag = np.abs(xv).astype(np.float64).sum(1, keepdims=True) * 140.0 * float(np.abs(sv).max())
    ref = O.activation(exact.astype(np.float32), act)
    assert (np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) + 1.13 * (2.0 ** -7 * np.abs(exact) + 1e-5 * mag) + 1e-30).all(), info
    # and against the kernel's own pre-activation output only the activation and one more rounding lie between
    pre = O.bf16_bits_to_f32(plain)
    assert (exact != 0).any() and not np.array_equal(bits, plain)
    if act == O.ACT_RELU:
        assert np.array_equal(bits, np.where(pre < 0, np.uint16(0), plain))


@pytest.mark.parametrize("mode", [ms_custom_ops.GRAPH_MODE, ms_custom_ops.PYNATIVE_MODE])
def test_v4_act_type_through_the_python_entry(mode):
    rng = np.random.default_rng(9)
    m, k, n, e = 96, 128, 256, 8
    counts = np.array([10, 0, 30, 5, 0, 20, 15, 16], dtype=np.int64)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    for act in ACTS:
        with ms_custom_ops.exec_mode(mode):
            out = ms_custom_ops.grouped_matmul_v4_cops([t(x)], [t(w)], None, [t(scale).bfloat16()], None, None, None, [t(pt)],
                                                       t(counts), split_item=3, group_type=0, group_list_type=1, act_type=act)[0]
        assert out.dtype == torch.bfloat16
        sc_bf = O.bf16_bits_to_f32(O.f32_to_bf16_bits(scale))
        _, ref64 = _reference(x, w, counts.cumsum(), None, sc_bf, pt, act)
        _assert_close(out.float().cpu().numpy(), ref64, "bf16", f"act {act}")


def test_act_type_errors():
    x = torch.zeros(32, 64, dtype=torch.int8, device="cuda")
    w = torch.zeros(8, 64, 128, dtype=torch.int8, device="cuda")
    gl = torch.full((8,), 4, dtype=torch.int64, device="cuda")
    sc = torch.ones(8, 128, dtype=torch.bfloat16, device="cuda")
    f = ms_custom_ops.grouped_matmul_v4_cops
    for bad in (3, 6, -1):
        with pytest.raises(ValueError, match="act_type must be 0"):
            f([x], [w], None, [sc], group_list=gl, split_item=3, group_type=0, act_type=bad)
    with pytest.raises(ValueError, match="needs a floating-point output"):
        f([x], [w], group_list=gl, split_item=3, group_type=0, act_type=1)
    with pytest.raises(RuntimeError, match="'activation_input'"):
        f([x], [w], None, [sc], group_list=gl, activation_input=[x], split_item=3, group_type=0)
    with pytest.raises(cabi.BackendError):
        cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_I32, group_list_dtype=cabi.DT_I64, act_type=cabi.ACT_RELU)
    with pytest.raises(cabi.BackendError):
        cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64, act_type=cabi.ACT_GELU_ERF)
