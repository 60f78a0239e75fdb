"""CPU oracle for the grouped quantized matmul path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests, the smoke check and
the CPU-baseline leg of the benchmark may import it.  The shipped operators run
on the HIP backend and must fail loudly when that backend is missing.

It restates, in numpy, the arithmetic that the reference pins for this path in
its own system tests (the device kernels themselves are closed binaries):

* grouped W8A8 golden         tests/st/test_grouped_matmul.py:62-71  (np_qbmm_compute)
* row / weight splitting      tests/st/test_grouped_matmul.py:44-59,97-120
* random boundaries           tests/st/test_grouped_matmul.py:162-169
* int64 scale wire format     tests/st/test_grouped_matmul.py:39-41  (process_deq_scale)
* V4 per-token golden         tests/st/test_grouped_matmul_v4_cops.py:291-301
* V4 per-channel+bias golden  tests/st/test_grouped_matmul_v4_cops.py:348-359
* V4 a16w8 golden             tests/st/test_grouped_matmul_v4_cops.py:159-174
* dense goldens               tests/st/test_quant_batch_matmul.py:71-80,136-151,168-184,201-212
* int64 dense scale format    tests/st/test_quant_batch_matmul.py:34-42  (trans_quant_param)
* count-based comparator      tests/st/st_utils.py:23-49             (custom_compare)
* A8W4 golden and nibble pack tests/st/test_grouped_matmul_w4.py:91-97,100-118
* fused activation            PARITY UNPINNED BY THE REFERENCE: act_type is passed through to aclnnGroupedMatmulV4
                              (ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:96,112,363) without values, a
                              description or a golden (grouped_matmul_v4_cops_doc.md:26 is one line); ``activation``
                              takes the values of CANN's GMMActType and the functions' textbook forms.

How each function is pinned (tests/test_oracle_pins.py):

* ``int32_matmul_exact``   brute-force integer loops on tiny shapes, int64 and
                           float64 matmuls, closed forms (ones, identity, +-127
                           saturation), K-chunk invariance.
* ``group_bounds`` / ``grouped_int32_acc``   hand-written boundaries including
                           empty groups, E=1 == dense, row permutation inside a
                           group, dependence on w[g] only, counts == cumsum.
* ``dequant_epilogue``     the reference's constant-scale known answers
                           (scale=10, per-token=10 -> 100*acc; scale=10, bias=1
                           -> 10*(acc+1); scale=1 and int32 out -> acc) and the
                           operation order of np_qbmm_compute.
* ``f32_to_bf16_bits``     hand-computed round-to-nearest-even ties, torch's
                           float32 -> bfloat16 cast on random and special values.
* ``golden_*`` functions   literal restatements of the reference formulas; they
                           are compared against the exact path under the
                           reference's own tolerances.
* ``a16w8_*``              float64 evaluation of x @ ((w + o) * s) on the exact
                           bf16 operand values; closed forms with constant scale.
* ``golden_v4_a16w4``      the reference's own packing loop written out per byte, the a16w8 formula on the unpacked
                           values in float64, and the closed form of its test data (weights in {0, 1}, scale 0.01,
                           offset 1: row sums of x times 0.01 plus 0.01 times the sum over the ones).
* ``decode_scale_int64``   round trip against the two wire formats above.
* ``activation``           what the mathematics fixes: torch's relu / silu / gelu(approximate="tanh") in float64,
                           the tanh form of the gelu against the sigmoid form used here, CANN's published fast-gelu
                           expression against x * sigmoid(1.702 x), silu(x) - silu(-x) = x, limits at +-40.
* ``pack_int4`` / ``unpack_int4``   per-element loops, hand-written bytes, round trip.
* ``golden_grouped_a8w4``  a float64 evaluation of the integer form
                           x_scale * sum_g scale_g * (exact int32 sum over the K group), a brute-force loop on a tiny
                           case, and the closed forms that constant scales give.
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "pack_int4", "unpack_int4", "quant_int4_groups", "golden_grouped_a8w4", "grouped_a8w4_f64",
    "f32_to_bf16_bits", "bf16_bits_to_f32", "f32_to_f16", "int32_matmul_exact", "int32_matmul_bruteforce",
    "group_bounds", "grouped_int32_acc", "dequant_epilogue", "grouped_matmul_w8a8", "golden_np_qbmm",
    "golden_grouped_w8a8", "golden_v4_pertoken", "golden_v4_perchannel_bias", "golden_v4_a16w8", "golden_v4_a16w4",
    "quant_batch_matmul_oracle", "a16w8_grouped_f64", "encode_scale_int64", "encode_scale_int64_qbmm", "pack_weights",
    "decode_scale_int64", "random_group_list", "count_compare", "bf16_ulp_check", "activation",
    "ACT_NONE", "ACT_RELU", "ACT_GELU_TANH", "ACT_GELU_ERF", "ACT_FAST_GELU", "ACT_SILU",
]

# act_type values (CANN's GMMActType; 3, the erf form of the gelu, is the one CANN lists as unsupported)
ACT_NONE, ACT_RELU, ACT_GELU_TANH, ACT_GELU_ERF, ACT_FAST_GELU, ACT_SILU = range(6)

# K-chunk for the exact accumulator: 127*127*1024 = 16 516 096 < 2**24, so every
# partial sum inside one chunk is an integer that float32 represents exactly.
_EXACT_K_CHUNK = 1024


# --------------------------------------------------------------------------
# float formats
# --------------------------------------------------------------------------
def f32_to_bf16_bits(a) -> np.ndarray:
    """float32 -> bfloat16 bit pattern (uint16), round-to-nearest-even, NaN kept quiet."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    nan = np.isnan(a)
    out = rounded.astype(np.uint16)
    if nan.any():
        out = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), out)
    return out


def bf16_bits_to_f32(bits) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_f16(a) -> np.ndarray:
    """float32 -> float16 (IEEE RNE, what numpy's astype does; reference cast at test_grouped_matmul.py:70)."""
    with np.errstate(over="ignore"):
        return np.asarray(a, dtype=np.float32).astype(np.float16)


# --------------------------------------------------------------------------
# exact int32 accumulators
# --------------------------------------------------------------------------
def int32_matmul_bruteforce(a, b) -> np.ndarray:
    """Pure-Python integer triple loop; only for tiny shapes.  a [M,K], b [K,N] integer arrays."""
    a = np.asarray(a)
    b = np.asarray(b)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.zeros((m, n), dtype=np.int64)
    al = a.tolist()
    bl = b.tolist()
    for i in range(m):
        for j in range(n):
            s = 0
            for t in range(k):
                s += int(al[i][t]) * int(bl[t][j])
            out[i, j] = s
    # int32 wrap-around semantics of the accumulator
    return out.astype(np.int64).astype(np.int32)


def int32_matmul_exact(a, b) -> np.ndarray:
    """Exact int32 result of int8[M,K] @ int8[K,N].

    float32 sgemm over K-chunks of at most 1024; each chunk's result is an integer
    of magnitude < 2**24, hence exact in float32, and the chunks are summed in
    int32 (two's-complement wrap like a hardware accumulator; |sum| <= 127*127*K
    cannot wrap for K < 133 000).
    """
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == np.int8 and b.dtype == np.int8, (a.dtype, b.dtype)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2, (a.shape, b.shape)
    acc = np.zeros((m, n), dtype=np.int32)
    if m == 0 or n == 0:
        return acc
    for k0 in range(0, k, _EXACT_K_CHUNK):
        k1 = min(k, k0 + _EXACT_K_CHUNK)
        part = np.dot(a[:, k0:k1].astype(np.float32), b[k0:k1, :].astype(np.float32))
        acc += part.astype(np.int32)
    return acc


# --------------------------------------------------------------------------
# grouping
# --------------------------------------------------------------------------
def group_bounds(group_list, group_list_type: int = 0):
    """Row range [start, end) of every group.

    type 0: cumulative ends (reference split_x, test_grouped_matmul.py:44-52);
    type 1: per-group counts, turned into ends by a running sum
            (test_grouped_matmul_v4_cops.py:296, 353).
    Equal neighbours give an empty group (random boundaries may repeat,
    test_grouped_matmul.py:162-169).
    """
    gl = np.asarray(group_list).astype(np.int64).reshape(-1)
    ends = np.cumsum(gl) if group_list_type == 1 else gl
    starts = np.concatenate([[0], ends[:-1]])
    if (ends < starts).any() or (len(ends) and starts[0] < 0):
        raise ValueError("group_list must be non-decreasing and non-negative")
    return starts, ends


def grouped_int32_acc(x, w, group_list, group_list_type: int = 0, transpose_b: bool = False) -> np.ndarray:
    """acc[m, n] = sum_k x[m, k] * w[g(m), k, n]; rows past the last boundary stay zero."""
    x = np.asarray(x)
    w = np.asarray(w)
    starts, ends = group_bounds(group_list, group_list_type)
    e = w.shape[0]
    assert len(ends) == e, (len(ends), e)
    n = w.shape[1] if transpose_b else w.shape[2]
    acc = np.zeros((x.shape[0], n), dtype=np.int32)
    for g in range(e):
        s, t = int(starts[g]), int(ends[g])
        if t <= s:
            continue
        wg = w[g].T if transpose_b else w[g]
        acc[s:t] = int32_matmul_exact(x[s:t], np.ascontiguousarray(wg))
    return acc


# --------------------------------------------------------------------------
# dequant epilogue
# --------------------------------------------------------------------------
def dequant_epilogue(acc, bias=None, scale=None, per_token=None, out_dtype: str = "bf16"):
    """Epilogue in the operation order of np_qbmm_compute (test_grouped_matmul.py:63-70):

        c = acc (+ bias, int32)  ->  float32(c) * scale[n]  ->  * per_token[m]  ->  cast

    every product is a separate float32 rounding.  ``bias``/``scale`` are [N] or
    [M,N]-broadcastable rows already selected per row's group; ``per_token`` is [M].
    out_dtype: "bf16" (returns uint16 bit patterns), "f16", "f32" (pre-cast value) or
    "i32" (accumulator + bias, no scaling).
    """
    c = np.asarray(acc, dtype=np.int32)
    if bias is not None:
        c = (c.astype(np.int64) + np.asarray(bias).astype(np.int64)).astype(np.int32)
    if out_dtype == "i32":
        return c
    f = c.astype(np.float32)
    if scale is not None:
        f = f * np.asarray(scale, dtype=np.float32)
    if per_token is not None:
        f = f * np.asarray(per_token, dtype=np.float32).reshape(-1, 1)
    f = f.astype(np.float32)
    if out_dtype == "f32":
        return f
    if out_dtype == "f16":
        return f32_to_f16(f)
    if out_dtype == "bf16":
        return f32_to_bf16_bits(f)
    raise ValueError(out_dtype)


def activation(v, act_type: int) -> np.ndarray:
    """Activation of the dequantised float32 values, evaluated in float64 (the caller rounds to the output type).
    relu max(v, 0); gelu_tanh v * sigmoid(2 sqrt(2/pi) (v + 0.044715 v^3)); fast_gelu v * sigmoid(1.702 v);
    silu v * sigmoid(v).  sigmoid(t) is taken as exp(-logaddexp(0, -t)), which neither overflows nor cancels."""
    v = np.asarray(v, dtype=np.float32).astype(np.float64)
    if act_type == ACT_NONE:
        return v
    if act_type == ACT_RELU:
        return np.where(v < 0, 0.0, v)
    if act_type == ACT_GELU_TANH:
        t = 2.0 * np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)
    elif act_type == ACT_FAST_GELU:
        t = 1.702 * v
    elif act_type == ACT_SILU:
        t = v
    else:
        raise ValueError(f"act_type {act_type} is not supported")
    return v * np.exp(-np.logaddexp(0.0, -t))


def _rows_of(param, starts, ends, m):
    """Expand a per-group [E, N] parameter to per-row [M, N] following the group of each row."""
    param = np.asarray(param)
    out = np.zeros((m, param.shape[-1]), dtype=param.dtype)
    for g in range(len(ends)):
        out[int(starts[g]):int(ends[g])] = param[g]
    return out


def grouped_matmul_w8a8(x, w, group_list, bias=None, scale=None, per_token=None, *, group_list_type: int = 0,
                        transpose_b: bool = False, out_dtype: str = "bf16", return_acc: bool = False):
    """Full grouped W8A8 path.  x int8 [M,K]; w int8 [E,K,N] ([E,N,K] when transpose_b);
    bias int32 [E,N]; scale float32 [E,N]; per_token float32 [M].  Rows at or past the
    last boundary are zero in every output."""
    x = np.asarray(x)
    m = x.shape[0]
    starts, ends = group_bounds(group_list, group_list_type)
    acc = grouped_int32_acc(x, w, group_list, group_list_type, transpose_b)
    b_rows = None if bias is None else _rows_of(bias, starts, ends, m)
    s_rows = None if scale is None else _rows_of(np.asarray(scale, dtype=np.float32), starts, ends, m)
    out = dequant_epilogue(acc, b_rows, s_rows, per_token, out_dtype)
    last = int(ends[-1]) if len(ends) else 0
    if last < m:
        out = out.copy()
        out[last:] = 0
    return (out, acc) if return_acc else out


# --------------------------------------------------------------------------
# literal restatements of the reference goldens (used to show the exact path
# above agrees with them under the reference's own tolerances, and as the timed
# CPU baseline)
# --------------------------------------------------------------------------
def golden_np_qbmm(a, b, scale, bias=None, per_token=None, out: str = "f16"):
    """One group of the reference golden, test_grouped_matmul.py:62-71: a single float32
    dot truncated to int32 (exact only while every partial sum stays below 2**24)."""
    c = np.dot(a.astype(np.float32), b.astype(np.float32)).astype(np.int32)
    if bias is not None:
        c = c + bias
    c = c.astype(np.float32) * scale
    if per_token is not None:
        c = c * per_token[:, np.newaxis]
    if out == "f16":
        return c.astype(np.float16)
    if out == "bf16":
        return f32_to_bf16_bits(c)
    return c


def golden_grouped_w8a8(x, w, group_list, bias=None, scale=None, per_token=None, out: str = "f16"):
    """Split / per-group golden / row-concat, test_grouped_matmul.py:97-120."""
    starts, ends = group_bounds(group_list, 0)
    parts = []
    for g in range(w.shape[0]):
        s, t = int(starts[g]), int(ends[g])
        parts.append(golden_np_qbmm(x[s:t], w[g], scale[g], None if bias is None else bias[g],
                                    None if per_token is None else per_token[s:t], out))
    return np.concatenate(parts, axis=0)


def golden_v4_pertoken(x, w, scale, per_token, counts):
    """test_grouped_matmul_v4_cops.py:296-301: matmul(x_g, w_g * s_g) row-concat, then * per_token."""
    starts, ends = group_bounds(counts, 1)
    parts = [np.matmul(x[int(s):int(t)], w[g] * scale[g]) for g, (s, t) in enumerate(zip(starts, ends))]
    return np.concatenate(parts, axis=0) * per_token.reshape(-1, 1)


def golden_v4_perchannel_bias(x, w, scale, bias, counts):
    """test_grouped_matmul_v4_cops.py:353-359: matmul(x_g, w_g * s_g) + b_g * s_g."""
    starts, ends = group_bounds(counts, 1)
    parts = [np.matmul(x[int(s):int(t)], w[g] * scale[g]) + bias[g] * scale[g]
             for g, (s, t) in enumerate(zip(starts, ends))]
    return np.concatenate(parts, axis=0)


def encode_scale_uint64(scale_f32) -> np.ndarray:
    """float32 scales -> the uint64 wire format of the V4 A8W4 test (float32 bits zero-extended,
    tests/st/test_grouped_matmul_v4_cops.py:462)."""
    return np.frombuffer(np.ascontiguousarray(scale_f32, dtype=np.float32).tobytes(), dtype=np.uint32).astype(np.uint64).reshape(np.shape(scale_f32))


def golden_v4_a8w4(x, w, scale_u64, per_token, counts):
    """The reference's expected value for grouped_matmul_v4_cops with 4-bit weights, literally
    (tests/st/test_grouped_matmul_v4_cops.py:467-476): x int8 [m, k]; w the int8 VALUES [e, k, n] in [-8, 7] (the op itself
    receives them as pack_int4(w), two per byte along n, :458-460); scale_u64 [e, 1, n] float32 bits in uint64; per_token
    float32 [m, 1]; counts int64 [e].  float32 [sum(counts), n]; the test's float32 bias (:463) does not enter."""
    index = np.cumsum(counts)
    x_split = np.split(x, index, axis=0)
    pt_split = np.split(per_token, index, axis=0)
    scale_fp32 = np.asarray(scale_u64).astype(np.uint32)
    scale_fp32.dtype = np.float32
    out = []
    for i in range(w.shape[0]):
        mm = np.matmul(x_split[i].astype(np.int32), w[i].astype(np.int32)).astype(np.float32)
        mm = mm * scale_fp32[i] * pt_split[i]
        out.append(mm)
    return np.concatenate(out, axis=0)


def golden_v4_a16w8(x, w, antiquant_scale, antiquant_offset, ends):
    """test_grouped_matmul_v4_cops.py:166-174: matmul(x_g, (w_g + o_g) * s_g) in the dtype numpy picks
    (x's float dtype); only rows below the last boundary exist."""
    starts, ends_ = group_bounds(ends, 0)
    parts = [np.matmul(x[int(s):int(t)], (w[g] + antiquant_offset[g]) * antiquant_scale[g])
             for g, (s, t) in enumerate(zip(starts, ends_))]
    return np.concatenate(parts, axis=0)


def golden_v4_a16w4(x, w, antiquant_scale, antiquant_offset, ends):
    """The reference's expected value for grouped_matmul_v4_cops with float16 / bfloat16 x and 4-bit weights
    (tests/st/test_grouped_matmul_v4_cops.py:223-241): w holds the int8 VALUES [e, k, n] (the op itself receives
    pack_int4(w): value 2 i in the low nibble and 2 i + 1 in the high nibble of byte i along the flattened tensor, i.e.
    pairs along n, :229-233); the expected value is the a16w8 formula on those values, matmul(x_g, (w_g + o_g) * s_g)."""
    return golden_v4_a16w8(x, w, antiquant_scale, antiquant_offset, ends)


# --------------------------------------------------------------------------
# dense single-group path (quant_batch_matmul)
# --------------------------------------------------------------------------
def quant_batch_matmul_oracle(x1, x2, scale, bias=None, per_token=None, transpose_x1: bool = False,
                              transpose_x2: bool = False, out_dtype: str = "bf16"):
    """Dense / batched W8A8 (tests/st/test_quant_batch_matmul.py:71-80,136-151,168-184).

    x1 [..., M, K] ([..., K, M] when transposed), x2 [..., K, N]; batch dims broadcast as in
    BatchMatMulMakeShape (ops/c_api/utils/common_utils.cc:79-138).  scale is [1] or [N],
    bias int32 [N], per_token [M].  Same epilogue order as the grouped path."""
    x1 = np.asarray(x1)
    x2 = np.asarray(x2)
    if transpose_x1:
        x1 = np.swapaxes(x1, -1, -2)
    if transpose_x2:
        x2 = np.swapaxes(x2, -1, -2)
    batch = np.broadcast_shapes(x1.shape[:-2], x2.shape[:-2])
    m, n = x1.shape[-2], x2.shape[-1]
    x1b = np.broadcast_to(x1, batch + x1.shape[-2:]).reshape((-1,) + x1.shape[-2:])
    x2b = np.broadcast_to(x2, batch + x2.shape[-2:]).reshape((-1,) + x2.shape[-2:])
    scale = np.asarray(scale, dtype=np.float32).reshape(-1)
    outs = []
    for i in range(x1b.shape[0]):
        acc = int32_matmul_exact(np.ascontiguousarray(x1b[i]), np.ascontiguousarray(x2b[i]))
        outs.append(dequant_epilogue(acc, bias, scale, per_token, out_dtype))
    return np.stack(outs, 0).reshape(batch + (m, n)) if outs else np.zeros(batch + (m, n))


# --------------------------------------------------------------------------
# weight-only W8A16
# --------------------------------------------------------------------------
def a16w8_grouped_f64(x, w, antiquant_scale, antiquant_offset, group_list, group_list_type: int = 0):
    """Ground truth for the weight-only path in float64:
    out[m, n] = sum_k x[m, k] * (w[g, k, n] + o[g, n]) * s[g, n]  on the exact values of the
    (already bf16/fp16-rounded) operands.  Formula: test_grouped_matmul_v4_cops.py:166-174."""
    x = np.asarray(x, dtype=np.float64)
    starts, ends = group_bounds(group_list, group_list_type)
    n = w.shape[2]
    out = np.zeros((x.shape[0], n), dtype=np.float64)
    for g in range(w.shape[0]):
        s, t = int(starts[g]), int(ends[g])
        if t <= s:
            continue
        wd = (w[g].astype(np.float64) + np.asarray(antiquant_offset[g], dtype=np.float64)) \
            * np.asarray(antiquant_scale[g], dtype=np.float64)
        out[s:t] = x[s:t] @ wd
    return out


# --------------------------------------------------------------------------
# scale wire formats
# --------------------------------------------------------------------------
def encode_scale_int64(scale_f32) -> np.ndarray:
    """float32 bits zero-extended into int64 (process_deq_scale, test_grouped_matmul.py:39-41)."""
    s = np.ascontiguousarray(scale_f32, dtype=np.float32)
    return s.view(np.uint32).astype(np.int64).reshape(s.shape)


def encode_scale_int64_qbmm(scale_f32) -> np.ndarray:
    """Dense-op wire format (trans_quant_param, test_quant_batch_matmul.py:34-42): keep the top 19
    bits of the float32 pattern, zero-extend to 64 bits and set bit 46."""
    s = np.ascontiguousarray(scale_f32, dtype=np.float32)
    u = (s.view(np.uint32) & np.uint32(0xFFFFE000)).astype(np.uint64)
    u = u | np.uint64(1 << 46)
    return u.astype(np.int64).reshape(s.shape)


def decode_scale_int64(scale_i64) -> np.ndarray:
    """Low 32 bits of each int64/uint64 element reinterpreted as float32."""
    u = np.ascontiguousarray(scale_i64).view(np.uint64) & np.uint64(0xFFFFFFFF)
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(scale_i64))


# --------------------------------------------------------------------------
# helpers used by tests
# --------------------------------------------------------------------------
def random_group_list(m: int, e: int, rng) -> np.ndarray:
    """e-1 boundaries drawn with replacement from 1..m, plus m, sorted: duplicates give empty
    groups (generate_random_numbers, test_grouped_matmul.py:162-169)."""
    cuts = rng.integers(1, m + 1, size=e - 1) if e > 1 else np.zeros(0, dtype=np.int64)
    return np.sort(np.concatenate([cuts, [m]])).astype(np.int64)


def count_compare(output, expect, limit: float) -> bool:
    """The reference's count-based bar (custom_compare, st_utils.py:23-49): at most size*limit
    elements may have relative error above ``limit`` (0.004 fp16, 0.03 bf16)."""
    o = np.asarray(output, dtype=np.float64).ravel()
    x = np.asarray(expect, dtype=np.float64).ravel()
    with np.errstate(divide="ignore", invalid="ignore"):
        bad = np.abs(o - x) / np.abs(x) > limit
    return int(bad.sum()) <= int(o.size * limit)


def bf16_ulp_check(out_bits, ref_bits):
    """Return (max |out-ref| / |ref|, number of elements violating |err| <= 2**-7 * |ref|)."""
    o = bf16_bits_to_f32(out_bits).astype(np.float64)
    r = bf16_bits_to_f32(ref_bits).astype(np.float64)
    err = np.abs(o - r)
    bad = err > (2.0 ** -7) * np.abs(r)
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(r != 0, err / np.abs(r), np.where(err == 0, 0.0, np.inf))
    return (float(rel.max()) if rel.size else 0.0), int(bad.sum())


def pack_weights(w):
    """[E,K,N] int8 -> the backend's packed weight layout, as a flat int8 array per group: [E, bytes].

    This layout has no counterpart in the reference (whose blocked weight format, FRACTAL_NZ, is produced by its
    closed trans_data kernel); it is restated here from the layout's definition so that the device-side packing can be
    checked: per group ceil(N/16) column groups of ceil(K/64) blocks of 1024 bytes, zero outside K x N; byte
    16 l + i (l = 0..63, i = 0..15) of block (a, b) holds w[k = 64 b + 16 (l // 16) + i][n = 16 a + (l % 16)].
    Pinned in tests/test_oracle_pins.py by a per-byte loop over the definition."""
    w = np.asarray(w, dtype=np.int8)
    e, k, n = w.shape
    kb, ng = (k + 63) // 64, (n + 15) // 16
    wp = np.zeros((e, kb * 64, ng * 16), dtype=np.int8)
    wp[:, :k, :n] = w
    # k = 64 b + 16 q + i, n = 16 a + c  ->  [e, a, b, q, c, i]
    return np.ascontiguousarray(wp.reshape(e, kb, 4, 16, ng, 16).transpose(0, 4, 1, 2, 5, 3)).reshape(e, -1)


# ------------------------------------------------------------------------------------------ A8W4
def pack_int4(w):
    """int8 values in [-8, 7], last axis of even length -> bytes, two per byte, even index in the low nibble
    (i8toi4, tests/st/test_grouped_matmul_w4.py:115-118)."""
    u = ((np.asarray(w).astype(np.int16) + 16) % 16).astype(np.uint8)
    return (u[..., 1::2] << 4) | u[..., ::2]


def unpack_int4(packed):
    """Inverse of pack_int4: bytes [..., k/2] -> int8 [..., k] in [-8, 7]."""
    p = np.asarray(packed).astype(np.uint8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int8)
    lo, hi = (p & 0x0F).astype(np.int8), (p >> 4).astype(np.int8)
    out[..., ::2] = np.where(lo >= 8, lo - 16, lo)
    out[..., 1::2] = np.where(hi >= 8, hi - 16, hi)
    return out


def quant_int4_groups(w_fp, group):
    """The reference test's weight quantiser (quant, test_grouped_matmul_w4.py:91-97): float weights [e, k, n] -> int8
    values in [-7, 7] [e, k, n] and float32 scales [e, k / group, 1, n] (max |w| over the K group / 7)."""
    e, k, n = w_fp.shape
    y = np.asarray(w_fp).reshape(e, k // group, group, n)
    y_max = np.max(np.abs(y), keepdims=True, axis=-2)
    scale = y_max.astype(np.float32) / 7.0
    q = np.round(y.astype(np.float32) / scale).astype(np.int8).reshape(e, k, n)
    return q, scale


def golden_grouped_a8w4(x, w_packed, group_list, x_scale, w_scale, group):
    """tests/st/test_grouped_matmul_w4.py:103-113 with the weights taken as the op gets them ([e, n, k/2] nibbles):
    w_deq = int4 * scale per K group (float32); per expert matmul(x as float16, w_deq) * x_scale rows; float32 result
    (the test compares the op's float16 output against it with custom_compare, limit 0.004)."""
    x = np.asarray(x)
    w = unpack_int4(w_packed).transpose(0, 2, 1)                        # [e, k, n]
    e, k, n = w.shape
    w_deq = (w.reshape(e, k // group, group, n).astype(np.float32) * np.asarray(w_scale, dtype=np.float32).reshape(e, k // group, 1, n))
    w_deq = w_deq.reshape(e, k, n)
    gl = [int(v) for v in np.asarray(group_list)]
    out = np.zeros((x.shape[0], n), dtype=np.float32)
    start = 0
    for g in range(e):
        end = gl[g]
        if end > start:
            out[start:end] = np.matmul(x[start:end].astype(np.float16), w_deq[g]) * np.asarray(x_scale, dtype=np.float32)[start:end, None]
        start = max(start, end)
    return out


def grouped_a8w4_f64(x, w_packed, group_list, x_scale, w_scale, group):
    """The same quantity from exact integers: x_scale * sum_g scale_g * (int sum over K group g), in float64."""
    x = np.asarray(x).astype(np.int64)
    w = unpack_int4(w_packed).transpose(0, 2, 1).astype(np.int64)
    e, k, n = w.shape
    sc = np.asarray(w_scale, dtype=np.float64).reshape(e, k // group, n)
    gl = [int(v) for v in np.asarray(group_list)]
    out = np.zeros((x.shape[0], n), dtype=np.float64)
    start = 0
    for g in range(e):
        end = gl[g]
        for kg in range(k // group):
            if end > start:
                part = x[start:end, kg * group:(kg + 1) * group] @ w[g, kg * group:(kg + 1) * group]
                out[start:end] += part.astype(np.float64) * sc[g, kg][None, :]
        start = max(start, end)
    return out * np.asarray(x_scale, dtype=np.float64)[:, None]
