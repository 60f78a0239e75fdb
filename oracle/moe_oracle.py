"""CPU oracle of the MoE routing / un-permutation operators (numpy).  TEST INFRASTRUCTURE ONLY: nothing
in the product imports this module; tests, the smoke check and bench.py's CPU baseline use it as the checker.

Restated from the reference's own goldens (read, not imported -- the test modules import MindSpore):
  * moe_init_routing_v2     tests/st/test_custom_moe_init_routing_v2.py:33-93 (dropless branch :58-65,
                            count / cumulative count :41-57); the op only accepts active_num = 0,
                            expert_capacity = 0, drop_pad_mode = 0 (ops/c_api/moe_init_routing_v2/moe_init_routing_v2.cc:107-109)
  * moe_token_unpermute     tests/st/test_custom_moe_token_unpermute.py:37-47
  * dyn_quant               tests/st/test_grouped_matmul_w4.py:83-89 (per-row dynamic int8 quantisation of the
                            activations in front of an int8-activation grouped matmul)

Pins (tests/test_moe_routing.py): the routing restatement against an independent per-entry Python sort, against the
permutation / gather invariants and against hand-written tiny cases; the un-permutation against scalar loops that
round with an independent float16 / bfloat16 implementation (torch), against the K = 1 gather and the all-ones cases;
dyn_quant against a per-element loop in Python floats with exact rational tie handling, and against what the
formula fixes (the row maximum maps to +-127, scale * 127 gives the maximum back, |x - q * scale| <= scale / 2).
No function here is "parity unpinned".
"""
from __future__ import annotations

import numpy as np

__all__ = ["moe_init_routing_v2", "moe_init_routing_v2_by_loops", "moe_token_unpermute", "moe_token_unpermute_bf16",
           "dyn_quant", "bf16_bits_to_f32"]


def moe_init_routing_v2(x, expert_idx, expert_num: int, count_or_cumsum_flag: int = 1):
    """Dropless routing.  Returns (expanded_x, expanded_row_idx int32, expert_tokens int32 or None)."""
    x = np.asarray(x)
    expert_idx = np.asarray(expert_idx)
    k = expert_idx.shape[-1]
    flat = expert_idx.reshape(-1)
    sorted_row_idx = np.argsort(flat, axis=-1, kind="stable")                        # golden :38
    hist = np.bincount(np.clip(flat, 0, expert_num - 1), minlength=expert_num)       # golden :46 (ids inside [0, E))
    expanded_row_idx = np.zeros(sorted_row_idx.shape, dtype=np.int32)
    expanded_row_idx[sorted_row_idx] = np.arange(sorted_row_idx.shape[-1], dtype=np.int32)   # golden :59-60
    expanded_x = x[sorted_row_idx // k, :]                                           # golden :65 (active_num = 0: all rows)
    tokens = None
    if count_or_cumsum_flag == 1:
        tokens = np.cumsum(hist).astype(np.int32)                                    # golden :54-55
    elif count_or_cumsum_flag == 2:
        tokens = hist.astype(np.int32)                                               # golden :56-57
    return expanded_x, expanded_row_idx, tokens


def moe_init_routing_v2_by_loops(x, expert_idx, expert_num: int):
    """Independent statement of the same thing: sort the (expert, flat position) pairs, then place row by row."""
    x = np.asarray(x)
    expert_idx = np.asarray(expert_idx)
    n_rows, k = expert_idx.shape
    pairs = sorted((int(expert_idx[t, j]), t * k + j) for t in range(n_rows) for j in range(k))
    expanded_x = np.empty((n_rows * k, x.shape[1]), dtype=x.dtype)
    expanded_row_idx = np.empty(n_rows * k, dtype=np.int32)
    counts = [0] * expert_num
    for dest, (e, pos) in enumerate(pairs):
        expanded_x[dest] = x[pos // k]
        expanded_row_idx[pos] = dest
        counts[e] += 1
    return expanded_x, expanded_row_idx, np.asarray(counts, dtype=np.int32)


def moe_token_unpermute(permuted_tokens, sorted_indices, probs):
    """float16 golden, test_custom_moe_token_unpermute.py:37-47: out[i] += probs[i, k] * permuted[sorted[i*K + k]] with
    numpy float16 arrays, i.e. the product and the running sum are both rounded to float16 (numpy computes half
    arithmetic in float32 and rounds the result)."""
    permuted_tokens = np.asarray(permuted_tokens, dtype=np.float16)
    probs = np.asarray(probs, dtype=np.float16)
    token_num, top_k = probs.shape
    out = np.zeros((token_num, permuted_tokens.shape[1]), dtype=np.float16)
    rows = np.asarray(sorted_indices).reshape(token_num, top_k)
    for k in range(top_k):                                   # the k loop is the golden's accumulation order
        out += probs[:, k:k + 1] * permuted_tokens[rows[:, k], :]
    return out


def _bf16_round(a):
    """float32 -> nearest-even bfloat16, returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


def moe_token_unpermute_bf16(permuted_bits, sorted_indices, probs_bits):
    """The same accumulation for bfloat16 data given as uint16 bit patterns (an extension of this backend: the
    reference op is float16 only).  Returns uint16 bit patterns."""
    pt = (np.asarray(permuted_bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
    pr = (np.asarray(probs_bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
    token_num, top_k = pr.shape
    rows = np.asarray(sorted_indices).reshape(token_num, top_k)
    out = np.zeros((token_num, pt.shape[1]), dtype=np.float32)
    for k in range(top_k):
        out = _bf16_round(out + _bf16_round(pr[:, k:k + 1] * pt[rows[:, k], :]))
    return (out.view(np.uint32) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits):
    """uint16 bfloat16 patterns -> float32 (exact)."""
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32)


def dyn_quant(x):
    """Per-row dynamic int8 quantisation, test_grouped_matmul_w4.py:83-89:
        x_max = max |x| over the row (in x's type);  scale = float32(x_max) / 127;  q = int8(round(float32(x) / scale))
    with numpy's round (half to even) and float32 divisions.  x: float16 array, or float32 array holding values that are
    exact in the activation type (bfloat16 rows widened with bf16_bits_to_f32).  Returns (q int8 [rows, h], scale
    float32 [rows]).  A row of zeros divides 0 by 0 in the golden; here it gets scale 0 and zeros."""
    x = np.asarray(x)
    x32 = x.astype(np.float32)
    x_max = np.max(np.abs(x32), axis=-1, keepdims=True)                  # exact: a maximum rounds nothing
    scale = x_max.astype(np.float32) / np.float32(127.0)
    safe = np.where(scale == 0, np.float32(1.0), scale)
    q = np.round(x32 / safe).astype(np.int8)
    q[np.broadcast_to(scale == 0, q.shape)] = 0
    return q, scale[..., 0]
