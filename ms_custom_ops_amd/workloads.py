"""Synthetic workloads for the grouped quantized matmul path (numpy, host side).

Every workload is drawn from numpy's legacy global stream seeded with 0, in the fixed order
x, weight, weight scale, activation scale, bias, routing logits.  int8 tensors are true
uniform integers in [-127, 127].  Routing follows an MoE layer: softmax of the logits,
top-k experts per token, the (token, expert) rows stably sorted by expert, and a cumulative
int64 ``group_list`` of the per-expert row counts.

Names
-----
c1          single group,  M=128  K=4096 N=4096, zero int32 bias
c2_m{M}     dense linear,  K=4096 N=11008, M in {1, 16, 256, 2048}, int32 bias in [-1000, 1000]
c3          MoE E=8 top-2 over 4096 tokens (8192 rows), K=4096 N=14336
c4          MoE E=64 top-6 over 8192 tokens (49152 rows), Zipf(1.2) expert popularity, K=2048 N=2816
c5          weight-only decode, E=8 top-2 over 16 tokens (32 rows), bf16 x, K=4096 N=14336 (c5_t<T>: T tokens)
c3_decode   the c3 layer at decode time: E=8 top-2 over 16 tokens (32 rows), int8 x, K=4096 N=14336 (not one of the
            published configurations: c3's weights with c5's routing, the W8A8 counterpart of c5)
ref_m{M}_k{K}_n{N}_e{E}
            the shapes the reference's own tests time or call "real": M rows cut into E groups at sorted random
            boundaries (empty groups allowed), per-channel and per-token scales -- E=8, M=1024, K=5120, N in {2688, 1344}
            (tests/st/test_grouped_matmul.py:325-345) and E=256 with (M, K, N) in {(40, 512, 7168), (1024, 2048, 7168),
            (1024, 7168, 4096)} (:190-204).  Weights beyond 1 GiB are not drawn on the host: ``w`` is None and
            ``meta["w_shape"]`` says what to draw on the device (timing only).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np

__all__ = ["Workload", "make", "names", "route_topk", "algorithmic_work", "f32_to_bf16_bits"]


def f32_to_bf16_bits(a) -> np.ndarray:
    """float32 -> bfloat16 bit pattern with round-to-nearest-even (finite inputs)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


@dataclass
class Workload:
    name: str
    kind: str                      # "w8a8" or "a16w8"
    m: int
    k: int
    n: int
    e: int
    x: np.ndarray                  # int8 [M,K]  (uint16 bf16 bits for a16w8)
    w: np.ndarray                  # int8 [E,K,N]
    scale: Optional[np.ndarray]    # f32 [E,N]   (a16w8: bf16 bits uint16 [E,N] antiquant scale)
    per_token: Optional[np.ndarray]  # f32 [M]
    bias: Optional[np.ndarray]     # int32 [E,N]
    offset: Optional[np.ndarray]   # a16w8: bf16 bits uint16 [E,N] antiquant offset
    group_list: np.ndarray         # int64 [E], cumulative
    meta: Dict = field(default_factory=dict)

    @property
    def ops(self) -> float:
        return 2.0 * int(self.group_list[-1]) * self.k * self.n

    @property
    def bytes(self) -> float:
        return algorithmic_work(self)["bytes"]


def _int8(shape):
    return np.random.randint(-127, 128, size=shape, dtype=np.int8)


def _scale(shape):
    return np.random.uniform(1e-3, 1e-2, size=shape).astype(np.float32)


def route_topk(logits: np.ndarray, top_k: int, n_experts: int):
    """Softmax -> top-k -> rows stably sorted by expert.  Returns (group_list int64 [E] cumulative,
    sorted expert id per row, source token per row)."""
    z = logits - logits.max(axis=1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(axis=1, keepdims=True)
    topk = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    expert_of_row = topk.reshape(-1)
    token_of_row = np.repeat(np.arange(logits.shape[0]), top_k)
    order = np.argsort(expert_of_row, kind="stable")
    counts = np.bincount(expert_of_row, minlength=n_experts)
    return np.cumsum(counts).astype(np.int64), expert_of_row[order], token_of_row[order]


def names():
    return ["c1", "c2_m1", "c2_m16", "c2_m256", "c2_m2048", "c3", "c4", "c5"]


def make(name: str, *, scale_down: int = 1) -> Workload:
    """Build a named workload.  ``scale_down`` > 1 divides K and N (and tokens for the MoE
    workloads) for quick tests; 1 gives the full-size configuration."""
    np.random.seed(0)
    sd = int(scale_down)
    if name == "c1":
        m, k, n, e = 128, 4096 // sd, 4096 // sd, 1
        x = _int8((m, k)); w = _int8((e, k, n)); s = _scale((e, n)); pt = _scale((m,))
        bias = np.zeros((e, n), dtype=np.int32)
        gl = np.array([m], dtype=np.int64)
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, bias, None, gl)
    if name.startswith("c2_m"):
        m = int(name[4:])
        k, n, e = 4096 // sd, 11008 // sd, 1
        x = _int8((m, k)); w = _int8((e, k, n)); s = _scale((e, n)); pt = _scale((m,))
        bias = np.random.randint(-1000, 1001, size=(e, n)).astype(np.int32)
        gl = np.array([m], dtype=np.int64)
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, bias, None, gl)
    if name == "c3":
        t, e, top_k = 4096 // sd, 8, 2
        k, n = 4096 // sd, 14336 // sd
        m = t * top_k
        x = _int8((m, k)); w = _int8((e, k, n)); s = _scale((e, n)); pt = _scale((m,))
        logits = np.random.randn(t, e)
        gl, _, _ = route_topk(logits, top_k, e)
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, None, None, gl)
    if name == "c3_decode" or name.startswith("c3_t"):   # c3_t<T>: the MoE layer of c3 with T tokens (c3_decode = c3_t16)
        t, e, top_k = (16 if name == "c3_decode" else int(name[4:])), 8, 2
        k, n = 4096 // sd, 14336 // sd
        m = t * top_k
        x = _int8((m, k)); w = _int8((e, k, n)); s = _scale((e, n)); pt = _scale((m,))
        logits = np.random.randn(t, e)
        gl, _, _ = route_topk(logits, top_k, e)
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, None, None, gl)
    if name == "c4":
        t, e, top_k = 8192 // sd, 64, 6
        k, n = 2048 // sd, 2816 // sd
        m = t * top_k
        x = _int8((m, k)); w = _int8((e, k, n)); s = _scale((e, n)); pt = _scale((m,))
        pop = 1.0 / np.arange(1, e + 1) ** 1.2
        pop /= pop.sum()
        logits = np.random.randn(t, e) + np.log(pop)[None, :]
        gl, _, _ = route_topk(logits, top_k, e)
        counts = np.diff(np.concatenate([[0], gl]))
        meta = {"empty_groups": int((counts == 0).sum()), "max_over_mean": float(counts.max() / counts.mean())}
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, None, None, gl, meta)
    if name == "c5" or name.startswith("c5_t"):   # c5_t<T>: the weight-only layer of c5 with T tokens (c5 = c5_t16)
        t, e, top_k = (16 if name == "c5" else int(name[4:])), 8, 2
        k, n = 4096 // sd, 14336 // sd
        m = t * top_k
        x = f32_to_bf16_bits(np.random.randn(m, k).astype(np.float32))
        w = _int8((e, k, n))
        s = f32_to_bf16_bits(np.random.uniform(1e-3, 1e-2, size=(e, n)).astype(np.float32))
        off_i8 = np.random.randint(-8, 9, size=(e, n)).astype(np.int8)
        off = f32_to_bf16_bits(off_i8.astype(np.float32))
        logits = np.random.randn(t, e)
        gl, _, _ = route_topk(logits, top_k, e)
        return Workload(name, "a16w8", m, k, n, e, x, w, s, None, None, off, gl, {"offset_int8": off_i8})
    if name.startswith("ref_m"):
        parts = dict((p[0], int(p[1:])) for p in name[4:].split("_"))
        m, k, n, e = parts["m"], parts["k"] // sd, parts["n"] // sd, parts["e"]
        x = _int8((m, k))
        big = e * k * n > (1 << 30)
        w = None if big else _int8((e, k, n))
        s = _scale((e, n)); pt = _scale((m,))
        cuts = np.sort(np.random.randint(0, m + 1, size=e - 1))   # duplicates allowed: empty groups (test_grouped_matmul.py:162-169)
        gl = np.concatenate([cuts, [m]]).astype(np.int64)
        return Workload(name, "w8a8", m, k, n, e, x, w, s, pt, None, None, gl, {"w_shape": (e, k, n)})
    raise KeyError(name)


def algorithmic_work(wl: Workload) -> Dict[str, float]:
    """Algorithmic ops and bytes of one pass: ops = 2*M*K*N with M = group_list[-1]; bytes = x +
    weights of the non-empty experts + 2-byte output + scales / bias / group_list."""
    m = int(wl.group_list[-1])
    counts = np.diff(np.concatenate([[0], wl.group_list]))
    nonempty = int((counts > 0).sum())
    sx = 1 if wl.kind == "w8a8" else 2
    b = m * wl.k * sx + nonempty * wl.k * wl.n + m * wl.n * 2 + wl.group_list.nbytes
    for extra in (wl.scale, wl.per_token, wl.bias, wl.offset):
        if extra is not None:
            # per-group rows ([E, N]) are read for the groups that hold rows only
            per_group = extra.ndim == 2 and extra.shape[0] == wl.e and wl.e > 1
            b += extra.nbytes * nonempty // wl.e if per_group else extra.nbytes
    return {"ops": 2.0 * m * wl.k * wl.n, "bytes": float(b), "rows": m, "nonempty_groups": nonempty}
