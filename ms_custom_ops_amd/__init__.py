"""ms_custom_ops grouped quantized matmul operators on AMD Instinct MI355X (gfx950).

Drop-in for the grouped / dense quantized matmul entries of ms_custom_ops
(python/ms_custom_ops/__init__.py:76 re-exports them from the compiled module):

    grouped_matmul(x, weight, group_list, bias=None, scale=None, per_token_scale=None,
                   antiquant_scale=None, transpose_a=False, transpose_b=False, x_format=0)
    grouped_matmul_v4_cops(x, weight, bias=None, scale=None, offset=None, antiquant_scale=None,
                           antiquant_offset=None, per_token_scale=None, group_list=None,
                           activation_input=None, activation_quant_scale=None,
                           activation_quant_offset=None, split_item=0, group_type=-1,
                           group_list_type=0, act_type=0, weight_format="ND", output_dtype=None)
    quant_batch_matmul(x1, x2, scale, offset=None, bias=None, pertoken_scale=None,
                       transpose_x1=False, transpose_x2=False, x2_format="ND", output_dtype=float16)
    grouped_matmul_w4(x, weight, group_list, bias, x_scale, weight_scale)

and for the two MoE steps on either side of the grouped matmul:

    moe_init_routing_v2(x, expert_idx, active_num, expert_capacity, expert_num, drop_pad_mode,
                        expert_tokens_count_or_cumsum_flag, expert_tokens_before_capacity_flag)
    moe_token_unpermute(permuted_tokens, sorted_indices, probs, padded_mode=False, restore_shape=None)

plus one fusion the reference has no operator for: moe_init_routing_quant(x, expert_idx, expert_num, flag), the routing
step with the per-token int8 quantisation of the activations done on the way.

Tensors are PyTorch-ROCm tensors on the GPU; PyTorch only provides device memory and the current
stream.  The compiled operator layer (``ms_custom_ops_amd.ms_custom_ops``, pybind11) validates and
plans, and the HIP backend behind the C ABI (``lib/libmsco_gmm.so``) does the work.  There is no
CPU or eager fallback: importing this package without the compiled modules raises.

Both execution modes of the reference are available: "pynative" calls the pybind entry directly,
"graph" runs the registered infer implementation and kernel module (Init / Resize / Launch).
"""
from __future__ import annotations

import contextlib
import os
from typing import List, Optional, Sequence

import torch

from . import cabi

try:
    from . import ms_custom_ops as _C  # the compiled operator layer
except ImportError as exc:  # pragma: no cover - exercised only on a broken install
    raise ImportError(
        "ms_custom_ops_amd: the compiled operator module is missing; run `python ms_custom_ops_amd/build.py` "
        "(needs hipcc for gfx950 and g++). There is no fallback implementation.") from exc

__all__ = ["grouped_matmul", "grouped_matmul_v4_cops", "grouped_matmul_w4", "quant_batch_matmul", "moe_init_routing_v2", "moe_init_routing_quant",
           "moe_token_unpermute", "set_context", "get_context", "exec_mode",
           "GRAPH_MODE", "PYNATIVE_MODE", "dtype_to_type_id", "type_id_to_dtype", "plan_cache_stats", "trans_data",
           "qint4x2", "QInt4x2", "as_qint4x2", "widen_qint4x2"]

GRAPH_MODE = 0
PYNATIVE_MODE = 1
_mode = PYNATIVE_MODE

# MindSpore TypeId values (the integer form of dtype arguments; float16 == 42 is the default
# output_dtype of quant_batch_matmul, ops/c_api/quant_batch_matmul/quant_batch_matmul.cc:161)
_TYPE_IDS = {
    torch.bool: 30, torch.int8: 32, torch.int16: 33, torch.int32: 34, torch.int64: 35, torch.uint8: 37,
    torch.float16: 42, torch.float32: 43, torch.float64: 44, torch.bfloat16: 45,
}
if hasattr(torch, "uint64"):
    _TYPE_IDS[torch.uint64] = 40
_DTYPES = {v: k for k, v in _TYPE_IDS.items()}


def dtype_to_type_id(dtype) -> Optional[int]:
    """torch dtype (or TypeId int, or None) -> TypeId int, the reference's ``dtype_to_type_id`` arg handler."""
    if dtype is None or isinstance(dtype, int):
        return dtype
    try:
        return _TYPE_IDS[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}") from None


def type_id_to_dtype(type_id: int):
    return _DTYPES[int(type_id)]


def set_context(mode: int):
    """Select GRAPH_MODE or PYNATIVE_MODE for subsequent operator calls."""
    global _mode
    if mode not in (GRAPH_MODE, PYNATIVE_MODE):
        raise ValueError("mode must be GRAPH_MODE or PYNATIVE_MODE")
    _mode = mode


def get_context() -> int:
    return _mode


@contextlib.contextmanager
def exec_mode(mode: int):
    prev = get_context()
    set_context(mode)
    try:
        yield
    finally:
        set_context(prev)


qint4x2 = 50   # TypeId of MindSpore's packed 4-bit type (two signed 4-bit values per stored element)


class QInt4x2:
    """Marks an int8 / uint8 tensor as qint4x2 data (torch has no 4-bit dtype): every byte holds two signed 4-bit values,
    the even-indexed one in the low nibble, and the stored shape is the logical shape with the last axis halved -- what
    ``Tensor(w_int4_np, dtype=ms.qint4x2)`` is in the reference (tests/st/test_grouped_matmul_v4_cops.py:458-460,479)."""

    def __init__(self, tensor: torch.Tensor):
        if not isinstance(tensor, torch.Tensor) or tensor.dtype not in (torch.int8, torch.uint8):
            raise TypeError("qint4x2 data is carried by an int8 or uint8 tensor")
        self.tensor = tensor


def as_qint4x2(tensor: torch.Tensor) -> QInt4x2:
    return QInt4x2(tensor)


def widen_qint4x2(weight) -> torch.Tensor:
    """4-bit weights widened to int8 once, at load time: [..., N / 2] nibble pairs (a QInt4x2 or the int8 / uint8 bytes
    themselves; low nibble first, signed) become an int8 tensor [..., N] that grouped_matmul_v4_cops takes like any int8
    weight.  The op widens a qint4x2 weight on every call (one more pass over the weights); a caller whose weights do
    not change does it here and keeps the result.  No counterpart in the reference, whose kernels read 4-bit weights
    directly (ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:56-66)."""
    t = weight.tensor if isinstance(weight, QInt4x2) else QInt4x2(weight).tensor
    if not t.is_cuda:
        raise RuntimeError("widen_qint4x2 takes a GPU tensor (the operators have no CPU path)")
    from . import cabi
    src = t.contiguous()
    out = torch.empty(tuple(src.shape[:-1]) + (2 * src.shape[-1],), dtype=torch.int8, device=src.device)
    with torch.cuda.device(src.device):
        cabi.unpack_int4(src.data_ptr(), out.data_ptr(), src.numel(), torch.cuda.current_stream().cuda_stream)
    return out


# ---- framework hooks: PyTorch owns device memory and streams -------------------------------------
def _wrap(t: Optional[torch.Tensor]):
    if t is None:
        return None
    if isinstance(t, QInt4x2):
        w = t.tensor
        if not w.is_cuda:
            raise ValueError("ms_custom_ops_amd operators take GPU tensors; got a tensor on " + str(w.device))
        return _C.Tensor(w.data_ptr(), qint4x2, list(w.shape), list(w.stride()), w)
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"expected a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError("ms_custom_ops_amd operators take GPU tensors; got a tensor on " + str(t.device))
    return _C.Tensor(t.data_ptr(), dtype_to_type_id(t.dtype), list(t.shape), list(t.stride()), t)


def _wrap_list(ts):
    if ts is None:
        return None
    if isinstance(ts, torch.Tensor):
        raise TypeError("expected a list of tensors")
    return [_wrap(t) for t in ts]


_CUDA = torch.device("cuda")


def _allocate(type_id: int, shape: Sequence[int]):
    # (called once or twice per operator call from the C++ layer: kept free of argument checks and string parsing)
    t = torch.empty(tuple(shape), dtype=_DTYPES[type_id], device=_CUDA)
    return _C.Tensor(t.data_ptr(), type_id, list(shape), list(t.stride()), t)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream() -> int:
    # the raw getter skips the construction of a torch.cuda.Stream object (a few microseconds per operator call)
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


_C._set_framework_hooks(_allocate, _current_stream)


def plan_cache_stats():
    """(hits, misses, size) of the kernel-plan cache of the operator layer."""
    return tuple(_C._plan_cache_stats())


# ---- operators ---------------------------------------------------------------------------------------
def grouped_matmul(x, weight, group_list, bias=None, scale=None, per_token_scale=None, antiquant_scale=None,
                   transpose_a=False, transpose_b=False, x_format=0, output_dtype=None):
    """Grouped matmul; see the module docstring.  ``output_dtype`` (None = float16 as in the reference,
    or torch.bfloat16) is an optional trailing extension."""
    od = dtype_to_type_id(output_dtype)
    if _mode == GRAPH_MODE:
        args = [_wrap(x), _wrap(weight), _wrap(group_list), _wrap(bias), _wrap(scale), _wrap(per_token_scale),
                _wrap(antiquant_scale), bool(transpose_a), bool(transpose_b), int(x_format), od]
        return _C._graph_run("grouped_matmul", args)[0].owner
    return _C.grouped_matmul(_wrap(x), _wrap(weight), _wrap(group_list), _wrap(bias), _wrap(scale),
                             _wrap(per_token_scale), _wrap(antiquant_scale), bool(transpose_a), bool(transpose_b),
                             int(x_format), od).owner


def grouped_matmul_v4_cops(x, weight, bias=None, scale=None, offset=None, antiquant_scale=None, antiquant_offset=None,
                           per_token_scale=None, group_list=None, activation_input=None, activation_quant_scale=None,
                           activation_quant_offset=None, split_item=0, group_type=-1, group_list_type=0, act_type=0,
                           weight_format="ND", output_dtype=None) -> List[torch.Tensor]:
    """List-of-tensor grouped matmul (GMM V4); returns a list of tensors."""
    od = dtype_to_type_id(output_dtype)
    lists = [_wrap_list(v) for v in (x, weight, bias, scale, offset, antiquant_scale, antiquant_offset,
                                     per_token_scale)]
    acts = [_wrap_list(v) for v in (activation_input, activation_quant_scale, activation_quant_offset)]
    gl = _wrap(group_list)
    if _mode == GRAPH_MODE:
        args = lists + [gl] + acts + [int(split_item), int(group_type), int(group_list_type), int(act_type),
                                      str(weight_format), od]
        outs = _C._graph_run("grouped_matmul_v4_cops", args)
    else:
        outs = _C.grouped_matmul_v4_cops(*lists, gl, *acts, int(split_item), int(group_type), int(group_list_type),
                                         int(act_type), str(weight_format), od)
    return [o.owner for o in outs]


def quant_batch_matmul(x1, x2, scale, offset=None, bias=None, pertoken_scale=None, transpose_x1=False,
                       transpose_x2=False, x2_format="ND", output_dtype=torch.float16):
    """Dense / batched W8A8 matmul with dequant epilogue."""
    od = dtype_to_type_id(output_dtype)
    if _mode == GRAPH_MODE:
        args = [_wrap(x1), _wrap(x2), _wrap(scale), _wrap(offset), _wrap(bias), _wrap(pertoken_scale),
                bool(transpose_x1), bool(transpose_x2), str(x2_format), od]
        return _C._graph_run("quant_batch_matmul", args)[0].owner
    return _C.quant_batch_matmul(_wrap(x1), _wrap(x2), _wrap(scale), _wrap(offset), _wrap(bias), _wrap(pertoken_scale),
                                 bool(transpose_x1), bool(transpose_x2), str(x2_format), od).owner


def grouped_matmul_w4(x, weight, group_list, bias, x_scale, weight_scale):
    """Grouped matmul of int8 activations with int4 weights (ops/c_api/grouped_matmul_w4/grouped_matmul_w4.cc:254-255;
    golden tests/st/test_grouped_matmul_w4.py:100-113): out[m] = x_scale[m] * sum over K groups g of
    weight_scale[e, g] * (x[m, K group g] @ w[e, K group g]) for the expert e of row m, float16 [m, n].
    x int8 [m, k]; weight [e, n, k/2], two signed 4-bit values per byte (even k in the low nibble), as an int8 or uint8
    tensor (torch has no 4-bit type); group_list int32 [e], cumulative; bias float32 [e, n] (the reference kernel's
    compensation term 8 * column sums of the dequantised weight: checked, not read, the nibbles are multiplied signed
    here); x_scale float32 [m]; weight_scale float32 [e, k/group_size, n]."""
    args = [_wrap(x), _wrap(weight), _wrap(group_list), _wrap(bias), _wrap(x_scale), _wrap(weight_scale)]
    if _mode == GRAPH_MODE:
        return _C._graph_run("grouped_matmul_w4", args)[0].owner
    return _C.grouped_matmul_w4(*args).owner


def moe_init_routing_v2(x, expert_idx, active_num, expert_capacity, expert_num, drop_pad_mode,
                        expert_tokens_count_or_cumsum_flag, expert_tokens_before_capacity_flag):
    """Dropless MoE routing in front of the grouped matmul (ops/c_api/moe_init_routing_v2/moe_init_routing_v2.cc:238-242):
    returns (expanded_x, expanded_row_idx, expert_tokens_count_or_cumsum, expert_tokens_before_capacity)."""
    if _mode == GRAPH_MODE:
        args = [_wrap(x), _wrap(expert_idx), int(active_num), int(expert_capacity), int(expert_num), int(drop_pad_mode),
                int(expert_tokens_count_or_cumsum_flag), bool(expert_tokens_before_capacity_flag)]
        outs = _C._graph_run("moe_init_routing_v2", args)
    else:
        outs = _C.moe_init_routing_v2(_wrap(x), _wrap(expert_idx), int(active_num), int(expert_capacity), int(expert_num),
                                      int(drop_pad_mode), int(expert_tokens_count_or_cumsum_flag),
                                      bool(expert_tokens_before_capacity_flag))
    return tuple(o.owner for o in outs)


def moe_init_routing_quant(x, expert_idx, expert_num, expert_tokens_count_or_cumsum_flag=1):
    """moe_init_routing_v2's dropless routing with the activations quantised to int8 per token on the way, for an
    int8-activation grouped matmul behind it.  The reference has no operator for the pair; the arithmetic per gathered row
    is the dynamic quantisation its test applies to such activations (tests/st/test_grouped_matmul_w4.py:83-89):
    scale = float32(max |row|) / 127, q = int8(round(float32(row) / scale)).
    x float16 or bfloat16 [rows, hidden] (hidden a multiple of 8), expert_idx int32 [rows, k].
    Returns (expanded_x int8 [rows*k, hidden], expanded_scale float32 [rows*k], expanded_row_idx, expert_tokens_count_or_cumsum):
    x, per_token_scale and (flag 1) group_list of grouped_matmul_v4_cops."""
    if _mode == GRAPH_MODE:
        outs = _C._graph_run("moe_init_routing_quant", [_wrap(x), _wrap(expert_idx), int(expert_num),
                                                        int(expert_tokens_count_or_cumsum_flag)])
    else:
        outs = _C.moe_init_routing_quant(_wrap(x), _wrap(expert_idx), int(expert_num), int(expert_tokens_count_or_cumsum_flag))
    return tuple(o.owner for o in outs)


def moe_token_unpermute(permuted_tokens, sorted_indices, probs, padded_mode=False, restore_shape=None):
    """Weighted un-permutation behind the grouped matmul
    (ops/c_api/moe_token_unpermute/moe_token_unpermute.cc:152-156): out[i] = sum_k probs[i, k] * permuted_tokens[sorted_indices[i*K + k]]."""
    if _mode == GRAPH_MODE:
        args = [_wrap(permuted_tokens), _wrap(sorted_indices), _wrap(probs), bool(padded_mode),
                None if restore_shape is None else str(tuple(restore_shape))]
        return _C._graph_run("moe_token_unpermute", args)[0].owner
    return _C.moe_token_unpermute(_wrap(permuted_tokens), _wrap(sorted_indices), _wrap(probs), bool(padded_mode),
                                  None if restore_shape is None else [int(v) for v in restore_shape]).owner


def trans_data(tensor, transdata_type=1, nd_shape=None, transposed=False):
    """Weight prepack, once at load time (ops/c_api/trans_data/trans_data.cc:203-223; the reference converts weights to the
    device's blocked FRACTAL_NZ format before grouped_matmul, tests/st/test_grouped_matmul.py:131-133, and
    grouped_matmul_v4_cops takes them with weight_format="FRACTAL_NZ", tests/st/test_grouped_matmul_v4_cops.py:514-519).

    transdata_type 1 (ND_TO_FRACTAL_NZ): an int8 weight [E, K, N] (or [K, N]) on the GPU becomes an int8 tensor
    [E, N/16, ceil(K/64), 1024] (or [N/16, ceil(K/64), 1024]) in this backend's blocked layout; N must be a multiple
    of 16.  `grouped_matmul` recognises such a tensor by its shape, `grouped_matmul_v4_cops` takes it with
    weight_format="FRACTAL_NZ".  Decode shapes stream it at the rate of a contiguous read.  The blocked layout is
    defined on (k, n), not on rows and columns of whatever was stored: a weight kept as [E, N, K] (what transpose_b=True
    describes) is packed with transposed=True, and the packed tensor is then passed with transpose_b=False.
    transdata_type 0 (FRACTAL_NZ_TO_ND): the inverse; a torch tensor carries no logical shape besides its own, so
    `nd_shape` ([E, K, N] or [K, N]) says what to cut the zero padding back to (default: the padded shape);
    transposed=True returns [E, N, K].
    Tensors of other dtypes are returned unchanged: only int8 weights have a blocked form here."""
    if transdata_type not in (0, 1):
        raise ValueError("transdata_type must be 0 (FRACTAL_NZ_TO_ND) or 1 (ND_TO_FRACTAL_NZ)")
    if not isinstance(tensor, torch.Tensor) or tensor.dtype != torch.int8:
        return tensor
    from . import cabi
    if transdata_type == 1:
        if tensor.dim() not in (2, 3):
            raise ValueError(f"For TransData, an int8 weight must be [K, N] or [E, K, N], but got {tuple(tensor.shape)}")
        if not tensor.is_cuda:
            raise RuntimeError("For TransData, the input must be on the GPU (the operators have no CPU path)")
        w = tensor.contiguous()
        lead = (w.shape[0],) if w.dim() == 3 else ()
        e = w.shape[0] if w.dim() == 3 else 1
        k, n = (int(w.shape[-1]), int(w.shape[-2])) if transposed else (int(w.shape[-2]), int(w.shape[-1]))
        if n % 16 != 0:
            raise ValueError(f"For TransData, the N dimension must be aligned to 16, but got {n}")
        out = torch.empty(lead + (n // 16, (k + 63) // 64, 1024), dtype=torch.int8, device=w.device)
        with torch.cuda.device(w.device):
            cabi.pack_weight(w.data_ptr(), out.data_ptr(), e, k, n, bool(transposed), torch.cuda.current_stream().cuda_stream)
        return out
    if tensor.dim() not in (3, 4) or tensor.shape[-1] != 1024:
        raise ValueError("For TransData, FRACTAL_NZ_TO_ND takes a tensor made by ND_TO_FRACTAL_NZ "
                         f"([E, N/16, ceil(K/64), 1024] or [N/16, ceil(K/64), 1024]), but got {tuple(tensor.shape)}")
    lead = tuple(tensor.shape[:-3])
    ng, kb = int(tensor.shape[-3]), int(tensor.shape[-2])
    # byte 16 l + i of block (a, b): k = 64 b + 16 (l // 16) + i, n = 16 a + (l % 16)  ->  [.., a, b, q, c, i] -> [.., b, q, i, a, c]
    d = len(lead)
    v = tensor.contiguous().view(lead + (ng, kb, 4, 16, 16))
    nd = v.permute(*range(d), d + 1, d + 2, d + 4, d + 0, d + 3).reshape(lead + (kb * 64, ng * 16))
    if nd_shape is not None:
        nd = nd[..., :int(nd_shape[-2]), :int(nd_shape[-1])]
    return (nd.transpose(-1, -2) if transposed else nd).contiguous()
