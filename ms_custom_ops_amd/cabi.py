"""ctypes binding of the backend's C ABI (include/msco_gmm.h).

This is the thinnest possible host: it loads libmsco_gmm.so, mirrors ``msco_gmm_desc`` and hands
raw device pointers to the library.  Tests and the benchmark use it to call the backend exactly the
way a foreign-language binding would; the operator layer proper is the pybind11 module.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
# MSCO_GMM_LIB selects another build of the backend library (used to compare kernel versions side by side)
LIB_PATH = os.environ.get("MSCO_GMM_LIB") or os.path.join(_HERE, "lib", "libmsco_gmm.so")

ABI_VERSION = 1

# msco_dtype
DT_NONE, DT_I8, DT_I32, DT_I64, DT_U64, DT_F16, DT_BF16, DT_F32 = range(8)

# positional launch inputs
IN_X, IN_WEIGHT, IN_BIAS, IN_SCALE, IN_GROUP_LIST, IN_PER_TOKEN_SCALE, IN_ANTIQUANT_SCALE, IN_ANTIQUANT_OFFSET = range(8)
IN_COUNT = 8

# msco_gmm_desc.kernel_override
OV_AUTO, OV_TILE_256, OV_TILE_128, OV_TILE_64, OV_SKINNY, OV_GENERIC, OV_TILE_256_W4, OV_TILE_128x256, OV_TILE_256_W4_MFMA32, OV_ROWS128, OV_ROWS256, OV_ROWS160 = range(12)

# msco_gmm_desc.act_type
ACT_NONE, ACT_RELU, ACT_GELU_TANH, ACT_GELU_ERF, ACT_FAST_GELU, ACT_SILU = range(6)

# msco_gmm_desc.weight_layout
WL_ROW_MAJOR, WL_PACKED = 0, 1

EXPORTED_SYMBOLS = ("msco_gmm_create", "msco_gmm_plan", "msco_gmm_launch", "msco_gmm_plan_info", "msco_gmm_destroy",
                    "msco_status_string", "msco_gmm_abi_version", "msco_transpose_2d",
                    "msco_packed_weight_bytes", "msco_pack_weight", "msco_gmm_a8w4", "msco_unpack_int4",
                    "msco_moe_init_routing_v2_workspace_bytes", "msco_moe_init_routing_v2", "msco_moe_init_routing_v2_quant",
                    "msco_moe_token_unpermute", "msco_gmm_launch_static")
PROBE_SYMBOLS = ("msco_probe_mfma_issue", "msco_probe_read")   # libmsco_probes.so, include/msco_probes.h
STATIC_WORKSPACE_BYTES = 32 << 20
PROBE_MFMA_WORKGROUPS, PROBE_MFMA_OPERAND_BYTES = 256, 8 * 256 * 16


class GmmDesc(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int32) for name in (
        "abi_version", "x_dtype", "weight_dtype", "out_dtype", "group_list_dtype", "group_list_type", "bias_dtype",
        "scale_dtype", "per_token_dtype", "antiquant_dtype", "has_antiquant_offset", "transpose_b", "scale_per_group",
        "scale_is_scalar", "kernel_override", "weight_layout", "act_type", "force_split_k")] + [("reserved", ctypes.c_int32 * 2)]


class BackendError(RuntimeError):
    def __init__(self, where: str, status: int, text: str):
        super().__init__(f"{where} failed: status {status} ({text})")
        self.status = status


_lib = None


_probes = None
PROBES_LIB_PATH = os.path.join(_HERE, "lib", "libmsco_probes.so")


def load_probes():
    """Load the library of measurement aids (the benchmark's yardstick kernels; the operators never need it)."""
    global _probes
    if _probes is None:
        if not os.path.exists(PROBES_LIB_PATH):
            raise ImportError(f"probe library missing: {PROBES_LIB_PATH}; build it with `python ms_custom_ops_amd/build.py`")
        lib = ctypes.CDLL(PROBES_LIB_PATH)
        lib.msco_probe_read.restype = ctypes.c_int
        lib.msco_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p]
        lib.msco_probe_mfma_issue.restype = ctypes.c_int
        lib.msco_probe_mfma_issue.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
        _probes = lib
    return _probes


def load():
    """Load the backend library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"HIP backend library missing: {LIB_PATH}; build it with "
                              "`python ms_custom_ops_amd/build.py`")
        lib = ctypes.CDLL(LIB_PATH)
        lib.msco_gmm_create.restype = ctypes.c_int
        lib.msco_gmm_create.argtypes = [ctypes.POINTER(GmmDesc), ctypes.POINTER(ctypes.c_void_p)]
        lib.msco_gmm_plan.restype = ctypes.c_int
        lib.msco_gmm_plan.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                      ctypes.POINTER(ctypes.c_size_t)]
        lib.msco_gmm_launch.restype = ctypes.c_int
        lib.msco_gmm_launch.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                                        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        lib.msco_gmm_plan_info.restype = ctypes.c_int
        lib.msco_gmm_plan_info.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]
        lib.msco_gmm_destroy.restype = ctypes.c_int
        lib.msco_gmm_destroy.argtypes = [ctypes.c_void_p]
        lib.msco_status_string.restype = ctypes.c_char_p
        lib.msco_status_string.argtypes = [ctypes.c_int]
        lib.msco_gmm_abi_version.restype = ctypes.c_int
        lib.msco_gmm_abi_version.argtypes = []
        lib.msco_transpose_2d.restype = ctypes.c_int
        lib.msco_transpose_2d.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                          ctypes.c_int32, ctypes.c_void_p]
        lib.msco_packed_weight_bytes.restype = ctypes.c_size_t
        lib.msco_packed_weight_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64]
        lib.msco_pack_weight.restype = ctypes.c_int
        lib.msco_pack_weight.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_int32, ctypes.c_void_p]
        lib.msco_moe_init_routing_v2_workspace_bytes.restype = ctypes.c_size_t
        lib.msco_moe_init_routing_v2_workspace_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
        lib.msco_moe_init_routing_v2.restype = ctypes.c_int
        lib.msco_moe_init_routing_v2.argtypes = [ctypes.c_void_p] * 7 + [ctypes.c_size_t] + [ctypes.c_int64] * 4 + \
                                                [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
        lib.msco_unpack_int4.restype = ctypes.c_int
        lib.msco_unpack_int4.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        lib.msco_gmm_a8w4.restype = ctypes.c_int
        lib.msco_gmm_a8w4.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 5 + [ctypes.c_void_p]
        lib.msco_moe_init_routing_v2_quant.restype = ctypes.c_int
        lib.msco_moe_init_routing_v2_quant.argtypes = [ctypes.c_void_p] * 8 + [ctypes.c_size_t] + [ctypes.c_int64] * 4 + \
            [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
        lib.msco_moe_token_unpermute.restype = ctypes.c_int
        lib.msco_moe_token_unpermute.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int64] * 3 + [ctypes.c_int32, ctypes.c_void_p]
        lib.msco_gmm_launch_static.restype = ctypes.c_int
        lib.msco_gmm_launch_static.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p]
        _lib = lib
    return _lib


def status_string(status: int) -> str:
    return load().msco_status_string(int(status)).decode()


def _check(where: str, status: int):
    if status != 0:
        raise BackendError(where, status, status_string(status))


def transpose_2d(src: int, dst: int, batch: int, rows: int, cols: int, elem_bytes: int, stream: Optional[int] = None):
    """src [batch, rows, cols] -> dst [batch, cols, rows] on the device (the weight prepack: [E,K,N] -> [E,N,K])."""
    _check("msco_transpose_2d", load().msco_transpose_2d(ctypes.c_void_p(src), ctypes.c_void_p(dst), batch, rows, cols,
                                                         elem_bytes, ctypes.c_void_p(stream if stream else None)))


def packed_weight_bytes(k: int, n: int) -> int:
    """Bytes of one group's K x N int8 weights in the packed layout."""
    return int(load().msco_packed_weight_bytes(k, n))


def pack_weight(src: int, dst: int, e: int, k: int, n: int, src_transposed: bool = False, stream: Optional[int] = None):
    """src [e,k,n] int8 (or [e,n,k] when src_transposed) -> dst, e * packed_weight_bytes(k, n) bytes in the packed
    layout that GmmOp(weight_layout=WL_PACKED) reads."""
    _check("msco_pack_weight", load().msco_pack_weight(ctypes.c_void_p(src), ctypes.c_void_p(dst), e, k, n,
                                                       int(bool(src_transposed)), ctypes.c_void_p(stream if stream else None)))


def gmm_a8w4(x: int, weight: int, group_list: int, x_scale: int, weight_scale: int, out: int, m: int, k: int, n: int, e: int,
             group_size: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_gmm_a8w4 (see include/msco_gmm.h)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_gmm_a8w4", load().msco_gmm_a8w4(vp(x), vp(weight), vp(group_list), vp(x_scale), vp(weight_scale), vp(out),
                                                 m, k, n, e, group_size, vp(stream)))


def unpack_int4(src: int, dst: int, src_bytes: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_unpack_int4 (see include/msco_gmm.h): src_bytes bytes of nibble pairs -> 2 * src_bytes int8."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_unpack_int4", load().msco_unpack_int4(vp(src), vp(dst), src_bytes, vp(stream)))


def probe_mfma_issue(operands: int, sink: int, clocks: int, pattern: int, iters: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_probe_mfma_issue (see include/msco_probes.h): `pattern` names the memory operations woven
    into rounds of 64 (32) MFMAs, PROBE_MFMA_WORKGROUPS * 4 * iters * 2 ** 21 int8 operations per launch; `clocks` receives
    two int64 (core clocks, 100 MHz ticks of the loop)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_probe_mfma_issue", load_probes().msco_probe_mfma_issue(vp(operands), vp(sink), vp(clocks), pattern, iters, vp(stream)))


def probe_read(src: int, nbytes: int, sink: int, workgroups: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_probe_read (see include/msco_probes.h)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_probe_read", load_probes().msco_probe_read(vp(src), nbytes, vp(sink), workgroups, vp(stream)))


def moe_init_routing_v2_workspace_bytes(num_rows: int, k: int, expert_num: int) -> int:
    return int(load().msco_moe_init_routing_v2_workspace_bytes(num_rows, k, expert_num))


def moe_init_routing_v2(x: int, expert_idx: int, expanded_x: int, expanded_row_idx: int, tokens: Optional[int],
                        before_capacity: Optional[int], workspace: int, workspace_bytes: int, num_rows: int, hidden: int,
                        k: int, expert_num: int, elem_bytes: int, flag: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_moe_init_routing_v2 (see include/msco_moe.h)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_moe_init_routing_v2", load().msco_moe_init_routing_v2(
        vp(x), vp(expert_idx), vp(expanded_x), vp(expanded_row_idx), vp(tokens), vp(before_capacity), vp(workspace),
        workspace_bytes, num_rows, hidden, k, expert_num, elem_bytes, flag, vp(stream)))


def moe_init_routing_v2_quant(x: int, expert_idx: int, expanded_x: int, expanded_scale: int, expanded_row_idx: int,
                              tokens: Optional[int], before_capacity: Optional[int], workspace: int, workspace_bytes: int,
                              num_rows: int, hidden: int, k: int, expert_num: int, x_dtype: int, flag: int,
                              stream: Optional[int] = None):
    """Raw-pointer call of msco_moe_init_routing_v2_quant (see include/msco_moe.h)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_moe_init_routing_v2_quant", load().msco_moe_init_routing_v2_quant(
        vp(x), vp(expert_idx), vp(expanded_x), vp(expanded_scale), vp(expanded_row_idx), vp(tokens), vp(before_capacity),
        vp(workspace), workspace_bytes, num_rows, hidden, k, expert_num, x_dtype, flag, vp(stream)))


def moe_token_unpermute(permuted: int, sorted_indices: int, probs: int, out: int, num_tokens: int, top_k: int, hidden: int,
                        dtype: int, stream: Optional[int] = None):
    """Raw-pointer call of msco_moe_token_unpermute (see include/msco_moe.h)."""
    vp = lambda v: ctypes.c_void_p(v if v else None)
    _check("msco_moe_token_unpermute", load().msco_moe_token_unpermute(vp(permuted), vp(sorted_indices), vp(probs), vp(out),
                                                                       num_tokens, top_k, hidden, dtype, vp(stream)))


class GmmOp:
    """One backend operator instance: create -> plan -> launch* -> destroy."""

    def __init__(self, **fields):
        lib = load()
        desc = GmmDesc()
        desc.abi_version = ABI_VERSION
        desc.weight_dtype = DT_I8
        desc.scale_per_group = 1
        for key, value in fields.items():
            if not hasattr(desc, key):
                raise AttributeError(key)
            setattr(desc, key, int(value))
        self.desc = desc
        self._h = ctypes.c_void_p()
        _check("msco_gmm_create", lib.msco_gmm_create(ctypes.byref(desc), ctypes.byref(self._h)))
        self.workspace_bytes = 0

    def plan(self, m: int, k: int, n: int, e: int) -> int:
        ws = ctypes.c_size_t(0)
        _check("msco_gmm_plan", load().msco_gmm_plan(self._h, m, k, n, e, ctypes.byref(ws)))
        self.workspace_bytes = int(ws.value)
        return self.workspace_bytes

    def plan_info(self) -> str:
        buf = ctypes.create_string_buffer(512)
        load().msco_gmm_plan_info(self._h, buf, 512)
        return buf.value.decode()

    def launch(self, inputs: Sequence[Optional[int]], out: int, workspace: Optional[int] = None,
               workspace_bytes: int = 0, stream: Optional[int] = None):
        """inputs: IN_COUNT device addresses (None/0 = absent)."""
        arr = (ctypes.c_void_p * IN_COUNT)()
        for i in range(IN_COUNT):
            v = inputs[i] if i < len(inputs) else None
            arr[i] = ctypes.c_void_p(v if v else None)
        _check("msco_gmm_launch", load().msco_gmm_launch(self._h, arr, ctypes.c_void_p(out),
                                                         ctypes.c_void_p(workspace if workspace else None),
                                                         workspace_bytes, ctypes.c_void_p(stream if stream else None)))

    def launch_static(self, inputs: Sequence[Optional[int]], out: int, stream: Optional[int] = None):
        """msco_gmm_launch_static: the launch that takes its split-K workspace from the library's fixed device array."""
        arr = (ctypes.c_void_p * IN_COUNT)()
        for i in range(IN_COUNT):
            v = inputs[i] if i < len(inputs) else None
            arr[i] = ctypes.c_void_p(v if v else None)
        _check("msco_gmm_launch_static", load().msco_gmm_launch_static(self._h, arr, ctypes.c_void_p(out),
                                                                       ctypes.c_void_p(stream if stream else None)))

    def close(self):
        if self._h:
            load().msco_gmm_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass
