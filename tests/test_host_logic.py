"""CPU-side tests: the C ABI library loads and exports what include/msco_gmm.h declares, status
codes, shape / dtype inference and error messages of the operator layer, prototype/pybind parity,
workload generators.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import yaml

import ms_custom_ops_amd as mco
from ms_custom_ops_amd import cabi, workloads

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_C = mco._C


def fake(shape, dtype_id, strides=None):
    """A tensor view with no memory behind it: enough for inference, which never dereferences."""
    shape = list(shape)
    if strides is None:
        strides, acc = [], 1
        for d in reversed(shape):
            strides.insert(0, acc)
            acc *= d
    return _C.Tensor(0x1000, dtype_id, shape, strides, None)


I8, I32, I64, U64, F16, F32, BF16 = 32, 34, 35, 40, 42, 43, 45


# ------------------------------------------------------------------------------------- C ABI surface
def test_header_symbols_are_exported():
    declared, probes = set(), set()
    for name in sorted(os.listdir(os.path.join(REPO, "include"))):   # every header: msco_gmm.h, msco_moe.h, msco_probes.h
        header = open(os.path.join(REPO, "include", name)).read()
        found = set(re.findall(r"MSCO_API\s+[\w\s\*]+?\b(msco_\w+)\s*\(", header))
        if name == "msco_probes.h":
            probes |= found
        else:
            declared |= found
    assert declared == set(cabi.EXPORTED_SYMBOLS) and probes == set(cabi.PROBE_SYMBOLS)
    lib = cabi.load()
    for name in declared:
        assert hasattr(lib, name), name
    for name in probes:   # the measurement aids live in a library of their own; the operator library does not export them
        assert hasattr(cabi.load_probes(), name), name
        assert not hasattr(lib, name), name
    assert lib.msco_gmm_abi_version() == cabi.ABI_VERSION == _C._backend_abi_version()


def test_desc_struct_matches_header_layout():
    header = open(os.path.join(REPO, "include", "msco_gmm.h")).read()
    body = header[header.index("typedef struct msco_gmm_desc {"):header.index("} msco_gmm_desc;")]
    fields = re.findall(r"int32_t\s+(\w+)(?:\[\d+\])?;", body)
    assert fields == [f[0] for f in cabi.GmmDesc._fields_]
    assert ctypes.sizeof(cabi.GmmDesc) == 4 * 20


def test_status_codes_and_argument_checks_without_a_gpu():
    assert cabi.status_string(0) == "ok"
    with pytest.raises(cabi.BackendError) as e:
        cabi.GmmOp(x_dtype=cabi.DT_F32, out_dtype=cabi.DT_BF16)
    assert e.value.status == 2
    with pytest.raises(cabi.BackendError) as e:
        cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, abi_version=99)
    assert e.value.status == 1
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64, scale_dtype=cabi.DT_F32)
    with pytest.raises(cabi.BackendError) as e:   # launch before plan
        op.launch([1, 1, None, 1, 1, None, None, None], 1)
    assert e.value.status == 4
    with pytest.raises(cabi.BackendError) as e:
        op.plan(8, 0, 16, 1)
    assert e.value.status == 3
    op.plan(8192, 4096, 14336, 8)
    assert "tile_256x256" in op.plan_info() and op.workspace_bytes == 0
    with pytest.raises(cabi.BackendError) as e:   # scale promised by the descriptor but not passed
        op.launch([1, 1, None, None, 1, None, None, None], 1)
    assert e.value.status == 1
    op.plan(37, 100, 24, 1)
    assert "generic" in op.plan_info()
    op.plan(40, 4096, 14336, 64)   # enough strips x groups that K is not split (a split plan allocates counters on the device)
    assert "skinny" in op.plan_info() and "split_k=1 " in op.plan_info()
    op.close()
    dense = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, scale_dtype=cabi.DT_F32)
    with pytest.raises(cabi.BackendError) as e:   # equal groups need M % E == 0
        dense.plan(10, 64, 64, 3)
    assert e.value.status == 3


# ------------------------------------------------------------------------------------- grouped_matmul infer
def _gmm_args(x=(64, 64), w=(8, 64, 128), gl=(8,), xt=I8, wt=I8, glt=I32, bias=None, scale=F32, pts=None, aq=None,
              ta=False, tb=False, xf=0, od=None):
    e, n = w[0], (w[1] if tb else w[-1])
    return [fake(x, xt), fake(w, wt), fake(gl, glt), None if bias is None else fake((e, n), bias),
            None if scale is None else fake((e, n), scale), None if pts is None else fake((x[0],), pts),
            None if aq is None else fake((e, w[-2], 1), aq), ta, tb, xf, od]


def test_plan_of_the_serving_range_on_packed_weights_without_a_gpu():
    # shapes only: eight experts, K = 4096, N = 14336 (no device: the plan assumes 256 CUs).  Packed weights take the row-chunk
    # kernels up to about 155 rows per group (chunks of 128 rows up to 116 per group, of 160 up to 146), in strips of 14 column
    # groups (512 workgroups);
    # other layouts and few columns keep the tiles; the forced forms fall back to tiles on row-major weights.
    def plan(m, n=14336, k=4096, e=8, packed=True, override=0):
        op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64, scale_dtype=cabi.DT_F32,
                        per_token_dtype=cabi.DT_F32, weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR,
                        kernel_override=override)
        ws = op.plan(m, k, n, e)
        info = op.plan_info()
        op.close()
        return info, ws
    for m, want in ((128, "tile_rows128"), (896, "tile_rows128"), (8 * 116, "tile_rows128"), (8 * 117, "tile_rows160"), (1024, "tile_rows160"),
                    (8 * 146, "tile_rows160"), (8 * 147, "tile_rows256"), (8 * 155, "tile_rows256"), (8 * 156, "tile_256x256x128_w4"),
                    (2048, "tile_256x256x128_w4"), (64, "w8a8_stream")):
        info, ws = plan(m)
        assert want in info and ws == 0, (m, info)
    assert "strips=64 " in plan(896)[0] and "strips=64 " in plan(1024)[0]
    assert "rows" not in plan(896, packed=False)[0]
    assert "rows" not in plan(1024, n=1344, k=5120)[0]                 # few columns: CUs would idle
    assert "rows" not in plan(896, k=512)[0]
    assert "tile_128x256" in plan(896, packed=False, override=cabi.OV_ROWS128)[0]
    assert "tile_256x256x128_w4" in plan(896, packed=False, override=cabi.OV_ROWS256)[0]
    assert "tile_rows256" in plan(300, n=512, k=256, e=2, override=cabi.OV_ROWS256)[0]
    assert "tile_rows160" in plan(300, n=512, k=256, e=2, override=cabi.OV_ROWS160)[0]


def test_grouped_matmul_infer_shape_and_type():
    shapes, types = _C._graph_infer("grouped_matmul", _gmm_args())
    assert shapes == [[64, 128]] and types == [F16]          # the reference's float16 output
    shapes, types = _C._graph_infer("grouped_matmul", _gmm_args(w=(8, 128, 64), tb=True, od=BF16))
    assert shapes == [[64, 128]] and types == [BF16]


@pytest.mark.parametrize("kwargs,msg", [
    (dict(x=(4, 64, 64)), "input 'x' must be 2D"),
    (dict(w=(64, 128)), "input 'weight' must be 3D"),
    (dict(gl=(8, 1)), "input 'group_list' must be 1D"),
    (dict(w=(8, 96, 128)), "must have the same dimension of 'k'"),
    (dict(x=(64, 48), w=(8, 48, 128)), "K dimension must be aligned to 32 for int8"),
    (dict(w=(8, 64, 120)), "N dimension must be aligned to 16"),
    (dict(w=(6, 64, 128), gl=(6,)), "E dimension (group count) must be aligned to 8"),
])
def test_grouped_matmul_shape_errors(kwargs, msg):
    with pytest.raises(RuntimeError, match=re.escape(msg)):
        _C._graph_infer("grouped_matmul", _gmm_args(**kwargs))


@pytest.mark.parametrize("kwargs,msg", [
    (dict(xt=F32, wt=F32), "input 'x' must be float16 or int8"),
    (dict(wt=F16), "input 'weight' must be the same type as 'x'"),
    (dict(glt=I64), "input 'group_list' must be int32"),
    (dict(bias=F32), "input 'bias' must be one of"),
    (dict(scale=F16), "input 'scale' must be one of"),
    (dict(pts=F16), "input 'per_token_scale' must be one of"),
    (dict(aq=I8), "input 'antiquant_scale' must be one of"),
])
def test_grouped_matmul_dtype_errors(kwargs, msg):
    with pytest.raises(RuntimeError, match=re.escape(msg)):
        _C._graph_infer("grouped_matmul", _gmm_args(**kwargs))


def test_grouped_matmul_output_dtype_extension_is_validated():
    with pytest.raises(ValueError, match="'output_dtype' must be Float16 or BFloat16"):
        _C._graph_infer("grouped_matmul", _gmm_args(od=F32))


# ------------------------------------------------------------------------------------- V4 infer
def _v4_args(x, w, scale=None, gl=None, group_type=0, od=None, split_item=3):
    return [x, w, None, scale, None, None, None, None, gl, None, None, None, split_item, group_type, 0, 0, "ND", od]


def test_v4_output_dtype_rules():
    x, w, gl = [fake((32, 256), I8)], [fake((8, 256, 128), I8)], fake((8,), I64)
    t = lambda **kw: _C._graph_infer("grouped_matmul_v4_cops", _v4_args(x, w, gl=gl, **kw))
    assert t() == ([[32, 128]], [I32])                                   # no scale: raw int32
    assert t(scale=[fake((8, 128), BF16)])[1] == [BF16]                  # bf16 scale -> bf16
    assert t(scale=[fake((8, 128), F32)])[1] == [F16]                    # f32 scale -> f16 (reference rule)
    assert t(scale=[fake((8, 128), F32)], od=BF16)[1] == [BF16]          # explicit output_dtype wins (extension)
    assert t(scale=[fake((8, 128), U64)])[1] == [I8]
    with pytest.raises(ValueError, match="the scale only support"):
        t(scale=[fake((8, 128), F16)])
    xa = [fake((32, 256), BF16)]
    assert _C._graph_infer("grouped_matmul_v4_cops", _v4_args(xa, w, gl=gl))[1] == [BF16]   # weight-only keeps x's dtype


def test_v4_shape_rules():
    x = [fake((2, 3, 16, 256), I8), fake((127, 88), I8)]
    w = [fake((256, 128), I8), fake((88, 64), I8)]
    shapes, _ = _C._graph_infer("grouped_matmul_v4_cops", _v4_args(x, w, group_type=-1, split_item=0))
    assert shapes == [[2, 3, 16, 128], [127, 64]]
    with pytest.raises(ValueError, match="x's size should be equal to weight"):
        _C._graph_infer("grouped_matmul_v4_cops", _v4_args(x, w[:1], group_type=-1, split_item=0))
    with pytest.raises(ValueError, match="the size of x and weight should both be 1"):
        _C._graph_infer("grouped_matmul_v4_cops", _v4_args(x, w, gl=fake((8,), I64), group_type=0))
    with pytest.raises(ValueError, match="group_list's rank must be equal to 1"):
        _C._graph_infer("grouped_matmul_v4_cops", _v4_args(x[1:], [fake((8, 88, 64), I8)], gl=fake((8, 1), I64)))


# ------------------------------------------------------------------------------------- quant_batch_matmul infer
def test_quant_batch_matmul_infer():
    q = lambda x1, x2, t1=False, t2=False, od=None: _C._graph_infer(
        "quant_batch_matmul", [fake(x1, I8), fake(x2, I8), fake((1,), F32), None, None, None, t1, t2, "ND", od])
    assert q((128, 256), (256, 128)) == ([[128, 128]], [F16])           # default output float16 (TypeId 42)
    assert q((2, 128, 256), (2, 256, 64), od=BF16) == ([[2, 128, 64]], [BF16])
    assert q((8, 64, 32), (8, 512, 64), True, True)[0] == [[8, 32, 512]]
    assert q((3, 1, 16, 64), (5, 64, 32))[0] == [[3, 5, 16, 32]]        # broadcast batch dims
    with pytest.raises(RuntimeError, match="the K dimension of 'x1' and 'x2' must be equal"):
        q((16, 64), (32, 16))
    with pytest.raises(RuntimeError, match="batch dimensions must be equal or one of them must be 1"):
        q((3, 16, 64), (5, 64, 32))
    with pytest.raises(RuntimeError, match="should be at least 2"):
        q((64,), (64, 32))


# ------------------------------------------------------------------------------------- registration surface
def test_registry_and_module_surface():
    ops = ("grouped_matmul", "grouped_matmul_v4_cops", "grouped_matmul_w4", "quant_batch_matmul", "moe_init_routing_v2", "moe_init_routing_quant",
           "moe_token_unpermute")
    assert set(_C._registered_graph_ops()) == set(ops)
    for name in ops:
        assert callable(getattr(_C, name)) and callable(getattr(mco, name))
    header = open(os.path.join(REPO, "ms_custom_ops_amd", "csrc", "ops", "framework", "module.h")).read()
    for token in ("REG_GRAPH_MODE_OP", "MS_CUSTOM_OPS_EXTENSION_MODULE", "class ModuleRegistry", "RegisterAll"):
        assert token in header


@pytest.mark.parametrize("op", ["grouped_matmul", "grouped_matmul_v4_cops", "grouped_matmul_w4", "quant_batch_matmul",
                                "moe_init_routing_v2", "moe_init_routing_quant", "moe_token_unpermute"])
def test_yaml_prototype_agrees_with_pybind_signature(op):
    """The prototype and the pybind definition must agree on names, order and defaults
    (the reference's rule, docs/ops_develop_guide.md:378)."""
    proto = yaml.safe_load(open(os.path.join(REPO, "ms_custom_ops_amd", "csrc", "ops", "c_api", "op_prototypes.yaml")))[op]
    args = [a.split("=", 1) for a in proto["args"]]
    names = [a[0] for a in args]
    doc = getattr(_C, op).__doc__
    sig = doc[doc.index("(") + 1:doc.index(") ->")]
    got = [a.split(":")[0].strip() for a in re.split(r",\s*(?=\w+:)", sig)]
    assert got == names
    for a in args:
        name = a[0]
        m = re.search(r"\b%s: [^=,]+? = ([^,]+?)(?:,|$)" % name, sig)
        if len(a) == 1:
            assert m is None, name
            continue
        want = a[1].strip("'\"").replace("mstype.float16", "42")
        have = m.group(1).strip().strip("'\"")
        assert have.lower() == want.lower(), (name, have, want)
    assert len(proto["returns"]) >= 1


def test_cpu_tensors_and_noncontiguous_inputs_are_rejected():
    import torch
    with pytest.raises(ValueError, match="take GPU tensors"):
        mco.quant_batch_matmul(torch.zeros(4, 32, dtype=torch.int8), torch.zeros(32, 16, dtype=torch.int8),
                               torch.ones(1))
    t = fake((8, 16), I8, strides=[1, 8])
    assert not t.is_contiguous() and fake((8, 16), I8).is_contiguous()


# ------------------------------------------------------------------------------------- workloads
def test_workloads_are_deterministic_and_shaped_as_specified():
    a, b = workloads.make("c4", scale_down=8), workloads.make("c4", scale_down=8)
    assert np.array_equal(a.x, b.x) and np.array_equal(a.group_list, b.group_list)
    c3 = workloads.make("c3", scale_down=8)
    assert c3.x.shape == (1024, 512) and c3.w.shape == (8, 512, 1792) and c3.group_list[-1] == 1024
    assert (np.diff(c3.group_list) >= 0).all() and c3.x.min() >= -127 and c3.x.max() <= 127
    c5 = workloads.make("c5", scale_down=8)
    assert c5.kind == "a16w8" and c5.x.dtype == np.uint16 and c5.m == 32 and c5.group_list[-1] == 32
    full = workloads.make("c4", scale_down=8)
    counts = np.diff(np.concatenate([[0], full.group_list]))
    assert (counts == 0).any() and counts.max() > 2 * counts.mean()       # Zipf skew: empty and oversized groups
    work = workloads.algorithmic_work(workloads.make("c1"))
    assert work["ops"] == 2.0 * 128 * 4096 * 4096 and abs(work["bytes"] - 18.4e6) < 0.3e6
