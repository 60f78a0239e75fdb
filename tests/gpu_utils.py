"""Helpers shared by the GPU parity tests: run the backend through its C ABI on numpy inputs."""
import numpy as np
import torch

from ms_custom_ops_amd import cabi

_NP2DT = {np.dtype(np.int32): cabi.DT_I32, np.dtype(np.int64): cabi.DT_I64}


def to_dev(a, device="cuda:0"):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:  # bf16 / f16 bit patterns travel as int16
        return torch.from_numpy(a.view(np.int16)).to(device)
    return torch.from_numpy(a).to(device)


def ptr(t):
    return None if t is None else t.data_ptr()


def pack_on_device(tw, e, k, n, src_transposed=False):
    """Row-major device weights ([e,k,n], or [e,n,k] when src_transposed) -> packed layout, through msco_pack_weight."""
    dst = torch.empty(e * cabi.packed_weight_bytes(k, n), dtype=torch.int8, device=tw.device)
    cabi.pack_weight(tw.data_ptr(), dst.data_ptr(), e, k, n, src_transposed, torch.cuda.current_stream().cuda_stream)
    return dst


def run_w8a8(x, w, group_list, bias=None, scale=None, per_token=None, *, out="bf16", transpose_b=False, override=0,
             group_list_type=0, gl_dtype=np.int64, scale_dtype=cabi.DT_F32, scale_per_group=1, scale_is_scalar=0,
             launches=1, poison=True, packed=False, act_type=0, force_split_k=0):
    """x int8 [M,K]; w int8 [E,K,N] in logical layout (transposed here when transpose_b; with `packed` that row-major
    tensor is then packed on the device and the op reads the packed layout).  Returns (numpy output, plan info)."""
    m, k = x.shape
    e, _, n = w.shape
    wd = np.ascontiguousarray(w.transpose(0, 2, 1)) if transpose_b else w
    out_dt = {"bf16": cabi.DT_BF16, "f16": cabi.DT_F16, "i32": cabi.DT_I32}[out]
    raw = out == "i32"
    tx, tw, tb = to_dev(x), to_dev(wd), to_dev(bias)
    if packed:
        tw = pack_on_device(tw, e, k, n, transpose_b)
    ts = None if (raw or scale is None) else to_dev(scale)
    tp = None if (raw or per_token is None) else to_dev(per_token)
    tg = None if group_list is None else to_dev(np.asarray(group_list).astype(gl_dtype))
    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=out_dt,
                    group_list_dtype=cabi.DT_NONE if tg is None else _NP2DT[np.dtype(gl_dtype)],
                    group_list_type=group_list_type, bias_dtype=cabi.DT_I32 if tb is not None else cabi.DT_NONE,
                    scale_dtype=scale_dtype if ts is not None else cabi.DT_NONE,
                    per_token_dtype=cabi.DT_F32 if tp is not None else cabi.DT_NONE,
                    transpose_b=0 if packed else int(transpose_b), weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR,
                    scale_per_group=scale_per_group, scale_is_scalar=scale_is_scalar, kernel_override=override,
                    act_type=act_type, force_split_k=force_split_k)
    ws = op.plan(m, k, n, e)
    tws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda:0")
    fill = -7777 if raw else 0x7FC0  # poison: a value no correct run produces (bf16/f16 NaN pattern)
    tout = torch.full((m, n), fill if poison else 0, dtype=torch.int32 if raw else torch.int16, device="cuda:0")
    ins = [ptr(tx), ptr(tw), ptr(tb), ptr(ts), ptr(tg), ptr(tp), None, None]
    for _ in range(launches):
        op.launch(ins, tout.data_ptr(), tws.data_ptr(), ws, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    info = op.plan_info()
    op.close()
    res = tout.cpu().numpy()
    return (res if raw else res.view(np.uint16)), info


def run_a16w8(x_bits, w, scale_bits, offset_bits, group_list, *, dtype="bf16", override=0, group_list_type=0, packed=False,
              act_type=0):
    m, k = x_bits.shape
    e, _, n = w.shape
    dt = cabi.DT_BF16 if dtype == "bf16" else cabi.DT_F16
    tx, tw, ts, to = to_dev(x_bits), to_dev(w), to_dev(scale_bits), to_dev(offset_bits)
    tg = to_dev(np.asarray(group_list).astype(np.int64))
    if packed:
        tw = pack_on_device(tw, e, k, n)
    op = cabi.GmmOp(x_dtype=dt, out_dtype=dt, group_list_dtype=cabi.DT_I64, group_list_type=group_list_type,
                    antiquant_dtype=dt, has_antiquant_offset=int(to is not None), kernel_override=override, act_type=act_type,
                    weight_layout=cabi.WL_PACKED if packed else cabi.WL_ROW_MAJOR)
    ws = op.plan(m, k, n, e)
    tws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda:0")
    tout = torch.full((m, n), 0x7FC0, dtype=torch.int16, device="cuda:0")
    ins = [ptr(tx), ptr(tw), None, None, ptr(tg), None, ptr(ts), ptr(to)]
    op.launch(ins, tout.data_ptr(), tws.data_ptr(), ws, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    info = op.plan_info()
    op.close()
    return tout.cpu().numpy().view(np.uint16), info
