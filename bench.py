#!/usr/bin/env python3
"""Benchmark of the grouped W8A8 matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--layout packed|nk|kn] [--no-sweep] [--no-cpu]
    python bench.py --probe c3|c2_m16|...|copy|moe|mfma|issue|read|plan [--layout packed|nk|kn] [--steps K]     (for rocprofv3 counter runs;
                                                            `plan`: the planner's picks against forced kernel families)

A step is one pass of the hot path over one batch of synthetic input (inputs resident in HBM before
the timed region).  The headline workload is the Mixtral-shaped MoE configuration (E=8, top-2 over
4096 tokens = 8192 rows, K=4096, N=14336); `value` is its int8 throughput.  The weights are generated
[E,K,N] as the configuration states and prepacked once, on the device, to the backend's blocked layout
(msco_pack_weight; the reference prepacks weights too, to its FRACTAL_NZ format, before the op runs); the
prepack is outside the timed region and its duration is reported as `prepack_ms`.  `--layout nk` times the op
on weights transposed once to [E,N,K], `--layout kn` on the unpacked [E,K,N] weights; the sweep always carries
all three.
Prints ONE JSON line.  Besides the contract keys it carries
  roofline      the dominant kernel's achieved algorithmic rate against the MI355X peak,
  cpu_baseline  the numpy restatement of the reference golden timed on this box's host cores,
  sweep         the other configurations (dense decode / prefill sweep, skewed MoE, weight-only decode, serving sizes,
                the reference's own timing shapes) per weight layout, one row each under `columns`: launch period and
                the int8 / HBM roofline fractions (TOP/s = int8_frac x 5000, GB/s = hbm_frac x 8000).
`mfma_pipe` (and `--probe mfma`) is a yardstick: loops of nothing but int8 MFMAs, either instruction shape, on random and on zero operands;
`--probe issue` times the same loops with the K loop's memory operations woven in at different places.
--probe runs a few untimed launches of one workload (or, for `copy`, of a plain device-to-device copy
of COPY_BYTES bytes, the reference a counter reading is scaled by) so that a profiler sees nothing else.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s
ROTATE_BYTES = 768e6      # HBM-bound cases rotate over weight copies totalling more than the 256 MB Infinity Cache
LAYOUT_TEXT = {"nk": "prepacked once to [E,N,K]", "kn": "[E,K,N] as generated",
               "packed": "prepacked once to the blocked layout"}
WARM_MIN_LAUNCHES, WARM_MIN_MS, WARM_MAX_MS, WARM_TOLERANCE = 60, 30.0, 1500.0, 0.01
COPY_BYTES = 1 << 29      # --probe copy: one launch reads and writes this many bytes
TRAFFIC_FILE = os.path.join(REPO, "ms_custom_ops_amd", "measured_traffic.json")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=40,
                    help="untimed steps, a floor: warm-up goes on until the launch period is stable (see DeviceProblem.time)")
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--layout", default="packed", choices=["kn", "nk", "packed"],
                    help="weight storage the op sees: packed=the blocked layout of msco_pack_weight (prepacked once, the default), "
                         "nk=[E,N,K] (prepacked once by a transpose), kn=[E,K,N] as generated")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--zero-operands", nargs="?", const="both", default=None, choices=["both", "x", "w"],
                    help="with --probe <workload>: all-zero x and weights, or only one of them (same kernel, less or nothing toggles)")
    ap.add_argument("--probe", default=None, help="workload name, `copy` or `moe` (the routing / un-permutation pair): launches only, for counter collection")
    return ap.parse_args()


class DeviceProblem:
    """One workload resident on the GPU plus a planned backend operator."""

    def __init__(self, wl, layout="kn", copies=1, zero_operands=False, act_type=0, force_split_k=0, kernel_override=0):
        import torch
        from ms_custom_ops_amd import cabi
        self.torch, self.cabi, self.wl = torch, cabi, wl
        dev = torch.device("cuda:0")
        nk = layout == "nk"
        self.a16 = wl.kind == "a16w8"
        t = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
        self.x = t(wl.x.view(np.int16)) if self.a16 else t(wl.x)
        if wl.w is None:   # weights too large to draw on the host: uniform int8 drawn on the device (timing only)
            w0 = torch.randint(-127, 128, tuple(wl.meta["w_shape"]), dtype=torch.int8, device=dev)
        else:
            w0 = t(wl.w)
        # same shapes, routing and kernel, operands that toggle nothing: a timing yardstick only (True or "both", "x", "w")
        if zero_operands in (True, "both", "x"):
            self.x.zero_()
        if zero_operands in (True, "both", "w"):
            w0.zero_()
        self.prepack_ms = None
        if nk:
            # one-time prepack [E,K,N] -> [E,N,K] through the backend's own transpose entry point
            packed = torch.empty((wl.e, wl.n, wl.k), dtype=torch.int8, device=dev)
            st = torch.cuda.current_stream().cuda_stream
            cabi.transpose_2d(w0.data_ptr(), packed.data_ptr(), wl.e, wl.k, wl.n, 1, st)   # warm
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            cabi.transpose_2d(w0.data_ptr(), packed.data_ptr(), wl.e, wl.k, wl.n, 1, st)
            b.record()
            torch.cuda.synchronize()
            self.prepack_ms = a.elapsed_time(b)
            w0 = packed
        elif layout == "packed":
            # one-time prepack into the backend's blocked layout (the counterpart of the reference's trans_data step)
            packed = torch.empty(wl.e * cabi.packed_weight_bytes(wl.k, wl.n), dtype=torch.int8, device=dev)
            st = torch.cuda.current_stream().cuda_stream
            cabi.pack_weight(w0.data_ptr(), packed.data_ptr(), wl.e, wl.k, wl.n, False, st)   # warm
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            cabi.pack_weight(w0.data_ptr(), packed.data_ptr(), wl.e, wl.k, wl.n, False, st)
            b.record()
            torch.cuda.synchronize()
            self.prepack_ms = a.elapsed_time(b)
            w0 = packed
        # extra weight copies (random bytes; only the timing uses them) defeat the Infinity Cache
        self.w = [w0] + [torch.randint(-127, 128, w0.shape, dtype=torch.int8, device=dev) for _ in range(copies - 1)]
        self.gl = t(wl.group_list)
        self.out = torch.empty((wl.m, wl.n), dtype=torch.int16, device=dev)
        if self.a16:
            self.scale, self.offset = t(wl.scale.view(np.int16)), t(wl.offset.view(np.int16))
            self.op = cabi.GmmOp(x_dtype=cabi.DT_BF16, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64,
                                 antiquant_dtype=cabi.DT_BF16, has_antiquant_offset=1,
                                 weight_layout=cabi.WL_PACKED if layout == "packed" else cabi.WL_ROW_MAJOR)
        else:
            self.scale, self.pt, self.bias = t(wl.scale), t(wl.per_token), t(wl.bias)
            self.op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64,
                                 scale_dtype=cabi.DT_F32, per_token_dtype=cabi.DT_F32,
                                 bias_dtype=cabi.DT_I32 if self.bias is not None else cabi.DT_NONE,
                                 transpose_b=int(nk), act_type=act_type, force_split_k=force_split_k, kernel_override=kernel_override,
                                 weight_layout=cabi.WL_PACKED if layout == "packed" else cabi.WL_ROW_MAJOR)
        self.ws_bytes = self.op.plan(wl.m, wl.k, wl.n, wl.e)
        self.ws = torch.empty(max(self.ws_bytes, 1), dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream
        self.i = 0

    def step(self):
        w = self.w[self.i % len(self.w)]
        self.i += 1
        p = lambda v: None if v is None else v.data_ptr()
        if self.a16:
            ins = [p(self.x), p(w), None, None, p(self.gl), None, p(self.scale), p(self.offset)]
        else:
            ins = [p(self.x), p(w), p(self.bias), p(self.scale), p(self.gl), p(self.pt), None, None]
        self.op.launch(ins, self.out.data_ptr(), self.ws.data_ptr(), self.ws_bytes, self.stream)

    def time(self, steps, warmup):
        """Returns (wall seconds of `steps` steps, mean per-launch seconds, details).  The per-launch figure comes from
        one pair of HIP events on the launch stream around the `steps` back-to-back launches, so it is the
        launch-to-launch period of a running stream and agrees with a profiler's kernel durations.

        `warmup` is a floor.  The shader clock takes tens of launches to settle under this load, so the untimed phase
        goes on (in batches of ten launches, each timed with events) until at least WARM_MIN_LAUNCHES launches and
        WARM_MIN_MS of device time have passed and three batches in a row agree within WARM_TOLERANCE, or WARM_MAX_MS is
        used up.  `details` records the warm-up launches actually made and the period of the first and the last
        quarter of the timed steps, so a figure taken while the clock still moved shows."""
        torch = self.torch
        ev = lambda: torch.cuda.Event(enable_timing=True)
        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize()
        done, spent_ms, recent, stable = warmup, 0.0, [], False
        while spent_ms < WARM_MAX_MS:
            a, b = ev(), ev()
            a.record()
            for _ in range(10):
                self.step()
            b.record()
            torch.cuda.synchronize()
            batch = a.elapsed_time(b)
            done += 10
            spent_ms += batch
            recent = (recent + [batch])[-3:]
            stable = len(recent) == 3 and max(recent) - min(recent) <= WARM_TOLERANCE * min(recent)
            if stable and done >= WARM_MIN_LAUNCHES and spent_ms >= WARM_MIN_MS:
                break
        marks = sorted({0, steps // 4, steps - steps // 4, steps})
        events = {}
        t0 = time.perf_counter()
        for i in range(steps + 1):
            if i in marks:
                events[i] = ev()
                events[i].record()
            if i < steps:
                self.step()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        per_launch = events[0].elapsed_time(events[steps]) / steps * 1e-3
        details = {"warmup_launches": done, "warmup_settled": bool(stable)}
        if steps >= 4:
            q = steps // 4
            details["first_quarter_us"] = events[0].elapsed_time(events[q]) / q * 1e3
            details["last_quarter_us"] = events[steps - q].elapsed_time(events[steps]) / q * 1e3
        return wall, per_launch, details


def rates(wl, seconds):
    from ms_custom_ops_amd import workloads
    work = workloads.algorithmic_work(wl)
    tops = work["ops"] / seconds / 1e12
    gbs = work["bytes"] / seconds / 1e9
    return work, tops, gbs


def cpu_baseline(wl, budget_s=15.0):
    """The reference golden restated in numpy (one float32 dot per group, then the dequant epilogue,
    bf16 cast), timed group by group on the host until the budget is used up."""
    from oracle import gmm_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    starts, ends = O.group_bounds(wl.group_list)
    done_ops, spent, groups = 0.0, 0.0, 0
    for g in range(wl.e):
        a, b = int(starts[g]), int(ends[g])
        if b <= a:
            continue
        t0 = time.perf_counter()
        O.golden_np_qbmm(wl.x[a:b], wl.w[g], wl.scale[g], None if wl.bias is None else wl.bias[g], wl.per_token[a:b],
                         out="bf16")
        dt = time.perf_counter() - t0
        spent += dt
        done_ops += 2.0 * (b - a) * wl.k * wl.n
        groups += 1
        if spent > budget_s:
            break
    return {"value": done_ops / spent / 1e12, "unit": "TOPS", "cores": int(threads), "kind": "port",
            "sample": f"{groups} of {wl.e} expert groups of the {wl.name} workload ({done_ops:.3g} ops in {spent:.2f} s), "
                      "numpy float32 dot per group + dequant epilogue + bf16 cast"}


def moe_neighbours(steps, warmup):
    """The routing step in front of the grouped matmul and the un-permutation behind it, on the shapes of the
    headline MoE layer: HBM-bound row copies, reported as algorithmic bytes per second."""
    import torch
    from ms_custom_ops_amd import cabi
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    out = []

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        for _ in range(steps):
            fn()
        last.record()
        torch.cuda.synchronize()
        return first.elapsed_time(last) / steps * 1e-3

    # routing: 4096 tokens x top-2 of 8 experts, int8 activations of width K = 4096 (the x of c3)
    rows, k, e, h = 4096, 2, 8, 4096
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    # (launches take their input and output rows from `sets` buffer pairs in turn, more than the 256 MB memory-side cache
    # holds: one pair would stay in that cache from launch to launch and the figure would not be an HBM figure)
    idx = torch.argsort(torch.randn(rows, e, device=dev, generator=g), dim=1, descending=True)[:, :k].to(torch.int32).contiguous()
    ridx = torch.empty(rows * k, dtype=torch.int32, device=dev)
    tok = torch.empty(e, dtype=torch.int32, device=dev)
    wsb = cabi.moe_init_routing_v2_workspace_bytes(rows, k, e)
    ws = torch.empty(max(wsb, 1), dtype=torch.uint8, device=dev)
    byts = rows * h + rows * k * h + rows * k * 4 * 2 + e * 4          # x read once, expanded_x written, indices in and out
    sets = int(np.ceil(ROTATE_BYTES / byts)) + 1
    xs = [torch.randint(-127, 128, (rows, h), dtype=torch.int8, device=dev, generator=g) for _ in range(sets)]
    exs = [torch.empty((rows * k, h), dtype=torch.int8, device=dev) for _ in range(sets)]
    turn_r = [0]
    def route():
        turn_r[0] += 1
        i = turn_r[0] % sets
        cabi.moe_init_routing_v2(xs[i].data_ptr(), idx.data_ptr(), exs[i].data_ptr(), ridx.data_ptr(), tok.data_ptr(), None,
                                 ws.data_ptr(), wsb, rows, h, k, e, 1, 1, st)
    sec = timed(route)
    out.append({"workload": f"moe_init_routing_v2: {rows} tokens x top-{k} of {e} experts, int8 rows of {h}", "launch_us": sec * 1e6,
                "gbs": byts / sec / 1e9, "hbm_frac": byts / sec / 1e9 / PEAK_HBM_GBS, "bytes_per_launch": byts, "buffer_sets_rotated": sets})
    del xs

    # the same routing on bfloat16 activations, quantised to int8 per token on the way (what c3's x and per-token scale
    # come from when the layer's input is not quantised yet)
    sc = torch.empty(rows * k, dtype=torch.float32, device=dev)
    byts = rows * h * 2 + rows * k * h + rows * k * 4 * 3 + e * 4      # x read once, int8 rows and scales written, indices in and out
    sets = int(np.ceil(ROTATE_BYTES / byts)) + 1
    xbs = [torch.randn((rows, h), dtype=torch.bfloat16, device=dev, generator=g) for _ in range(sets)]
    exs = exs[:sets]
    def route_quant():
        turn_r[0] += 1
        i = turn_r[0] % sets
        cabi.moe_init_routing_v2_quant(xbs[i].data_ptr(), idx.data_ptr(), exs[i].data_ptr(), sc.data_ptr(), ridx.data_ptr(),
                                       tok.data_ptr(), None, ws.data_ptr(), wsb, rows, h, k, e, cabi.DT_BF16, 1, st)
    sec = timed(route_quant)
    out.append({"workload": f"moe_init_routing_v2_quant: {rows} tokens x top-{k} of {e} experts, bfloat16 rows of {h} -> int8",
                "launch_us": sec * 1e6, "gbs": byts / sec / 1e9, "hbm_frac": byts / sec / 1e9 / PEAK_HBM_GBS, "bytes_per_launch": byts,
                "buffer_sets_rotated": sets})
    del xbs, exs

    # grouped A8W4 at the reference test's shape: 32 rows routed to 256 experts, K = 7168, N = 256, K groups of 256
    # (tests/st/test_grouped_matmul_w4.py:146-152).  Bytes: the int4 weights and scales of the experts that got rows.
    m4, k4, n4, e4, g4 = 32, 7168, 256, 256, 256
    x4 = torch.randint(-127, 128, (m4, k4), dtype=torch.int8, device=dev, generator=g)
    # (four copies of the 235 MB of weights, taken in turn: one copy would stay in the 256 MB Infinity Cache between launches)
    w4 = [torch.randint(0, 256, (e4, n4, k4 // 2), dtype=torch.uint8, device=dev, generator=g) for _ in range(4)]
    turn = [0]
    ws4 = torch.rand((e4, k4 // g4, n4), dtype=torch.float32, device=dev, generator=g) * 1e-2
    xs4 = torch.rand(m4, dtype=torch.float32, device=dev, generator=g) * 1e-2
    ends = torch.sort(torch.randint(1, m4 + 1, (e4 - 1,), device=dev, generator=g)).values.tolist() + [m4]
    gl4 = torch.tensor(ends, dtype=torch.int32, device=dev)
    o4 = torch.empty((m4, n4), dtype=torch.float16, device=dev)
    def a8w4():
        turn[0] += 1
        cabi.gmm_a8w4(x4.data_ptr(), w4[turn[0] % 4].data_ptr(), gl4.data_ptr(), xs4.data_ptr(), ws4.data_ptr(), o4.data_ptr(),
                      m4, k4, n4, e4, g4, st)
    sec = timed(a8w4)
    hit = len(set(ends))                                               # experts with at least one row
    byts = hit * (n4 * k4 // 2 + (k4 // g4) * n4 * 4) + m4 * k4 + m4 * n4 * 2 + m4 * 4 + e4 * 4
    out.append({"workload": f"grouped_matmul_w4: {m4} rows over {e4} experts ({hit} hit), K={k4}, N={n4}, K groups of {g4}",
                "launch_us": sec * 1e6, "gbs": byts / sec / 1e9, "hbm_frac": byts / sec / 1e9 / PEAK_HBM_GBS, "bytes_per_launch": byts})

    # un-permutation: 4096 tokens x top-8, float16 rows of 7168 (the reference op's largest supported shape class)
    t, k, h = 4096, 8, 7168
    pt = torch.randn((t * k, h), dtype=torch.float16, device=dev, generator=g)
    si = torch.randperm(t * k, device=dev, generator=g).to(torch.int32)
    pr = torch.randn((t, k), dtype=torch.float16, device=dev, generator=g)
    o = torch.empty((t, h), dtype=torch.float16, device=dev)
    sec = timed(lambda: cabi.moe_token_unpermute(pt.data_ptr(), si.data_ptr(), pr.data_ptr(), o.data_ptr(), t, k, h, cabi.DT_F16, st))
    byts = t * k * h * 2 + t * h * 2 + t * k * (4 + 2)
    out.append({"workload": f"moe_token_unpermute: {t} tokens x top-{k}, float16 rows of {h}", "launch_us": sec * 1e6,
                "gbs": byts / sec / 1e9, "hbm_frac": byts / sec / 1e9 / PEAK_HBM_GBS, "bytes_per_launch": byts})
    return out


def mfma_pipe_probe(iters=20000, launches=12):
    """Rate of a loop of nothing but int8 MFMAs (msco_probe_mfma_issue, patterns 0 and 12: 256 workgroups, one wavefront per
    SIMD, no memory traffic) for both instruction shapes the tile kernels use, on uniformly random int8 operands, the
    distribution of the workloads, and on zeros: what the matrix pipe sustains at the clock the chip holds under each.
    Every figure is the mean over the last half of the launches (one pair of events around them), after the first half
    has let the clock settle."""
    import torch
    from ms_custom_ops_amd import cabi
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    sink = torch.empty(cabi.PROBE_MFMA_WORKGROUPS * 256, dtype=torch.int32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    ops = cabi.PROBE_MFMA_WORKGROUPS * 4 * iters * 2.0 ** 21
    out = {"ops_per_launch": ops, "iters": iters}
    for shape, pattern in (("16x16x64", 0), ("32x32x32", 12)):
        for name, operands in (("random_int8", torch.randint(-127, 128, (cabi.PROBE_MFMA_OPERAND_BYTES,), dtype=torch.int8, device=dev, generator=g)),
                               ("zeros", torch.zeros(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device=dev))):
            run = lambda: cabi.probe_mfma_issue(operands.data_ptr(), sink.data_ptr(), clocks.data_ptr(), pattern, iters, st)
            for _ in range(launches // 2):
                run()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(launches - launches // 2):
                run()
            b.record()
            torch.cuda.synchronize()
            sec = a.elapsed_time(b) * 1e-3 / (launches - launches // 2)
            c = clocks.cpu().numpy()
            out[f"{shape}/{name}"] = {"launch_us": sec * 1e6, "tops": ops / sec / 1e12, "int8_frac": ops / sec / 1e12 / PEAK_INT8_TOPS,
                                      "ghz": float(c[0]) / (float(c[1]) * 10.0)}
    return out


ISSUE_PATTERNS = (
    (0, "16x16x64 MFMAs only"), (1, "+ 16 ds_read_b128"), (2, "+ 16 reads + 8 buffer loads"),
    (3, "+ 8 ds_write_b128 alone"), (4, "+ 16 ds_write_b64 alone"), (5, "+ 32 ds_write_b32 alone"),
    (6, "reads + loads + 8 ds_write_b128, a read one MFMA later"), (7, "reads + loads + 8 ds_write_b128, the next read three MFMAs later"),
    (8, "reads + loads + 16 ds_write_b64 in slots of their own"), (9, "reads + loads + 16 ds_write_b64 sharing the reads' slots"),
    (10, "as 8, loads sharing a write's slot"), (11, "reads + loads + 32 ds_write_b32"),
    (12, "32x32x32 MFMAs only"), (13, "32x32x32: reads + loads + 8 ds_write_b128"), (14, "32x32x32: reads + loads + 16 ds_write_b64"))


def mfma_issue_probe(iters=20000):
    """What a wavefront that is alone on its SIMD can issue between MFMAs (msco_probe_mfma_issue): core clocks per round of
    64 v_mfma_i32_16x16x64_i8 (32 v_mfma_i32_32x32x32_i8) with the K loop's memory operations woven in at different
    places, on zero operands (the nominal clock).  A row reads [pattern, what it adds, clocks per round, clocks beyond
    the bare loop of its instruction shape]."""
    import torch
    from ms_custom_ops_amd import cabi
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.empty(cabi.PROBE_MFMA_WORKGROUPS * 256, dtype=torch.int32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    operands = torch.zeros(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device=dev)
    rows, bare = [], {}
    for pattern, what in ISSUE_PATTERNS:
        for _ in range(3):
            cabi.probe_mfma_issue(operands.data_ptr(), sink.data_ptr(), clocks.data_ptr(), pattern, iters, st)
        torch.cuda.synchronize()
        per_round = float(clocks.cpu().numpy()[0]) / iters
        shape = "32" if pattern >= 12 else "16"
        bare.setdefault(shape, per_round)
        rows.append([pattern, what, round(per_round, 1), round(per_round - bare[shape], 1)])
    return {"iters": iters, "columns": ["pattern", "adds", "clocks_per_round", "beyond_bare_loop"], "rows": rows}


def read_floor(sizes=(45.09e6, 469.8e6), steps=60):
    """Duration of one launch that only reads a buffer of the given size front to back (msco_probe_read), the floor under
    a single-launch decode kernel whose weights have that size.  Successive launches read successive windows of a
    buffer larger than the 256 MB memory-side cache, so every launch streams from HBM.  The best of a few workgroup
    counts is reported."""
    import torch
    from ms_custom_ops_amd import cabi
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    out = []
    for size in sizes:
        size = int(size) // 4096 * 4096
        windows = max(3, int(np.ceil(ROTATE_BYTES / size)) + 1)
        buf = torch.randint(-127, 128, (windows * size,), dtype=torch.int8, device=dev)
        best = None
        for wgs in (256, 344, 512, 1024, 2048):
            sink = torch.empty(wgs * 256, dtype=torch.int32, device=dev)
            turn = [0]
            def one():
                turn[0] += 1
                cabi.probe_read(buf.data_ptr() + (turn[0] % windows) * size, size, sink.data_ptr(), wgs, st)
            for _ in range(10):
                one()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(steps):
                one()
            b.record()
            torch.cuda.synchronize()
            sec = a.elapsed_time(b) / steps * 1e-3
            if best is None or sec < best[0]:
                best = (sec, wgs)
        out.append({"bytes": size, "launch_us": best[0] * 1e6, "workgroups": best[1], "gbs": size / best[0] / 1e9,
                    "hbm_frac": size / best[0] / 1e9 / PEAK_HBM_GBS})
        del buf
        torch.cuda.empty_cache()
    return out


def library_reference(wl, steps=20):
    """The vendor library on the same operands, for scale: torch._int_mm (hipBLASLt) on ONE dense int8 matmul with the
    headline's M, K and N (all rows against one expert's weights; int32 out, no grouping, no epilogue), weights [K,N] as
    generated and [N,K] (passed as a transposed view).  Reported, not used."""
    import torch
    out = {}
    try:
        dev = torch.device("cuda:0")
        x = torch.from_numpy(np.ascontiguousarray(wl.x)).to(dev)
        w_kn = torch.from_numpy(np.ascontiguousarray(wl.w[0])).to(dev)
        w_nk = w_kn.t().contiguous()
        ops = 2.0 * wl.x.shape[0] * wl.k * wl.n
        for name, b in (("kn", w_kn), ("nk", w_nk.t())):
            for _ in range(10):
                torch._int_mm(x, b)
            first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            first.record()
            for _ in range(steps):
                torch._int_mm(x, b)
            last.record()
            torch.cuda.synchronize()
            sec = first.elapsed_time(last) / steps * 1e-3
            out[name] = {"launch_us": sec * 1e6, "tops": ops / sec / 1e12, "int8_frac": ops / sec / 1e12 / PEAK_INT8_TOPS}
        out["what"] = f"torch._int_mm, dense [{wl.x.shape[0]},{wl.k}] x [{wl.k},{wl.n}] int8 -> int32"
    except Exception as exc:   # not every build of torch carries the routine
        out["error"] = repr(exc)
    return out


def measured_traffic(workload, layout, kernel):
    """HBM bytes per launch of the dominant kernel from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs (scaled by
    the same counters' reading for a copy of known size); None when no measurement of this kernel is on file."""
    try:
        table = json.load(open(TRAFFIC_FILE))
    except OSError:
        return None
    entry = table.get(f"{workload}/{layout}")
    if not entry or entry.get("kernel") != kernel:
        return None
    return entry["hbm_bytes_per_launch"]


def plan_regret(steps=30):
    """What the planner's pick costs against the kernel families it could have picked: neighbouring shapes of the dense
    linear (K=4096, N=11008) and of the MoE layer (8 experts, top-2, K=4096, N=14336) on packed and on [E,K,N] weights,
    each timed with the plan's own choice and with every family forced through msco_gmm_desc.kernel_override.
    A row reads [workload, layout, picked kernel, us, best forced family, us, pick / best]; a ratio well above 1 is a
    planner rule that is wrong for that shape."""
    import torch
    from ms_custom_ops_amd import cabi, workloads
    forced = (("tile_256", cabi.OV_TILE_256), ("tile_256_w4", cabi.OV_TILE_256_W4), ("tile_256_w4_mfma32", cabi.OV_TILE_256_W4_MFMA32),
              ("tile_128x256", cabi.OV_TILE_128x256),
              ("tile_128", cabi.OV_TILE_128), ("tile_64", cabi.OV_TILE_64), ("decode", cabi.OV_SKINNY),
              ("rows_128", cabi.OV_ROWS128), ("rows_160", cabi.OV_ROWS160), ("rows_256", cabi.OV_ROWS256))
    names = ["c2_m%d" % m for m in (1, 16, 17, 32, 64, 65, 128, 192, 256, 320, 384, 448, 512, 640, 704, 768, 1024, 1280, 1536, 2048, 3072)]
    names += ["c3_t%d" % t for t in (8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 448, 512, 576, 768, 1024, 2048)]
    rows = []
    for name in names:
        wl = workloads.make(name)
        per_group = wl.m / wl.e
        for layout in ("packed", "kn"):
            copies = max(1, int(np.ceil(ROTATE_BYTES / (wl.e * wl.k * wl.n))))
            prob = DeviceProblem(wl, layout, copies)

            def period():   # (the warm-up of the headline measurement: until the launch period has settled)
                return prob.time(steps, 10)[1] * 1e6

            picked = prob.op.plan_info().split("kernel=")[1].split(" ")[0]
            picked_op, picked_ws, picked_bytes = prob.op, prob.ws, prob.ws_bytes
            period()        # (the first kernel after the set-up meets a cold chip: its figure is taken again at the end)
            best = (None, float("inf"))
            for fam, ov in forced:
                # (families that would stream the weights dozens of times, or multiply mostly padding, are not candidates)
                if (fam == "decode" and per_group > 64) or (fam == "tile_64" and per_group > 512) or \
                        (fam in ("tile_256", "tile_256_w4") and wl.m < 64) or (fam in ("tile_128", "tile_128x256") and wl.m < 32) or \
                        (fam in ("rows_128", "rows_160", "rows_256") and (layout != "packed" or wl.e == 1 or wl.m < 32)):
                    continue
                try:
                    op = cabi.GmmOp(x_dtype=cabi.DT_I8, out_dtype=cabi.DT_BF16, group_list_dtype=cabi.DT_I64,
                                    scale_dtype=cabi.DT_F32, per_token_dtype=cabi.DT_F32,
                                    bias_dtype=cabi.DT_I32 if prob.bias is not None else cabi.DT_NONE, kernel_override=ov,
                                    weight_layout=cabi.WL_PACKED if layout == "packed" else cabi.WL_ROW_MAJOR)
                    ws_bytes = op.plan(wl.m, wl.k, wl.n, wl.e)
                except cabi.BackendError:
                    continue
                prob.op, prob.ws_bytes = op, ws_bytes
                prob.ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda:0")
                us = period()
                if us < best[1]:
                    best = (fam, us)
            prob.op, prob.ws, prob.ws_bytes = picked_op, picked_ws, picked_bytes
            us_pick = period()
            rows.append([name, layout, picked, us_pick, best[0], best[1], us_pick / best[1] if best[0] else None])
            del prob
            torch.cuda.empty_cache()
            print("plan_regret", rows[-1], file=sys.stderr, flush=True)
    worst = max((r for r in rows if r[6] is not None), key=lambda r: r[6])
    return {"columns": ["workload", "layout", "picked", "us", "best_forced_family", "us_forced", "pick_over_best"], "rows": rows,
            "worst": worst}


def probe(args):
    import torch
    from ms_custom_ops_amd import workloads
    if args.probe == "plan":
        print(json.dumps(compact({"probe": "plan", "plan_regret": plan_regret()})))
        return
    if args.probe == "copy":
        src = torch.randint(-127, 128, (COPY_BYTES,), dtype=torch.int8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "copy", "bytes_read": COPY_BYTES, "bytes_written": COPY_BYTES, "launches": args.steps}))
        return
    if args.probe == "read":
        print(json.dumps({"probe": "read", "read_floor": read_floor()}))
        return
    if args.probe == "mfma":
        print(json.dumps({"probe": "mfma", "mfma_pipe": mfma_pipe_probe()}))
        return
    if args.probe == "issue":
        print(json.dumps({"probe": "issue", "mfma_issue": mfma_issue_probe()}))
        return
    if args.probe == "moe":
        print(json.dumps({"probe": "moe", "moe_neighbours": moe_neighbours(args.steps, 5)}))
        return
    wl = workloads.make(args.probe)
    prob = DeviceProblem(wl, args.layout, zero_operands=args.zero_operands)
    for _ in range(args.steps):
        prob.step()
    torch.cuda.synchronize()
    print(json.dumps({"probe": args.probe, "zero_operands": args.zero_operands, "plan": prob.op.plan_info(), "launches": args.steps}))


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this build has no multi-GPU path)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from ms_custom_ops_amd import workloads

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the operators have no CPU path)", file=sys.stderr)
        sys.exit(1)

    if args.probe:
        probe(args)
        return
    wl = workloads.make(args.workload)
    prob = DeviceProblem(wl, args.layout)
    wall, per_launch, timing = prob.time(args.steps, args.warmup)
    work, _, _ = rates(wl, per_launch)
    step_s = wall / args.steps
    tops_wall = work["ops"] / step_s / 1e12
    tops_kernel = work["ops"] / per_launch / 1e12
    plan = prob.op.plan_info()
    mfma_bound = (work["ops"] / work["bytes"]) > (PEAK_INT8_TOPS * 1e12) / (PEAK_HBM_GBS * 1e9)
    if mfma_bound:
        roof = {"bound": "mfma", "achieved": tops_kernel, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": tops_kernel / PEAK_INT8_TOPS, "traffic": None}
    else:
        gbs = work["bytes"] / per_launch / 1e9
        roof = {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                "traffic": None}
    roof["kernel"] = plan.split("kernel=")[1].split(" ")[0]
    roof["traffic"] = measured_traffic(wl.name, args.layout, roof["kernel"])
    roof["traffic_source"] = None if roof["traffic"] is None else \
        "stored: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised under profiles/ (not re-measured in this run)"
    roof["launch_us"] = per_launch * 1e6
    roof["ops_per_launch"] = work["ops"]
    roof["bytes_per_launch"] = work["bytes"]

    result = {
        "metric": "int8 TOPS and HBM GB/s (% roofline) for grouped W8A8 GEMM, 1 MI355X",
        "value": tops_wall, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": step_s * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (int32 accumulate, bf16 out)", "data": "synthetic",
        "config": {"workload": f"{wl.name}: grouped W8A8, E={wl.e}, rows={work['rows']}, K={wl.k}, N={wl.n}, "
                               f"weights {LAYOUT_TEXT[args.layout]}, "
                               "routing top-2 of softmax(N(0,1))",
                   "plan": plan, "prepack_ms": prob.prepack_ms, "timing": timing},
        "hbm_gbs": work["bytes"] / step_s / 1e9, "hbm_frac": work["bytes"] / step_s / 1e9 / PEAK_HBM_GBS,
        "int8_frac": tops_wall / PEAK_INT8_TOPS,
        "roofline": roof,
    }
    del prob
    torch.cuda.empty_cache()

    if not args.no_sweep:
        sweep = []
        cached = [None, None]
        others = [l for l in ("packed", "nk", "kn") if l != args.layout]
        for name, layout in [("c3", others[0]), ("c3", others[1]), ("c2_m2048", "packed"), ("c2_m2048", "nk"), ("c2_m2048", "kn"),
                             ("c4", "packed"), ("c4", "nk"), ("c4", "kn"), ("c1", "packed"), ("c2_m256", "packed"),
                             ("c1", "nk"), ("c1", "kn"), ("c2_m256", "nk"), ("c2_m256", "kn"), ("c2_m16", "nk"),
                             ("c2_m16", "kn"), ("c2_m16", "packed"), ("c2_m1", "kn"), ("c2_m1", "packed"), ("c5", "kn"),
                             ("c5", "packed"), ("c3_decode", "kn"), ("c3_decode", "packed"),
                             # the headline MoE layer at serving batch sizes (T tokens, top-2 of 8): bound by the 470 MB of weights
                             ("c3_t64", "packed"), ("c3_t128", "packed"), ("c3_t256", "packed"), ("c3_t448", "packed"), ("c3_t512", "packed"),
                             ("c3_t1024", "packed"),
                             # the weight-only layer beyond decode: chunks of 32 .. 128 rows share a pass over the weights
                             ("c5_t64", "packed"), ("c5_t256", "packed"), ("c5_t256", "kn"),
                             # the shapes the reference's own tests time or call real (its weights are [E,N,K] there):
                             # 1024 rows over 8 experts, and 256 experts with 40 or 1024 rows
                             ("ref_m1024_k5120_n2688_e8", "nk"), ("ref_m1024_k5120_n2688_e8", "packed"),
                             ("ref_m1024_k5120_n1344_e8", "nk"), ("ref_m1024_k5120_n1344_e8", "packed"),
                             ("ref_m40_k512_n7168_e256", "nk"), ("ref_m40_k512_n7168_e256", "packed"),
                             ("ref_m1024_k2048_n7168_e256", "nk"), ("ref_m1024_k2048_n7168_e256", "packed"),
                             ("ref_m1024_k7168_n4096_e256", "nk"), ("ref_m1024_k7168_n4096_e256", "packed")]:
            if cached[0] != name:   # (one draw serves every layout of a workload)
                cached[:] = [name, workloads.make(name)]
            w2 = cached[1]
            w_bytes = w2.e * w2.k * w2.n
            # (what a launch reads of the weights: the experts that hold rows)
            w_read = workloads.algorithmic_work(w2)["nonempty_groups"] * w2.k * w2.n
            hbm_bound_guess = name in ("c1", "c2_m256", "c2_m16", "c2_m1", "c5", "c3_decode") or name.startswith(("c3_t", "c5_t")) or \
                (name.startswith("ref_") and w_read < 2 * ROTATE_BYTES)
            copies = max(1, int(np.ceil(ROTATE_BYTES / (w_read if name.startswith("ref_") else w_bytes)))) if hbm_bound_guess else 1
            p2 = DeviceProblem(w2, layout, copies)
            _, sec, _ = p2.time(max(20, min(200, args.steps)), args.warmup)
            wk, tops, gbs = rates(w2, sec)
            sweep.append([name, layout, sec * 1e6, tops / PEAK_INT8_TOPS, gbs / PEAK_HBM_GBS, copies,
                          p2.op.plan_info().split("kernel=")[1].split(" ")[0]])
            del p2
            torch.cuda.empty_cache()
        # (one row per case, columnar: the whole line has to survive a log tail; TOP/s = int8_frac x 5000, GB/s = hbm_frac x 8000)
        result["sweep"] = {"columns": ["workload", "layout", "launch_us", "int8_frac", "hbm_frac", "weight_copies_rotated", "kernel"],
                           "rows": sweep}
        result["moe_neighbours"] = moe_neighbours(max(20, min(100, args.steps)), 10)
        result["mfma_pipe"] = mfma_pipe_probe()
        result["read_floor"] = read_floor()
        result["library_reference"] = library_reference(wl)
        # the headline kernel once more on all-zero x and weights: same instruction stream and memory traffic, but the
        # matrix pipe toggles nothing, so the chip holds a higher clock; the gap to the figure above is what the
        # operand distribution costs, the gap to the peak is what the kernel's own stalls and padding cost
        pz = DeviceProblem(wl, args.layout, zero_operands=True)
        _, secz, _ = pz.time(max(20, min(100, args.steps)), args.warmup)
        result["zero_operand_check"] = {"workload": wl.name, "layout": args.layout, "launch_us": secz * 1e6,
                                        "tops": work["ops"] / secz / 1e12, "int8_frac": work["ops"] / secz / 1e12 / PEAK_INT8_TOPS}
        del pz
        torch.cuda.empty_cache()
        # and with an activation fused into the epilogue (act_type 5, silu)
        pa = DeviceProblem(wl, args.layout, act_type=5)
        _, seca, _ = pa.time(max(20, min(100, args.steps)), args.warmup)
        result["fused_activation"] = {"workload": wl.name, "layout": args.layout, "act_type": 5, "launch_us": seca * 1e6,
                                      "tops": work["ops"] / seca / 1e12, "int8_frac": work["ops"] / seca / 1e12 / PEAK_INT8_TOPS}
        del pa
        torch.cuda.empty_cache()

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(wl)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(compact(result)))


def compact(v):
    """Floats to five significant digits: the line stays short enough to be read whole from a log tail."""
    if isinstance(v, float):
        return float(f"{v:.5g}")
    if isinstance(v, dict):
        return {k: compact(x) for k, x in v.items()}
    if isinstance(v, (list, tuple)):
        return [compact(x) for x in v]
    return v


if __name__ == "__main__":
    main()
