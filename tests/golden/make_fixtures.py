"""Writes the committed fixtures of tests/golden/ with the CPU oracle.

    python tests/golden/make_fixtures.py          # small known-answer files + digests of the scaled workloads
    python tests/golden/make_fixtures.py --full   # additionally digests of the full-size workloads (minutes, ~4 GB)

Fixtures are data only: seeded inputs and the oracle's outputs (int32 accumulators, float32
pre-cast values, bf16 / f16 bit patterns), or sha256 digests where the arrays are too large to
commit.  The oracle itself is pinned independently in tests/test_oracle_pins.py.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from ms_custom_ops_amd import workloads  # noqa: E402
from oracle import gmm_oracle as O  # noqa: E402


def sha(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def kat_tiny():
    rng = np.random.default_rng(20251125)
    m, k, n, e = 24, 64, 32, 4
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    bias = rng.integers(-1000, 1001, (e, n)).astype(np.int32)
    scale = rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32)
    pt = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    gl = np.array([7, 7, 19, 24], dtype=np.int64)  # group 1 is empty, the others are ragged
    acc = O.grouped_int32_acc(x, w, gl)
    f32 = O.grouped_matmul_w8a8(x, w, gl, bias, scale, pt, out_dtype="f32")
    np.savez_compressed(os.path.join(HERE, "kat_tiny.npz"), x=x, w=w, bias=bias, scale=scale, per_token=pt,
                        group_list=gl, acc=acc, acc_plus_bias=O.grouped_matmul_w8a8(x, w, gl, bias, out_dtype="i32"),
                        pre_cast_f32=f32, bf16_bits=O.f32_to_bf16_bits(f32), f16_bits=O.f32_to_f16(f32).view(np.uint16))


def kat_const_scale():
    """The reference's constant-scale cases (tests/st/test_grouped_matmul_v4_cops.py:281-301,338-359):
    m=32 k=256 n=128 e=8, counts [1,2,7,4,4,4,2,8], scale 10, per-token 10 / bias 1."""
    rng = np.random.default_rng(7)
    x = rng.integers(-128, 128, (32, 256)).astype(np.int8)
    w = rng.integers(-128, 128, (8, 256, 128)).astype(np.int8)
    counts = np.array([1, 2, 7, 4, 4, 4, 2, 8], dtype=np.int64)
    acc = O.grouped_int32_acc(x, w, counts, 1)
    np.savez_compressed(os.path.join(HERE, "kat_const_scale.npz"), x=x, w=w, counts=counts, acc=acc,
                        pertoken_expected=acc.astype(np.float32) * 100.0,
                        perchannel_bias_expected=(acc + 1).astype(np.float32) * 10.0)


def kat_a16w8():
    rng = np.random.default_rng(11)
    m, k, n, e = 32, 256, 128, 8
    ends = np.array([1, 3, 10, 14, 18, 22, 24, 30], dtype=np.int64)  # last boundary below M
    x = O.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    w = rng.integers(-128, 128, (e, k, n)).astype(np.int8)
    s = O.f32_to_bf16_bits(rng.uniform(1e-3, 1e-2, (e, n)).astype(np.float32))
    o = O.f32_to_bf16_bits(rng.integers(-8, 9, (e, n)).astype(np.float32))
    xf, sf, of = (O.bf16_bits_to_f32(v) for v in (x, s, o))
    exact = O.a16w8_grouped_f64(xf, w, sf, of, ends)
    mag = np.zeros_like(exact)
    starts = np.concatenate([[0], ends[:-1]])
    for g in range(e):
        a, b = int(starts[g]), int(ends[g])
        mag[a:b] = np.abs(xf[a:b].astype(np.float64)) @ (np.abs(w[g].astype(np.float64) + of[g]) * np.abs(sf[g]))
    np.savez_compressed(os.path.join(HERE, "kat_a16w8.npz"), x_bf16=x, w=w, scale_bf16=s, offset_bf16=o, ends=ends,
                        expected_f64=exact, abs_sum_f64=mag)


def digest_workload(name, scale_down):
    wl = workloads.make(name, scale_down=scale_down)
    d = {"x": sha(wl.x), "w": sha(wl.w), "group_list": wl.group_list.tolist(), "m": wl.m, "k": wl.k, "n": wl.n,
         "e": wl.e}
    if wl.kind == "w8a8":
        acc = O.grouped_int32_acc(wl.x, wl.w, wl.group_list)
        d["acc"] = sha(acc)
        bits = O.grouped_matmul_w8a8(wl.x, wl.w, wl.group_list, wl.bias, wl.scale, wl.per_token)
        d["bf16"] = sha(bits)
        d["acc_plus_bias"] = sha(O.grouped_matmul_w8a8(wl.x, wl.w, wl.group_list, wl.bias, out_dtype="i32"))
    d.update({k: v for k, v in wl.meta.items() if not isinstance(v, np.ndarray)})
    return d


def main():
    kat_tiny()
    kat_const_scale()
    kat_a16w8()
    path = os.path.join(HERE, "digests.json")
    digests = json.load(open(path)) if os.path.exists(path) else {}
    for name in ["c1", "c2_m1", "c2_m16", "c2_m256", "c3", "c4"]:
        digests[f"{name}/4"] = digest_workload(name, 4)
        print("digest", name, "/4", flush=True)
    if "--full" in sys.argv:
        for name in ["c1", "c2_m1", "c2_m16", "c2_m256", "c2_m2048", "c3", "c4"]:
            digests[f"{name}/1"] = digest_workload(name, 1)
            print("digest", name, "/1", flush=True)
    json.dump(digests, open(path, "w"), indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
