"""In-tree build of the native parts: the HIP backend behind the C ABI (libmsco_gmm.so) and the
pybind11 operator-registration module (ms_custom_ops.*.so).  hipcc cross-compiles gfx950 code
objects without a GPU, so this runs anywhere the ROCm toolchain is installed."""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(PKG_DIR, "lib", "obj")
INCLUDE = os.path.join(REPO_DIR, "include")

BACKEND_LIB = os.path.join(LIB_DIR, "libmsco_gmm.so")
PROBES_LIB = os.path.join(LIB_DIR, "libmsco_probes.so")   # measurement aids: not part of the operator library
HIP_SOURCES = ["gmm_tile_w8a8.hip", "gmm_tile4_w8a8.hip", "gmm_tile4m_w8a8.hip", "gmm_rows_w8a8.hip", "gmm_skinny_w8a8.hip", "gmm_skinny_a16w8.hip", "gmm_generic.hip", "gmm_stream.hip", "msco_gmm.hip", "moe_routing.hip", "gmm_w4.hip"]
PROBE_SOURCES = ["probes.hip"]
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP backend cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def build_backend(verbose: bool = False, tuning: bool = False) -> str:
    """Compile every HIP source for gfx950 and link libmsco_gmm.so (the operators) and libmsco_probes.so (the
    benchmark's two yardstick kernels)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()
    hip_dir = os.path.join(CSRC, "hip")

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        cmd = [hipcc] + HIP_FLAGS + ["-DMSCO_BUILDING_LIB", "-I", INCLUDE, "-I", hip_dir, "-c",
                                     os.path.join(hip_dir, src), "-o", obj]
        if tuning:   # development build: the planner's constants can be overridden from the environment (MSCO_TILE_CFG, ...)
            cmd.insert(1, "-DMSCO_TUNING_SWITCHES")
        out = _run(cmd)
        if verbose and out.strip():
            print(out)
        return obj

    with cf.ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES + PROBE_SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", BACKEND_LIB] + objs[:len(HIP_SOURCES)])
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBES_LIB] + objs[len(HIP_SOURCES):])
    return BACKEND_LIB


ATTRIBUTION_BUILDS = {"noepi": 1, "nomfma": 2, "nomfma_noepi": 3, "nostore": 4,
                      # the K loop alone (no epilogue) without its memory requests, its LDS writes, its barriers, and with
                      # nothing but MFMAs and fragment reads
                      "kloop_noload": 1 | 8, "kloop_nowrite": 1 | 16, "kloop_nobarrier": 1 | 32, "kloop_mfma_lds": 1 | 8 | 16,
                      "kloop_mfma": 1 | 8 | 16 | 64, "kloop_noread": 1 | 64}


def build_attribution(verbose: bool = False):
    """Measurement builds of the backend, never the shipped one: lib/attr/libmsco_gmm_<name>.so is libmsco_gmm.so with
    one part of the persistent tile kernels taken out (MSCO_TILE4_ATTR in gmm_tile4_w8a8.hip and gmm_tile4m_w8a8.hip), so that timing the rest
    says what that part costs.  Select one with MSCO_GMM_LIB=<path>; their results are wrong on purpose."""
    build_backend(verbose)
    hipcc = _hipcc()
    hip_dir = os.path.join(CSRC, "hip")
    out_dir = os.path.join(LIB_DIR, "attr")
    os.makedirs(out_dir, exist_ok=True)
    tile4 = ("gmm_tile4_w8a8.hip", "gmm_tile4m_w8a8.hip")
    others = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in HIP_SOURCES if s not in tile4]

    def build_one(item):
        name, mask = item
        objs = []
        for src in tile4:
            objs.append(os.path.join(out_dir, "%s_%s.o" % (src[:-4], name)))
            _run([hipcc] + HIP_FLAGS + ["-DMSCO_BUILDING_LIB", "-DMSCO_TILE4_ATTR=%d" % mask, "-I", INCLUDE, "-I", hip_dir, "-c",
                                        os.path.join(hip_dir, src), "-o", objs[-1]])
        lib = os.path.join(out_dir, "libmsco_gmm_%s.so" % name)
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + others + objs)
        for obj in objs:
            os.remove(obj)
        return lib

    with cf.ThreadPoolExecutor(max_workers=4) as pool:
        only = [a for a in sys.argv if a in ATTRIBUTION_BUILDS]
        return list(pool.map(build_one, [(k, v) for k, v in ATTRIBUTION_BUILDS.items() if not only or k in only]))


def pybind_module_path() -> str:
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(PKG_DIR, "ms_custom_ops" + suffix)


def build_pybind(verbose: bool = False) -> str:
    """Compile the C++ operator layer (framework + one translation unit per op) into a pybind11
    module that links against libmsco_gmm.so."""
    import pybind11

    cxx = shutil.which("g++") or "g++"
    srcs = []
    for root, _, files in os.walk(os.path.join(CSRC, "ops")):
        for f in sorted(files):
            if f.endswith(".cc"):
                srcs.append(os.path.join(root, f))
    os.makedirs(OBJ_DIR, exist_ok=True)
    flags = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-DMS_EXTENSION_NAME=ms_custom_ops",
             "-I", INCLUDE, "-I", CSRC, "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"]]

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.relpath(src, CSRC).replace(os.sep, "_").replace(".cc", ".o"))
        out = _run([cxx] + flags + ["-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with cf.ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(compile_one, srcs))
    target = pybind_module_path()
    _run([cxx, "-shared", "-o", target] + objs + ["-L", LIB_DIR, "-lmsco_gmm", "-Wl,-rpath,$ORIGIN/lib"])
    return target


def build_all(verbose: bool = False, tuning: bool = False):
    return build_backend(verbose, tuning), build_pybind(verbose)


if __name__ == "__main__":
    paths = build_attribution("-v" in sys.argv) if "--attribution" in sys.argv else build_all(verbose="-v" in sys.argv, tuning="--tuning" in sys.argv)
    for path in paths:
        print("built", path)
