"""Builds libdcnv4_gfx950.so from dcnv4_amd/csrc/*.hip with hipcc, for gfx950 only.

Takes the place of the reference's CUDAExtension build (DCNv4_op/setup.py:24-60): there is no
hipify pass and no torch extension machinery, just hipcc on hand-written HIP sources and a C ABI.
Usage: ``python dcnv4_amd/build.py [--force]`` (run as a script: importing the package needs the library).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libdcnv4_gfx950.so")
SOURCES = ["capi.hip", "dcnv4_kernels.hip", "dcnv4_tiled_gather.hip", "dcnv4_grad_value.hip", "dcnv4_backward_dual.hip", "fda_kernels.hip", "fda_grad_value.hip",
           "depthwise_conv.hip", "layer_norm.hip", "center_feature.hip"]
HEADERS = [os.path.join(CSRC, "common.hpp"), os.path.join(CSRC, "launch.hpp"), os.path.join(CSRC, "dcnv4_tiled_gather.hpp"), os.path.join(CSRC, "dcnv4_grad_value.hpp"),
           os.path.join(os.path.dirname(HERE), "include", "dcnv4_gfx950.h")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 instructions.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-pass-failed", "-Wno-unused-function", "-Wno-unknown-attributes"]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + HEADERS):
        cmd = [HIPCC] + FLAGS + ["-c", path, "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), err))
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(force=False, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), SOURCES))
    if force or _stale(LIB_PATH, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("link failed: %s\n%s" % (" ".join(cmd), proc.stderr))
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(force="--force" in sys.argv)
