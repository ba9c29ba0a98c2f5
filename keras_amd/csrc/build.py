"""Compile the k3q HIP sources into keras_amd/libk3q.so for gfx950.

Run as `python -m keras_amd.csrc.build` or through `__graft_entry__.build()`.
hipcc cross-compiles, so no GPU is needed to build.
"""

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libk3q.so")

SOURCES = [
    "k3q_api.hip",
    "k3q_pack.hip",
    "k3q_quantize.hip",
    "k3q_weight_quantize.hip",
    "k3q_gemv_w4.hip",
    "k3q_gemv_w4s.hip",
    "k3q_gemv_w4_nk.hip",
    "k3q_gemv_w8.hip",
    "k3q_gemm_i8.hip",
    "k3q_gemm_i8_skinny.hip",
    "k3q_embedding.hip",
    "k3q_decode_attn.hip",
    "k3q_gemv_w8s.hip",
    "k3q_glue.hip",
]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    # packed-fp32 VALU forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the k3q kernels need the ROCm toolchain")
    return exe


def build(verbose=True, jobs=8):
    srcs = [os.path.join(HERE, s) for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in srcs:
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [hipcc(), *FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out = p.communicate()[0].decode()
        # hipcc's host pass does not know the packed-fp32 feature: harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            sys.stderr.write(out + "\n")
            raise RuntimeError(f"hipcc failed on {src}")
        if out.strip():
            print(out)


if __name__ == "__main__":
    build()
