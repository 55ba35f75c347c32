"""Builds libsmh.so (the HIP kernels and their C ABI) in-tree for gfx950.

`python -m spec_mcts_amd.build` or `spec_mcts_amd.build.build()`.  hipcc cross-compiles, so this
works on a machine without a GPU; the library is then loaded by spec_mcts_amd._lib.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsmh.so")
SOURCES = ["smh_api.hip", "q40_codec.hip", "q40_gemv.hip", "q40_gemm.hip", "partial_ops.hip", "elementwise.hip", "attn_decode.hip", "f16_head.hip"]
# packed fp32 VALU ops are disabled on purpose (device code only; the host pass ignores the feature)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, pr in procs:
        out, _ = pr.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if pr.returncode != 0:
            failed = True
            print(f"[build] {src} FAILED\n{out}", file=sys.stderr)
        elif out.strip() and verbose:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    tmp = LIB + ".tmp"
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
