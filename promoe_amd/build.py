"""Compile the HIP/C++ sources of the library for gfx950 into promoe_amd/libmoe_engine.so.

Usage: python -m promoe_amd.build            (or call build())
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe_engine.so")

HIP_SOURCES = ["moe_kernels.hip", "moe_prefill.hip"]
CXX_SOURCES = ["moe_common.cpp", "engine_cfg.cpp", "engine_core.cpp", "engine_forward.cpp", "engine_predict.cpp", "backends.cpp"]

# -packed-fp32-ops: keep hipcc from forming v_pk_*_f32 out of scalar float code.
HIP_FLAGS = [
    "-Wno-inline-asm",
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("MOE_EXTRA_HIPFLAGS", "").split()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out, file=sys.stderr)


def build(verbose: bool = True) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    objs = []
    for src in HIP_SOURCES + CXX_SOURCES:
        obj = os.path.join(objdir, src.rsplit(".", 1)[0] + ".o")
        cmd = [hipcc] + HIP_FLAGS + inc + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print("[build]", src, flush=True)
        _run(cmd)
        objs.append(obj)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread"])
    if verbose:
        print("[build] ->", LIB, flush=True)
    return LIB


if __name__ == "__main__":
    build()
