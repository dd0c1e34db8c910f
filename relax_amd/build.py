"""Compiles the HIP/C++ sources under ``relax_amd/csrc`` into ``librelax_amd_wq.so`` (gfx950).

hipcc cross-compiles without a GPU.  The library is built in-tree so that it
travels with the source tree to the machine that runs it.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librelax_amd_wq.so")
OBJDIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".cc")))


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    if src.endswith(".cc"):
        cmd.insert(1, "-x")
        cmd.insert(2, "hip")
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    """Compile every source and link the shared library; returns its path."""
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.check_call(cmd)
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources", flush=True)
    return LIB


if __name__ == "__main__":
    build()
