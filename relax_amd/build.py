"""Compiles the HIP/C++ sources under ``relax_amd/csrc`` into ``librelax_amd_wq.so`` (gfx950), and
the calibration kernels (``calibrate.hip``: measurement only) into ``librelax_amd_wq_calibrate.so``.

hipcc cross-compiles without a GPU.  The library is built in-tree so that it
travels with the source tree to the machine that runs it.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
if os.path.dirname(HERE) not in sys.path:
    sys.path.insert(0, os.path.dirname(HERE))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librelax_amd_wq.so")
CALIBRATE_LIB = os.path.join(HERE, "librelax_amd_wq_calibrate.so")
CALIBRATE_SOURCES = ("calibrate.hip",)  # not linked into the product library
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


def _deps(src: str, seen=None):
    """`src` and every file it includes with quotes, transitively."""
    seen = seen if seen is not None else set()
    if src in seen or not os.path.exists(src):
        return seen
    seen.add(src)
    with open(src) as f:
        for line in f:
            line = line.strip()
            if line.startswith('#include "'):
                _deps(os.path.normpath(os.path.join(os.path.dirname(src), line.split('"')[1])), seen)
    return seen


def _stale(src: str) -> bool:
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in _deps(src))


def build(verbose: bool = True, incremental: bool = False) -> str:
    """Compile every source (with `incremental`, only those newer than their object file, headers
    included) and link the shared library; returns its path."""
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    todo = [s for s in srcs if _stale(s)] if incremental else srcs
    if todo:
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(todo))) as ex:
            list(ex.map(_compile, todo))
    from relax_amd import check_ring_asm

    ring = [os.path.basename(s) for s in todo if os.path.basename(s) in check_ring_asm.SOURCES]
    if ring:
        # those kernels wait for their inline-assembly loads by hand: verify the generated code
        try:
            check_ring_asm.main(HIPCC, [f for f in FLAGS if f != "-fPIC"], ring)
        except Exception:
            for name in ring:  # an incremental build must not take the refused objects for up to date
                os.remove(os.path.join(OBJDIR, name + ".o"))
            raise
    for lib, want in ((LIB, False), (CALIBRATE_LIB, True)):
        objs = [os.path.join(OBJDIR, os.path.basename(s) + ".o") for s in srcs
                if (os.path.basename(s) in CALIBRATE_SOURCES) == want]
        subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs])
    if verbose:
        print(f"built {LIB}: compiled {len(todo)} of {len(srcs)} sources", flush=True)
    return LIB


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
