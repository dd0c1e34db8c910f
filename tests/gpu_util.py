"""Helpers shared by the GPU parity tests."""
import os
import subprocess

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def build_cpp_program(name: str, force: bool = False) -> str:
    """Compiles tests/cpp/<name>.cc (host code against include/ and the shared library, HIP runtime API
    only) into tests/cpp/bin/<name> unless an up-to-date binary is there; returns its path."""
    src = os.path.join(ROOT, "tests", "cpp", name + ".cc")
    exe = os.path.join(ROOT, "tests", "cpp", "bin", name)
    libdir = os.path.join(ROOT, "relax_amd")
    if force or not os.path.exists(exe) or os.path.getmtime(exe) < os.path.getmtime(src):
        os.makedirs(os.path.dirname(exe), exist_ok=True)
        subprocess.check_call(["g++", "-std=c++17", "-O1", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
                               "-I", "/opt/rocm/include", src, "-o", exe, "-L", libdir, "-lrelax_amd_wq",
                               "-L", "/opt/rocm/lib", "-lamdhip64", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"])
    return exe


def dev(a: np.ndarray) -> torch.Tensor:
    """numpy -> device tensor (uint32 travels as int32: same bytes)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).cuda()


def host(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


# Tolerance of the fused kernels against the fp32-accumulated oracle.  The
# requirement is a maximum relative error of 1e-2; the reference's own tests use
# assert_allclose(rtol=1e-2, atol=1e-2) (tests/python/relax/test_codegen_cutlass.py:1609).
# That absolute term is meant for outputs of magnitude O(1); for larger outputs it is
# scaled by their rms (at |y| ~ 50 one fp16 ulp is already 0.03).  All kernels
# accumulate in fp32 and differ from the oracle only in summation order and, for the
# streaming kernels, in applying the scale after the sum instead of rounding every
# weight to fp16 first, so a 10x tighter normalised bound is asserted as well.
RTOL = 1e-2
ATOL = 1e-2
NORM_TOL = 1e-3


def assert_close(got: np.ndarray, ref: np.ndarray, what: str = ""):
    g = got.astype(np.float64)
    r = ref.astype(np.float64)
    assert g.shape == r.shape, (what, g.shape, r.shape)
    assert np.all(np.isfinite(g)), what
    err = np.abs(g - r)
    atol = ATOL * max(1.0, float(np.sqrt(np.mean(r * r))))
    bad = err > RTOL * np.abs(r) + atol
    assert not bad.any(), f"{what}: {bad.sum()} elements outside rtol={RTOL} atol={ATOL}; max err {err.max()}"
    # An output is rounded to fp16 once, or twice where a residual is added to the rounded
    # y + bias: two results of the same arithmetic in another summation order can then lie
    # two fp16 steps apart, three where the residual takes the sum down one binade (a step of
    # the binade above and one of its own), which near the largest output is 1.0e-3..1.5e-3
    # of it.  Such an element passes; anything further off must meet the normalised bound.
    scale = max(np.abs(r).max(), 1e-6)
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    far = err > 3.0 * ulp
    worst = float((err * far).max()) if far.any() else 0.0
    assert worst / scale <= NORM_TOL, f"{what}: normalised max error {worst / scale:.3e} > {NORM_TOL}"
