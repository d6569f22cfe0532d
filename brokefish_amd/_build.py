"""Build glue: compiles the native pieces in-tree with hipcc / gcc.

Plays the role of the reference's extension loader (brokefish/nn/_build.py:149-190) for
gfx950.  Two shared libraries live next to this file:

* ``libbrokefish_hip.so``  -- the HIP kernels and the C-ABI of ``include/brokefish_hip.h``
* ``libbf_chessgen.so``    -- the CPU rules engine that makes synthetic positions
"""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
HIP_LIB = os.path.join(HERE, "libbrokefish_hip.so")
CHESSGEN_LIB = os.path.join(HERE, "libbf_chessgen.so")

HIP_SOURCES = ["bf_eval.hip"]
# -ffp-contract=off: the kernel's fp32 arithmetic is specified operation by operation
# (fused multiply-adds are written explicitly), so the compiler must not fuse on its own.
# The packed-fp32 feature is disabled so no v_pk_*_f32 instructions are generated.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-ffp-contract=off", "-fno-fast-math",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def hipcc_path() -> str:
    p = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(p):
        raise RuntimeError("hipcc not found; the evaluator needs ROCm to build")
    return p


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"build failed: {' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    return r


def build_hip(verbose: bool = False, extra=()) -> str:
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    cmd = [hipcc_path()] + HIPCC_FLAGS + list(extra) + ["-I", INCLUDE, "-I", CSRC, "-o", HIP_LIB] + srcs
    r = _run(cmd)
    if verbose:
        print(r.stderr)
    return HIP_LIB


def build_chessgen() -> str:
    _run(["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", CHESSGEN_LIB,
          os.path.join(CSRC, "chessgen.c")])
    return CHESSGEN_LIB


def build_all(verbose: bool = False) -> None:
    build_chessgen()
    build_hip(verbose)
