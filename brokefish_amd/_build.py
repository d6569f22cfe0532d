"""Build glue: compiles the native pieces in-tree with hipcc / gcc.

Plays the role of the reference's extension loader (brokefish/nn/_build.py:149-190) for
gfx950.  Two shared libraries live next to this file:

* ``libbrokefish_hip.so``  -- the HIP kernels and the C-ABI of ``include/brokefish_hip.h``
* ``libbf_chessgen.so``    -- the CPU rules engine that makes synthetic positions
* ``_bf_torch.so``         -- the PyTorch extension module over that C-ABI (tensors in, current stream)
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
TORCH_EXT = os.path.join(HERE, "_bf_torch.so")

# the four-positions-per-workgroup kernels take minutes each to compile (the e4m3 ones five): they
# go first so that the pool's last minutes are not spent waiting for one of them alone
HIP_SOURCES = ["bf_variant_prod_fp8.hip", "bf_variant_taps_fp8.hip", "bf_variant_prof_fp8.hip",
               "bf_variant_prod.hip", "bf_variant_taps.hip", "bf_variant_prof.hip",
               "bf_variant_board512.hip", "bf_variant_board512_taps.hip", "bf_variant_board512_prof.hip",
               "bf_host.hip", "bf_expand.hip", "bf_movegen.hip", "bf_probe.hip",
               "bf_variant_board256.hip", "bf_variant_board256_taps.hip", "bf_variant_board256_prof.hip",
               "bf_variant_twin256.hip", "bf_variant_twin256_taps.hip", "bf_variant_twin256_prof.hip",
               "bf_variant_twin256_fp8.hip", "bf_variant_twin256_fp8_taps.hip", "bf_variant_twin256_fp8_prof.hip",
               "bf_variant_board256_fp8.hip", "bf_variant_board256_fp8_taps.hip", "bf_variant_board256_fp8_prof.hip",
               "bf_variant_octo512.hip", "bf_variant_octo512_taps.hip", "bf_variant_octo512_prof.hip",
               "bf_variant_octo256_fp8.hip", "bf_variant_octo256_fp8_taps.hip", "bf_variant_octo256_fp8_prof.hip",
               "bf_variant_duo256.hip", "bf_variant_duo256_taps.hip", "bf_variant_duo256_prof.hip",
               "bf_variant_duo256_fp8.hip", "bf_variant_duo256_fp8_taps.hip", "bf_variant_duo256_fp8_prof.hip",
               "bf_variant_solo256.hip", "bf_variant_solo256_taps.hip", "bf_variant_solo256_prof.hip"]
# -ffp-contract=off: the kernel's fp32 arithmetic is specified operation by operation
# (fused multiply-adds are written explicitly), so the compiler must not fuse on its own.
# The packed-fp32 feature is disabled so no v_pk_*_f32 instructions are generated.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
               "-ffp-contract=off", "-fno-fast-math",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # the layer body is one fully unrolled straight-line block; the default
               # unroll budgets would leave the last loops rolled and their register
               # arrays in scratch memory
               "-mllvm", "-pragma-unroll-threshold=10000000", "-mllvm", "-unroll-threshold=10000000",
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
    """Compile every translation unit (in parallel: the kernel variants take minutes each)
    and link them into libbrokefish_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    # the kernels' timing experiments give wrong results by construction: never in the library
    if any("BF_EXP_" in f or "BF_TIMING_BUILD" in f for f in list(extra) + HIPCC_FLAGS):
        raise ValueError("BF_EXP_* / BF_TIMING_BUILD switches are timing experiments and must not be built into the library")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc_path()] + HIPCC_FLAGS + list(extra) + ["-I", INCLUDE, "-I", CSRC, "-c",
                                                            os.path.join(CSRC, src), "-o", obj]
        r = _run(cmd)
        if verbose:
            print(r.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(HIP_SOURCES), os.cpu_count() or 4)) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    _run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    # the extension module is compiled against this library's header: one built earlier may not
    # match the library any more, so it goes and build_torch_ext() makes the new one
    if os.path.exists(TORCH_EXT):
        os.remove(TORCH_EXT)
    return HIP_LIB


def build_chessgen() -> str:
    _run(["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", CHESSGEN_LIB,
          os.path.join(CSRC, "chessgen.c")])
    return CHESSGEN_LIB


def build_torch_ext() -> str:
    """The PyTorch extension module brokefish_amd._bf_torch (host code only: it calls the C-ABI of
    libbrokefish_hip.so, which must have been built).  The counterpart of the reference's
    ``load_extension`` (brokefish/nn/_build.py:149-190), compiled in-tree with the flags
    ``torch.utils.cpp_extension`` uses for a ROCm build."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    if not os.path.exists(HIP_LIB):
        raise RuntimeError("build the HIP library first (build_hip)")
    inc = ce.include_paths("cuda") + [sysconfig.get_paths()["include"], INCLUDE]
    libdirs = ce.library_paths("cuda")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=_bf_torch", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"]
    cmd += [f"-I{p}" for p in inc]
    cmd += [os.path.join(CSRC, "bf_torch_ext.cpp"), "-o", TORCH_EXT]
    cmd += [f"-L{p}" for p in libdirs if os.path.isdir(p)] + [f"-L{HERE}"]
    cmd += ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python", "-lbrokefish_hip",
            "-Wl,-rpath,$ORIGIN"] + [f"-Wl,-rpath,{p}" for p in libdirs if os.path.isdir(p)]
    _run(cmd)
    return TORCH_EXT


C_DRIVER = os.path.join(os.path.dirname(HERE), "tests", "abi", "c_driver")


def build_c_driver() -> str:
    """tests/abi/c_driver: a host program over the C-ABI and the HIP runtime alone (no PyTorch), for
    the GPU test that runs the library without Python.  Host code only; the library must be built."""
    _run([hipcc_path(), "-O2", "-std=c++17", "-I", INCLUDE, C_DRIVER + ".cpp", "-o", C_DRIVER,
          "-L", HERE, "-lbrokefish_hip", "-Wl,-rpath," + HERE])
    return C_DRIVER


def build_all(verbose: bool = False) -> None:
    build_chessgen()
    build_hip(verbose)
    build_torch_ext()
    build_c_driver()
