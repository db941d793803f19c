"""Builds the native parts in-tree: libm2dscan.so (pure HIP, C ABI) and the PyTorch shim.

    python -m mamba2d_amd.build            # both
    python -m mamba2d_amd.build --lib      # only the HIP library

hipcc cross-compiles for gfx950 without a GPU.  Nothing here runs at import time: the
package loads what has been built and fails loudly when it is missing.
"""
from __future__ import annotations

import glob
import os
import re
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libm2dscan.so")
SHIM = os.path.join(HERE, "_m2d_torch.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-inline-asm",
]

# Source -> flags of its own.  The scan kernels are long straight-line VALU code at two waves per
# SIMD: the iterative ILP scheduler orders the backward kernel 4 % faster than the default one
# (0.92 -> 0.88 ms at B=128, E=64, 56x56, bf16) and costs the forward kernel 2 %.  The projection
# kernels are memory-bound and do better with the default scheduler.
SOURCES = {
    "m2dscan.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"],
    "m2dproj.hip": [],
    "m2dblock.hip": [],
    "m2dcompat.hip": [],
}


# Kernels that may keep a few values in scratch memory, and how many bytes per lane.  Only the backward kernel of
# 8 waves in its replaying form (m2d_bwd_kernel<..., 8, true>: a checkpoint interval of 8 or 16 steps, not the
# default): the same sweep as the default kernel, which fills all 256 registers, plus the addresses of the replay.
# It reloads two to nine values a few times per block of steps; every other kernel must not spill at all.
SPILL_ALLOWANCE = [(re.compile(r"m2d_bwd_kernelI\w*Li8ELb1E\w*EEv"), 64)]   # (<..., 8 waves, REPLAY = true, snapshot type>)

# A kernel that runs out of scalar registers parks some in lanes of a vector register; the compiler then reserves a
# few bytes of scratch for that register without ever storing it.  Allowed up to this many bytes per lane, and only
# where the kernel has no scratch load or store at all.
UNTOUCHED_SCRATCH = 64


def build_lib(verbose: bool = True) -> str:
    """Compiles the HIP sources into libm2dscan.so.  The device assembly of the same compile is
    kept (-save-temps) and checked for the hazards that inline assembly hides from the compiler
    (asmcheck.py); the library is only put in place if the check passes."""
    from . import asmcheck
    scratch = os.path.join(HERE, "build")   # in-tree, ignored by git
    os.makedirs(scratch, exist_ok=True)
    tmp = tempfile.mkdtemp(prefix="lib_", dir=scratch)

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd, cwd=tmp)

    try:
        objs = []
        for name, extra in SOURCES.items():
            obj = os.path.join(tmp, name.replace(".hip", ".o"))
            run(["hipcc", *HIPCC_FLAGS, *extra, "-save-temps=obj", "-I", os.path.join(ROOT, "include"),
                 "-c", os.path.join(HERE, "csrc", name), "-o", obj])
            objs.append(obj)
        listings = sorted(glob.glob(os.path.join(tmp, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
        if len(listings) != len(SOURCES):
            raise RuntimeError(f"expected the device assembly of {len(SOURCES)} sources, found {listings}")
        for path in listings:
            ndpp, bad = asmcheck.check_file(path)
            if verbose:
                print(f"asmcheck {os.path.basename(path)}: {ndpp} DPP instructions, {len(bad)} hazards", flush=True)
            if bad:
                raise RuntimeError("hazard between inline-assembly DPP instructions and their producers:\n" +
                                   "\n".join(f"  {k}: {p}  ->  {c}" for k, p, c in bad[:8]))
            with open(path) as f:
                accesses = asmcheck.scratch_accesses(f.read())
            spills = [(k, n) for k, n in asmcheck.spills_in_file(path)
                      if not any(pat.search(k) and n <= cap for pat, cap in SPILL_ALLOWANCE)
                      and not (n <= UNTOUCHED_SCRATCH and accesses.get(k, 1) == 0)]
            if spills:
                raise RuntimeError("kernels that spill registers to scratch memory:\n" +
                                   "\n".join(f"  {k}: {n} bytes per lane" for k, n in spills[:8]))
        out = os.path.join(tmp, "libm2dscan.so")
        run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs])
        shutil.move(out, LIB)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return LIB


def build_shim(verbose: bool = True) -> str:
    """Compile csrc/m2d_torch.cpp (host only) against torch and link it to libm2dscan.so."""
    import torch
    from torch.utils import cpp_extension as ce

    src = os.path.join(HERE, "csrc", "m2d_torch.cpp")
    inc = [f"-I{p}" for p in ce.include_paths(device_type="cuda")] + [f"-I{os.path.join(ROOT, 'include')}"]
    libdirs = ce.library_paths(device_type="cuda")
    cmd = ["hipcc", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-unused-result",
           *inc, "-o", SHIM, src,
           *[f"-L{d}" for d in libdirs], f"-L{HERE}", "-lm2dscan", "-lc10", "-lc10_hip", "-ltorch_cpu",
           "-ltorch_hip", "-ltorch", "-Wl,-rpath,$ORIGIN", *[f"-Wl,-rpath,{d}" for d in libdirs]]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return SHIM


def main(argv):
    build_lib()
    if "--lib" not in argv:
        build_shim()


if __name__ == "__main__":
    main(sys.argv[1:])
