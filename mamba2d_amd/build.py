"""Builds the native parts in-tree: libm2dscan.so (pure HIP, C ABI) and the PyTorch shim.

    python -m mamba2d_amd.build            # both
    python -m mamba2d_amd.build --lib      # only the HIP library

hipcc cross-compiles for gfx950 without a GPU.  Nothing here runs at import time: the
package loads what has been built and fails loudly when it is missing.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libm2dscan.so")
SHIM = os.path.join(HERE, "_m2d_torch.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-inline-asm",
]


def build_lib(verbose: bool = True) -> str:
    srcs = [os.path.join(HERE, "csrc", n) for n in ("m2dscan.hip", "m2dproj.hip")]
    cmd = ["hipcc", *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-o", LIB, *srcs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
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
