"""Build-time check of the generated gfx950 assembly for hazards that the compiler cannot see.

The scan kernels fold DPP row shifts into arithmetic instructions with inline assembly
(v_fmac_f32_dpp, v_mul_f32_dpp, v_add_f32_dpp).  The compiler's hazard recogniser does not look
inside inline assembly, so two rules of the ISA are the source's own responsibility:

* a VGPR that a DPP instruction reads through the lane shift (its src0) must not have been
  written by a vector instruction in the two preceding issue slots;
* a VGPR written by a transcendental instruction (v_exp/v_log/v_rcp/v_rsq/v_sqrt) must not be
  read by a vector instruction in the next issue slot.

The source arranges its code so that neither can happen; this module verifies it on the assembly
that was actually produced, and the build fails if it finds a violation.

It also reads the compiler's own per-kernel summary for register spills: the scan kernels are
written to fit the 256 vector registers of a wave at two waves per SIMD, and a change that pushes
one of them over the edge spills to scratch memory silently and costs tens of percent.
"""
from __future__ import annotations

import re

_DPP = re.compile(r"(v_\w+_dpp)\s+v(\d+),\s*v(\d+),\s*v(\d+)")
_WRITE = re.compile(r"(v_\w+|ds_read\w*|global_load\w*|scratch_load\w*|buffer_load\w*)\s+(?:v\[(\d+):(\d+)\]|v(\d+))")
_TRANS = re.compile(r"v_(exp|log|rcp|rsq|sqrt)_f32")
_NOP = re.compile(r"s_nop (\d+)")
_KERNEL = re.compile(r"^(_Z\w+):")


def _written(inst: str) -> set:
    m = _WRITE.match(inst)
    if not m:
        return set()
    if m.group(2) is not None:
        return set(range(int(m.group(2)), int(m.group(3)) + 1))
    return {int(m.group(4))}


def check_text(text: str):
    """Returns (number of DPP instructions seen, list of (kernel, producer, consumer) violations)."""
    kernel, hist, ndpp, bad = None, [], 0, []
    for line in text.splitlines():
        t = line.strip()
        k = _KERNEL.match(t)
        if k:
            kernel, hist = k.group(1), []
            continue
        if not line.startswith("\t") or not t or t[0] in ".;":
            continue
        m = _DPP.match(t)
        if m:
            ndpp += 1
            regs = {int(m.group(2)), int(m.group(3)), int(m.group(4))}
            shifted = int(m.group(3))
            slots = 0
            for prev, width in reversed(hist):
                w = _written(prev)
                if slots < 1 and _TRANS.match(prev) and w & regs:
                    bad.append((kernel, prev, t))
                    break
                if slots < 2 and prev.startswith("v_") and shifted in w:
                    bad.append((kernel, prev, t))
                    break
                slots += width
                if slots >= 2:
                    break
        n = _NOP.match(t)
        hist.append((t, int(n.group(1)) + 1 if n else 1))
        del hist[:-8]
    return ndpp, bad


def check_file(path: str):
    with open(path) as f:
        return check_text(f.read())


_SCRATCH = re.compile(r"^\s*\.amdhsa_private_segment_fixed_size\s+(\d+)")
_HSA_KERNEL = re.compile(r"^\s*\.amdhsa_kernel\s+(\S+)")


def spilling_kernels(text: str):
    """Kernels whose descriptor asks for scratch memory: list of (kernel, bytes per lane)."""
    out, kernel = [], None
    for line in text.splitlines():
        k = _HSA_KERNEL.match(line)
        if k:
            kernel = k.group(1)
            continue
        m = _SCRATCH.match(line)
        if m and int(m.group(1)) > 0:
            out.append((kernel, int(m.group(1))))
    return out


_LABEL = re.compile(r"^(_Z\w+):")
_SCRATCH_OP = re.compile(r"^\s+scratch_(load|store)")


def scratch_accesses(text: str):
    """Number of scratch loads and stores in the body of every kernel: {kernel: count}.  A kernel whose descriptor asks
    for scratch memory and which has none of them only parks scalar registers in lanes of a vector register; the
    compiler reserves a few bytes for that register and never touches them."""
    out, kernel = {}, None
    for line in text.splitlines():
        m = _LABEL.match(line)
        if m:
            kernel = m.group(1)
            out.setdefault(kernel, 0)
        elif kernel and _SCRATCH_OP.match(line):
            out[kernel] += 1
    return out


def spills_in_file(path: str):
    with open(path) as f:
        return spilling_kernels(f.read())
