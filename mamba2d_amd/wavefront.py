"""Scan operator with the reference's Python surface, backed by the HIP library.

Mirrors ``models/kernels/wavefront_cuda.py`` of cocoalex00/Mamba2D: the same public names
(``wavefront_scan_cuda``, ``wf_cuda_fn_pr``, ``wf_cuda_fn_fr``, ``proj_params``), the same
argument order and the same error behaviour, so that ``M2DBlock.ssm``
(``models/mamba2d.py:180-188``) runs unchanged.  Differences, all internal:

* ``mamba2d::wf_fwd`` / ``mamba2d::wf_bwd`` and the tensor algebra around them
  (``wavefront_cuda.py:152-156``, ``:169-194``) are replaced by two fused operators,
  ``m2dscan::scan_fwd`` and ``m2dscan::scan_bwd`` (csrc/m2d_torch.cpp -> include/m2dscan.h);
  the (B,H,W,E,N) state tensor never exists in memory.
* state and accumulation are fp32 also for bf16 tensors.

There is no fallback path: importing this module raises if the native parts are not built.
"""
from __future__ import annotations

import ctypes
import os

import torch
import torch.nn.functional as F

from . import cabi

_SHIM = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_m2d_torch.so")
if not os.path.exists(_SHIM):
    raise ImportError(f"{_SHIM} is missing: build it with `python -m mamba2d_amd.build` "
                      "(there is no CPU or eager fallback for the scan)")
torch.ops.load_library(_SHIM)

scan_fwd_op = torch.ops.m2dscan.scan_fwd
scan_bwd_op = torch.ops.m2dscan.scan_bwd

# Keep the forward's anti-diagonal checkpoints for the backward (faster backward, more saved
# memory) or rebuild them inside the backward (nothing saved beyond the inputs, like the
# reference's partial recomputation).  Module-level switch, read at forward time.
SAVE_CHECKPOINTS = os.environ.get("M2D_SAVE_CHECKPOINTS", "1") != "0"


def _ckpt_bytes(x, N, flip=False) -> int:
    d = cabi.make_desc(x, N, flip)
    return int(cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d)))


@torch.library.register_fake("m2dscan::scan_fwd")
def _scan_fwd_fake(x, deltaT, deltaL, AT, AL, BT, BL, C, D, save_ckpt, flip):
    n = _ckpt_bytes(x, AT.shape[1]) if save_ckpt else 1
    return torch.empty_like(x), x.new_empty((max(n, 1),), dtype=torch.uint8)


@torch.library.register_fake("m2dscan::scan_bwd")
def _scan_bwd_fake(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy, ckpt, flip):
    return [torch.empty_like(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]


def proj_params(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b):
    """SSM parameters from x (reference ``wavefront_cuda.py:63-95``): x_proj, split
    [R, R, N, N, N], two dt projections with softplus, A = -exp(A_log); all cast to x.dtype."""
    d_state = AT_log.shape[1]
    dt_rank = dt_projT_w.shape[1]
    AT = -torch.exp(AT_log.float())
    AL = -torch.exp(AL_log.float())
    delta2BC = F.linear(x, x_proj_w)
    deltaT, deltaL, BT, BL, C = torch.split(delta2BC, [dt_rank, dt_rank, d_state, d_state, d_state], dim=-1)
    deltaT = F.softplus(F.linear(deltaT, dt_projT_w, dt_projT_b))
    deltaL = F.softplus(F.linear(deltaL, dt_projL_w, dt_projL_b))
    dt = x.dtype
    return (deltaT.to(dt), deltaL.to(dt), AT.to(dt), AL.to(dt), BT.to(dt), BL.to(dt), C.to(dt))


def _c(t):
    return t if t.is_contiguous() else t.contiguous()


class wf_cuda_fn_pr(torch.autograd.Function):
    """Scan + output projection on precomputed parameters (reference ``wavefront_cuda.py:146-196``).

    ``apply(x, deltaT, deltaL, AT, AL, BT, BL, C, D[, flip]) -> y``; backward returns the nine
    gradients in input order.  ``flip=True`` (not in the reference) scans from the bottom-right
    corner, which equals flipping every spatial tensor before and y after
    (``models/mamba2d.py:163-173``) without the copies."""

    @staticmethod
    def forward(ctx, x, deltaT, deltaL, AT, AL, BT, BL, C, D, flip=False):
        args = [_c(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]
        # (grad mode is always off inside forward(); needs_input_grad is what tells training from inference)
        keep = SAVE_CHECKPOINTS and any(ctx.needs_input_grad)
        y, ck = scan_fwd_op(*args, keep, bool(flip))
        ctx.save_for_backward(*args, ck)
        ctx.flip = bool(flip)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        *args, ck = ctx.saved_tensors
        dy = _c(grad_output.to(args[0].dtype))
        return (*scan_bwd_op(*args, dy, ck, ctx.flip), None)


class wf_cuda_fn_fr(torch.autograd.Function):
    """Full-recompute variant (reference ``wavefront_cuda.py:199-313``): only x and the weights
    are saved; projections, checkpoints and states are rebuilt in the backward."""

    @staticmethod
    def forward(ctx, x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D, flip=False):
        with torch.no_grad():
            deltaT, deltaL, AT, AL, BT, BL, C = proj_params(
                x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b)
            y, _ = scan_fwd_op(_c(x), _c(deltaT), _c(deltaL), _c(AT), _c(AL), _c(BT), _c(BL), _c(C), _c(D),
                               False, bool(flip))
        ctx.save_for_backward(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D)
        ctx.flip = bool(flip)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D = ctx.saved_tensors
        dy = _c(grad_output.to(x.dtype))
        with torch.enable_grad():
            leaves = [t.detach().requires_grad_(True) for t in
                      (x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b)]
            deltaT, deltaL, AT, AL, BT, BL, C = proj_params(*leaves)
        det = [_c(t.detach()) for t in (deltaT, deltaL, AT, AL, BT, BL, C)]
        none = x.new_empty((1,), dtype=torch.uint8)
        d_x_scan, d_dT, d_dL, d_AT, d_AL, d_BT, d_BL, d_C, d_D = scan_bwd_op(
            _c(x), det[0], det[1], det[2], det[3], det[4], det[5], det[6], _c(D), dy, none, ctx.flip)
        grads = torch.autograd.grad([deltaT, deltaL, BT, BL, C, AT, AL], leaves,
                                    [d_dT, d_dL, d_BT, d_BL, d_C, d_AT, d_AL])
        d_x = d_x_scan + grads[0]   # d_x_scan already contains dy*D
        return (d_x, *grads[1:], d_D, None)


def wavefront_scan_cuda(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D,
                        recomp="partial", *, flip=False):
    """Entry point with the reference's signature (``wavefront_cuda.py:315-347``).

    recomp: 'partial' computes the projections once (autograd-tracked) and runs the scan on them;
            'full' recomputes the projections in the backward (minimal saved memory).
    flip:   (not in the reference) scan from the bottom-right corner by index arithmetic.
    """
    _, H, W, _ = x.shape
    if H < 2 or W < 2:
        raise ValueError(f"Wavefront scan kernel requires spatial dims > 1. Got H={H}, W={W}.")

    x_proj_w = x_proj_w.to(x.dtype)
    dt_projT_w = dt_projT_w.to(x.dtype)
    dt_projT_b = dt_projT_b.to(x.dtype)
    dt_projL_w = dt_projL_w.to(x.dtype)
    dt_projL_b = dt_projL_b.to(x.dtype)
    D = D.to(x.dtype)

    if recomp == "partial":
        deltaT, deltaL, AT, AL, BT, BL, C = proj_params(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b,
                                                        dt_projL_w, dt_projL_b)
        return wf_cuda_fn_pr.apply(x, deltaT, deltaL, AT, AL, BT, BL, C, D, flip)
    if recomp == "full":
        return wf_cuda_fn_fr.apply(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w,
                                   dt_projL_b, D, flip)
    raise ValueError(f"Unknown recomputation mode, got {recomp}...")
