"""CPU oracle for the Mamba2D wavefront 2-D selective scan -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the ``cpu_baseline`` leg of the benchmark may import
this module.  The shipped package never does: its operators fail loudly when the HIP
library is missing.

Three independent restatements of the reference (cocoalex00/Mamba2D) live here:

* ``CScan`` -- ctypes front end of ``m2d_oracle.c`` (scalar C, fp64 and fp32), which
  follows the reference's data flow: ``models/kernels/wf_cuda/wf_cuda.cu:40-69``
  (forward), ``:108-160`` (adjoint), ``models/kernels/wavefront_cuda.py:102-139``
  (parameter gradients) and ``:146-196`` (autograd data flow).
* ``scan_forward_torch`` -- a differentiable, diagonal-vectorised PyTorch version of
  the forward recurrence; ``torch.autograd`` through it is the independent check of
  the explicit adjoint (the reference backward is the exact adjoint of its forward).
* ``scan_forward_loops`` -- a pure-Python triple loop for tiny inputs.

``proj_params_ref`` / ``wavefront_scan_ref`` restate the projection step and the entry
point (``wavefront_cuda.py:63-95`` and ``:315-347``) with stock torch ops.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libm2d_oracle.so")


def build(force: bool = False) -> str:
    """Compile ``m2d_oracle.c`` into ``libm2d_oracle.so`` next to it."""
    src = os.path.join(_HERE, "m2d_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(
            ["gcc", "-O2", "-fPIC", "-fopenmp", "-std=c11", "-fno-fast-math", "-shared",
             "-o", _SO, src, "-lm"])
    return _SO


# --------------------------------------------------------------------------------------
# seeded synthetic inputs (fixed draw order, reference layout)
# --------------------------------------------------------------------------------------
INPUT_NAMES = ("x", "deltaT", "deltaL", "AT", "AL", "BT", "BL", "C", "D")


def make_inputs(B, H, W, E, N=16, seed=0, dtype=torch.float32, with_dy=True):
    """x~N(0,1); delta=softplus(N(0,1)); A=-exp(U(-4,0)); B,C~N(0,1); D~N(0,1); dy~N(0,1).

    Drawn in fp32 on the CPU in a fixed order, then rounded to ``dtype``.
    Returns a dict of CPU tensors in the reference's channel-last layout.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    out = {}
    out["x"] = r(B, H, W, E)
    out["deltaT"] = F.softplus(r(B, H, W, E))
    out["deltaL"] = F.softplus(r(B, H, W, E))
    out["AT"] = -torch.exp(-4.0 * torch.rand(E, N, generator=g, dtype=torch.float32))
    out["AL"] = -torch.exp(-4.0 * torch.rand(E, N, generator=g, dtype=torch.float32))
    out["BT"] = r(B, H, W, N)
    out["BL"] = r(B, H, W, N)
    out["C"] = r(B, H, W, N)
    out["D"] = r(E)
    if with_dy:
        out["dy"] = r(B, H, W, E)
    return {k: v.to(dtype).contiguous() for k, v in out.items()}


# --------------------------------------------------------------------------------------
# C oracle
# --------------------------------------------------------------------------------------
class CScan:
    """ctypes wrapper around libm2d_oracle.so (numpy in, numpy out)."""

    GRADS = ("d_x", "d_deltaT", "d_deltaL", "d_AT", "d_AL", "d_BT", "d_BL", "d_C", "d_D")

    def __init__(self):
        self.lib = ctypes.CDLL(build())
        self.lib.m2d_oracle_threads.restype = ctypes.c_int

    @property
    def threads(self) -> int:
        return int(self.lib.m2d_oracle_threads())

    def set_threads(self, n: int) -> None:
        self.lib.m2d_oracle_set_threads(ctypes.c_int(n))

    @staticmethod
    def _np(t, dt):
        if isinstance(t, torch.Tensor):
            t = t.detach().cpu().to(torch.float64 if dt == np.float64 else torch.float32).numpy()
        return np.ascontiguousarray(t, dtype=dt)

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p)

    def forward(self, x, deltaT, deltaL, AT, AL, BT, BL, C, D, dtype=np.float64, want_hs=False):
        dt = np.dtype(dtype).type
        suf = "f64" if dt == np.float64 else "f32"
        a = [self._np(t, dt) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]
        B, H, W, E = a[0].shape
        N = a[3].shape[1]
        hs = np.empty((B, H, W, E, N), dt)
        y = np.empty((B, H, W, E), dt)
        rc = getattr(self.lib, "m2d_oracle_fwd_" + suf)(
            B, H, W, E, N, *[self._p(v) for v in a], self._p(hs), self._p(y))
        if rc:
            raise ValueError(f"Wavefront scan kernel requires spatial dims > 1. Got H={H}, W={W}.")
        return (y, hs) if want_hs else y

    def backward(self, x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy, dtype=np.float64,
                 want_intermediates=False):
        dt = np.dtype(dtype).type
        suf = "f64" if dt == np.float64 else "f32"
        a = [self._np(t, dt) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy)]
        B, H, W, E = a[0].shape
        N = a[3].shape[1]
        big = [np.empty((B, H, W, E, N), dt) for _ in range(4)]  # hs, dBX, dDAT, dDAL
        outs = [np.empty(s, dt) for s in ((B, H, W, E),) * 3 + ((E, N),) * 2 +
                ((B, H, W, N),) * 3 + ((E,),)]
        rc = getattr(self.lib, "m2d_oracle_bwd_" + suf)(
            B, H, W, E, N, *[self._p(v) for v in a], *[self._p(v) for v in big],
            *[self._p(v) for v in outs])
        if rc == 1:
            raise ValueError(f"Wavefront scan kernel requires spatial dims > 1. Got H={H}, W={W}.")
        if rc:
            raise MemoryError("oracle backward: allocation failed")
        res = dict(zip(self.GRADS, outs))
        if want_intermediates:
            res.update(hs=big[0], dBX=big[1], dDAT=big[2], dDAL=big[3])
        return res


# --------------------------------------------------------------------------------------
# independent restatements used to pin the C oracle
# --------------------------------------------------------------------------------------
def scan_forward_loops(x, deltaT, deltaL, AT, AL, BT, BL, C, D):
    """Pure-Python loops in row-major cell order (tiny inputs only). Returns (y, hs)."""
    import math
    x, deltaT, deltaL, AT, AL, BT, BL, C, D = [
        np.asarray(t, dtype=np.float64) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]
    Bn, H, W, E = x.shape
    N = AT.shape[1]
    hs = np.zeros((Bn, H, W, E, N))
    y = np.zeros((Bn, H, W, E))
    for b in range(Bn):
        for i in range(H):
            for j in range(W):
                for e in range(E):
                    acc = 0.0
                    for n in range(N):
                        left = (math.exp(deltaL[b, i, j, e] * AL[e, n]) * hs[b, i, j - 1, e, n]
                                if j > 0 else 0.0) + deltaL[b, i, j, e] * BL[b, i, j, n] * x[b, i, j, e]
                        top = (math.exp(deltaT[b, i, j, e] * AT[e, n]) * hs[b, i - 1, j, e, n]
                               if i > 0 else 0.0) + deltaT[b, i, j, e] * BT[b, i, j, n] * x[b, i, j, e]
                        if i == 0:
                            v = left          # first row (and the origin): L direction only
                        elif j == 0:
                            v = top           # first column: T direction only
                        else:
                            v = 0.5 * (left + top)
                        hs[b, i, j, e, n] = v
                        acc += v * C[b, i, j, n]
                    y[b, i, j, e] = acc + x[b, i, j, e] * D[e]
    return y, hs


def scan_core_torch(gT, gL, uT, uL):
    """hs (B,H,W,E,N) from explicit gates and input terms, each (B,H,W,E,N); differentiable."""
    _, H, W = gT.shape[:3]
    rows = [[None] * W for _ in range(H)]
    for d in range(H + W - 1):
        for i in range(max(0, d - W + 1), min(d, H - 1) + 1):
            j = d - i
            if i == 0 and j == 0:
                h = uL[:, 0, 0]
            elif i == 0:
                h = gL[:, i, j] * rows[i][j - 1] + uL[:, i, j]
            elif j == 0:
                h = gT[:, i, j] * rows[i - 1][j] + uT[:, i, j]
            else:
                h = 0.5 * (gL[:, i, j] * rows[i][j - 1] + uL[:, i, j]
                           + gT[:, i, j] * rows[i - 1][j] + uT[:, i, j])
            rows[i][j] = h
    return torch.stack([torch.stack(r, dim=1) for r in rows], dim=1)


def scan_forward_torch(x, deltaT, deltaL, AT, AL, BT, BL, C, D, return_hs=False):
    """Differentiable forward, one update per cell in anti-diagonal order, out-of-place.

    Works in the dtype of ``x`` (use fp64 for oracle duty).  ``torch.autograd`` through
    this function yields all nine gradients of the fused operator.
    """
    gT = torch.exp(deltaT.unsqueeze(-1) * AT)                       # (B,H,W,E,N)
    gL = torch.exp(deltaL.unsqueeze(-1) * AL)
    uT = (deltaT.unsqueeze(-1) * BT.unsqueeze(-2)) * x.unsqueeze(-1)
    uL = (deltaL.unsqueeze(-1) * BL.unsqueeze(-2)) * x.unsqueeze(-1)
    hs = scan_core_torch(gT, gL, uT, uL)
    y = (hs * C.unsqueeze(-2)).sum(-1) + x * D
    return (y, hs) if return_hs else y


def scan_grads_autograd(inputs: dict, dtype=torch.float64):
    """y and the nine gradients by autograd through ``scan_forward_torch``."""
    leaves = [inputs[k].detach().to(dtype).clone().requires_grad_(True) for k in INPUT_NAMES]
    y = scan_forward_torch(*leaves)
    grads = torch.autograd.grad(y, leaves, inputs["dy"].to(dtype))
    return y.detach(), dict(zip(CScan.GRADS, [g.detach() for g in grads]))


# --------------------------------------------------------------------------------------
# projections and entry point with stock torch ops
# --------------------------------------------------------------------------------------
def proj_params_ref(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b):
    """wavefront_cuda.py:63-95 -- split order [R, R, N, N, N], everything cast to x.dtype."""
    N = AT_log.shape[1]
    R = dt_projT_w.shape[1]
    AT = -torch.exp(AT_log.float())
    AL = -torch.exp(AL_log.float())
    z = F.linear(x, x_proj_w)
    dT, dL, BT, BL, C = torch.split(z, [R, R, N, N, N], dim=-1)
    dT = F.softplus(F.linear(dT, dt_projT_w, dt_projT_b))
    dL = F.softplus(F.linear(dL, dt_projL_w, dt_projL_b))
    return tuple(t.to(x.dtype) for t in (dT, dL, AT, AL, BT, BL, C))


def wavefront_scan_ref(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w,
                       dt_projL_b, D, compute_dtype=torch.float64):
    """Entry point restated (wavefront_cuda.py:315-347): casts, projections, scan.

    The projections run in ``x.dtype`` as in the reference; the scan itself is evaluated
    in ``compute_dtype`` on the (rounded) projection outputs.
    """
    _, H, W, _ = x.shape
    if H < 2 or W < 2:
        raise ValueError(f"Wavefront scan kernel requires spatial dims > 1. Got H={H}, W={W}.")
    cast = lambda t: t.to(x.dtype)
    dT, dL, AT, AL, BT, BL, C = proj_params_ref(
        x, AT_log, AL_log, cast(x_proj_w), cast(dt_projT_w), cast(dt_projT_b),
        cast(dt_projL_w), cast(dt_projL_b))
    up = lambda t: t.to(compute_dtype)
    y = scan_forward_torch(up(x), up(dT), up(dL), up(AT), up(AL), up(BT), up(BL), up(C),
                           up(cast(D)))
    return y


class _RoundBothWays(torch.autograd.Function):
    """Rounds a float64 tensor to bfloat16 values on the way forward and its gradient on the way back:
    what a bf16 tensor between two stock operators does to the reference's data flow."""

    @staticmethod
    def forward(ctx, t):
        return t.bfloat16().double()

    @staticmethod
    def backward(ctx, g):
        return g.bfloat16().double()


PARAM_ORDER = ("AT_log", "AL_log", "x_proj_w", "dt_projT_w", "dt_projT_b", "dt_projL_w", "dt_projL_b", "D")


def entry_point_reference(x, params, dy, round_intermediates=False):
    """The entry point (wavefront_cuda.py:315-347) in float64 for activations of x.dtype: the weights
    are rounded to x.dtype first, as the reference's casts do (:327-332, and :88-94 for A), and every
    product, the softplus and the scan are evaluated in float64.  With ``round_intermediates`` the
    outputs of the three linear layers and of the softplus, and the gradients that flow back through
    them, are rounded to bfloat16 as they are when the reference runs these stock operators on bf16
    tensors (its own data flow, with exact arithmetic inside every operator).

    Returns y, the nine gradients in the entry point's argument order, and for each of the five
    projection weights the sum of the absolute values of the terms its gradient adds up
    (``scales``): d_w = sum_p a_p b_p can cancel to far below sum_p |a_p b_p|, and an error bound that
    is relative per term is relative to the latter.
    """
    dt = x.dtype
    rw = lambda t: t.to(dt).double()
    leaves = [x.double().requires_grad_(True)]
    leaves += [(params[k].double() if k in ("AT_log", "AL_log") else rw(params[k])).requires_grad_(True) for k in PARAM_ORDER]
    xx, ATl, ALl, xw, tw, tb, lw, lb, D = leaves
    N, R = ATl.shape[1], tw.shape[1]
    rb = _RoundBothWays.apply if round_intermediates else (lambda t: t)
    AT = -torch.exp(ATl)
    AL = -torch.exp(ALl)
    if dt != torch.float64:   # A reaches the scan in x.dtype
        AT = AT + (AT.detach().to(dt).double() - AT.detach())
        AL = AL + (AL.detach().to(dt).double() - AL.detach())
    z = rb(F.linear(xx, xw))
    z.retain_grad()
    rT, rL, BT, BL, C = torch.split(z, [R, R, N, N, N], dim=-1)
    preT = rb(F.linear(rT, tw, tb))
    preL = rb(F.linear(rL, lw, lb))
    preT.retain_grad()
    preL.retain_grad()
    y = scan_forward_torch(xx, rb(F.softplus(preT)), rb(F.softplus(preL)), AT, AL, BT, BL, C, D)
    y.backward(dy.double())
    grads = [t.grad.detach() for t in leaves]
    flat = lambda t: t.detach().reshape(-1, t.shape[-1]).abs()
    scales = {
        "x_proj_w": flat(z.grad).t() @ flat(xx),
        "dt_projT_w": flat(preT.grad).t() @ flat(rT), "dt_projT_b": flat(preT.grad).sum(0),
        "dt_projL_w": flat(preL.grad).t() @ flat(rL), "dt_projL_b": flat(preL.grad).sum(0),
    }
    return y.detach(), grads, scales


# --------------------------------------------------------------------------------------
# error metrics used by every parity test
# --------------------------------------------------------------------------------------
def rel_err(a, b):
    """Tensor-normalised max error: max|a-b| / max|b|."""
    a = torch.as_tensor(np.asarray(a) if not isinstance(a, torch.Tensor) else a).double().cpu()
    b = torch.as_tensor(np.asarray(b) if not isinstance(b, torch.Tensor) else b).double().cpu()
    den = b.abs().max().item()
    return (a - b).abs().max().item() / (den if den > 0 else 1.0)


def elem_rel_err(a, b, eps=1e-3):
    """Elementwise |a-b| / (|b| + eps*max|b|), maximum over the tensor."""
    a = torch.as_tensor(np.asarray(a) if not isinstance(a, torch.Tensor) else a).double().cpu()
    b = torch.as_tensor(np.asarray(b) if not isinstance(b, torch.Tensor) else b).double().cpu()
    den = b.abs().max().item()
    return ((a - b).abs() / (b.abs() + eps * (den if den > 0 else 1.0))).max().item()
