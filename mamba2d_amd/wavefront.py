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
* the entry point runs the projections (``proj_params``, ``wavefront_cuda.py:63-95``) and their
  backward in the library's own kernels (``wf_cuda_fn_proj``); ``proj_params``, ``wf_cuda_fn_pr``
  and ``wf_cuda_fn_fr`` keep the reference's form for callers that use them directly.

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
# the reference's own pair of in-place operators, same names and mutated arguments (wavefront_cuda.py:25-57): hs is
# materialised, any number of states, float64 / float32 / bfloat16.  Not on the fast path.
wf_fwd_op = torch.ops.mamba2d.wf_fwd
wf_bwd_op = torch.ops.mamba2d.wf_bwd
proj_fwd_op = torch.ops.m2dscan.proj_fwd
proj_bwd_op = torch.ops.m2dscan.proj_bwd
layernorm_fwd_op = torch.ops.m2dscan.layernorm_fwd
dwconv3x3_fwd_op = torch.ops.m2dscan.dwconv3x3_fwd
starrelu_fwd_op = torch.ops.m2dscan.starrelu_fwd
scale_residual_fwd_op = torch.ops.m2dscan.scale_residual_fwd
scale_residual_layernorm_fwd_op = torch.ops.m2dscan.scale_residual_layernorm_fwd
rope_qknorm_fwd_op = torch.ops.m2dscan.rope_qknorm_fwd
rope_attention_fwd_op = torch.ops.m2dscan.rope_attention_fwd
mlp_fwd_op = torch.ops.m2dscan.mlp_fwd
linear_act_fwd_op = torch.ops.m2dscan.linear_act_fwd
layernorm_linear_act_fwd_op = torch.ops.m2dscan.layernorm_linear_act_fwd

# Keep the forward's anti-diagonal checkpoints for the backward (faster backward, more saved
# memory) or rebuild them inside the backward (nothing saved beyond the inputs, like the
# reference's partial recomputation).  Module-level switch, read at forward time.
SAVE_CHECKPOINTS = os.environ.get("M2D_SAVE_CHECKPOINTS", "1") != "0"

# Steps between the state snapshots that a forward keeps for its backward (m2d_desc.ckpt_interval).  0: the library
# chooses (2 for batches of images that are swept one stream each, 4 for few large images); 2 or 4 ask for that
# interval where the schedule has it; 8 or 16 keep a half or a quarter of the snapshots of 4, and the backward replays
# the forward over the steps in between.  Read at forward time; a backward uses the value its forward ran with.
# There is one switch: mamba2d_amd.cabi.CKPT_INTERVAL (environment: M2D_CKPT_INTERVAL); this module reads it there.
CKPT_INTERVALS = cabi.CKPT_INTERVALS


# bf16 tensors keep their snapshots rounded to bf16, as the reference keeps its whole hidden-state tensor
# (wf_cuda.cu:5,59-67).  True: kept in fp32 (M2D_FLAG_FP32_SNAPSHOTS: an interval of 4 steps, twice the bytes, slower
# kernels; gradient elements then meet the bound of the forward).  Read at forward time like the interval, and handed
# to the operators as the interval -4 ("every 4 steps, in fp32"), so that a backward uses what its forward ran with.
FP32_SNAPSHOTS = os.environ.get("M2D_FP32_SNAPSHOTS", "0") == "1"
FP32_SNAPSHOT_INTERVAL = -4


def _interval() -> int:
    v = cabi.CKPT_INTERVAL
    if v not in CKPT_INTERVALS:
        raise ValueError(f"m2dscan: CKPT_INTERVAL must be one of {CKPT_INTERVALS}, got {v!r}")
    if FP32_SNAPSHOTS:
        if v not in (0, 4):
            raise ValueError(f"m2dscan: FP32_SNAPSHOTS keeps a snapshot every 4 steps, CKPT_INTERVAL is {v}")
        return FP32_SNAPSHOT_INTERVAL
    return v


def __getattr__(name):   # wavefront.CKPT_INTERVAL reads the one switch
    if name == "CKPT_INTERVAL":
        return cabi.CKPT_INTERVAL
    raise AttributeError(name)


# The entry point computes the projections with the library's own kernels (wf_cuda_fn_proj) or
# with stock torch operators followed by wf_cuda_fn_pr / wf_cuda_fn_fr.  Read at call time.
FUSED_PROJECTIONS = os.environ.get("M2D_FUSED_PROJECTIONS", "1") != "0"


def _ckpt_bytes(x, N, flip=False, packed_bc=False, ckpt_interval=0) -> int:
    d = cabi.make_desc(x, N, flip)
    d.ckpt_interval = 4 if ckpt_interval == FP32_SNAPSHOT_INTERVAL else ckpt_interval
    if ckpt_interval == FP32_SNAPSHOT_INTERVAL:
        d.flags |= cabi.M2D_FLAG_FP32_SNAPSHOTS
    if packed_bc:   # the caller brings the packed B/C records: the buffer has no room for them
        d.flags |= cabi.M2D_FLAG_PACKED_BC
    return int(cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d)))


@torch.library.register_fake("m2dscan::scan_fwd")
def _scan_fwd_fake(x, deltaT, deltaL, AT, AL, BT, BL, C, D, save_ckpt, flip, raw_params=False, packed_bc=False, ckpt_interval=0):
    n = _ckpt_bytes(x, AT.shape[1], packed_bc=packed_bc, ckpt_interval=ckpt_interval) if save_ckpt else 1
    return torch.empty_like(x), x.new_empty((max(n, 1),), dtype=torch.uint8)


@torch.library.register_fake("m2dscan::scan_bwd")
def _scan_bwd_fake(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy, ckpt, flip, raw_params=False, packed_bc=False, dpre=False,
                   ckpt_interval=0, sum_parts=False):
    bc = [x.new_empty((*x.shape[:3], AT.shape[1])) for _ in range(3)]
    if sum_parts:   # the per-workgroup sums of d_C, d_BT, d_BL in fp32, as many as the library's plan has channel groups
        d = cabi.Desc(*x.shape, AT.shape[1], cabi.M2D_BF16 if x.dtype == torch.bfloat16 else cabi.M2D_F32,
                      (cabi.M2D_FLAG_FLIP if flip else 0) | (cabi.M2D_FLAG_RAW_PARAMS if raw_params else 0)
                      | (cabi.M2D_FLAG_PACKED_BC if packed_bc else 0) | (cabi.M2D_FLAG_DPRE if dpre else 0) | cabi.M2D_FLAG_SUM_PARTS
                      | (cabi.M2D_FLAG_FP32_SNAPSHOTS if ckpt_interval == FP32_SNAPSHOT_INTERVAL else 0),
                      4 if ckpt_interval == FP32_SNAPSHOT_INTERVAL else ckpt_interval)
        parts = int(cabi.lib.m2d_scan_sum_parts(ctypes.byref(d)))
        bc = [x.new_empty((parts, *x.shape[:3], 3 * AT.shape[1]), dtype=torch.float32), x.new_empty((0,)), x.new_empty((0,))]
    return [torch.empty_like(x), torch.empty_like(deltaT), torch.empty_like(deltaL), torch.empty_like(AT), torch.empty_like(AL),
            *bc, torch.empty_like(D)]


@torch.library.register_fake("mamba2d::wf_fwd")
def _wf_fwd_fake(hs, x, deltaT, deltaL, BT, BL, AT, AL):
    return None


@torch.library.register_fake("mamba2d::wf_bwd")
def _wf_bwd_fake(hs, x, deltaT, deltaL, AT, AL, grad_output, dDAT, dDAL, omega):
    return None


@torch.library.register_fake("m2dscan::proj_fwd")
def _proj_fwd_fake(x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, d_state, round_weights, packed_bc=False):
    B, H, W, _ = x.shape
    R = dt_projT_w.shape[1]
    if packed_bc:
        bc = [x.new_empty((B, H, W, 3 * d_state), dtype=torch.float32), x.new_empty((0,)), x.new_empty((0,))]
    else:
        bc = [x.new_empty((B, H, W, d_state)) for _ in range(3)]
    return [x.new_empty((B, H, W, 2 * R)), torch.empty_like(x), torch.empty_like(x), *bc]


@torch.library.register_fake("m2dscan::proj_bwd")
def _proj_bwd_fake(x, lowrank, deltaT, deltaL, x_proj_w, dt_projT_w, dt_projL_w, d_deltaT, d_deltaL, d_BT, d_BL, d_C, dx,
                   round_weights, dpre=False, sum_parts=0):
    b = dt_projT_w.new_empty((x.shape[-1],))
    return torch.empty_like(x_proj_w), torch.empty_like(dt_projT_w), b, torch.empty_like(dt_projL_w), torch.empty_like(b)


@torch.library.register_fake("m2dscan::layernorm_fwd")
def _layernorm_fwd_fake(x, weight, bias, eps):
    return torch.empty_like(x)


@torch.library.register_fake("m2dscan::dwconv3x3_fwd")
def _dwconv3x3_fwd_fake(x, weight):
    return torch.empty_like(x)


@torch.library.register_fake("m2dscan::starrelu_fwd")
def _starrelu_fwd_fake(x, scale, bias):
    return torch.empty_like(x)


@torch.library.register_fake("m2dscan::scale_residual_layernorm_fwd")
def _scale_residual_layernorm_fwd_fake(x, scale, residual, residual2, weight, bias, eps):
    return torch.empty_like(x), torch.empty_like(x)


@torch.library.register_fake("m2dscan::scale_residual_fwd")
def _scale_residual_fwd_fake(x, scale, residual, residual2=None):
    return torch.empty_like(x)


@torch.library.register_fake("m2dscan::linear_act_fwd")
def _linear_act_fwd_fake(x, weight, bias, pre, pre_scale, pre_bias, post, post_scale, post_bias):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


@torch.library.register_fake("m2dscan::layernorm_linear_act_fwd")
def _layernorm_linear_act_fwd_fake(x, ln_weight, ln_bias, eps, weight, bias, post, post_scale, post_bias):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


@torch.library.register_fake("m2dscan::mlp_fwd")
def _mlp_fwd_fake(x, w1, b1, w2, b2, ln_weight=None, ln_bias=None, eps=1e-5):
    return torch.empty_like(x)


@torch.library.register_fake("m2dscan::rope_attention_fwd")
def _rope_attention_fwd_fake(qkv, cos, sin, q_weight, q_bias, k_weight, k_bias, eps, scale):
    B, L, _, nh, hd = qkv.shape
    return qkv.new_empty((B, L, nh, hd))


@torch.library.register_fake("m2dscan::rope_qknorm_fwd")
def _rope_qknorm_fwd_fake(qkv, cos, sin, q_weight, q_bias, k_weight, k_bias, eps, token_major=False):
    B, L, _, nh, hd = qkv.shape
    if token_major:
        return qkv.new_empty((B, L, nh, hd)).permute(0, 2, 1, 3), qkv.new_empty((B, L, nh, hd)).permute(0, 2, 1, 3)
    return qkv.new_empty((B, nh, L, hd)), qkv.new_empty((B, nh, L, hd))


def fused_backward_math(dDAT, dDAL, dHS_total, deltaT, deltaL, AT, AL, BT, BL, x):
    """The reference's tensor algebra behind ``wf_bwd`` (``wavefront_cuda.py:97-139``), for callers of the
    operator pair ``wf_fwd_op`` / ``wf_bwd_op``: from ``dDAT``, ``dDAL`` and ``dBX`` (``dHS_total``), all
    (B,H,W,E,N), the gradients ``(d_x_scan, d_deltaT, d_deltaL, d_AT, d_AL, d_BT, d_BL)``.  The fused backward
    (``m2dscan::scan_bwd``) computes the same sums inside its kernel and never forms these tensors."""
    H, W = dHS_total.shape[1:3]
    zT = dDAT * torch.exp(deltaT.unsqueeze(-1) * AT)              # gradients with respect to the gate exponents
    zL = dDAL * torch.exp(deltaL.unsqueeze(-1) * AL)
    d_AT = torch.einsum("bhwen,bhwe->en", zT, deltaT)
    d_AL = torch.einsum("bhwen,bhwe->en", zL, deltaL)
    rows = torch.arange(H, device=x.device).view(1, H, 1, 1, 1)
    cols = torch.arange(W, device=x.device).view(1, 1, W, 1, 1)
    gT = dHS_total * (rows > 0)                                   # the T input reaches every row but the first,
    gL = dHS_total * ((cols > 0) | (rows == 0))                   # the L input every column but the first, and the origin
    d_deltaT = (zT * AT).sum(-1) + torch.einsum("bhwen,bhwn->bhwe", gT, BT) * x
    d_deltaL = (zL * AL).sum(-1) + torch.einsum("bhwen,bhwn->bhwe", gL, BL) * x
    d_BT = torch.einsum("bhwen,bhwe->bhwn", gT, deltaT * x)
    d_BL = torch.einsum("bhwen,bhwe->bhwn", gL, deltaL * x)
    d_x_scan = torch.einsum("bhwen,bhwn->bhwe", gT, BT) * deltaT + torch.einsum("bhwen,bhwn->bhwe", gL, BL) * deltaL
    return d_x_scan, d_deltaT, d_deltaL, d_AT, d_AL, d_BT, d_BL


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
    """Contiguous and 16-byte aligned (a contiguous view into a larger buffer may start anywhere)."""
    if not t.is_contiguous():
        return t.contiguous()
    if torch.compiler.is_compiling():   # addresses are not known while tracing; the shim rejects a misaligned one
        return t
    return t if t.data_ptr() % 16 == 0 else t.clone()


def _as_f32(t):
    """The parameter as a contiguous, aligned fp32 tensor: fp32 parameters (the reference trains
    bf16-mixed with fp32 parameters) pass through, others are cast on every call (no copy is kept: a
    parameter can change through ``.data`` without any trace a cache could check)."""
    if t.dtype == torch.float32:
        return _c(t)
    return _c(t.detach().float())


# The kernels hold the 16 states of a cell in the registers of one lane (d_state of every
# published Mamba2D configuration, models/mamba2d.py:23).  The recurrence is independent per state
# and y is a sum over states (wf_cuda.cu:40-69, wavefront_cuda.py:156), so any other d_state is the
# sum of scans over groups of 16 states, the last group padded with states whose B and C are zero
# (they stay at zero; their gradients are dropped); the skip term x*D goes with the first group.
STATES_PER_CALL = 16


def _state_groups(AT, AL, BT, BL, C):
    """(AT, AL, BT, BL, C) cut along the state axis into contiguous groups of 16, the last one padded."""
    pad = (-AT.shape[1]) % STATES_PER_CALL
    if pad:
        AT, AL = F.pad(AT, (0, pad), value=-1.0), F.pad(AL, (0, pad), value=-1.0)
        BT, BL, C = F.pad(BT, (0, pad)), F.pad(BL, (0, pad)), F.pad(C, (0, pad))
    return [tuple(t[..., n0:n0 + STATES_PER_CALL].contiguous() for t in (AT, AL, BT, BL, C))
            for n0 in range(0, AT.shape[1], STATES_PER_CALL)]


def _grouped_scan_fwd(x, deltaT, deltaL, AT, AL, BT, BL, C, D, keep, flip, interval=0):
    """scan_fwd for d_state != 16: y summed over the groups in fp32; one checkpoint buffer per group."""
    if AT.shape[1] < 1:
        raise ValueError(f"d_state must be positive, got {AT.shape[1]}")
    y, cks, no_skip = None, [], torch.zeros_like(D)
    for gi, grp in enumerate(_state_groups(AT, AL, BT, BL, C)):
        part, ck = scan_fwd_op(x, deltaT, deltaL, *grp, D if gi == 0 else no_skip, keep, flip, ckpt_interval=interval)
        y = part.float() if y is None else y + part.float()
        cks.append(ck)
    return y.to(x.dtype), cks


def _grouped_scan_bwd(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy, cks, flip, interval=0):
    """scan_bwd for d_state != 16: gradients of x and the step sizes summed over the groups in fp32,
    those of A, B, C put together along the state axis (padding dropped); d_D comes with the first group."""
    N = AT.shape[1]
    sums, per_state, d_D, no_skip = None, [], None, torch.zeros_like(D)
    for gi, grp in enumerate(_state_groups(AT, AL, BT, BL, C)):
        g = scan_bwd_op(x, deltaT, deltaL, *grp, D if gi == 0 else no_skip, dy, cks[gi], flip, ckpt_interval=interval)
        if gi == 0:
            sums, d_D = [t.float() for t in g[:3]], g[8]
        else:
            sums = [a + t.float() for a, t in zip(sums, g[:3])]
        per_state.append(g[3:8])
    joined = [torch.cat([grp[k] for grp in per_state], dim=-1)[..., :N].contiguous() for k in range(5)]
    return (*[t.to(x.dtype) for t in sums], *joined, d_D)


class _ScanOnParams(torch.autograd.Function):
    """The Function behind ``wf_cuda_fn_pr``: 16 states, and told by its caller whether autograd
    records the call (``recording``)."""

    @staticmethod
    def forward(ctx, x, deltaT, deltaL, AT, AL, BT, BL, C, D, flip=False, recording=True):
        args = [_c(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]
        keep = SAVE_CHECKPOINTS and recording and any(ctx.needs_input_grad)
        ctx.flip = bool(flip)
        ctx.interval = _interval()
        if AT.shape[1] != STATES_PER_CALL:
            y, cks = _grouped_scan_fwd(*args, keep, ctx.flip, ctx.interval)
            ctx.save_for_backward(*args, *cks)
            return y
        y, ck = scan_fwd_op(*args, keep, ctx.flip, ckpt_interval=ctx.interval)
        ctx.save_for_backward(*args, ck)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        args, cks = ctx.saved_tensors[:9], ctx.saved_tensors[9:]
        dy = _c(grad_output.to(args[0].dtype))
        if args[3].shape[1] != STATES_PER_CALL:
            return (*_grouped_scan_bwd(*args, dy, cks, ctx.flip, ctx.interval), None, None)
        return (*scan_bwd_op(*args, dy, cks[0], ctx.flip, ckpt_interval=ctx.interval), None, None)


class wf_cuda_fn_pr(torch.autograd.Function):
    """Scan + output projection on precomputed parameters (reference ``wavefront_cuda.py:146-196``).

    ``apply(x, deltaT, deltaL, AT, AL, BT, BL, C, D[, flip]) -> y``; backward returns the nine
    gradients in input order.  ``flip=True`` (not in the reference) scans from the bottom-right
    corner, which equals flipping every spatial tensor before and y after
    (``models/mamba2d.py:163-173``) without the copies.

    ``apply`` hands the call to ``_ScanOnParams`` (the node that shows up as ``y.grad_fn``) together
    with the grad mode of the caller: forward() always runs with grad mode off, and
    needs_input_grad is also set for parameters under torch.no_grad(), so whether autograd records
    the call is only known out here.  Written without ``super()``, and with forward and backward
    that are complete without it (torch.compile may trace either), so that a compiled caller can
    trace through the scan as it can through the reference's operator (``wavefront_cuda.py:25-57``)."""

    forward = staticmethod(_ScanOnParams.forward)
    backward = staticmethod(_ScanOnParams.backward)

    @classmethod
    def apply(cls, x, deltaT, deltaL, AT, AL, BT, BL, C, D, flip=False):
        return _ScanOnParams.apply(x, deltaT, deltaL, AT, AL, BT, BL, C, D, flip, torch.is_grad_enabled())


class wf_cuda_fn_fr(torch.autograd.Function):
    """Full-recompute variant (reference ``wavefront_cuda.py:199-313``): only x and the weights
    are saved; projections, checkpoints and states are rebuilt in the backward."""

    @staticmethod
    def forward(ctx, x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D, flip=False):
        with torch.no_grad():
            deltaT, deltaL, AT, AL, BT, BL, C = proj_params(
                x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b)
            if AT.shape[1] != STATES_PER_CALL:
                y, _ = _grouped_scan_fwd(*[_c(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)], False, bool(flip))
            else:
                y, _ = scan_fwd_op(_c(x), _c(deltaT), _c(deltaL), _c(AT), _c(AL), _c(BT), _c(BL), _c(C), _c(D),
                                   False, bool(flip))
        ctx.save_for_backward(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D)
        ctx.flip = bool(flip)
        ctx.interval = _interval()   # (no snapshots are kept: only the rebuilding forward inside the backward uses it)
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
        if AT_log.shape[1] != STATES_PER_CALL:
            n_groups = -(-AT_log.shape[1] // STATES_PER_CALL)
            d_x_scan, d_dT, d_dL, d_AT, d_AL, d_BT, d_BL, d_C, d_D = _grouped_scan_bwd(
                _c(x), *det, _c(D), dy, [none] * n_groups, ctx.flip, ctx.interval)
        else:
            d_x_scan, d_dT, d_dL, d_AT, d_AL, d_BT, d_BL, d_C, d_D = scan_bwd_op(
                _c(x), det[0], det[1], det[2], det[3], det[4], det[5], det[6], _c(D), dy, none, ctx.flip, ckpt_interval=ctx.interval)
        grads = torch.autograd.grad([deltaT, deltaL, BT, BL, C, AT, AL], leaves,
                                    [d_dT, d_dL, d_BT, d_BL, d_C, d_AT, d_AL])
        d_x = d_x_scan + grads[0]   # d_x_scan already contains dy*D
        return (d_x, *grads[1:], d_D, None)


def _proj_kernels_cover(x, AT_log, dt_projT_w) -> bool:
    """Shapes the projection kernels are built for; anything else takes the stock operators."""
    return AT_log.shape[1] == STATES_PER_CALL and dt_projT_w.shape[1] <= 32 and x.shape[-1] <= 4096


class wf_cuda_fn_proj(torch.autograd.Function):
    """Projections and scan behind one Function, all in the library's own kernels.

    Same function of the nine raw inputs as the reference's entry point: the projection weights
    are rounded to ``x.dtype`` (``wavefront_cuda.py:327-332``; here inside the kernels that pack
    them), then ``proj_params`` and ``wf_cuda_fn_pr`` (``:63-95``, ``:146-196``) or ``wf_cuda_fn_fr``
    (``:199-313``).  ``full=False`` keeps the projection outputs and the scan's checkpoints for the
    backward; ``full=True`` keeps only x and the weights and rebuilds the rest in the backward.
    ``recording``: the caller's grad mode (see wf_cuda_fn_pr); the entry point passes it."""

    @staticmethod
    def _params(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D):
        """The parameters as fp32 tensors (no copy if they already are): the library itself forms
        A = -exp(A_log) and rounds everything to x.dtype as the reference's casts do."""
        return [_as_f32(t) for t in (AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D)]

    @staticmethod
    def forward(ctx, x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D,
                full=False, flip=False, recording=True):
        x = _c(x)
        raw = (AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D)
        At, Al, *w32, D32 = wf_cuda_fn_proj._params(x, *raw)
        # B_T, B_L, C go from the projection kernel to the scan as packed records (BT) and two empty tensors
        low, dT, dL, BT, BL, C = proj_fwd_op(x, *w32, AT_log.shape[1], True, True)
        keep = SAVE_CHECKPOINTS and not full and recording and any(ctx.needs_input_grad)
        ctx.interval = _interval()
        y, ck = scan_fwd_op(x, dT, dL, At, Al, BT, BL, C, D32, keep, bool(flip), True, True, ctx.interval)
        if full:
            ctx.save_for_backward(x, *raw)
        else:
            ctx.save_for_backward(x, *raw, low, dT, dL, BT, BL, C, ck)
        ctx.full, ctx.flip = bool(full), bool(flip)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, *raw = ctx.saved_tensors[:9]
        At, Al, *w32, D32 = wf_cuda_fn_proj._params(x, *raw)
        dy = _c(grad_output.to(x.dtype))
        if ctx.full:
            low, dT, dL, BT, BL, C = proj_fwd_op(x, *w32, At.shape[1], True, True)
            ck = x.new_empty((1,), dtype=torch.uint8)
        else:
            low, dT, dL, BT, BL, C, ck = ctx.saved_tensors[9:]
        # with raw parameters the gradients of A_log and D come back in fp32; the gradients of the two
        # step sizes come back as gradients before the softplus, which is what the projections' backward wants
        # the sums over channels d_BT, d_BL, d_C have one reader here, the projections' backward: where its products run on the
        # matrix cores it takes the scan's per-workgroup sums as they are and adds them up while it loads them
        parts = x.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0
        d_x, d_dT, d_dL, d_At, d_Al, d_BT, d_BL, d_C, d_D = scan_bwd_op(x, dT, dL, At, Al, BT, BL, C, D32, dy, ck, ctx.flip,
                                                                        True, True, True, ctx.interval, parts)
        # d_x holds the scan's own gradient (dy*D included); the projections add theirs in place
        g = proj_bwd_op(x, low, dT, dL, w32[0], w32[1], w32[3], d_dT, d_dL, d_BT, d_BL, d_C, d_x, True, True,
                        d_BT.shape[0] if parts else 0)
        grads = (d_At, d_Al, *g, d_D)
        return (d_x, *[t.to(r.dtype) for t, r in zip(grads, raw)], None, None, None)


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

    if recomp not in ("partial", "full"):
        raise ValueError(f"Unknown recomputation mode, got {recomp}...")
    if FUSED_PROJECTIONS and _proj_kernels_cover(x, AT_log, dt_projT_w):
        # the casts of the weights to x.dtype happen inside (no copies of the parameters)
        return wf_cuda_fn_proj.apply(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, D,
                                     recomp == "full", flip, torch.is_grad_enabled())

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
    return wf_cuda_fn_fr.apply(x, AT_log, AL_log, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w,
                               dt_projL_b, D, flip)
