"""ctypes view of libm2dscan.so -- the C ABI declared in include/m2dscan.h.

PyTorch appears here only as the owner of device memory and of the current HIP stream.
There is no fallback: if the library has not been built, importing this module raises.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("M2D_LIB") or os.path.join(_HERE, "libm2dscan.so")

M2D_F32, M2D_BF16 = 0, 1
M2D_FLAG_FLIP = 1
M2D_FLAG_ROUND_WEIGHTS = 2
M2D_FLAG_RAW_PARAMS = 4
M2D_FLAG_PACKED_BC = 8
M2D_FLAG_DPRE = 16
M2D_FLAG_SPLIT_STATES = 32
M2D_FLAG_WHOLE_STATES = 64
M2D_FLAG_TEST_DEAD_LINK = 128
M2D_FLAG_SUM_PARTS = 256
M2D_FLAG_FP32_SNAPSHOTS = 512
M2D_PASS_FWD, M2D_PASS_BWD = 0, 1

EXPORTS = ("m2d_version", "m2d_status_str", "m2d_desc_check", "m2d_scan_workspace_bytes",
           "m2d_scan_ckpt_bytes", "m2d_scan_fwd", "m2d_scan_fwd_noalloc", "m2d_scan_link_error", "m2d_scan_plan", "m2d_scan_bwd", "m2d_proj_workspace_bytes", "m2d_proj_fwd",
           "m2d_proj_bwd", "m2d_proj_bwd_parts", "m2d_scan_sum_parts", "m2d_layernorm_fwd", "m2d_dwconv3x3_fwd", "m2d_starrelu_fwd",
           "m2d_scale_residual_fwd", "m2d_scale_residual_layernorm_fwd", "m2d_rope_qknorm_fwd", "m2d_rope_attention_fwd", "m2d_mlp_fwd", "m2d_layernorm_linear_fwd", "m2d_linear_fwd", "m2d_profile_enable", "m2d_profile_last_ms", "m2d_valu_rate_probe", "m2d_wf_fwd", "m2d_wf_bwd")


class Desc(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in ("B", "H", "W", "E", "N", "dtype", "flags", "ckpt_interval")]


class M2DError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(f"m2dscan: {text} (status {status})")
        self.status = status


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m mamba2d_amd.build` "
            "(there is no CPU or eager fallback for the scan)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    dp = ctypes.POINTER(Desc)
    lib.m2d_version.restype = i32
    lib.m2d_status_str.restype = ctypes.c_char_p
    lib.m2d_status_str.argtypes = [i32]
    lib.m2d_desc_check.restype = i32
    lib.m2d_desc_check.argtypes = [dp]
    lib.m2d_scan_workspace_bytes.restype = sz
    lib.m2d_scan_workspace_bytes.argtypes = [dp, i32, i32]
    lib.m2d_scan_ckpt_bytes.restype = sz
    lib.m2d_scan_ckpt_bytes.argtypes = [dp]
    lib.m2d_scan_fwd.restype = i32
    lib.m2d_scan_fwd.argtypes = [dp] + [vp] * 9 + [vp, vp, sz, vp, sz, vp]
    lib.m2d_scan_link_error.restype = i32
    lib.m2d_scan_link_error.argtypes = [dp, vp, vp, ctypes.POINTER(ctypes.c_int)]
    lib.m2d_valu_rate_probe.restype = i32
    lib.m2d_valu_rate_probe.argtypes = [i32, i32, vp, sz, vp, ctypes.POINTER(ctypes.c_double)]
    lib.m2d_wf_fwd.restype = i32
    lib.m2d_wf_fwd.argtypes = [i32] * 6 + [vp] * 9
    lib.m2d_wf_bwd.restype = i32
    lib.m2d_wf_bwd.argtypes = [i32] * 6 + [vp] * 11
    lib.m2d_scan_plan.restype = i32
    lib.m2d_scan_plan.argtypes = [dp, i32, ctypes.c_char_p, sz]
    lib.m2d_scan_fwd_noalloc.restype = i32
    lib.m2d_scan_fwd_noalloc.argtypes = [dp] + [vp] * 9 + [vp, vp]
    lib.m2d_scan_bwd.restype = i32
    lib.m2d_scan_bwd.argtypes = [dp] + [vp] * 10 + [vp, sz] + [vp] * 9 + [vp, sz, vp]
    lib.m2d_proj_workspace_bytes.restype = sz
    lib.m2d_proj_workspace_bytes.argtypes = [dp, i32, i32]
    lib.m2d_proj_fwd.restype = i32
    lib.m2d_proj_fwd.argtypes = [dp, i32] + [vp] * 12 + [vp, sz, vp]
    lib.m2d_proj_bwd.restype = i32
    lib.m2d_proj_bwd.argtypes = [dp, i32] + [vp] * 18 + [vp, sz, vp]
    lib.m2d_proj_bwd_parts.restype = i32
    lib.m2d_proj_bwd_parts.argtypes = [dp, i32, i32] + [vp] * 18 + [vp, sz, vp]
    lib.m2d_scan_sum_parts.restype = i32
    lib.m2d_scan_sum_parts.argtypes = [dp]
    lib.m2d_layernorm_fwd.restype = i32
    lib.m2d_layernorm_fwd.argtypes = [ctypes.c_int64, i32, i32, i32, vp, vp, vp, ctypes.c_float, vp, vp]
    lib.m2d_dwconv3x3_fwd.restype = i32
    lib.m2d_dwconv3x3_fwd.argtypes = [i32, i32, i32, i32, i32, i32, vp, vp, vp, vp]
    lib.m2d_starrelu_fwd.restype = i32
    lib.m2d_starrelu_fwd.argtypes = [ctypes.c_int64, i32, i32, vp, vp, vp, vp, vp]
    lib.m2d_scale_residual_layernorm_fwd.restype = i32
    lib.m2d_scale_residual_layernorm_fwd.argtypes = [ctypes.c_int64, i32, i32, i32] + [vp] * 6 + [ctypes.c_float, vp, vp, vp]
    lib.m2d_scale_residual_fwd.restype = i32
    lib.m2d_scale_residual_fwd.argtypes = [ctypes.c_int64, i32, i32, i32, vp, vp, vp, vp, vp, vp]
    lib.m2d_mlp_fwd.restype = i32
    lib.m2d_mlp_fwd.argtypes = [ctypes.c_int64, i32, i32, i32, vp, vp, vp, ctypes.c_float] + [vp] * 6
    lib.m2d_layernorm_linear_fwd.restype = i32
    lib.m2d_layernorm_linear_fwd.argtypes = [ctypes.c_int64, i32, i32, i32, vp, vp, vp, ctypes.c_float, vp, vp, i32, vp, vp, vp, vp]
    lib.m2d_rope_attention_fwd.restype = i32
    lib.m2d_rope_attention_fwd.argtypes = [i32] * 5 + [vp] * 7 + [ctypes.c_float, ctypes.c_float, vp, vp]
    lib.m2d_rope_qknorm_fwd.restype = i32
    lib.m2d_rope_qknorm_fwd.argtypes = [i32] * 6 + [vp] * 7 + [ctypes.c_float, i32, vp, vp, vp]
    lib.m2d_linear_fwd.restype = i32
    lib.m2d_linear_fwd.argtypes = [ctypes.c_int64, i32, i32, i32, vp, vp, vp, i32, vp, vp, i32, vp, vp, vp, vp]
    lib.m2d_profile_enable.restype = i32
    lib.m2d_profile_enable.argtypes = [i32]
    lib.m2d_profile_last_ms.restype = i32
    lib.m2d_profile_last_ms.argtypes = [i32, ctypes.POINTER(ctypes.c_float)]
    return lib


lib = _load()


def profile_enable(on: bool) -> None:
    check(lib.m2d_profile_enable(int(on)))


def profile_last_ms(which: int) -> float:
    ms = ctypes.c_float(0.0)
    check(lib.m2d_profile_last_ms(which, ctypes.byref(ms)))
    return float(ms.value)


RATE_KINDS = {"fma": 0, "fma_dependent": 1, "exp": 2, "exp_dependent": 3, "scan_fwd_unit": 4}


def valu_rate_probe(kind: str, waves_per_simd: int = 2, device=None) -> float:
    """Lane-operations per second (units per second for "scan_fwd_unit") that the vector ALUs of the device issue,
    measured by m2d_valu_rate_probe."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    scratch = torch.empty(1024 * torch.cuda.get_device_properties(dev).multi_processor_count * waves_per_simd, dtype=torch.uint8, device=dev)
    rate = ctypes.c_double(0.0)
    check(lib.m2d_valu_rate_probe(RATE_KINDS[kind], waves_per_simd, _ptr(scratch), scratch.numel(), _stream(dev), ctypes.byref(rate)))
    return float(rate.value)


def status_str(code: int) -> str:
    return lib.m2d_status_str(int(code)).decode()


def check(code: int) -> None:
    if code != 0:
        raise M2DError(code, status_str(code))


# M2D_FLAG_SPLIT_STATES or M2D_FLAG_WHOLE_STATES to override the library's choice of lane layout in
# scan_fwd / scan_bwd (0: the library decides); the tests run every case all three ways.
SCHEDULE_HINT = 0
# Steps between the state snapshots that the forward keeps for the backward (m2d_desc.ckpt_interval).  0: the
# library chooses (2 for batches of images swept one stream each, 4 for few large images); 2 or 4: that interval
# where the schedule has it; 8 or 16: a half or a quarter of the snapshots of 4, and the backward replays the
# forward over the steps in between.  Set once, before the forward of a problem, and leave until its backward.
# The one switch of the package (mamba2d_amd.wavefront reads it here); environment: M2D_CKPT_INTERVAL.
CKPT_INTERVALS = (0, 2, 4, 8, 16)


def _interval_from_env() -> int:
    text = os.environ.get("M2D_CKPT_INTERVAL", "0")
    try:
        v = int(text)
    except ValueError:
        v = None
    if v not in CKPT_INTERVALS:
        raise ValueError(f"m2dscan: M2D_CKPT_INTERVAL must be one of {CKPT_INTERVALS}, got {text!r}")
    return v


CKPT_INTERVAL = _interval_from_env()


def make_desc(x: torch.Tensor, N: int, flip: bool = False) -> Desc:
    B, H, W, E = x.shape
    if x.dtype == torch.float32:
        dt = M2D_F32
    elif x.dtype == torch.bfloat16:
        dt = M2D_BF16
    else:
        raise TypeError(f"m2dscan supports float32 and bfloat16, got {x.dtype}")
    return Desc(B, H, W, E, N, dt, (M2D_FLAG_FLIP if flip else 0) | SCHEDULE_HINT, CKPT_INTERVAL)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _same(x, *ts):
    for t in ts:
        if t.dtype != x.dtype or t.device != x.device or not t.is_contiguous():
            raise ValueError("m2dscan: all tensors must be contiguous, on one device and of one dtype")


def _shapes(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy=None):
    """The library only sees pointers, so every extent it will index is checked here."""
    if x.dim() != 4 or AT.dim() != 2:
        raise ValueError("m2dscan: x must be (B,H,W,E) and AT (E,N)")
    B, H, W, E = x.shape
    N = AT.shape[1]
    want = {"deltaT": (deltaT, (B, H, W, E)), "deltaL": (deltaL, (B, H, W, E)), "AT": (AT, (E, N)),
            "AL": (AL, (E, N)), "BT": (BT, (B, H, W, N)), "BL": (BL, (B, H, W, N)), "C": (C, (B, H, W, N)),
            "D": (D, (E,))}
    if dy is not None:
        want["dy"] = (dy, (B, H, W, E))
    for k, (t, shp) in want.items():
        if tuple(t.shape) != shp:
            raise ValueError(f"m2dscan: {k} has shape {tuple(t.shape)}, expected {shp}")
    if not x.is_cuda:
        raise ValueError("m2dscan: tensors must live on the GPU")


def _bytes(n, dev):
    # torch's caching allocator returns 512-byte aligned blocks
    return torch.empty(max(int(n), 1), dtype=torch.uint8, device=dev)


CHECK_LINKS = False   # tests set this: every scan call then synchronises and raises if a workgroup gave up waiting


def _check_links(d, ws, dev):
    if CHECK_LINKS:
        flag = ctypes.c_int(0)
        check(lib.m2d_scan_link_error(ctypes.byref(d), _ptr(ws), _stream(dev), ctypes.byref(flag)))
        if flag.value:
            raise RuntimeError("m2dscan: a workgroup of the linked sweep gave up waiting for its neighbour")


def scan_plan(B, H, W, E, dtype, pass_=M2D_PASS_FWD, N=16, flags=None, ckpt_interval=None):
    """The library's one-line description of how it will run a pass of this problem (m2d_scan_plan)."""
    dt = M2D_F32 if dtype in (torch.float32, "f32") else M2D_BF16
    d = Desc(B, H, W, E, N, dt, SCHEDULE_HINT if flags is None else flags, CKPT_INTERVAL if ckpt_interval is None else ckpt_interval)
    buf = ctypes.create_string_buffer(320)
    check(lib.m2d_scan_plan(ctypes.byref(d), pass_, buf, len(buf)))
    return buf.value.decode()


def scan_fwd(x, deltaT, deltaL, AT, AL, BT, BL, C, D, save_ckpt=False, flip=False):
    """y (and the checkpoint buffer when ``save_ckpt``) through m2d_scan_fwd."""
    _same(x, deltaT, deltaL, AT, AL, BT, BL, C, D)
    _shapes(x, deltaT, deltaL, AT, AL, BT, BL, C, D)
    d = make_desc(x, AT.shape[1], flip)
    check(lib.m2d_desc_check(ctypes.byref(d)))
    y = torch.empty_like(x)
    ck = _bytes(lib.m2d_scan_ckpt_bytes(ctypes.byref(d)), x.device) if save_ckpt else None
    ws = _bytes(lib.m2d_scan_workspace_bytes(ctypes.byref(d), M2D_PASS_FWD, int(save_ckpt)), x.device)
    check(lib.m2d_scan_fwd(ctypes.byref(d), *[_ptr(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)],
                           _ptr(y), _ptr(ck), ck.numel() if ck is not None else 0, _ptr(ws), ws.numel(),
                           _stream(x.device)))
    _check_links(d, ws, x.device)
    return (y, ck) if save_ckpt else y


NOALLOC_SCRATCH_BYTES = 32 << 20
M2D_ERR_TOO_LARGE = 7


def scan_fwd_noalloc(x, deltaT, deltaL, AT, AL, BT, BL, C, D, y, flip=False):
    """y through m2d_scan_fwd_noalloc: the caller brings the output too, the library's scratch is a
    static device array, and nothing is allocated anywhere in the call."""
    _same(x, deltaT, deltaL, AT, AL, BT, BL, C, D, y)
    _shapes(x, deltaT, deltaL, AT, AL, BT, BL, C, D, y)
    d = make_desc(x, AT.shape[1], flip)
    check(lib.m2d_scan_fwd_noalloc(ctypes.byref(d), *[_ptr(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)],
                                   _ptr(y), _stream(x.device)))
    return y


def scan_bwd(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy, ckpt=None, flip=False, dpre=False, sum_parts=False):
    """The nine gradients (order of the inputs) through m2d_scan_bwd.  ``dpre``: d_deltaT and d_deltaL
    come multiplied by the slope of the softplus that made the deltas (M2D_FLAG_DPRE).  ``sum_parts``:
    d_BT comes back as the float32 per-workgroup sums (parts,B,H,W,3N) for ``proj_bwd(sum_parts=parts)``,
    d_BL and d_C as None (M2D_FLAG_SUM_PARTS)."""
    _same(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy)
    _shapes(x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy)
    d = make_desc(x, AT.shape[1], flip)
    if dpre:
        d.flags |= M2D_FLAG_DPRE
    check(lib.m2d_desc_check(ctypes.byref(d)))
    outs = [torch.empty_like(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D)]
    if sum_parts:
        d.flags |= M2D_FLAG_SUM_PARTS
        parts = lib.m2d_scan_sum_parts(ctypes.byref(d))
        outs[5:8] = [x.new_empty((parts, *x.shape[:3], 3 * AT.shape[1]), dtype=torch.float32), None, None]
    ws = _bytes(lib.m2d_scan_workspace_bytes(ctypes.byref(d), M2D_PASS_BWD, int(ckpt is not None)), x.device)
    check(lib.m2d_scan_bwd(ctypes.byref(d), *[_ptr(t) for t in (x, deltaT, deltaL, AT, AL, BT, BL, C, D, dy)],
                           _ptr(ckpt), ckpt.numel() if ckpt is not None else 0, *[_ptr(t) for t in outs],
                           _ptr(ws), ws.numel(), _stream(x.device)))
    _check_links(d, ws, x.device)
    return tuple(outs)


def _proj_check(x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, N):
    if x.dim() != 4 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("m2dscan: x must be a contiguous (B,H,W,E) tensor on the GPU")
    E = x.shape[-1]
    R = dt_projT_w.shape[1]
    want = {"x_proj_w": (x_proj_w, (2 * R + 3 * N, E)), "dt_projT_w": (dt_projT_w, (E, R)), "dt_projT_b": (dt_projT_b, (E,)),
            "dt_projL_w": (dt_projL_w, (E, R)), "dt_projL_b": (dt_projL_b, (E,))}
    for k, (t, shp) in want.items():
        if tuple(t.shape) != shp or t.dtype != torch.float32 or t.device != x.device or not t.is_contiguous():
            raise ValueError(f"m2dscan: {k} must be a contiguous float32 tensor of shape {shp} on {x.device}")
    return R


def proj_fwd(x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, N=16, round_weights=False):
    """(lowrank, deltaT, deltaL, BT, BL, C) through m2d_proj_fwd; weights are float32 tensors
    (``round_weights``: the library rounds them to x.dtype first)."""
    R = _proj_check(x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, N)
    B, H, W, E = x.shape
    d = make_desc(x, N)
    d.flags = M2D_FLAG_ROUND_WEIGHTS if round_weights else 0
    low = x.new_empty((B, H, W, 2 * R))
    dT, dL = torch.empty_like(x), torch.empty_like(x)
    BT, BL, C = (x.new_empty((B, H, W, N)) for _ in range(3))
    ws = _bytes(lib.m2d_proj_workspace_bytes(ctypes.byref(d), R, M2D_PASS_FWD), x.device)
    check(lib.m2d_proj_fwd(ctypes.byref(d), R, *[_ptr(t) for t in (x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w,
                                                                  dt_projL_b, low, dT, dL, BT, BL, C)],
                           _ptr(ws), ws.numel(), _stream(x.device)))
    return low, dT, dL, BT, BL, C


def proj_bwd(x, lowrank, deltaT, deltaL, x_proj_w, dt_projT_w, dt_projL_w, d_deltaT, d_deltaL, d_BT, d_BL, d_C, dx,
             round_weights=False, dpre=False, sum_parts=0):
    """Adds the gradient through the projections to ``dx`` in place and returns the five weight
    gradients (x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b; float32) through m2d_proj_bwd.
    ``dpre``: d_deltaT and d_deltaL are gradients before the softplus (M2D_FLAG_DPRE); deltaT and deltaL
    may then be None.  ``sum_parts`` > 0: d_BT is the (sum_parts,B,H,W,3N) float32 tensor of
    ``scan_bwd(sum_parts=True)``, d_BL and d_C are None (m2d_proj_bwd_parts)."""
    N = d_BT.shape[-1] // 3 if sum_parts else d_BT.shape[-1]
    zb = torch.zeros(x.shape[-1], device=x.device)
    R = _proj_check(x, x_proj_w, dt_projT_w, zb, dt_projL_w, zb, N)
    B, H, W, E = x.shape
    given = [t for t in (deltaT, deltaL) if t is not None]
    if not dpre and len(given) < 2:
        raise ValueError("m2dscan: deltaT and deltaL are needed unless dpre is set")
    if sum_parts:
        _same(x, lowrank, *given, d_deltaT, d_deltaL, dx)
        if d_BT.dtype != torch.float32 or d_BT.device != x.device or not d_BT.is_contiguous():
            raise ValueError("m2dscan: with sum_parts d_BT must be a contiguous float32 tensor on x's device")
        bc = {"d_BT": (d_BT, (sum_parts, B, H, W, 3 * N))}
    else:
        _same(x, lowrank, *given, d_deltaT, d_deltaL, d_BT, d_BL, d_C, dx)
        bc = {"d_BT": (d_BT, (B, H, W, N)), "d_BL": (d_BL, (B, H, W, N)), "d_C": (d_C, (B, H, W, N))}
    want = {"lowrank": (lowrank, (B, H, W, 2 * R)),
            "d_deltaT": (d_deltaT, (B, H, W, E)), "d_deltaL": (d_deltaL, (B, H, W, E)), **bc, "dx": (dx, (B, H, W, E))}
    for k, t in zip(("deltaT", "deltaL"), (deltaT, deltaL)):
        if t is not None:
            want[k] = (t, (B, H, W, E))
    for k, (t, shp) in want.items():
        if tuple(t.shape) != shp:
            raise ValueError(f"m2dscan: {k} has shape {tuple(t.shape)}, expected {shp}")
    d = make_desc(x, N)
    d.flags = (M2D_FLAG_ROUND_WEIGHTS if round_weights else 0) | (M2D_FLAG_DPRE if dpre else 0)
    outs = [torch.empty_like(t) for t in (x_proj_w, dt_projT_w, zb, dt_projL_w, zb)]
    ws = _bytes(lib.m2d_proj_workspace_bytes(ctypes.byref(d), R, M2D_PASS_BWD), x.device)
    check(lib.m2d_proj_bwd_parts(ctypes.byref(d), R, int(sum_parts), *[_ptr(t) for t in (x, lowrank, deltaT, deltaL, x_proj_w, dt_projT_w,
                                                                  dt_projL_w, d_deltaT, d_deltaL, d_BT, d_BL, d_C, dx)],
                           *[_ptr(t) for t in outs], _ptr(ws), ws.numel(), _stream(x.device)))
    return tuple(outs)


def _dtype_code(t):
    if t.dtype == torch.float32:
        return M2D_F32
    if t.dtype == torch.bfloat16:
        return M2D_BF16
    raise TypeError(f"m2dscan supports float32 and bfloat16, got {t.dtype}")


def layernorm_fwd(x, weight, bias, eps=1e-5):
    """LayerNorm over the last axis of a contiguous tensor through m2d_layernorm_fwd (inference forward)."""
    C = x.shape[-1]
    if not x.is_cuda or not x.is_contiguous():
        raise ValueError("m2dscan: x must be a contiguous tensor on the GPU")
    for k, t in (("weight", weight), ("bias", bias)):
        if tuple(t.shape) != (C,) or t.device != x.device or not t.is_contiguous() or t.dtype != weight.dtype:
            raise ValueError(f"m2dscan: {k} must be a contiguous ({C},) tensor on {x.device}, both of one dtype")
    y = torch.empty_like(x)
    check(lib.m2d_layernorm_fwd(x.numel() // C, C, _dtype_code(x), _dtype_code(weight), _ptr(x), _ptr(weight), _ptr(bias),
                                float(eps), _ptr(y), _stream(x.device)))
    return y


def dwconv3x3_fwd(x, weight):
    """Depthwise 3x3 convolution (padding 1, no bias) of a channel-last (B,H,W,C) tensor with the
    (C,1,3,3) weight of nn.Conv2d(C, C, 3, padding=1, groups=C), through m2d_dwconv3x3_fwd."""
    if x.dim() != 4 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("m2dscan: x must be a contiguous (B,H,W,C) tensor on the GPU")
    B, H, W, C = x.shape
    if tuple(weight.shape) != (C, 1, 3, 3) or weight.device != x.device or not weight.is_contiguous():
        raise ValueError(f"m2dscan: weight must be a contiguous ({C},1,3,3) tensor on {x.device}")
    y = torch.empty_like(x)
    check(lib.m2d_dwconv3x3_fwd(B, H, W, C, _dtype_code(x), _dtype_code(weight), _ptr(x), _ptr(weight), _ptr(y),
                                _stream(x.device)))
    return y


def starrelu_fwd(x, scale, bias):
    """scale * relu(x)^2 + bias with one-element scale and bias, through m2d_starrelu_fwd."""
    if not x.is_cuda or not x.is_contiguous():
        raise ValueError("m2dscan: x must be a contiguous tensor on the GPU")
    for k, t in (("scale", scale), ("bias", bias)):
        if t.numel() != 1 or t.device != x.device or t.dtype != scale.dtype:
            raise ValueError(f"m2dscan: {k} must hold one element on {x.device}, both of one dtype")
    y = torch.empty_like(x)
    check(lib.m2d_starrelu_fwd(x.numel(), _dtype_code(x), _dtype_code(scale), _ptr(x), _ptr(scale), _ptr(bias), _ptr(y),
                               _stream(x.device)))
    return y


def scale_residual_fwd(x, scale, residual, residual2=None):
    """x * scale + residual (+ residual2) with a per-channel scale (last axis), through m2d_scale_residual_fwd."""
    C = x.shape[-1]
    for r in (residual,) if residual2 is None else (residual, residual2):
        if not x.is_cuda or not x.is_contiguous() or not r.is_contiguous() or r.shape != x.shape or r.dtype != x.dtype or r.device != x.device:
            raise ValueError("m2dscan: x and the residuals must be contiguous tensors of one shape and dtype on the GPU")
    if tuple(scale.shape) != (C,) or scale.device != x.device or not scale.is_contiguous():
        raise ValueError(f"m2dscan: scale must be a contiguous ({C},) tensor on {x.device}")
    y = torch.empty_like(x)
    check(lib.m2d_scale_residual_fwd(x.numel() // C, C, _dtype_code(x), _dtype_code(scale), _ptr(x), _ptr(scale), _ptr(residual),
                                     None if residual2 is None else _ptr(residual2), _ptr(y), _stream(x.device)))
    return y


def scale_residual_layernorm_fwd(x, scale, residual, residual2, weight, bias, eps=1e-5):
    """(x * scale + residual (+ residual2), LayerNorm of it over the last axis), through
    m2d_scale_residual_layernorm_fwd."""
    C = x.shape[-1]
    for r in (residual,) if residual2 is None else (residual, residual2):
        if not x.is_cuda or not x.is_contiguous() or not r.is_contiguous() or r.shape != x.shape or r.dtype != x.dtype or r.device != x.device:
            raise ValueError("m2dscan: x and the residuals must be contiguous tensors of one shape and dtype on the GPU")
    for t in (scale, weight, bias):
        if tuple(t.shape) != (C,) or t.device != x.device or not t.is_contiguous() or t.dtype != scale.dtype:
            raise ValueError(f"m2dscan: scale, weight and bias must be contiguous ({C},) tensors of one dtype on {x.device}")
    xo, y = torch.empty_like(x), torch.empty_like(x)
    check(lib.m2d_scale_residual_layernorm_fwd(x.numel() // C, C, _dtype_code(x), _dtype_code(scale), _ptr(x), _ptr(scale),
                                               _ptr(residual), None if residual2 is None else _ptr(residual2), _ptr(weight),
                                               _ptr(bias), float(eps), _ptr(xo), _ptr(y), _stream(x.device)))
    return xo, y


def mlp_fwd(x, w1, b1, w2, b2, ln_weight=None, ln_bias=None, eps=1e-5):
    """fc2(GELU(fc1 x)) on a contiguous bf16 (..., C) tensor, through m2d_mlp_fwd (C = 32 or 64, hidden = 4 C); with
    ``ln_weight`` and ``ln_bias`` x passes through LayerNorm first."""
    C = x.shape[-1]
    if not x.is_cuda or not x.is_contiguous() or x.dtype != torch.bfloat16:
        raise ValueError("m2dscan: x must be a contiguous bfloat16 tensor on the GPU")
    H = w1.shape[0]
    if w1.dim() != 2 or w1.shape[1] != C or tuple(w2.shape) != (C, H) or w2.dtype != w1.dtype:
        raise ValueError(f"m2dscan: w1 must be (hidden,{C}) and w2 ({C},hidden), of one dtype")
    for t, n in ((w1, None), (w2, None), (b1, H), (b2, C), (ln_weight, C), (ln_bias, C)):
        if t is None:
            continue
        if t.device != x.device or not t.is_contiguous() or t.dtype != w1.dtype or (n is not None and t.numel() != n):
            raise ValueError(f"m2dscan: weights and biases must be contiguous tensors of one dtype on {x.device}")
    y = torch.empty_like(x)
    check(lib.m2d_mlp_fwd(x.numel() // C, C, H, _dtype_code(w1), _ptr(x), _ptr(ln_weight), _ptr(ln_bias), float(eps), _ptr(w1),
                          _ptr(b1), _ptr(w2), _ptr(b2), _ptr(y), _stream(x.device)))
    return y


def rope_attention_fwd(qkv, cos, sin, q_weight, q_bias, k_weight, k_bias, eps=1e-5, scale=None):
    """(B, L, heads, head_dim): the attention of a rotary stage (rotation and per-head LayerNorm of q and k, softmax
    attention) from a contiguous bf16 (B, L, 3, heads, head_dim) projection, through m2d_rope_attention_fwd."""
    if qkv.dim() != 5 or qkv.shape[2] != 3 or not qkv.is_cuda or not qkv.is_contiguous():
        raise ValueError("m2dscan: qkv must be a contiguous (B, L, 3, heads, head_dim) tensor on the GPU")
    B, L, _, nh, hd = qkv.shape
    for t in (cos, sin):
        if tuple(t.shape) != (L, hd) or t.dtype != qkv.dtype or t.device != qkv.device or not t.is_contiguous():
            raise ValueError(f"m2dscan: cos and sin must be contiguous ({L},{hd}) tensors of qkv's dtype and device")
    for t in (q_weight, q_bias, k_weight, k_bias):
        if tuple(t.shape) != (hd,) or t.dtype != q_weight.dtype or t.device != qkv.device or not t.is_contiguous():
            raise ValueError(f"m2dscan: the LayerNorm weights must be contiguous ({hd},) tensors of one dtype on {qkv.device}")
    if qkv.dtype != torch.bfloat16:
        raise ValueError("m2dscan: the attention kernel takes bfloat16")
    out = qkv.new_empty((B, L, nh, hd))
    check(lib.m2d_rope_attention_fwd(B, L, nh, hd, _dtype_code(q_weight), _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(q_weight),
                                     _ptr(q_bias), _ptr(k_weight), _ptr(k_bias), float(eps),
                                     float(hd ** -0.5 if scale is None else scale), _ptr(out), _stream(qkv.device)))
    return out


def rope_qknorm_fwd(qkv, cos, sin, q_weight, q_bias, k_weight, k_bias, eps=1e-5, token_major=False):
    """(q, k), each (B, heads, L, head_dim): rotary embedding and per-head LayerNorm of the q and k parts of
    a contiguous (B, L, 3, heads, head_dim) projection, through m2d_rope_qknorm_fwd.  ``token_major``: the
    same tensors as views of (B, L, heads, head_dim) memory."""
    if qkv.dim() != 5 or qkv.shape[2] != 3 or not qkv.is_cuda or not qkv.is_contiguous():
        raise ValueError("m2dscan: qkv must be a contiguous (B, L, 3, heads, head_dim) tensor on the GPU")
    B, L, _, nh, hd = qkv.shape
    for k_, t in (("cos", cos), ("sin", sin)):
        if tuple(t.shape) != (L, hd) or t.dtype != qkv.dtype or t.device != qkv.device or not t.is_contiguous():
            raise ValueError(f"m2dscan: {k_} must be a contiguous ({L},{hd}) tensor of qkv's dtype and device")
    for k_, t in (("q_weight", q_weight), ("q_bias", q_bias), ("k_weight", k_weight), ("k_bias", k_bias)):
        if tuple(t.shape) != (hd,) or t.dtype != q_weight.dtype or t.device != qkv.device or not t.is_contiguous():
            raise ValueError(f"m2dscan: {k_} must be a contiguous ({hd},) tensor, all four of one dtype, on qkv's device")
    shape = (B, L, nh, hd) if token_major else (B, nh, L, hd)
    q, k = qkv.new_empty(shape), qkv.new_empty(shape)
    check(lib.m2d_rope_qknorm_fwd(B, L, nh, hd, _dtype_code(qkv), _dtype_code(q_weight), _ptr(qkv), _ptr(cos), _ptr(sin),
                                  _ptr(q_weight), _ptr(q_bias), _ptr(k_weight), _ptr(k_bias), float(eps), int(token_major),
                                  _ptr(q), _ptr(k), _stream(qkv.device)))
    return (q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3)) if token_major else (q, k)


ACT_NONE, ACT_GELU, ACT_STARRELU = 0, 1, 2


def linear_fwd(x, weight, bias=None, pre=ACT_NONE, pre_params=None, post=ACT_NONE, post_params=None, ln=None):
    """post(pre(x) @ weight.T + bias) on bf16 activations through m2d_linear_fwd; ``*_params`` are the
    (scale, bias) one-element tensors of a StarReLU.  ``ln`` = (weight, bias, eps) of a LayerNorm over x's last
    axis in front of the layer (then through m2d_layernorm_linear_fwd, and no ``pre``)."""
    K = x.shape[-1]
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("m2dscan: x must be a contiguous bfloat16 tensor on the GPU")
    if tuple(weight.shape) != (N, K) or not weight.is_contiguous() or weight.device != x.device:
        raise ValueError(f"m2dscan: weight must be a contiguous (N,{K}) tensor on {x.device}")
    small = [t for t in (bias, *(pre_params or ()), *(post_params or ()), *((ln or ())[:2])) if t is not None]
    for t in small:
        if t.dtype != weight.dtype or t.device != x.device or not t.is_contiguous():
            raise ValueError("m2dscan: bias and activation parameters must have the weight's dtype and device")
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError(f"m2dscan: bias must have shape ({N},)")
    ps, pb = pre_params if pre == ACT_STARRELU else (None, None)
    qs, qb = post_params if post == ACT_STARRELU else (None, None)
    y = x.new_empty((*x.shape[:-1], N))
    if ln is not None:
        if pre != ACT_NONE or tuple(ln[0].shape) != (K,) or tuple(ln[1].shape) != (K,):
            raise ValueError(f"m2dscan: a LayerNorm in front of the layer takes ({K},) weights and no other activation before the layer")
        check(lib.m2d_layernorm_linear_fwd(x.numel() // K, K, N, _dtype_code(weight), _ptr(x), _ptr(ln[0]), _ptr(ln[1]), float(ln[2]),
                                           _ptr(weight), _ptr(bias), post, _ptr(qs), _ptr(qb), _ptr(y), _stream(x.device)))
        return y
    check(lib.m2d_linear_fwd(x.numel() // K, K, N, _dtype_code(weight), _ptr(x), _ptr(weight), _ptr(bias), pre, _ptr(ps), _ptr(pb),
                             post, _ptr(qs), _ptr(qb), _ptr(y), _stream(x.device)))
    return y
