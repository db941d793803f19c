"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol that
include/m2dscan.h declares, validates descriptors, and sizes its buffers consistently."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cabi():
    from mamba2d_amd import cabi as m
    return m


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "m2dscan.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(m2d_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(cabi):
    syms = declared_symbols()
    assert "m2d_scan_fwd" in syms and "m2d_scan_bwd" in syms
    raw = ctypes.CDLL(cabi.LIB_PATH)
    for s in syms:
        assert hasattr(raw, s), f"{s} declared in m2dscan.h but not exported"
    assert set(cabi.EXPORTS) == set(syms)


def test_version_and_status_strings(cabi):
    assert cabi.lib.m2d_version() >= 100
    assert cabi.status_str(0) == "ok"
    for code in range(1, 8):
        assert cabi.status_str(code) not in ("ok", "unknown status")
    assert cabi.status_str(99) == "unknown status"


def D(cabi, **kw):
    base = dict(B=2, H=14, W=14, E=32, N=16, dtype=0, flags=0, ckpt_interval=0)
    base.update(kw)
    return cabi.Desc(**base)


def test_descriptor_validation(cabi):
    chk = lambda d: cabi.lib.m2d_desc_check(ctypes.byref(d))
    assert chk(D(cabi)) == 0
    assert cabi.lib.m2d_desc_check(None) == 1
    # spatial dims must exceed 1, like the reference's ValueError (wavefront_cuda.py:323-324)
    assert chk(D(cabi, H=1)) == 2 and chk(D(cabi, W=1)) == 2 and chk(D(cabi, B=0)) == 2
    # flags 1 (flip), 4 (raw parameters), 8 (packed B/C), 16 (gradients before the softplus) and the two lane
    # layout hints 32 and 64 (one of them at most) belong to the scan, and so do the test aid 128, the
    # unfinished channel sums 256 and the fp32 snapshots of bf16 tensors 512 (at the default interval or 4); 2 is a projection
    # flag, 1024 nobody's
    assert chk(D(cabi, flags=4)) == 0 and chk(D(cabi, flags=29)) == 0 and chk(D(cabi, flags=2)) == 3
    assert chk(D(cabi, flags=32)) == 0 and chk(D(cabi, flags=64 | 1)) == 0 and chk(D(cabi, flags=96)) == 3
    assert chk(D(cabi, N=8)) == 3 and chk(D(cabi, dtype=7)) == 3 and chk(D(cabi, flags=128)) == 0 and chk(D(cabi, flags=256)) == 0 and chk(D(cabi, flags=512)) == 0 and chk(D(cabi, flags=1024)) == 3
    assert chk(D(cabi, dtype=1, flags=512, ckpt_interval=4)) == 0 and chk(D(cabi, dtype=1, flags=512, ckpt_interval=2)) == 3 and chk(D(cabi, dtype=0, flags=512, ckpt_interval=8)) == 0
    # steps between snapshots: the library's choice, 2, 4, 8 or 16
    assert all(chk(D(cabi, ckpt_interval=v)) == 0 for v in (0, 2, 4, 8, 16))
    assert all(chk(D(cabi, ckpt_interval=v)) == 3 for v in (1, 3, 12, 32, -4))
    # one image must fit 32-bit offsets: H*W < 2^24 cells, H*W*E < 2^30 elements
    assert chk(D(cabi, B=1, H=4096, W=4096, E=8)) == 3 and chk(D(cabi, B=1, H=2048, W=2048, E=256)) == 3
    assert chk(D(cabi, B=1, H=2048, W=2048, E=64)) == 0 and chk(D(cabi, B=4, H=4000, W=4000, E=32)) == 0


def test_argument_validation_happens_before_any_launch(cabi):
    """NULL pointers, misalignment and short buffers are rejected on the host (no GPU here)."""
    d = D(cabi)
    vp = ctypes.c_void_p
    good = [vp(4096)] * 9
    ws = cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(d), 0, 0)
    assert ws > 0
    f = cabi.lib.m2d_scan_fwd
    assert f(ctypes.byref(d), *([vp(0)] + good[1:]), vp(4096), vp(0), 0, vp(4096), ws, vp(0)) == 1
    assert f(ctypes.byref(d), *([vp(4100)] + good[1:]), vp(4096), vp(0), 0, vp(4096), ws, vp(0)) == 5
    assert f(ctypes.byref(d), *good, vp(4096), vp(0), 0, vp(4096 + 16), ws, vp(0)) == 5
    assert f(ctypes.byref(d), *good, vp(4096), vp(0), 0, vp(4096), ws - 1, vp(0)) == 4
    assert f(ctypes.byref(d), *good, vp(4096), vp(4096), 8, vp(4096), ws, vp(0)) == 4
    assert f(ctypes.byref(D(cabi, H=1)), *good, vp(4096), vp(0), 0, vp(4096), ws, vp(0)) == 2
    b = cabi.lib.m2d_scan_bwd
    wsb = cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(d), 1, 0)
    args = [vp(4096)] * 10 + [vp(0), 0] + [vp(4096)] * 9
    assert b(ctypes.byref(d), *args, vp(4096), wsb - 1, vp(0)) == 4
    args_null = list(args)
    args_null[15] = vp(0)
    assert b(ctypes.byref(d), *args_null, vp(4096), wsb, vp(0)) == 1


def test_buffer_sizes_scale_linearly_in_area(cabi):
    """Checkpoints and scratch grow with H*W (no quadratic term), and stay well below the full
    (B,H,W,E,N) fp32 state tensor for large grids."""
    sizes = {}
    for hw in (256, 512, 1024, 2048):
        # (one lane layout for all four sizes; the library's own choice is compared with it below)
        d = D(cabi, B=1, H=hw, W=hw, E=64, flags=cabi.M2D_FLAG_WHOLE_STATES)
        ck = cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d))
        wsb = cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(d), 1, 1)
        sizes[hw] = (ck, wsb)
        full_state = hw * hw * 64 * 16 * 4
        assert ck < 0.6 * full_state
        # splitting the states over the lanes keeps a set of channel sums per 8 channels (per 4 where few workgroups
        # are under way, with waves of their own to stage for them: 256x256, 512x512) instead of per 16 or 32: the library's own choice may cost up to that much more
        # scratch, never more checkpoints
        auto = D(cabi, B=1, H=hw, W=hw, E=64)
        assert cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(auto)) <= ck * 1.01
        assert cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(auto), 1, 1) <= (3.5 if hw <= 512 else 2.5) * wsb
    for a, b in ((256, 512), (512, 1024), (1024, 2048)):
        for k in range(2):
            ratio = sizes[b][k] / sizes[a][k]
            assert 3.5 < ratio < 4.5, (a, b, k, ratio)
    assert cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(D(cabi, H=1)), 0, 0) == 0
    assert cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(D(cabi, N=3))) == 0


def test_checkpoint_interval_shrinks_the_snapshots(cabi):
    """m2d_desc.ckpt_interval = 8 / 16: a half / a quarter of the snapshots (band boundary rows and, for fp32, the
    packed B|C stay), a small ring of replayed snapshots per workgroup in the backward's scratch, and the one
    backward kernel that replays, whatever layout was asked for."""
    import torch
    for dtype, shape in ((1, (128, 56, 56, 64)), (0, (1, 2048, 2048, 64)), (1, (1, 2048, 2048, 64)), (0, (300, 7, 7, 32))):
        B, H, W, E = shape
        ck, ws = {}, {}
        for iv in (0, 4, 8, 16):
            d = D(cabi, B=B, H=H, W=W, E=E, dtype=dtype, ckpt_interval=iv, flags=cabi.M2D_FLAG_WHOLE_STATES)
            ck[iv] = cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d))
            ws[iv] = cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(d), 1, 1)
        # left to itself the library keeps a snapshot every 2 steps for batches swept one stream per image or stack
        # (twice the snapshots of 4 steps, and one behind the sweep), every 4 steps for the few large images of a linked sweep
        if B > 1:
            assert ck[0] > ck[4] and ws[4] == ws[0]
        else:
            assert ck[4] == ck[0] and ws[4] == ws[0]
        if H > 14:   # (7x7 images are stacked at the shorter intervals and not at the others: other block counts)
            assert ck[4] > ck[8] > ck[16]
            # a half of the blocks dropped against three quarters (rounded up per window of a band)
            assert abs((ck[4] - ck[8]) / (ck[4] - ck[16]) - 2 / 3) < 0.05
            assert 0 < ws[8] - ws[4] < ws[16] - ws[4] <= 0.1 * ws[4] + (1 << 20)   # (three parked snapshots per workgroup)
    plan = cabi.scan_plan(1, 256, 256, 64, torch.float32, cabi.M2D_PASS_BWD, flags=cabi.M2D_FLAG_SPLIT_STATES, ckpt_interval=16)
    assert plan.startswith("m2d_bwd_kernel: linked sweep") and plan.endswith("a snapshot every 16 steps and the forward replayed in between")
    assert cabi.scan_plan(300, 7, 7, 32, torch.float32, cabi.M2D_PASS_FWD, ckpt_interval=8).startswith("m2d_fwd_kernel: one stream per image")
    assert cabi.scan_plan(300, 7, 7, 32, torch.float32, cabi.M2D_PASS_FWD, ckpt_interval=4).startswith("m2d_fwd_kernel: stacked images")


def test_plan_names_kernel_and_schedule(cabi):
    """m2d_scan_plan (host only): which kernel and schedule a problem gets on a 256-unit device."""
    import torch
    big = cabi.scan_plan(128, 56, 56, 64, torch.bfloat16, cabi.M2D_PASS_BWD)
    assert big.startswith("m2d_bwd2_kernel: one stream per image, 4 bands back to back, 256 workgroups of 8 waves, 32 channels each")
    assert big.endswith("a snapshot every 2 steps and one step in two recomputed")
    big4 = cabi.scan_plan(128, 56, 56, 64, torch.bfloat16, cabi.M2D_PASS_BWD, ckpt_interval=4)
    assert big4.startswith("m2d_bwd_kernel: one stream per image, 4 bands back to back, 256 workgroups of 8 waves, 32 channels each") and "snapshot" not in big4
    one = cabi.scan_plan(1, 256, 256, 64, torch.float32, cabi.M2D_PASS_BWD)
    assert one.startswith("m2d_bwd_split_kernel: linked sweep, 19 bands, 304 workgroups of 4 waves and 4 that stage, 4 channels each, 4 states per lane")
    two = cabi.scan_plan(1, 768, 768, 64, torch.float32, cabi.M2D_PASS_BWD)   # (more bands under way: workgroups of 8)
    assert two.startswith("m2d_bwd_split_kernel: linked sweep, 55 bands, 440 workgroups of 8 waves and 4 that stage, 8 channels each, 4 states per lane")
    ragged = cabi.scan_plan(1, 768, 768, 62, torch.float32, cabi.M2D_PASS_BWD)   # (rows that are no whole 16-byte chunks: no staging waves beside 8)
    assert ragged.startswith("m2d_bwd_split_kernel: linked sweep, 55 bands, 440 workgroups of 8 waves, 8 channels each, 4 states per lane")
    whole = cabi.scan_plan(1, 256, 256, 64, torch.float32, cabi.M2D_PASS_FWD, flags=cabi.M2D_FLAG_WHOLE_STATES)
    assert whole.startswith("m2d_fwd_kernel: linked sweep, 19 bands") and "16 states per lane" in whole
    small = cabi.scan_plan(128, 7, 7, 512, torch.bfloat16, cabi.M2D_PASS_FWD)
    assert small.startswith("m2d_fwd_kernel: stacked images, 8 per stream, 4 bands")   # two images of 7 rows per band
    # the bands of a stack have no neighbours: all 16 lanes are rows (two 8-row images or one 16-row image per band)
    assert cabi.scan_plan(128, 8, 8, 512, torch.bfloat16, cabi.M2D_PASS_BWD).startswith("m2d_bwd2_kernel: stacked images, 8 per stream, 4 bands")
    assert cabi.scan_plan(128, 16, 16, 320, torch.bfloat16, cabi.M2D_PASS_BWD).startswith("m2d_bwd2_kernel: stacked images, 6 per stream, 6 bands")
    assert cabi.scan_plan(2001, 3, 3, 8, torch.float32, cabi.M2D_PASS_FWD).startswith("m2d_fwd_kernel: stacked images, 8 per stream, 2 bands")   # five per band
    # a short buffer truncates, a bad descriptor reports its status and an empty text
    buf = ctypes.create_string_buffer(8)
    assert cabi.lib.m2d_scan_plan(ctypes.byref(D(cabi)), 0, buf, 8) == 0 and len(buf.value) == 7
    assert cabi.lib.m2d_scan_plan(ctypes.byref(D(cabi, H=1)), 0, buf, 8) == 2 and buf.value == b""


def test_python_surface_matches_reference_names():
    """models/kernels/wavefront_cuda.py exposes these names; models/mamba2d.py:10 imports one."""
    from mamba2d_amd.kernels import wavefront_cuda as w
    for name in ("wavefront_scan_cuda", "wf_cuda_fn_pr", "wf_cuda_fn_fr", "proj_params"):
        assert hasattr(w, name)
    import inspect
    sig = inspect.signature(w.wavefront_scan_cuda)
    positional = [n for n, q in sig.parameters.items() if q.kind is not inspect.Parameter.KEYWORD_ONLY]
    assert positional == ["x", "AT_log", "AL_log", "x_proj_w", "dt_projT_w", "dt_projT_b",
                          "dt_projL_w", "dt_projL_b", "D", "recomp"]
    assert sig.parameters["recomp"].default == "partial"
    # anything beyond the reference's signature is keyword-only and off by default
    extras = {n: q.default for n, q in sig.parameters.items() if q.kind is inspect.Parameter.KEYWORD_ONLY}
    assert extras == {"flip": False}


def test_entry_point_errors_match_reference():
    import torch
    from mamba2d_amd.wavefront import wavefront_scan_cuda
    z = torch.zeros
    with pytest.raises(ValueError, match=r"Wavefront scan kernel requires spatial dims > 1. Got H=1, W=5."):
        wavefront_scan_cuda(z(1, 1, 5, 4), *[None] * 8)
    E, N, R = 4, 16, 1
    a = (z(1, 3, 3, E), z(E, N), z(E, N), z(2 * R + 3 * N, E), z(E, R), z(E), z(E, R), z(E), z(E))
    with pytest.raises(ValueError, match="Unknown recomputation mode"):
        wavefront_scan_cuda(*a, recomp="sometimes")
