"""GPU tests of the unfinished channel sums between m2d_scan_bwd and m2d_proj_bwd_parts (M2D_FLAG_SUM_PARTS).

The scan's backward normally ends with a small kernel that adds the per-workgroup sums of d_C, d_BT, d_BL
and rounds them; with the flag the projections' backward adds them while it loads them.  Both do the
additions in the order of the parts and round once, so everything downstream has to agree bit for bit with
the two-step route, which the other tests check against the oracle.  (The reference forms these sums with
einsum in fused_backward_math, models/kernels/wavefront_cuda.py:218-227, and hands them to autograd,
wavefront_cuda.py:262-296.)
"""
import ctypes

import pytest
import torch

from tests.test_proj_gpu import N, WNAMES, make_case, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from mamba2d_amd import cabi
    return cabi


def scan_inputs(B, H, W, E, seed, dT, dL, BT, BL, C):
    g = torch.Generator().manual_seed(seed)
    A = -torch.exp(torch.rand(E, N, generator=g) * 2 - 1)
    bf = lambda t: t.to(torch.bfloat16).cuda()
    return dict(AT=bf(A), AL=bf(A.flip(0)), D=bf(torch.rand(E, generator=g)), dy=bf(torch.randn(B, H, W, E, generator=g)))


# (B, H, W, E, flip): one and several channel groups per image, a ragged last group, an image that is swept in
# linked bands, one image, the scan from the other corner
CASES = [(3, 14, 14, 64, False), (2, 20, 9, 192, False), (1, 33, 31, 328, True), (2, 150, 70, 64, False),
         (1, 2, 2, 8, False), (67, 16, 16, 64, True)]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{}_{}x{}_E{}_{}".format(*c))
@pytest.mark.parametrize("with_ckpt", [True, False], ids=["ckpt", "nockpt"])
def test_parts_route_equals_two_step_route(cabi, case, with_ckpt):
    B, H, W, E, flip = case
    say(f"\ncase sum_parts {case} ckpt={with_ckpt}")
    R, x, w, up, _ = make_case(B, H, W, E, seed=5, dtype=torch.bfloat16)
    xd = x.cuda()
    wd = {k: v.cuda() for k, v in w.items()}
    low, dT, dL, BT, BL, C = cabi.proj_fwd(xd, *[wd[k] for k in WNAMES], N)
    s = scan_inputs(B, H, W, E, 6, dT, dL, BT, BL, C)
    ck = None
    if with_ckpt:
        _, ck = cabi.scan_fwd(xd, dT, dL, s["AT"], s["AL"], BT, BL, C, s["D"], save_ckpt=True, flip=flip)
    args = (xd, dT, dL, s["AT"], s["AL"], BT, BL, C, s["D"], s["dy"])
    ga = cabi.scan_bwd(*args, ckpt=ck, flip=flip, dpre=True)
    gb = cabi.scan_bwd(*args, ckpt=ck, flip=flip, dpre=True, sum_parts=True)
    torch.cuda.synchronize()
    for i in (0, 1, 2, 3, 4, 8):
        assert torch.equal(ga[i], gb[i]), i
    parts = gb[5]
    d = cabi.make_desc(xd, N, flip)
    d.flags |= cabi.M2D_FLAG_DPRE | cabi.M2D_FLAG_SUM_PARTS
    assert parts.shape == (cabi.lib.m2d_scan_sum_parts(ctypes.byref(d)), B, H, W, 3 * N) and parts.dtype == torch.float32
    assert gb[6] is None and gb[7] is None
    total = parts[0].clone()
    for p in parts[1:]:
        total += p
    for k, i in zip(range(3), (7, 5, 6)):   # the records hold d_C, d_BT, d_BL
        assert torch.equal(total[..., k * N:(k + 1) * N].to(torch.bfloat16), ga[i]), i
    dxa, dxb = ga[0].clone(), gb[0].clone()
    wa = cabi.proj_bwd(xd, low, None, None, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], ga[1], ga[2], ga[5], ga[6], ga[7],
                       dxa, dpre=True)
    wb = cabi.proj_bwd(xd, low, None, None, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], gb[1], gb[2], parts, None, None,
                       dxb, dpre=True, sum_parts=parts.shape[0])
    torch.cuda.synchronize()
    assert torch.equal(dxa, dxb)
    for k, u, v in zip(WNAMES, wa, wb):
        assert torch.equal(u, v), k


def test_parts_are_refused_where_the_matrix_core_path_is_not_taken(cabi):
    """fp32 tensors and channel counts that are no multiple of 8 take the plain kernels, which read finished sums."""
    for dtype, E in ((torch.float32, 64), (torch.bfloat16, 12)):
        R, x, w, up, _ = make_case(1, 6, 6, E, seed=7, dtype=dtype)
        xd = x.cuda()
        wd = {k: v.cuda() for k, v in w.items()}
        low = cabi.proj_fwd(xd, *[wd[k] for k in WNAMES], N)[0]
        upd = {k: v.cuda() for k, v in up.items()}
        parts = torch.zeros(1, 1, 6, 6, 3 * N, device="cuda")
        with pytest.raises(RuntimeError, match="unsupported"):
            cabi.proj_bwd(xd, low, None, None, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], upd["d_deltaT"], upd["d_deltaL"],
                          parts, None, None, upd["dx"], dpre=True, sum_parts=1)
    torch.cuda.synchronize()
