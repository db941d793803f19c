"""GPU parity tests of the projection kernels (m2d_proj_fwd / m2d_proj_bwd) through the C ABI.

The checker is the restatement of the reference's proj_params with stock torch operators in
fp64 on the CPU (oracle.scan_oracle.proj_params_ref, models/kernels/wavefront_cuda.py:63-95)
and torch.autograd through it, which is how the reference itself differentiates the projections
(wavefront_cuda.py:262-296).  Tolerances: fp32 1e-4, bf16 tensors 2e-2 (max error over max value).
"""
import math

import pytest
import torch

from oracle import scan_oracle as so

pytestmark = pytest.mark.gpu

N = 16


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def cabi():
    from mamba2d_amd import cabi
    return cabi


def make_case(B, H, W, E, seed, dtype):
    """x and weights with the magnitudes of an M2D block (models/mamba2d.py:57-111); the weights are
    rounded to `dtype` as the reference's entry point does (wavefront_cuda.py:327-332)."""
    R = math.ceil(E / 16)
    g = torch.Generator().manual_seed(seed)
    dt = torch.exp(torch.rand(E, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
    w = dict(
        x_proj_w=(torch.rand(2 * R + 3 * N, E, generator=g) * 2 - 1) / math.sqrt(E),
        dt_projT_w=(torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5,
        dt_projT_b=dt + torch.log(-torch.expm1(-dt)),
        dt_projL_w=(torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5,
        dt_projL_b=(dt + torch.log(-torch.expm1(-dt))).flip(0).contiguous())
    raw = dict(w)
    w = {k: v.to(dtype).float() for k, v in w.items()}
    x = torch.randn(B, H, W, E, generator=g).to(dtype)
    up = {k: torch.randn(B, H, W, n, generator=g).to(dtype)
          for k, n in (("d_deltaT", E), ("d_deltaL", E), ("d_BT", N), ("d_BL", N), ("d_C", N), ("dx", E))}
    return R, x, w, up, raw


WNAMES = ("x_proj_w", "dt_projT_w", "dt_projT_b", "dt_projL_w", "dt_projL_b")

# (B, H, W, E): tiles that end inside the batch, fewer positions than one wave owns, channel counts
# that are no multiple of the 64-channel chunk, one to seven 16-wide chunks of outputs, the largest rank
SHAPES = [(2, 9, 12, 32), (1, 5, 7, 3), (2, 14, 14, 64), (1, 8, 8, 128), (1, 40, 4, 100), (1, 7, 9, 320),
          (3, 7, 7, 512), (5, 31, 30, 64), (1, 2, 2, 8), (1, 2, 3, 16), (1, 3, 3, 504), (1, 17, 1, 72)]


def reference(x, w, up, R):
    """fp64 outputs and gradients of the projections for the upstream gradients `up`."""
    x64 = x.double().requires_grad_(True)
    w64 = {k: v.double().requires_grad_(True) for k, v in w.items()}
    z = torch.nn.functional.linear(x64, w64["x_proj_w"])
    low = z[..., :2 * R]
    A = torch.zeros(x.shape[-1], N, dtype=torch.float64)
    dT, dL, _, _, BT, BL, C = so.proj_params_ref(x64, A, A, *[w64[k] for k in WNAMES])
    outs = dict(lowrank=low, deltaT=dT, deltaL=dL, BT=BT, BL=BL, C=C)
    loss = sum((outs[k] * up["d_" + k].double()).sum() for k in ("deltaT", "deltaL", "BT", "BL", "C"))
    grads = torch.autograd.grad(loss, [x64] + [w64[k] for k in WNAMES])
    g = dict(zip(("x",) + WNAMES, grads))
    g["x"] = g["x"] + up["dx"].double()
    return {k: v.detach() for k, v in outs.items()}, g


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_projections_match_reference(cabi, shape, dtype, tol):
    say(f"\ncase proj {shape} {dtype}")
    B, H, W, E = shape
    R, x, w, up, _ = make_case(B, H, W, E, seed=sum(shape), dtype=dtype)
    ref_out, ref_g = reference(x, w, up, R)
    xd = x.cuda()
    wd = {k: v.cuda() for k, v in w.items()}
    low, dT, dL, BT, BL, C = cabi.proj_fwd(xd, *[wd[k] for k in WNAMES], N)
    got = dict(lowrank=low, deltaT=dT, deltaL=dL, BT=BT, BL=BL, C=C)
    for k, v in got.items():
        assert v.dtype == dtype and v.shape == ref_out[k].shape
        assert so.rel_err(v.float().cpu(), ref_out[k]) < tol, k
    # the step sizes span two decades: also hold every element to the tolerance
    assert so.elem_rel_err(dT.float().cpu(), ref_out["deltaT"]) < 2 * tol

    upd = {k: v.cuda() for k, v in up.items()}
    dx = upd["dx"].clone()
    gw = cabi.proj_bwd(xd, low, dT, dL, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"],
                       upd["d_deltaT"], upd["d_deltaL"], upd["d_BT"], upd["d_BL"], upd["d_C"], dx)
    torch.cuda.synchronize()
    assert dx.dtype == dtype and so.rel_err(dx.float().cpu(), ref_g["x"]) < tol, "dx"
    for k, g in zip(WNAMES, gw):
        assert g.dtype == torch.float32 and g.shape == ref_g[k].shape
        assert so.rel_err(g.cpu(), ref_g[k]) < tol, k


@pytest.mark.parametrize("shape", [(2, 14, 14, 64), (1, 40, 4, 100)], ids=lambda s: "x".join(map(str, s)))
def test_library_rounds_weights_like_a_cast(cabi, shape):
    """M2D_FLAG_ROUND_WEIGHTS on fp32 weights gives bit for bit what weights cast to bf16 beforehand give."""
    say(f"\ncase proj round_weights {shape}")
    B, H, W, E = shape
    R, x, w, up, raw = make_case(B, H, W, E, seed=7, dtype=torch.bfloat16)
    xd = x.cuda()
    wd = {k: v.cuda() for k, v in w.items()}
    rd = {k: v.cuda() for k, v in raw.items()}
    assert any(not torch.equal(wd[k], rd[k]) for k in WNAMES)
    a = cabi.proj_fwd(xd, *[wd[k] for k in WNAMES], N)
    b = cabi.proj_fwd(xd, *[rd[k] for k in WNAMES], N, round_weights=True)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    upd = {k: v.cuda() for k, v in up.items()}
    dxa, dxb = upd["dx"].clone(), upd["dx"].clone()
    args = (upd["d_deltaT"], upd["d_deltaL"], upd["d_BT"], upd["d_BL"], upd["d_C"])
    ga = cabi.proj_bwd(xd, a[0], a[1], a[2], wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], *args, dxa)
    gb = cabi.proj_bwd(xd, a[0], a[1], a[2], rd["x_proj_w"], rd["dt_projT_w"], rd["dt_projL_w"], *args, dxb, round_weights=True)
    assert torch.equal(dxa, dxb)
    for u, v in zip(ga, gb):
        assert torch.equal(u, v)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(2, 14, 14, 64), (1, 40, 4, 100), (3, 7, 9, 24)], ids=lambda s: "x".join(map(str, s)))
def test_gradients_before_the_softplus_are_accepted(cabi, shape, dtype, tol):
    """M2D_FLAG_DPRE: handed d_delta * (1 - exp(-delta)) in place of d_delta, and no deltas, the backward gives
    what it gives for d_delta and delta."""
    say(f"\ncase proj dpre {shape} {dtype}")
    B, H, W, E = shape
    R, x, w, up, _ = make_case(B, H, W, E, seed=3, dtype=dtype)
    xd = x.cuda()
    wd = {k: v.cuda() for k, v in w.items()}
    low, dT, dL, BT, BL, C = cabi.proj_fwd(xd, *[wd[k] for k in WNAMES], N)
    upd = {k: v.cuda() for k, v in up.items()}
    rest = (upd["d_BT"], upd["d_BL"], upd["d_C"])
    dxa, dxb = upd["dx"].clone(), upd["dx"].clone()
    ga = cabi.proj_bwd(xd, low, dT, dL, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], upd["d_deltaT"], upd["d_deltaL"],
                       *rest, dxa)
    slope = lambda d: -torch.expm1(-d.double())
    preT = (upd["d_deltaT"].double() * slope(dT)).to(dtype)
    preL = (upd["d_deltaL"].double() * slope(dL)).to(dtype)
    gb = cabi.proj_bwd(xd, low, None, None, wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"], preT, preL, *rest, dxb,
                       dpre=True)
    torch.cuda.synchronize()
    assert so.rel_err(dxb.float().cpu(), dxa.float().cpu()) < tol
    for k, u, v in zip(WNAMES, ga, gb):
        assert so.rel_err(v.cpu(), u.cpu()) < tol, k


def test_projection_limits_are_reported(cabi):
    import ctypes
    d = cabi.Desc(1, 4, 4, 64, 16, cabi.M2D_F32, 0, 0)
    assert cabi.lib.m2d_proj_workspace_bytes(ctypes.byref(d), 4, cabi.M2D_PASS_FWD) > 0
    assert cabi.lib.m2d_proj_workspace_bytes(ctypes.byref(d), 33, cabi.M2D_PASS_FWD) == 0     # dt_rank > 32
    d8 = cabi.Desc(1, 4, 4, 64, 8, cabi.M2D_F32, 0, 0)
    assert cabi.lib.m2d_proj_workspace_bytes(ctypes.byref(d8), 4, cabi.M2D_PASS_BWD) == 0    # d_state != 16


def test_positions_beyond_two_giga_elements(cabi):
    """Maximum sizes: P*E = 2.16e9 elements (more than 2^31).  Positions are independent, so an input that
    repeats 256 seeded images 42 times must give, bit for bit, the outputs and dx of the 256 images
    on their own; the weight gradients (sums over positions) must be 42 times theirs."""
    say("\ncase proj beyond_two_giga_elements")
    free, _ = torch.cuda.mem_get_info()
    if free < 100 * 2**30:
        pytest.skip("needs 100 GB of free device memory")
    B0, reps, H, W, E = 256, 42, 56, 56, 64
    R, x, w, up, _ = make_case(B0, H, W, E, seed=11, dtype=torch.bfloat16)
    wd = {k: v.cuda() for k, v in w.items()}
    x0 = x.cuda()
    up0 = {k: v.cuda() for k, v in up.items()}
    out0 = cabi.proj_fwd(x0, *[wd[k] for k in WNAMES], N)
    dx0 = up0["dx"].clone()
    gw0 = cabi.proj_bwd(x0, out0[0], out0[1], out0[2], wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"],
                        up0["d_deltaT"], up0["d_deltaL"], up0["d_BT"], up0["d_BL"], up0["d_C"], dx0)
    xb = x0.repeat(reps, 1, 1, 1)
    assert xb.numel() > 2**31
    upb = {k: v.repeat(reps, 1, 1, 1) for k, v in up0.items()}
    out = cabi.proj_fwd(xb, *[wd[k] for k in WNAMES], N)
    dx = upb["dx"]   # read and written in place
    gw = cabi.proj_bwd(xb, out[0], out[1], out[2], wd["x_proj_w"], wd["dt_projT_w"], wd["dt_projL_w"],
                       upb["d_deltaT"], upb["d_deltaL"], upb["d_BT"], upb["d_BL"], upb["d_C"], dx)
    torch.cuda.synchronize()
    for r in range(reps):
        for u, v in zip(out, out0):
            assert torch.equal(u[r * B0:(r + 1) * B0], v), r
        assert torch.equal(dx[r * B0:(r + 1) * B0], dx0), r
    for k, g, s in zip(WNAMES, gw, gw0):
        e = so.rel_err(g.cpu(), reps * s.cpu())
        say(f"  {k} rel_err {e:.3e}")
        assert e < 5e-4, (k, e)
    del xb, upb, out, dx
    torch.cuda.empty_cache()
