"""The reference's operator pair at its own boundary: mamba2d::wf_fwd (hs materialised) and mamba2d::wf_bwd
(dBX in place over grad_output, dDAT, dDAL, the two-slot omega), models/kernels/wavefront_cuda.py:25-57 and
wf_cuda.cu:40-69, 108-160 -- any number of states, float64 / float32 / bfloat16.

Checked against the C oracle's intermediates (hs, dBX, dDAT, dDAL), which tests/test_oracle.py pins by autograd
through an independent forward, and end to end: the reference's own backward data flow (wavefront_cuda.py:169-196:
dC, dHS, wf_bwd, fused_backward_math, d_x) rebuilt on the two operators must give the nine gradients of the fused
path.  Tolerances: fp64 1e-10, fp32 1e-4, bf16 2e-2 (tensor-normalised).
"""
import numpy as np
import pytest
import torch

from oracle import scan_oracle as so

pytestmark = pytest.mark.gpu

TOL = {torch.float64: 1e-10, torch.float32: 1e-4, torch.bfloat16: 2e-2}


def _inputs(B, H, W, E, N, dtype, seed):
    inp = so.make_inputs(B, H, W, E, N, seed=seed, dtype=torch.float32 if dtype == torch.float64 else dtype)
    return {k: v.to(dtype) for k, v in inp.items()}


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.bfloat16], ids=["f64", "f32", "bf16"])
@pytest.mark.parametrize("shape", [(2, 14, 14, 32, 16), (3, 5, 9, 6, 8), (1, 2, 2, 1, 1), (2, 20, 7, 5, 24), (1, 1, 6, 3, 4), (1, 7, 1, 3, 4)],
                         ids=lambda s: "x".join(map(str, s)))
def test_wf_fwd_and_wf_bwd_against_the_oracle(cscan, shape, dtype):
    from mamba2d_amd import wavefront as wf
    B, H, W, E, N = shape
    print(f"\ncase wf ops {shape} {dtype}", flush=True)
    inp = _inputs(B, H, W, E, N, dtype, seed=sum(shape))
    dev = {k: v.cuda() for k, v in inp.items()}
    ref = {k: v.double() for k, v in inp.items()}
    hs = torch.empty(B, H, W, E, N, dtype=dtype, device="cuda")
    assert wf.wf_fwd_op(hs, dev["x"], dev["deltaT"], dev["deltaL"], dev["BT"], dev["BL"], dev["AT"], dev["AL"]) is None
    a_ref = [ref[k] for k in so.INPUT_NAMES]
    if H < 2 or W < 2:   # the oracle restates the entry point, which refuses such grids; the kernels themselves do not: row 0 / column 0 are 1-D scans
        g = torch.exp(ref["deltaL"].unsqueeze(-1) * ref["AL"]) if H == 1 else torch.exp(ref["deltaT"].unsqueeze(-1) * ref["AT"])
        u = (ref["deltaL"] * ref["x"]).unsqueeze(-1) * ref["BL"].unsqueeze(-2) if H == 1 else (ref["deltaT"] * ref["x"]).unsqueeze(-1) * ref["BT"].unsqueeze(-2)
        if W == 1:   # a single column: the origin takes the L input (wf_cuda.cu:58-59), the rest is the T scan
            u[:, 0] = ((ref["deltaL"] * ref["x"]).unsqueeze(-1) * ref["BL"].unsqueeze(-2))[:, 0]
        h_ref = torch.zeros_like(u)
        ax = 2 if H == 1 else 1
        prev = torch.zeros_like(u.select(ax, 0))
        for k in range(u.shape[ax]):
            prev = (g.select(ax, k) * prev if k else 0) + u.select(ax, k)
            h_ref.select(ax, k).copy_(prev)
        assert so.rel_err(hs.double().cpu(), h_ref) < TOL[dtype]
        return
    y_ref, hs_ref = cscan.forward(*a_ref, want_hs=True)
    e = so.rel_err(hs.double().cpu(), hs_ref)
    print(f"  hs rel_err {e:.3e}", flush=True)
    assert e < TOL[dtype]
    # backward at the reference's boundary: dHS = dy (x) C goes in, dBX comes back in its place
    res = cscan.backward(*a_ref, ref["dy"], want_intermediates=True)
    go = (dev["dy"].unsqueeze(-1) * dev["C"].unsqueeze(-2)).contiguous()
    dDAT, dDAL = torch.empty_like(hs), torch.empty_like(hs)
    omega = torch.zeros(2, B, H, E, N, dtype=dtype, device="cuda")
    hs_in = torch.from_numpy(np.ascontiguousarray(hs_ref)).to(dtype).cuda()   # the oracle's states, so that only wf_bwd is under test
    assert wf.wf_bwd_op(hs_in, dev["x"], dev["deltaT"], dev["deltaL"], dev["AT"], dev["AL"], go, dDAT, dDAL, omega) is None
    go_ref = (ref["dy"].to(dtype).double().unsqueeze(-1) * ref["C"].unsqueeze(-2))   # (what went in, rounded as the tensor holds it)
    for name, got in (("dBX", go), ("dDAT", dDAT), ("dDAL", dDAL)):
        e = so.rel_err(got.double().cpu(), res[name])
        print(f"  {name} rel_err {e:.3e}", flush=True)
        assert e < (TOL[dtype] if dtype != torch.bfloat16 else 3e-2), name


@pytest.mark.parametrize("dtype,N", [(torch.float32, 16), (torch.float32, 5), (torch.float64, 8)], ids=["f32-16", "f32-5", "f64-8"])
def test_reference_backward_data_flow_on_the_operator_pair(cscan, dtype, N):
    """wavefront_cuda.py:146-196 rebuilt on wf_fwd_op / wf_bwd_op / fused_backward_math: y and the nine gradients
    against the oracle (and so against the fused operators, which meet the same oracle)."""
    from mamba2d_amd import wavefront as wf
    B, H, W, E = 2, 9, 12, 6
    inp = _inputs(B, H, W, E, N, dtype, seed=77)
    d = {k: v.cuda() for k, v in inp.items()}
    hs = torch.empty(B, H, W, E, N, dtype=dtype, device="cuda")
    wf.wf_fwd_op(hs, d["x"], d["deltaT"], d["deltaL"], d["BT"], d["BL"], d["AT"], d["AL"])
    y = (hs * d["C"].unsqueeze(-2)).sum(-1) + d["x"] * d["D"]
    dD = (d["dy"] * d["x"]).sum((0, 1, 2))
    dC = (d["dy"].unsqueeze(-1) * hs).sum(-2)
    go = (d["dy"].unsqueeze(-1) * d["C"].unsqueeze(-2)).contiguous()
    dDAT, dDAL = torch.empty_like(hs), torch.empty_like(hs)
    omega = torch.empty(2, B, H, E, N, dtype=dtype, device="cuda")
    wf.wf_bwd_op(hs, d["x"], d["deltaT"], d["deltaL"], d["AT"], d["AL"], go, dDAT, dDAL, omega)
    d_x_scan, d_dT, d_dL, d_AT, d_AL, d_BT, d_BL = wf.fused_backward_math(dDAT, dDAL, go, d["deltaT"], d["deltaL"], d["AT"], d["AL"], d["BT"], d["BL"], d["x"])
    got = dict(d_x=d_x_scan + d["dy"] * d["D"], d_deltaT=d_dT, d_deltaL=d_dL, d_AT=d_AT, d_AL=d_AL, d_BT=d_BT, d_BL=d_BL, d_C=dC, d_D=dD)
    ref_in = [inp[k].double() for k in so.INPUT_NAMES]
    assert so.rel_err(y.double().cpu(), cscan.forward(*ref_in)) < TOL[dtype]
    g_ref = cscan.backward(*ref_in, inp["dy"].double())
    for k in so.CScan.GRADS:
        e = so.rel_err(got[k].double().cpu(), g_ref[k])
        print(f"  {k} rel_err {e:.3e}", flush=True)
        assert e < TOL[dtype] * (10 if dtype == torch.float32 else 1), k


def test_wf_ops_reject_mixed_dtypes_and_shapes():
    from mamba2d_amd import wavefront as wf
    hs = torch.empty(1, 3, 3, 2, 4, device="cuda")
    x = torch.zeros(1, 3, 3, 2, device="cuda")
    bc = torch.zeros(1, 3, 3, 4, device="cuda")
    A = torch.zeros(2, 4, device="cuda")
    with pytest.raises(RuntimeError, match="dtype"):
        wf.wf_fwd_op(hs, x.double(), x, x, bc, bc, A, A)
    with pytest.raises(RuntimeError, match="shape"):
        wf.wf_fwd_op(hs, x, x, x, bc, bc, A, A[:, :3].contiguous())
