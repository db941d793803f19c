"""The four operators of the shim trace without a device: their fake implementations (what
torch.compile sees, like the reference's register_fake no-ops at wavefront_cuda.py:33-57) return
outputs of the right shapes and dtypes for meta tensors."""
import math

import pytest
import torch


@pytest.fixture(scope="module")
def wf():
    from mamba2d_amd import wavefront
    return wavefront


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scan_ops_on_meta_tensors(wf, dtype):
    B, H, W, E, N = 2, 5, 7, 8, 16
    m = lambda *s: torch.empty(*s, dtype=dtype, device="meta")
    args = [m(B, H, W, E), m(B, H, W, E), m(B, H, W, E), m(E, N), m(E, N), m(B, H, W, N), m(B, H, W, N), m(B, H, W, N), m(E)]
    y, ck = wf.scan_fwd_op(*args, True, False)
    assert y.shape == (B, H, W, E) and y.dtype == dtype and y.device.type == "meta"
    assert ck.dtype == torch.uint8 and ck.numel() > 1
    y2, ck2 = wf.scan_fwd_op(*args, False, True)
    assert ck2.numel() == 1
    grads = wf.scan_bwd_op(*args, m(B, H, W, E), ck, False)
    assert [tuple(g.shape) for g in grads] == [tuple(a.shape) for a in args]
    assert all(g.dtype == dtype for g in grads)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_projection_ops_on_meta_tensors(wf, dtype):
    B, H, W, E, N = 2, 5, 7, 40, 16
    R = math.ceil(E / 16)
    x = torch.empty(B, H, W, E, dtype=dtype, device="meta")
    f = lambda *s: torch.empty(*s, dtype=torch.float32, device="meta")
    w = [f(2 * R + 3 * N, E), f(E, R), f(E), f(E, R), f(E)]
    low, dT, dL, BT, BL, C = wf.proj_fwd_op(x, *w, N, True)
    assert low.shape == (B, H, W, 2 * R) and dT.shape == dL.shape == x.shape
    assert BT.shape == BL.shape == C.shape == (B, H, W, N)
    assert all(t.dtype == dtype for t in (low, dT, dL, BT, BL, C))
    packed = wf.proj_fwd_op(x, *w, N, True, True)
    assert packed[3].shape == (B, H, W, 3 * N) and packed[3].dtype == torch.float32 and packed[4].numel() == packed[5].numel() == 0
    g = wf.proj_bwd_op(x, low, dT, dL, w[0], w[1], w[3], dT, dL, BT, BL, C, torch.empty_like(x), True)
    assert [tuple(t.shape) for t in g] == [tuple(t.shape) for t in w]
    assert all(t.dtype == torch.float32 for t in g)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("shape,dtype", [((2, 56, 56, 64), torch.bfloat16), ((1, 150, 90, 8), torch.float32), ((9, 7, 7, 32), torch.bfloat16)])
def test_fake_checkpoint_size_matches_the_library(shape, dtype, packed):
    """The fake of m2dscan::scan_fwd must size the checkpoint tensor as the real operator does, also when
    the caller brings packed B/C records (then the buffer holds no copy of them): a backend that plans
    memory from the fake's shapes would otherwise disagree with the kernel."""
    import ctypes
    from mamba2d_amd import cabi, wavefront  # noqa: F401  (registers the fakes)
    B, H, W, E = shape
    N = 16
    m = lambda *s, dt=dtype: torch.empty(*s, dtype=dt, device="meta")
    x = m(B, H, W, E)
    bc = m(B, H, W, 3 * N, dt=torch.float32) if packed else m(B, H, W, N)
    rest = (m(0), m(0)) if packed else (m(B, H, W, N), m(B, H, W, N))
    y, ck = torch.ops.m2dscan.scan_fwd(x, m(B, H, W, E), m(B, H, W, E), m(E, N), m(E, N), bc, *rest, m(E), True, False, False, packed)
    d = cabi.Desc(B, H, W, E, N, cabi.M2D_BF16 if dtype == torch.bfloat16 else cabi.M2D_F32,
                  cabi.M2D_FLAG_PACKED_BC if packed else 0, 0)
    assert ck.numel() == cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d)) and y.shape == x.shape


def test_reference_operator_pair_on_meta_tensors(wf):
    """mamba2d::wf_fwd / mamba2d::wf_bwd carry the reference's names, argument order and mutated arguments
    (wavefront_cuda.py:25-57) and trace on meta tensors (they return nothing, like the reference's fakes), and the
    reference module's names resolve in the import-path twin."""
    from mamba2d_amd.kernels import wavefront_cuda as twin
    for name in ("wavefront_scan_cuda", "wf_cuda_fn_pr", "wf_cuda_fn_fr", "proj_params", "fused_backward_math", "wf_fwd_op", "wf_bwd_op"):
        assert hasattr(twin, name), name
    B, H, W, E, N = 2, 3, 4, 5, 6
    m = lambda *s: torch.empty(*s, dtype=torch.float64, device="meta")
    hs = m(B, H, W, E, N)
    assert wf.wf_fwd_op(hs, m(B, H, W, E), m(B, H, W, E), m(B, H, W, E), m(B, H, W, N), m(B, H, W, N), m(E, N), m(E, N)) is None
    assert wf.wf_bwd_op(hs, m(B, H, W, E), m(B, H, W, E), m(B, H, W, E), m(E, N), m(E, N), m(B, H, W, E, N), m(B, H, W, E, N),
                        m(B, H, W, E, N), m(2, B, H, E, N)) is None
    s_fwd, s_bwd = torch.ops.mamba2d.wf_fwd.default._schema, torch.ops.mamba2d.wf_bwd.default._schema
    assert [a.name for a in s_fwd.arguments] == ["hs", "x", "deltaT", "deltaL", "BT", "BL", "AT", "AL"]
    assert [a.name for a in s_bwd.arguments] == ["hs", "x", "deltaT", "deltaL", "AT", "AL", "grad_output", "dDAT", "dDAL", "omega"]
    assert [a.name for a in s_fwd.arguments if a.is_write] == ["hs"]
    assert [a.name for a in s_bwd.arguments if a.is_write] == ["grad_output", "dDAT", "dDAL", "omega"]


def test_fused_backward_math_against_autograd():
    """wavefront.fused_backward_math (the reference's algebra behind wf_bwd, wavefront_cuda.py:97-139) in float64 on
    the CPU: fed the oracle's dDAT, dDAL, dBX it must return the oracle's gradients."""
    from mamba2d_amd import wavefront as wf
    from oracle import scan_oracle as so
    B, H, W, E, N = 2, 4, 5, 3, 6
    inp = {k: v.double() for k, v in so.make_inputs(B, H, W, E, N, seed=3, dtype=torch.float32).items()}
    cs = so.CScan()
    res = cs.backward(*[inp[k] for k in so.INPUT_NAMES], inp["dy"], want_intermediates=True)
    t = lambda a: torch.from_numpy(a)
    out = wf.fused_backward_math(t(res["dDAT"]), t(res["dDAL"]), t(res["dBX"]), inp["deltaT"], inp["deltaL"], inp["AT"], inp["AL"],
                                 inp["BT"], inp["BL"], inp["x"])
    want = [res["d_x"] - (inp["dy"] * inp["D"]).numpy(), res["d_deltaT"], res["d_deltaL"], res["d_AT"], res["d_AL"], res["d_BT"], res["d_BL"]]
    for got, w in zip(out, want):
        assert so.rel_err(got, w) < 1e-12
