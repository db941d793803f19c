"""GPU tests of the Python operator surface (mamba2d_amd.wavefront) through the PyTorch shim:
autograd Functions with the reference's signatures, entry point, both recompute modes."""
import math

import pytest
import torch

from oracle import scan_oracle as so

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def wf():
    from mamba2d_amd import wavefront
    return wavefront


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("save", [True, False], ids=["ckpt_saved", "ckpt_rebuilt"])
def test_fn_pr_forward_backward(wf, cscan, dtype, tol, save):
    say(f"\ncase fn_pr {dtype} save={save}")
    inp = so.make_inputs(4, 14, 14, 16, 16, seed=11, dtype=dtype)
    leaves = [inp[k].cuda().requires_grad_(True) for k in so.INPUT_NAMES]
    old = wf.SAVE_CHECKPOINTS
    wf.SAVE_CHECKPOINTS = save
    try:
        y = wf.wf_cuda_fn_pr.apply(*leaves)
        # the forward keeps its checkpoints exactly when asked to (a 1-byte tensor stands for none)
        assert (y.grad_fn.saved_tensors[-1].numel() > 1) == save
        grads = torch.autograd.grad(y, leaves, inp["dy"].cuda())
    finally:
        wf.SAVE_CHECKPOINTS = old
    ref_in = [inp[k].double() for k in so.INPUT_NAMES]
    assert y.dtype == dtype and so.rel_err(y.float().cpu(), cscan.forward(*ref_in)) < tol
    g_ref = cscan.backward(*ref_in, inp["dy"].double())
    for k, g, leaf in zip(so.CScan.GRADS, grads, leaves):
        assert g.dtype == leaf.dtype and g.shape == leaf.shape
        assert so.rel_err(g.float().cpu(), g_ref[k]) < tol, k


def make_block_params(E, N, R, seed, device):
    """Parameters shaped and initialised like M2DBlock's (models/mamba2d.py:57-111)."""
    g = torch.Generator().manual_seed(seed)
    dt = torch.exp(torch.rand(E, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
    inv_dt = dt + torch.log(-torch.expm1(-dt))
    std = R ** -0.5
    p = dict(
        AT_log=torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)),
        AL_log=torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)),
        x_proj_w=(torch.rand(2 * R + 3 * N, E, generator=g) * 2 - 1) / math.sqrt(E),
        dt_projT_w=(torch.rand(E, R, generator=g) * 2 - 1) * std, dt_projT_b=inv_dt.clone(),
        dt_projL_w=(torch.rand(E, R, generator=g) * 2 - 1) * std, dt_projL_b=inv_dt.clone(),
        D=torch.ones(E))
    return {k: v.to(device) for k, v in p.items()}


ORDER = ("AT_log", "AL_log", "x_proj_w", "dt_projT_w", "dt_projT_b", "dt_projL_w", "dt_projL_b", "D")


@pytest.fixture(params=[True, False], ids=["own_projections", "torch_projections"])
def projections(wf, request):
    """The entry point with the library's projection kernels and with stock torch operators."""
    old = wf.FUSED_PROJECTIONS
    wf.FUSED_PROJECTIONS = request.param
    yield request.param
    wf.FUSED_PROJECTIONS = old


@pytest.mark.parametrize("recomp", ["partial", "full"])
def test_entry_point_matches_oracle_fp32(wf, recomp, projections):
    say(f"\ncase entry_point {recomp} own_projections={projections}")
    B, H, W, E, N = 2, 9, 12, 32, 16
    R = math.ceil(E / 16)
    p = make_block_params(E, N, R, 0, "cuda")
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(1)).cuda()
    dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(2)).cuda()
    leaves = [x.clone().requires_grad_(True)] + [p[k].clone().requires_grad_(True) for k in ORDER]
    y = wf.wavefront_scan_cuda(*leaves, recomp=recomp)
    grads = torch.autograd.grad(y, leaves, dy)
    # oracle: same projections in fp64 on the CPU, scan by the differentiable restatement
    ref_leaves = [t.detach().double().cpu().requires_grad_(True) for t in leaves]
    y_ref = so.wavefront_scan_ref(*ref_leaves)
    g_ref = torch.autograd.grad(y_ref, ref_leaves, dy.double().cpu())
    assert so.rel_err(y.cpu(), y_ref.detach()) < 1e-4
    for name, g, gr in zip(("x",) + ORDER, grads, g_ref):
        assert so.rel_err(g.cpu(), gr) < 2e-4, name


@pytest.mark.parametrize("interval", [8, 16])
@pytest.mark.parametrize("recomp", ["partial", "full"])
def test_entry_point_with_longer_checkpoint_interval(wf, recomp, interval, monkeypatch):
    """cabi.CKPT_INTERVAL (the one switch, which mamba2d_amd.wavefront reads) reaches the library through the operators: fewer bytes saved for the backward,
    the same gradients (the oracle's, to the entry point's fp32 bound); 24 states run as two groups."""
    say(f"\ncase entry_point {recomp} ckpt_interval={interval}")
    for N in (16, 24):
        B, H, W, E = 2, 30, 12, 32
        R = math.ceil(E / 16)
        p = make_block_params(E, N, R, 0, "cuda")
        x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(1)).cuda()
        dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(2)).cuda()
        kept = {}
        for iv in (0, interval):
            monkeypatch.setattr(wf.cabi, "CKPT_INTERVAL", iv)
            real, seen = wf.scan_fwd_op, []

            def spy(*a, **kw):
                out = real(*a, **kw)
                seen.append(out[1].numel())
                return out

            monkeypatch.setattr(wf, "scan_fwd_op", spy)
            leaves = [x.clone().requires_grad_(True)] + [p[k].clone().requires_grad_(True) for k in ORDER]
            y = wf.wavefront_scan_cuda(*leaves, recomp=recomp)
            grads = torch.autograd.grad(y, leaves, dy)
            monkeypatch.setattr(wf, "scan_fwd_op", real)
            kept[iv] = sum(seen)
        if recomp == "partial":
            assert kept[interval] < kept[0], kept
        ref_leaves = [t.detach().double().cpu().requires_grad_(True) for t in leaves]
        y_ref = so.wavefront_scan_ref(*ref_leaves)
        g_ref = torch.autograd.grad(y_ref, ref_leaves, dy.double().cpu())
        assert so.rel_err(y.cpu(), y_ref.detach()) < 1e-4
        for name, g, gr in zip(("x",) + ORDER, grads, g_ref):
            assert so.rel_err(g.cpu(), gr) < 2e-4, (N, name)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("N", [1, 8, 24, 32])
def test_fn_pr_other_state_counts(wf, cscan, N, dtype, tol):
    """d_state other than 16 (a constructor argument of the reference's block, models/mamba2d.py:23):
    the operator splits the states into groups of 16, padding the last one."""
    say(f"\ncase fn_pr N={N} {dtype}")
    inp = so.make_inputs(3, 9, 17, 8, N, seed=21, dtype=dtype)
    leaves = [inp[k].cuda().requires_grad_(True) for k in so.INPUT_NAMES]
    y = wf.wf_cuda_fn_pr.apply(*leaves)
    grads = torch.autograd.grad(y, leaves, inp["dy"].cuda())
    ref_in = [inp[k].double() for k in so.INPUT_NAMES]
    assert y.dtype == dtype and so.rel_err(y.float().cpu(), cscan.forward(*ref_in)) < tol
    g_ref = cscan.backward(*ref_in, inp["dy"].double())
    for k, g, leaf in zip(so.CScan.GRADS, grads, leaves):
        assert g.dtype == leaf.dtype and g.shape == leaf.shape
        assert so.rel_err(g.float().cpu(), g_ref[k]) < tol, k


@pytest.mark.parametrize("recomp", ["partial", "full"])
@pytest.mark.parametrize("N", [8, 20])
def test_entry_point_other_state_counts_fp32(wf, recomp, N):
    say(f"\ncase entry_point {recomp} N={N}")
    B, H, W, E = 2, 16, 7, 32
    R = math.ceil(E / 16)
    p = make_block_params(E, N, R, 7, "cuda")
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(8)).cuda()
    dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(9)).cuda()
    leaves = [x.clone().requires_grad_(True)] + [p[k].clone().requires_grad_(True) for k in ORDER]
    y = wf.wavefront_scan_cuda(*leaves, recomp=recomp, flip=(N == 20))
    grads = torch.autograd.grad(y, leaves, dy)
    ref_leaves = [t.detach().double().cpu().requires_grad_(True) for t in leaves]
    xr, dyr = ref_leaves[0], dy.double().cpu()
    if N == 20:   # bottom-right scan = flipped input, flipped output (models/mamba2d.py:163-173)
        y_ref = torch.flip(so.wavefront_scan_ref(torch.flip(xr, (1, 2)), *ref_leaves[1:]), (1, 2))
    else:
        y_ref = so.wavefront_scan_ref(*ref_leaves)
    g_ref = torch.autograd.grad(y_ref, ref_leaves, dyr)
    assert so.rel_err(y.cpu(), y_ref.detach()) < 1e-4
    for name, g, gr in zip(("x",) + ORDER, grads, g_ref):
        assert g.shape == gr.shape and so.rel_err(g.cpu(), gr) < 2e-4, name


@pytest.mark.parametrize("recomp", ["partial", "full"])
@pytest.mark.parametrize("N", [16, 8])
def test_entry_point_under_torch_compile(wf, projections, recomp, N):
    """The reference registers its kernels as custom operators so that torch.compile traces through the
    scan (wavefront_cuda.py:25-57).  Here: the entry point compiled with the aot_eager backend (dynamo
    tracing, functionalisation, fake tensors of every operator; no code generation) gives the bits of
    the eager call, forward and backward."""
    say(f"\ncase torch.compile {recomp} N={N} own_projections={projections}")
    import torch._dynamo
    torch._dynamo.reset()
    B, H, W, E = 2, 14, 20, 32
    p = make_block_params(E, N, 2, 0, "cuda")
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(1)).cuda()
    dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(2)).cuda()

    def fn(*a):
        return wf.wavefront_scan_cuda(*a, recomp=recomp) * 2.0

    def run(f):
        leaves = [x.clone().requires_grad_(True)] + [p[k].clone().requires_grad_(True) for k in ORDER]
        y = f(*leaves)
        return y, torch.autograd.grad(y, leaves, dy)

    y0, g0 = run(fn)
    # wf_cuda_fn_fr re-derives the projections under autograd inside its backward (requires_grad_ on
    # detached copies, as the reference does at wavefront_cuda.py:262-296): dynamo breaks the graph there
    # and runs that Function eagerly, so only the other paths are asked for one whole graph
    through_fr = recomp == "full" and (N != 16 or not projections)
    y1, g1 = run(torch.compile(fn, backend="aot_eager", fullgraph=not through_fr))
    assert torch.equal(y0, y1)
    for name, a, b in zip(("x",) + ORDER, g0, g1):
        assert torch.equal(a, b), name
    torch._dynamo.reset()


def test_partial_and_full_agree_bf16(wf, projections):
    """The two recompute modes are the same function of the nine raw inputs."""
    say(f"\ncase partial_vs_full bf16 own_projections={projections}")
    B, H, W, E, N = 3, 14, 14, 64, 16
    R = math.ceil(E / 16)
    p = make_block_params(E, N, R, 3, "cuda")
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(4)).cuda().bfloat16()
    dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(5)).cuda().bfloat16()
    outs = {}
    for mode in ("partial", "full"):
        leaves = [x.clone().requires_grad_(True)] + [p[k].clone().requires_grad_(True) for k in ORDER]
        y = wf.wavefront_scan_cuda(*leaves, recomp=mode)
        outs[mode] = (y, torch.autograd.grad(y, leaves, dy))
    assert y.dtype == torch.bfloat16
    assert torch.equal(outs["partial"][0], outs["full"][0])
    for a, b in zip(outs["partial"][1], outs["full"][1]):
        assert a.dtype == b.dtype and so.rel_err(a.float().cpu(), b.float().cpu()) < 2e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)], ids=["f32", "bf16"])
def test_raw_parameters_match_cast_parameters(wf, dtype, tol):
    """M2D_FLAG_RAW_PARAMS: fp32 A_log and D in, the library forms A = -exp(A_log) and rounds like
    the reference's casts; gradients come back for A_log and D in fp32."""
    say(f"\ncase raw parameters {dtype}")
    inp = so.make_inputs(2, 9, 30, 8, 16, seed=5, dtype=torch.float32)
    a = {k: inp[k].cuda() for k in so.INPUT_NAMES}
    logT, logL = torch.log(-a["AT"]), torch.log(-a["AL"])
    act = [a[k].to(dtype) for k in ("x", "deltaT", "deltaL")]
    bc = [a[k].to(dtype) for k in ("BT", "BL", "C")]
    cast = [(-torch.exp(logT)).to(dtype), (-torch.exp(logL)).to(dtype)]
    dy = inp["dy"].cuda().to(dtype)
    y0, ck0 = wf.scan_fwd_op(*act, *cast, *bc, a["D"].to(dtype), True, False)
    y1, ck1 = wf.scan_fwd_op(*act, logT, logL, *bc, a["D"], True, False, True)
    assert y1.dtype == dtype and so.rel_err(y1.float().cpu(), y0.float().cpu()) < tol
    g0 = wf.scan_bwd_op(*act, *cast, *bc, a["D"].to(dtype), dy, ck0, False)
    g1 = wf.scan_bwd_op(*act, logT, logL, *bc, a["D"], dy, ck1, False, True)
    for i in (0, 1, 2, 5, 6, 7):
        assert g1[i].dtype == dtype and so.rel_err(g1[i].float().cpu(), g0[i].float().cpu()) < tol, i
    for i, lg in ((3, logT), (4, logL)):
        assert g1[i].dtype == torch.float32
        want = g0[i].float() * -torch.exp(lg)          # dA/dA_log = A
        assert so.rel_err(g1[i].cpu(), want.cpu()) < 2 * tol, i
    assert g1[8].dtype == torch.float32 and so.rel_err(g1[8].cpu(), g0[8].float().cpu()) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("E", [24, 12], ids=["matrix_core_shape", "vector_shape"])
def test_packed_records_equal_separate_tensors(wf, dtype, E):
    """M2D_FLAG_PACKED_BC: B_T, B_L, C handed from proj_fwd to the scan as records give bit for bit
    the scan results of the three separate tensors."""
    say(f"\ncase packed B/C {dtype} E={E}")
    N, R = 16, math.ceil(E / 16)
    p = make_block_params(E, N, R, 1, "cuda")
    x = torch.randn(2, 9, 30, E, generator=torch.Generator().manual_seed(3)).cuda().to(dtype)
    dy = torch.randn(2, 9, 30, E, generator=torch.Generator().manual_seed(4)).cuda().to(dtype)
    w = [p[k] for k in ("x_proj_w", "dt_projT_w", "dt_projT_b", "dt_projL_w", "dt_projL_b")]
    low, dT, dL, BT, BL, C = wf.proj_fwd_op(x, *w, N, True)
    low2, dT2, dL2, rec, e1, e2 = wf.proj_fwd_op(x, *w, N, True, True)
    assert torch.equal(dT, dT2) and torch.equal(low, low2) and rec.shape == (2, 9, 30, 48) and e1.numel() == 0
    logs = [p["AT_log"], p["AL_log"]]
    y0, ck0 = wf.scan_fwd_op(x, dT, dL, *logs, BT, BL, C, p["D"], True, False, True)
    y1, ck1 = wf.scan_fwd_op(x, dT, dL, *logs, rec, e1, e2, p["D"], True, False, True, True)
    assert torch.equal(y0, y1)
    g0 = wf.scan_bwd_op(x, dT, dL, *logs, BT, BL, C, p["D"], dy, ck0, False, True)
    g1 = wf.scan_bwd_op(x, dT, dL, *logs, rec, e1, e2, p["D"], dy, ck1, False, True, True)
    g2 = wf.scan_bwd_op(x, dT, dL, *logs, rec, e1, e2, p["D"], dy, torch.empty(1, dtype=torch.uint8, device="cuda"), False, True, True)
    for a, b, c in zip(g0, g1, g2):
        assert a.shape == b.shape and torch.equal(a, b) and torch.equal(a, c)


def test_no_checkpoints_are_kept_under_no_grad(wf, monkeypatch):
    """Parameters keep requires_grad=True at inference; torch.no_grad() must still give the
    inference forward (no checkpoint buffer), for the plain Function and for the entry point."""
    say("\ncase no_grad keeps nothing")
    seen = []
    real = wf.scan_fwd_op

    def spy(*a, **kw):
        seen.append(bool(a[9]))
        return real(*a, **kw)

    monkeypatch.setattr(wf, "scan_fwd_op", spy)
    inp = so.make_inputs(1, 6, 5, 8, 16, seed=2, dtype=torch.float32)
    leaves = [inp[k].cuda().requires_grad_(True) for k in so.INPUT_NAMES]
    E, N, R = 8, 16, 1
    p = make_block_params(E, N, R, 0, "cuda")
    params = [p[k].requires_grad_(True) for k in ORDER]
    with torch.no_grad():
        wf.wf_cuda_fn_pr.apply(*leaves)
        wf.wavefront_scan_cuda(leaves[0], *params)
    assert seen == [False, False]
    wf.wf_cuda_fn_pr.apply(*leaves)
    wf.wavefront_scan_cuda(leaves[0], *params)
    assert seen[2:] == [wf.SAVE_CHECKPOINTS, wf.SAVE_CHECKPOINTS]


@pytest.mark.parametrize("shape,dtype", [((1, 150, 90, 8), torch.float32), ((6, 30, 30, 64), torch.bfloat16)],
                         ids=["sliced_f32", "batch_bf16"])
def test_entry_point_replays_from_a_graph(wf, shape, dtype):
    """The library allocates nothing and never synchronises, so a caller can capture forward and backward
    in a HIP graph (here through torch).  Every replay, with eager work and synchronisations between the
    replays, must give the bits of an eager run on the same inputs; the first shape is the linked sweep
    of one image (a sequence of 40 launches per pass)."""
    say(f"\ncase graph {shape} {dtype}")
    B, H, W, E = shape
    N, R = 16, math.ceil(E / 16)
    p = make_block_params(E, N, R, 0, "cuda")
    gen = torch.Generator().manual_seed(1)
    xs = [torch.randn(B, H, W, E, generator=gen).to(dtype).cuda() for _ in range(4)]
    dy = torch.randn(B, H, W, E, generator=gen).to(dtype).cuda()
    x = xs[0].clone().requires_grad_(True)
    leaves = [x] + [p[k].clone().requires_grad_(True) for k in ORDER]

    def run():
        y = wf.wavefront_scan_cuda(*leaves)
        return (y, *torch.autograd.grad(y, leaves, dy))

    side = torch.cuda.Stream()   # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        outs = run()
    for i in range(1, 4):
        with torch.no_grad():
            x.copy_(xs[i])
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = run()            # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), i


def test_parameter_updates_through_data_show_in_the_next_call(wf):
    """Parameters held in bf16 are cast to fp32 on every call: an update of a parameter, also one made
    through ``.data`` (old-style optimisers, EMA swaps, weight clipping), which leaves no trace in the
    tensor's version counter, must show in the next call."""
    say("\ncase parameter updates through .data")
    B, H, W, E, N = 2, 6, 7, 32, 16
    R = math.ceil(E / 16)
    p = {k: torch.nn.Parameter(v.bfloat16()) for k, v in make_block_params(E, N, R, 1, "cuda").items()}
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(1)).cuda().bfloat16()
    args = [p[k] for k in ORDER]
    with torch.no_grad():
        y1 = wf.wavefront_scan_cuda(x, *args)
        assert torch.equal(y1, wf.wavefront_scan_cuda(x, *args))
        p["D"].data.mul_(2.0)                              # y = scan + x * D
        y3 = wf.wavefront_scan_cuda(x, *args)
        want = y1.float() + x.float() * (p["D"].float() / 2)
        assert so.rel_err(y3.float().cpu(), want.cpu()) < 2e-2 and not torch.equal(y1, y3)
        fresh = [t.detach().clone() for t in args]         # same values in new tensors
        assert torch.equal(wf.wavefront_scan_cuda(x, *fresh), y3)


def test_views_that_start_off_alignment_are_accepted(wf, cscan):
    """A contiguous view whose first element is not 16-byte aligned is copied, not rejected."""
    say("\ncase unaligned views")
    inp = so.make_inputs(1, 6, 5, 3, 16, seed=2, dtype=torch.float32)
    a = []
    for k in so.INPUT_NAMES:
        big = torch.zeros(inp[k].numel() + 1, device="cuda")
        big[1:] = inp[k].flatten().cuda()
        a.append(big[1:].view(inp[k].shape))
    assert any(t.data_ptr() % 16 for t in a)
    y = wf.wf_cuda_fn_pr.apply(*a)
    assert so.rel_err(y.cpu(), cscan.forward(*[inp[k].double() for k in so.INPUT_NAMES])) < 1e-4


def test_small_spatial_dims_raise_on_gpu(wf):
    p = make_block_params(4, 16, 1, 0, "cuda")
    with pytest.raises(ValueError, match="spatial dims > 1"):
        wf.wavefront_scan_cuda(torch.zeros(1, 1, 8, 4, device="cuda"), *[p[k] for k in ORDER])


def test_wrong_shapes_and_dtypes_are_rejected(wf):
    inp = so.make_inputs(1, 4, 4, 4, 16, seed=0)
    a = [inp[k].cuda() for k in so.INPUT_NAMES]
    bad = list(a)
    bad[5] = bad[5][:, :, :3].contiguous()          # BT with the wrong width
    with pytest.raises(RuntimeError, match="BT has shape"):
        wf.scan_fwd_op(*bad, False, False)
    bad = list(a)
    bad[1] = bad[1].bfloat16()
    with pytest.raises(RuntimeError, match="share one dtype"):
        wf.scan_fwd_op(*bad, False, False)
    bad = [t.double() for t in a]
    with pytest.raises(RuntimeError, match="float32 and bfloat16"):
        wf.scan_fwd_op(*bad, False, False)
    a8 = [inp[k][..., :8].contiguous().cuda() if k in ("AT", "AL", "BT", "BL", "C") else inp[k].cuda()
          for k in so.INPUT_NAMES]
    with pytest.raises(RuntimeError, match="unsupported"):
        wf.scan_fwd_op(*a8, False, False)
