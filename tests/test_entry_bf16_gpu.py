"""The entry point wavefront_scan_cuda on bf16 activations (projections + scan, both recompute modes)
against a float64 evaluation of the same function on the CPU (oracle.entry_point_reference: weights
rounded to bf16 as the reference's casts do, wavefront_cuda.py:327-332, exact arithmetic after that).

Bound: 2e-2 tensor-normalised for y and every gradient.  The gradients of the five projection
weights are sums over all B*H*W positions of products with both signs; with few channels (dt_rank 1,
E of 1 to 6) such a sum can cancel to a hundredth of the sum of its terms' magnitudes, and then the
bf16 rounding of the terms (the step-size gradients and the low-rank activations are bf16 tensors in
the reference too) is larger than 2 % of the result.  For those five tensors the bound is therefore
max(2e-2 * max|ref|, 4e-3 * S), S = largest sum of |terms| of the tensor: 4e-3 = 2^-8 is one bf16
rounding (half an ulp, 2^-9) on each of a term's two factors.  tests/test_oracle.py shows on the CPU
that a float64 emulation of the reference's own bf16 data flow needs exactly this allowance on the
seeds listed first below (it misses 2e-2 on them), so the allowance is the reference's own noise and
not the kernels'.
"""
import math

import pytest
import torch

from oracle import scan_oracle as so

from .test_wavefront_gpu import make_block_params, say, wf  # noqa: F401  (wf is a fixture)

pytestmark = pytest.mark.gpu

# B, H, W, E, recomp, seed
CANCELLING_SEEDS = [(2, 34, 8, 6, "full", 513480), (5, 11, 28, 1, "full", 999395), (5, 26, 23, 1, "partial", 118331)]
CASES = CANCELLING_SEEDS + [
    (3, 9, 12, 1, "partial", 1), (2, 20, 31, 1, "full", 2),
    (4, 14, 14, 6, "partial", 3), (1, 40, 17, 6, "full", 4), (7, 7, 7, 6, "partial", 5),
    (2, 28, 28, 32, "partial", 6), (2, 28, 28, 32, "full", 7), (5, 13, 30, 32, "full", 8), (1, 60, 45, 32, "partial", 9),
    (2, 56, 56, 64, "partial", 10), (2, 56, 56, 64, "full", 11), (9, 14, 14, 64, "partial", 12), (3, 33, 9, 64, "full", 13),
    (3, 14, 14, 320, "partial", 14), (3, 14, 14, 320, "full", 15), (16, 7, 7, 320, "partial", 16), (1, 30, 28, 320, "full", 17),
    (6, 7, 7, 512, "full", 18), (2, 28, 28, 128, "partial", 19), (1, 5, 3, 100, "full", 20), (2, 17, 4, 12, "partial", 21),
]


def entry_point_case(wf, B, H, W, E, recomp, seed, flip=False):
    R = math.ceil(E / 16)
    p = make_block_params(E, 16, R, seed, "cpu")
    x = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(seed + 1)).bfloat16()
    dy = torch.randn(B, H, W, E, generator=torch.Generator().manual_seed(seed + 2)).bfloat16()
    leaves = [x.cuda().requires_grad_(True)] + [p[k].cuda().requires_grad_(True) for k in so.PARAM_ORDER]
    y = wf.wavefront_scan_cuda(*leaves, recomp=recomp, flip=flip)
    grads = torch.autograd.grad(y, leaves, dy.cuda())
    torch.cuda.synchronize()
    fl = (lambda t: torch.flip(t, dims=(1, 2))) if flip else (lambda t: t)
    y_ref, g_ref, scales = so.entry_point_reference(fl(x), p, fl(dy))
    y_ref, g_ref[0] = fl(y_ref), fl(g_ref[0])
    e = so.rel_err(y.float().cpu(), y_ref)
    say(f"  y {e:.3e}")
    assert e < 2e-2, ("y", e)
    for name, g, gr in zip(("x",) + so.PARAM_ORDER, grads, g_ref):
        diff = (g.double().cpu() - gr).abs().max().item()
        allowed = 2e-2 * gr.abs().max().item()
        if name in scales:
            allowed = max(allowed, 4e-3 * scales[name].max().item())
        say(f"  {name} max|diff| {diff:.3e} allowed {allowed:.3e} (2e-2*max|ref| = {2e-2 * gr.abs().max().item():.3e})")
        assert math.isfinite(diff) and diff <= allowed, (name, diff, allowed)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{}_{}x{}_E{}_{}_s{}".format(*c))
def test_entry_point_bf16_against_float64(wf, case):
    say(f"\ncase entry_bf16 {case}")
    entry_point_case(wf, *case)


@pytest.mark.parametrize("case", [(2, 30, 28, 64, "partial", 31), (3, 14, 14, 6, "full", 32)], ids=lambda c: "B{}_{}x{}_E{}_{}_s{}".format(*c))
def test_entry_point_bf16_flipped(wf, case):
    say(f"\ncase entry_bf16 flipped {case}")
    entry_point_case(wf, *case, flip=True)
