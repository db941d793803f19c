"""GPU parity of the scan with a longer checkpoint interval (m2d_desc.ckpt_interval = 8 or 16 steps).

The forward then keeps the snapshot of one block of 4 steps in two or four, and the backward replays the
forward over the blocks in between before it sweeps them.  Checked against the CPU oracle to the same bounds
as the default interval, and against the library's own results at the default interval: y must be the same
bits (the forward's arithmetic does not depend on what it keeps), the gradients the same to rounding.
"""
import ctypes

import pytest
import torch

from oracle import scan_oracle as so

from .test_scan_gpu import cabi, run_case, say  # noqa: F401  (cabi is a fixture)

pytestmark = pytest.mark.gpu


@pytest.fixture
def interval(request, cabi):
    cabi.CKPT_INTERVAL = request.param
    yield request.param
    cabi.CKPT_INTERVAL = 0


SHAPES = [
    # B, H, W, E        schedule at these intervals (images are not stacked, states not split over lanes)
    (2, 14, 14, 32),    # one band, 7 blocks: groups of 2 and 4 with a shorter one at the end
    (3, 5, 9, 4),       # short band, most channels of the workgroup missing
    (301, 7, 7, 4),     # many small images (stacked at the default interval), one stream each
    (2, 33, 40, 2),     # three bands back to back
    (1, 70, 50, 2),     # linked sweep, five bands: a group never spans two bands' windows
    (2, 130, 20, 2),    # ten bands, padded windows of 9 blocks
    (1, 64, 17, 10),    # channels not a multiple of anything: x, deltas, dy read from memory, also in the replay
    (1, 150, 90, 8),    # linked sweep of 11 bands
    (70, 56, 30, 4),    # four bands back to back, workgroups of 8 waves
    (4, 20, 11, 50),    # workgroups of 4 waves, the last partly filled
    (3, 30, 28, 32),    # workgroups of 4 waves, stride = width
    (2, 100, 33, 48),   # linked sweep, three workgroups per band
    (1, 512, 512, 2),   # 37 bands of one large image
    (9, 56, 56, 64),    # stage-1 grid
]


@pytest.mark.parametrize("interval", [8, 16], indirect=True)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_parity_with_longer_interval(cabi, cscan, shape, dtype, interval):
    say(f"\ninterval {interval} shape {shape} {dtype}: {cabi.scan_plan(*shape, dtype, cabi.M2D_PASS_BWD)}")
    assert f"a snapshot every {interval} steps" in cabi.scan_plan(*shape, dtype, cabi.M2D_PASS_BWD)
    run_case(cabi, cscan, *shape, dtype)


@pytest.mark.parametrize("interval", [8, 16], indirect=True)
@pytest.mark.parametrize("shape", [(2, 14, 14, 4), (1, 70, 9, 2), (3, 33, 40, 6)], ids=lambda s: "x".join(map(str, s)))
def test_flipped_scan_and_rebuilt_checkpoints(cabi, cscan, shape, interval):
    run_case(cabi, cscan, *shape, torch.float32, flip=True)
    run_case(cabi, cscan, *shape, torch.bfloat16, with_ckpt=False)   # the backward runs the keeping forward itself


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(5, 40, 36, 32), (1, 90, 120, 16), (128, 28, 28, 64), (1, 1024, 1024, 64)], ids=lambda s: "x".join(map(str, s)))
def test_same_results_as_the_default_interval(cabi, shape, dtype):
    inp = so.make_inputs(*shape, 16, seed=5, dtype=dtype)
    a = [inp[k].cuda() for k in so.INPUT_NAMES]
    dy = inp["dy"].cuda()
    flags = cabi.M2D_FLAG_WHOLE_STATES   # the layout that the longer intervals use: the only difference left is the interval
    res, sizes = {}, {}
    try:
        cabi.SCHEDULE_HINT = flags
        for iv in (0, 8, 16):
            cabi.CKPT_INTERVAL = iv
            y, ck = cabi.scan_fwd(*a, save_ckpt=True)
            g = cabi.scan_bwd(*a, dy, ckpt=ck)
            torch.cuda.synchronize()
            res[iv] = (y.clone(), [t.clone() for t in g])
            d = cabi.Desc(*shape, 16, cabi.M2D_BF16 if dtype == torch.bfloat16 else cabi.M2D_F32, flags, iv)
            sizes[iv] = cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(d))
    finally:
        cabi.CKPT_INTERVAL = 0
        cabi.SCHEDULE_HINT = 0
    say(f"checkpoint bytes {sizes}")
    assert sizes[0] > sizes[8] > sizes[16]
    for iv in (8, 16):
        assert torch.equal(res[iv][0], res[0][0]), "y depends on the interval"
        for name, g, g0 in zip(so.CScan.GRADS, res[iv][1], res[0][1]):
            # fp32: the replay repeats the forward's own arithmetic; bf16: a replayed state is rounded to bf16 once
            # more than a kept one, which moves gradients as the snapshots' own rounding does
            e = so.rel_err(g.float().cpu(), g0.float().cpu().double().numpy())
            say(f"  interval {iv} {name}: {e:.2e} from the default interval's")
            assert e < (1e-5 if dtype == torch.float32 else 1e-2), (iv, name, e)
