"""GPU parity of the scan at every checkpoint interval (m2d_desc.ckpt_interval).

8 or 16 steps: the forward keeps the snapshot of one block of 4 steps in two or four, and the backward replays the
forward over the blocks in between before it sweeps them.  2 steps (what the library picks by itself for batches of
images swept one stream each): the forward keeps two snapshots per block, and m2d_bwd2_kernel recomputes one step
in two; asked for explicitly, 4 steps keeps such a batch on m2d_bwd_kernel.  Checked against the CPU oracle to the
same bounds whatever the interval, and against the library's own results at the other intervals: y must be the same
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


# shapes that the library sweeps one stream per image or stack (with what the two-step interval adds: every schedule,
# both workgroup sizes, channel counts that cannot be staged, a last stack that is shorter)
SHAPES_PER_IMAGE = [s for s in SHAPES if s not in ((1, 70, 50, 2), (2, 130, 20, 2), (1, 150, 90, 8), (2, 100, 33, 48), (1, 512, 512, 2), (1, 64, 17, 10))] + [
    (600, 14, 14, 4), (129, 8, 8, 512), (601, 5, 9, 8), (37, 5, 9, 8), (33, 57, 8, 48), (260, 20, 5, 64), (67, 56, 56, 64), (128, 28, 28, 128), (300, 16, 16, 32)]


@pytest.mark.parametrize("interval", [2, 4], indirect=True)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES_PER_IMAGE, ids=lambda s: "x".join(map(str, s)))
def test_parity_with_two_and_four_steps(cabi, cscan, shape, dtype, interval):
    cabi.SCHEDULE_HINT = cabi.M2D_FLAG_WHOLE_STATES   # (small batches would split the states of a channel over lanes: a snapshot every 4 steps)
    try:
        plan = cabi.scan_plan(*shape, dtype, cabi.M2D_PASS_BWD)
        say(f"\ninterval {interval} shape {shape} {dtype}: {plan}")
        two = interval == 2 and "linked sweep" not in plan
        assert plan.startswith("m2d_bwd2_kernel" if two else "m2d_bwd_kernel") and ("a snapshot every 2 steps" in plan) == two, plan
        run_case(cabi, cscan, *shape, dtype)
    finally:
        cabi.SCHEDULE_HINT = 0


@pytest.mark.parametrize("interval", [2, 4], indirect=True)
@pytest.mark.parametrize("shape", [(2, 14, 14, 4), (3, 33, 40, 6), (301, 7, 7, 4), (70, 56, 30, 12)], ids=lambda s: "x".join(map(str, s)))
def test_flipped_scan_and_rebuilt_checkpoints_two_and_four_steps(cabi, cscan, shape, interval):
    run_case(cabi, cscan, *shape, torch.float32, flip=True)
    run_case(cabi, cscan, *shape, torch.bfloat16, flip=True)
    run_case(cabi, cscan, *shape, torch.bfloat16, with_ckpt=False)   # the backward runs the keeping forward itself
    run_case(cabi, cscan, *shape, torch.float32, with_ckpt=False)


def test_few_large_images_keep_four_steps(cabi):
    """The two-step interval belongs to the schedules of many images; a linked sweep asked for it keeps a snapshot every
    4 steps (sizes and plan say so), and the library never picks it there by itself."""
    for iv in (0, 2):
        plan = cabi.scan_plan(1, 256, 256, 64, torch.float32, cabi.M2D_PASS_BWD, ckpt_interval=iv)
        assert "every 2 steps" not in plan and "linked sweep" in plan, plan
    size = lambda iv: cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(cabi.Desc(1, 256, 256, 64, 16, cabi.M2D_F32, 0, iv)))
    assert size(0) == size(2) == size(4)
    many = lambda iv: cabi.lib.m2d_scan_ckpt_bytes(ctypes.byref(cabi.Desc(128, 56, 56, 64, 16, cabi.M2D_BF16, 0, iv)))
    assert many(0) == many(2) > 1.7 * many(4)   # (twice the snapshots and one; the boundary rows stay)
    assert "every 2 steps" in cabi.scan_plan(128, 56, 56, 64, torch.bfloat16, cabi.M2D_PASS_FWD)


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
        for iv in (4, 2, 8, 16):
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
    assert sizes[2] >= sizes[4] > sizes[8] > sizes[16]   # (2: only where every image is one stream)
    for iv in (2, 8, 16):
        assert torch.equal(res[iv][0], res[4][0]), "y depends on the interval"
        for name, g, g0 in zip(so.CScan.GRADS, res[iv][1], res[4][1]):
            # fp32: the replay repeats the forward's own arithmetic; bf16: a replayed state is rounded to bf16 once
            # more than a kept one, which moves gradients as the snapshots' own rounding does
            e = so.rel_err(g.float().cpu(), g0.float().cpu().double().numpy())
            say(f"  interval {iv} {name}: {e:.2e} from the results at 4 steps")
            assert e < (1e-5 if dtype == torch.float32 else 1e-2), (iv, name, e)
