"""Parity at the shapes of the benchmark configurations themselves, through the C ABI.

cfg1 (B=128, E=64, 56x56, bf16): forward and backward against the C oracle on a batch large
enough for the schedule the full batch takes (workgroups of 8 waves, one per compute unit).
cfg2 stages 2-4 (E=128/320/512 at 28x28, 14x14, 7x7, B=128, bf16): full size against the oracle.
cfg4 (B=1, E=64, fp32): 256x256 against the oracle directly; 512x512, 1024x1024, 1280x1280 (where the
forward splits the states of a channel over lanes and the backward does not) and 2048x2048 through a
property tied to the oracle: channels are independent, so a problem whose 64 channels repeat a
2-channel problem 32 times must give the 2-channel answer in every pair of channels (y, d_x,
d_deltaT, d_deltaL, d_AT, d_AL, d_D), and 32 times its sums over channels (d_BT, d_BL, d_C); the
2-channel problem itself is compared with the oracle at that size.

Tolerances: fp32 1e-4, bf16 2e-2 (tensor-normalised), as everywhere.
"""
import numpy as np
import pytest
import torch

from oracle import scan_oracle as so

from .test_scan_gpu import TOL, cabi, run_case, say  # noqa: F401  (cabi is a fixture)

pytestmark = pytest.mark.gpu


def test_cfg1_forward_backward_at_full_channel_count(cabi, cscan):
    """65 images x 2 workgroups of 32 channels: more workgroups than half the compute units, so both
    passes run the kernels the 128-image batch runs (8 waves per workgroup)."""
    say("\ncase cfg1 B=65 E=64 56x56 bf16")
    run_case(cabi, cscan, 65, 56, 56, 64, torch.bfloat16, seed=101)


def test_cfg1_flipped_at_full_channel_count(cabi, cscan):
    say("\ncase cfg1 flipped B=33 E=64 56x56 bf16")
    run_case(cabi, cscan, 33, 56, 56, 64, torch.bfloat16, seed=102, flip=True)


@pytest.mark.parametrize("E,HW", [(128, 28), (320, 14), (512, 7)], ids=["stage2", "stage3", "stage4"])
def test_cfg2_stages_at_full_size(cabi, cscan, E, HW):
    say(f"\ncase cfg2 stage B=128 E={E} {HW}x{HW} bf16")
    run_case(cabi, cscan, 128, HW, HW, E, torch.bfloat16, seed=200 + HW)


@pytest.mark.parametrize("E,HW", [(320, 14), (512, 7)], ids=["stage3", "stage4"])
def test_cfg2_small_stages_fp32(cabi, cscan, E, HW):
    """The stacked schedule at full channel count with the fp32 bound (a batch of 37: a last stack
    that is shorter than the others)."""
    say(f"\ncase cfg2 stage fp32 B=37 E={E} {HW}x{HW}")
    run_case(cabi, cscan, 37, HW, HW, E, torch.float32, seed=300 + HW)


def test_cfg4_256_at_full_channel_count(cabi, cscan):
    say("\ncase cfg4 B=1 E=64 256x256 fp32")
    run_case(cabi, cscan, 1, 256, 256, 64, torch.float32, seed=401)


def _fwd_bwd(cabi, dev, keep=True):
    """keep=False: the forward keeps no snapshots and the backward rebuilds them with a forward sweep of its own."""
    a = [dev[k] for k in so.INPUT_NAMES]
    if keep:
        y, ck = cabi.scan_fwd(*a, save_ckpt=True)
    else:
        y, ck = cabi.scan_fwd(*a), None
    g = cabi.scan_bwd(*a, dev["dy"], ckpt=ck)
    torch.cuda.synchronize()
    return y, g


def _check_replicas(y, g, y0, g0, reps):
    assert so.rel_err(y.cpu(), y0.repeat(1, 1, 1, reps).cpu()) < 1e-6
    for k, got, base in zip(so.CScan.GRADS, g, g0):
        if k in ("d_x", "d_deltaT", "d_deltaL"):
            want = base.repeat(1, 1, 1, reps)
        elif k in ("d_AT", "d_AL"):
            want = base.repeat(reps, 1)
        elif k == "d_D":
            want = base.repeat(reps)
        else:   # sums over channels
            want = base * reps
        e = so.rel_err(got.cpu(), want.cpu())
        say(f"  E=64 {k} vs replicated E=2: {e:.3e}")
        assert e < 1e-5, (k, e)


@pytest.mark.parametrize("HW", [512, 1024, 1280, 2048])
def test_cfg4_large_grids_by_channel_replication(cabi, cscan, HW):
    say(f"\ncase cfg4 B=1 E=64 {HW}x{HW} fp32 by replication of an E=2 problem")
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * 2**30:
        pytest.skip("needs 40 GB of free device memory")
    E0, reps, dtype = 2, 32, torch.float32
    inp = so.make_inputs(1, HW, HW, E0, 16, seed=500 + HW, dtype=dtype)
    small = {k: v.cuda() for k, v in inp.items()}
    y0, g0 = _fwd_bwd(cabi, small)
    # the 2-channel problem against the oracle at this size
    ref_in = [inp[k].double() for k in so.INPUT_NAMES]
    y_ref = cscan.forward(*ref_in)
    e = so.rel_err(y0.cpu(), y_ref)
    say(f"  E=2 y rel_err {e:.3e}")
    assert e < TOL[dtype]
    del y_ref
    g_ref = cscan.backward(*ref_in, inp["dy"].double())
    for k, g in zip(so.CScan.GRADS, g0):
        e = so.rel_err(g.cpu(), g_ref[k])
        say(f"  E=2 {k} rel_err {e:.3e}")
        assert np.isfinite(e) and e < TOL[dtype], (k, e)
    del g_ref, ref_in
    # 64 channels = the two channels 32 times over
    rep = {"x": (1, 1, 1, reps), "deltaT": (1, 1, 1, reps), "deltaL": (1, 1, 1, reps), "dy": (1, 1, 1, reps),
           "AT": (reps, 1), "AL": (reps, 1), "D": (reps,)}
    big = {k: (v.repeat(*rep[k]) if k in rep else v) for k, v in small.items()}
    y, g = _fwd_bwd(cabi, big)
    _check_replicas(y, g, y0, g0, reps)
    if HW == 1280:
        # Between about 1180 and 1490 pixels a side the two passes of this problem take different lane layouts:
        # the forward splits the 16 states of a channel over the lanes of a wave, the backward (whose per-workgroup
        # channel sums would outgrow their bound) keeps them in one lane.  The backward then restarts from
        # snapshots and replays boundary rows that the other layout wrote, also where it rebuilds them itself.
        f, b = cabi.scan_plan(1, HW, HW, E0 * reps, dtype, cabi.M2D_PASS_FWD), cabi.scan_plan(1, HW, HW, E0 * reps, dtype, cabi.M2D_PASS_BWD)
        say(f"  forward: {f}\n  backward: {b}")
        assert f.startswith("m2d_fwd_split_kernel") and b.startswith("m2d_bwd_kernel"), (f, b)
        del y, g
        y, g = _fwd_bwd(cabi, big, keep=False)
        say("  without kept snapshots:")
        _check_replicas(y, g, y0, g0, reps)
