"""A linked sweep that fails must show in the caller's tensors.

Grids of many bands and few images run every band on workgroups of its own inside one launch; a band waits, with a
bound, for the band whose boundary rows it reads.  A wait that gives up (seconds of wall time: only another tenant
of the device holding the compute units can cause it) sets an error word that nobody reads on the operator path,
so the workgroup also overwrites its rows of the outputs with NaN, and so does every band after it.  The test
drives that path from the host: with M2D_FLAG_TEST_DEAD_LINK one band's neighbour never reports and every wait of
the launch gives up after a few polls, so every kernel still ends normally.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import scan_oracle as so

pytestmark = pytest.mark.gpu

RB = 14   # grid rows per band


@pytest.mark.parametrize("layout", ["split_states", "whole_states"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("flip", [False, True], ids=["tl", "br"])
def test_a_wait_that_gives_up_poisons_the_outputs(layout, dtype, flip):
    from mamba2d_amd import cabi
    B, H, W, E = 1, 70, 50, 6   # five bands of one image: linked sweep
    hint = {"split_states": cabi.M2D_FLAG_SPLIT_STATES, "whole_states": cabi.M2D_FLAG_WHOLE_STATES}[layout]
    inp = so.make_inputs(B, H, W, E, 16, seed=11, dtype=dtype)
    a = [inp[k].cuda() for k in so.INPUT_NAMES]
    dy = inp["dy"].cuda()
    nbands = -(-H // RB)
    rows = lambda t: t.flip(1, 2) if flip else t   # band k of a flipped scan covers the rows k*14.. of the flipped image
    try:
        cabi.CHECK_LINKS = False
        cabi.SCHEDULE_HINT = hint
        assert "linked sweep" in cabi.scan_plan(B, H, W, E, dtype, cabi.M2D_PASS_FWD)
        y_ok, ck = cabi.scan_fwd(*a, save_ckpt=True, flip=flip)
        g_ok = cabi.scan_bwd(*a, dy, ckpt=ck, flip=flip)
        torch.cuda.synchronize()
        assert all(torch.isfinite(t.float()).all() for t in (y_ok, *g_ok))

        cabi.SCHEDULE_HINT = hint | cabi.M2D_FLAG_TEST_DEAD_LINK
        print(f"\ncase dead link forward {layout} {dtype} flip={flip}", flush=True)
        y_bad, ck_bad = cabi.scan_fwd(*a, save_ckpt=True, flip=flip)
        torch.cuda.synchronize()
        # the first band never waits: its rows are the good ones; every band after it says NaN
        assert torch.equal(rows(y_bad)[:, :RB], rows(y_ok)[:, :RB])
        assert torch.isnan(rows(y_bad)[:, RB:].float()).all()

        print(f"case dead link backward {layout} {dtype} flip={flip}", flush=True)
        g_bad = cabi.scan_bwd(*a, dy, ckpt=ck, flip=flip)   # (the good forward's snapshots: only the backward's wait fails)
        torch.cuda.synchronize()
        last = (nbands - 1) * RB   # the last band is swept first and never waits
        for name, bad, ok in zip(so.CScan.GRADS[:3], g_bad[:3], g_ok[:3]):
            # (a band that ends after the error word was set says NaN as well, whether it waited or not: the last
            # band's rows are the good ones or NaN, depending on when it ended)
            assert torch.equal(rows(bad)[:, last:], rows(ok)[:, last:]) or torch.isnan(rows(bad)[:, last:].float()).all(), name
            assert torch.isnan(rows(bad)[:, :last].float()).all(), name
        for name, bad in zip(("d_AT", "d_AL", "d_D"), (g_bad[3], g_bad[4], g_bad[8])):
            assert torch.isnan(bad.float()).any(dim=-1).all() if bad.dim() == 2 else torch.isnan(bad.float()).all(), name

        # a backward that rebuilds the snapshots with a forward sweep of its own: that sweep's failure shows as well
        g_bad2 = cabi.scan_bwd(*a, dy, ckpt=None, flip=flip)
        torch.cuda.synchronize()
        assert torch.isnan(g_bad2[0].float()).any() and torch.isnan(g_bad2[8].float()).all()
    finally:
        cabi.SCHEDULE_HINT = 0
        cabi.CHECK_LINKS = False


def test_the_error_word_is_set_and_cleared():
    from mamba2d_amd import cabi
    inp = so.make_inputs(1, 70, 50, 6, 16, seed=12, dtype=torch.float32)
    a = [inp[k].cuda() for k in so.INPUT_NAMES]
    try:
        cabi.CHECK_LINKS = True
        cabi.SCHEDULE_HINT = cabi.M2D_FLAG_TEST_DEAD_LINK
        with pytest.raises(RuntimeError, match="gave up waiting"):
            cabi.scan_fwd(*a)
        cabi.SCHEDULE_HINT = 0
        y = cabi.scan_fwd(*a)   # the next call starts from a clean word
        assert torch.isfinite(y).all()
    finally:
        cabi.SCHEDULE_HINT = 0
        cabi.CHECK_LINKS = False
