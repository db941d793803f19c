"""m2d_scan_fwd_noalloc (the forward entry point whose scratch is a static device array) against
m2d_scan_fwd, through the C ABI.  Both run the same kernels on the same inputs, so the outputs must
agree bit for bit (the bar for the existing entry point itself -- 1e-4 fp32 / 2e-2 bf16 against the
oracle -- is checked here too).  Two calls in a row, the second on a smaller problem: the array keeps
the first call's contents, which must not leak into the second.  Collected last on purpose."""
import ctypes
import sys

import pytest
import torch

from oracle import scan_oracle as so



def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def one_call(cabi, cscan, B, H, W, E, dtype, seed, flip=False):
    say(f"\ncase no_alloc B={B} H={H} W={W} E={E} dtype={dtype} flip={flip} seed={seed}")
    inp = so.make_inputs(B, H, W, E, 16, seed=seed, dtype=dtype)
    a = [inp[k].cuda() for k in so.INPUT_NAMES]
    want = cabi.scan_fwd(*a, flip=flip)
    y = torch.full_like(a[0], float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    cabi.scan_fwd_noalloc(*a, y, flip=flip)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(y, want), float((y.float() - want.float()).abs().max())
    ref_in = [inp[k].double() for k in so.INPUT_NAMES]
    if flip:
        ref_in = [torch.flip(t, dims=(1, 2)).contiguous() if t.dim() == 4 else t for t in ref_in]
    y_ref = torch.from_numpy(cscan.forward(*ref_in).copy())
    if flip:
        y_ref = torch.flip(y_ref, dims=(1, 2))
    e = so.rel_err(y.float().cpu(), y_ref)
    say(f"  y rel_err vs oracle {e:.3e}")
    assert e < (1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.gpu
def test_two_calls_in_a_row_second_smaller(cscan):
    from mamba2d_amd import cabi
    # four bands back to back: uses the set-up area, the packed B/C records and the band boundary rows
    one_call(cabi, cscan, 4, 56, 56, 64, torch.bfloat16, seed=11)
    one_call(cabi, cscan, 2, 20, 9, 8, torch.float32, seed=12)
    # linked sweep (one image, five bands on workgroups of their own), then stacked images
    one_call(cabi, cscan, 1, 70, 50, 16, torch.float32, seed=13, flip=True)
    one_call(cabi, cscan, 9, 7, 7, 6, torch.bfloat16, seed=14)


def test_too_large_is_rejected_before_any_launch():
    from mamba2d_amd import cabi
    d = cabi.Desc(128, 56, 56, 64, 16, cabi.M2D_BF16, 0, 0)
    assert cabi.lib.m2d_scan_workspace_bytes(ctypes.byref(d), cabi.M2D_PASS_FWD, 0) > cabi.NOALLOC_SCRATCH_BYTES
    vp = ctypes.c_void_p
    rc = cabi.lib.m2d_scan_fwd_noalloc(ctypes.byref(d), *([vp(4096)] * 10), vp(0))
    assert rc == cabi.M2D_ERR_TOO_LARGE
    assert "M2D_NOALLOC_SCRATCH_BYTES" in cabi.status_str(rc)
