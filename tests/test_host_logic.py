"""Host-side logic that needs no GPU: the bench contract for more than one GPU, and the split of a
d_state other than 16 into groups of 16 states (checked against the CPU oracle)."""
import os
import subprocess
import sys

import numpy as np
import torch

from oracle import scan_oracle as so

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_state_groups_pad_and_cover_every_state():
    from mamba2d_amd import wavefront as wf
    E, N = 3, 21
    AT, AL = -torch.rand(E, N) - 0.1, -torch.rand(E, N) - 0.1
    BT, BL, C = torch.randn(2, 4, 5, N), torch.randn(2, 4, 5, N), torch.randn(2, 4, 5, N)
    groups = wf._state_groups(AT, AL, BT, BL, C)
    assert len(groups) == 2
    for grp in groups:
        assert all(t.shape[-1] == wf.STATES_PER_CALL and t.is_contiguous() for t in grp)
    for k, full in enumerate((AT, AL, BT, BL, C)):
        joined = torch.cat([grp[k] for grp in groups], dim=-1)
        assert torch.equal(joined[..., :N], full)
        pad = joined[..., N:]
        assert torch.all(pad == (-1.0 if k < 2 else 0.0))   # finite gates, zero B and C


def test_scan_is_the_sum_of_its_state_groups(cscan):
    """y = sum over states and the recurrence is independent per state (wf_cuda.cu:40-69,
    wavefront_cuda.py:156): the oracle at N=21 equals the sum of the oracle over padded groups of 16,
    the skip term counted once; gradients of A, B, C are those of the groups side by side."""
    from mamba2d_amd import wavefront as wf
    N = 21
    inp = so.make_inputs(2, 5, 6, 3, N, seed=3, dtype=torch.float32)
    a = [inp[k].double() for k in so.INPUT_NAMES]
    x, dT, dL, AT, AL, BT, BL, C, D = a
    dy = inp["dy"].double()
    y = cscan.forward(*a)
    g = cscan.backward(*a, dy)
    y_sum, parts = 0.0, []
    for gi, grp in enumerate(wf._state_groups(AT, AL, BT, BL, C)):
        Dg = D if gi == 0 else torch.zeros_like(D)
        y_sum = y_sum + cscan.forward(x, dT, dL, *grp, Dg)
        parts.append(cscan.backward(x, dT, dL, *grp, Dg, dy))
    assert np.abs(y_sum - y).max() < 1e-12 * max(1.0, np.abs(y).max())
    names = so.CScan.GRADS
    for k in (names[0], names[1], names[2]):   # x, deltaT, deltaL: sums over the groups
        tot = sum(p[k] for p in parts)
        assert np.abs(tot - g[k]).max() < 1e-10 * max(1.0, np.abs(g[k]).max()), k
    for k in names[3:8]:                       # A_T, A_L, B_T, B_L, C: side by side, padding dropped
        joined = np.concatenate([p[k] for p in parts], axis=-1)[..., :N]
        assert np.abs(joined - g[k]).max() < 1e-10 * max(1.0, np.abs(g[k]).max()), k
    assert np.abs(parts[0][names[8]] - g[names[8]]).max() < 1e-10 * max(1.0, np.abs(g[names[8]]).max())
