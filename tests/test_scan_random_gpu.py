"""Seeded random sweep of the scan against the CPU oracle, through the C ABI: shapes drawn from the
four regimes the launch logic distinguishes (many small single-band images, a few bands in one
stream, many bands of few images, wide channel counts), either dtype, either scan direction,
checkpoints kept or rebuilt.  Tolerances as in test_scan_gpu.py."""
import random

import pytest
import torch

from .test_scan_gpu import cabi, run_case, say  # noqa: F401  (cabi is a fixture)

pytestmark = pytest.mark.gpu


def draw_cases(seed, count):
    rng = random.Random(seed)
    cases = []
    for _ in range(count):
        kind = rng.random()
        if kind < 0.35:
            H, W, B, E = rng.randint(2, 14), rng.randint(2, 20), rng.randint(1, 400), rng.choice([1, 2, 3, 4, 5, 8, 12])
        elif kind < 0.7:
            H, W, B, E = rng.randint(15, 70), rng.randint(2, 70), rng.randint(1, 6), rng.choice([1, 2, 4, 6, 8, 9, 16, 33])
        elif kind < 0.9:
            H, W, B, E = rng.randint(57, 200), rng.randint(2, 120), rng.randint(1, 2), rng.choice([1, 2, 4, 8])
        else:
            H, W, B, E = rng.randint(2, 30), rng.randint(2, 30), rng.randint(1, 8), rng.choice([40, 64, 72, 100, 128])
        if B * H * W * E > 400000:   # keeps the oracle's share of a case well under a second
            B = max(1, 400000 // (H * W * E))
        cases.append((B, H, W, E, rng.choice(["f32", "bf16"]), rng.random() < 0.4, rng.random() < 0.6, rng.randint(0, 10 ** 6)))
    return cases


CASES = draw_cases(20240, 48)


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}x{c[3]}-{c[4]}{'-flip' if c[5] else ''}{'-ckpt' if c[6] else ''}")
def test_random_shape(cabi, cscan, case):
    B, H, W, E, dt, flip, ckpt, seed = case
    say(f"\ncase random B={B} H={H} W={W} E={E} {dt} flip={flip} ckpt={ckpt} seed={seed}")
    run_case(cabi, cscan, B, H, W, E, torch.float32 if dt == "f32" else torch.bfloat16, seed=seed, flip=flip, with_ckpt=ckpt)


INTERVAL_CASES = draw_cases(777, 32)


@pytest.mark.parametrize("case", INTERVAL_CASES, ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}x{c[3]}-{c[4]}{'-flip' if c[5] else ''}{'-ckpt' if c[6] else ''}")
def test_random_shape_with_longer_checkpoint_interval(cabi, cscan, case):
    """The same sweep with a snapshot every 8 or 16 steps (the backward replays the forward in between)."""
    B, H, W, E, dt, flip, ckpt, seed = case
    interval = 8 if seed % 2 else 16
    say(f"\ncase random interval={interval} B={B} H={H} W={W} E={E} {dt} flip={flip} ckpt={ckpt} seed={seed}")
    cabi.CKPT_INTERVAL = interval
    try:
        run_case(cabi, cscan, B, H, W, E, torch.float32 if dt == "f32" else torch.bfloat16, seed=seed, flip=flip, with_ckpt=ckpt)
    finally:
        cabi.CKPT_INTERVAL = 0
