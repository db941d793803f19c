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


# Many small images of 2 to 16 rows, drawn once (seed 31337) and kept where the library stacks them: several images
# to a band, bands whose two outer lanes are rows, a last stack of fewer images.
STACKED_CASES = [
    (566, 12, 18, 3, "f32", True, True, 112076), (412, 16, 12, 8, "f32", True, True, 719603), (963, 12, 7, 1, "f32", False, True, 165333),
    (595, 7, 13, 4, "f32", True, False, 367726), (1076, 2, 15, 3, "bf16", False, False, 81092), (659, 10, 18, 2, "bf16", False, False, 490492),
    (917, 16, 2, 3, "f32", True, True, 766715), (860, 6, 8, 3, "f32", True, False, 177671), (620, 16, 15, 1, "f32", False, False, 853535),
    (478, 3, 10, 6, "bf16", False, False, 57983), (314, 6, 21, 16, "bf16", False, False, 821958), (542, 3, 6, 12, "bf16", False, True, 736511),
    (425, 13, 13, 2, "f32", True, True, 422991), (663, 5, 7, 6, "bf16", True, False, 117636), (1175, 13, 21, 2, "f32", False, True, 205897),
    (1197, 3, 18, 6, "f32", True, True, 988088), (793, 16, 21, 2, "bf16", True, True, 640239), (854, 9, 15, 2, "f32", False, True, 971659),
    (383, 5, 16, 2, "bf16", False, True, 124604), (1141, 8, 6, 8, "bf16", True, False, 425108), (1186, 8, 10, 6, "f32", False, True, 406950),
    (465, 2, 13, 16, "f32", False, True, 19605), (308, 12, 18, 12, "bf16", True, False, 21272), (759, 3, 8, 40, "f32", False, False, 877286),
]


@pytest.mark.parametrize("case", STACKED_CASES, ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}x{c[3]}-{c[4]}{'-flip' if c[5] else ''}{'-ckpt' if c[6] else ''}")
def test_random_stacked_images(cabi, cscan, case):
    B, H, W, E, dt, flip, ckpt, seed = case
    dtype = torch.float32 if dt == "f32" else torch.bfloat16
    say(f"\ncase random stacked B={B} H={H} W={W} E={E} {dt} flip={flip} ckpt={ckpt} seed={seed}")
    assert "stacked images" in cabi.scan_plan(B, H, W, E, dtype, cabi.M2D_PASS_BWD)
    run_case(cabi, cscan, B, H, W, E, dtype, seed=seed, flip=flip, with_ckpt=ckpt)
