#!/usr/bin/env python3
"""Benchmark of the wavefront 2-D selective scan on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--workload cfg1|stage2|...]

One "step" is one forward + backward of the scan operator (``wf_cuda_fn_pr.apply`` and
``torch.autograd.grad`` of its output) on the M2D-T stage-1 shape: B=128, E=64, 56x56, N=16,
bf16 tensors with fp32 state, synthetic seeded inputs already resident in HBM.

Prints ONE JSON line.  ``value`` is the mean forward+backward latency in ms (lower is
better); ``fwd_ms`` the forward alone.  ``roofline`` prices the dominant kernel (the
backward scan kernel) against MI355X's 8 TB/s HBM peak with the algorithmic bytes of the
fused backward, s*[P*(7E+6N) + 4EN + 2E]; its duration is measured with HIP events the
library records around that kernel on the launch stream.  ``cpu_baseline`` times the CPU
oracle (a restatement of the reference, which has no CPU path of its own) on the host cores
on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (B, E, H, W, dtype)
    "cfg1": (128, 64, 56, 56, "bf16"),
    "stage2": (128, 128, 28, 28, "bf16"),
    "stage3": (128, 320, 14, 14, "bf16"),
    "stage4": (128, 512, 7, 7, "bf16"),
    "hires256": (1, 64, 256, 256, "f32"),
    "hires512": (1, 64, 512, 512, "f32"),
    "hires1024": (1, 64, 1024, 1024, "f32"),
    "hires2048": (1, 64, 2048, 2048, "f32"),
    "cfg0": (2, 32, 14, 14, "f32"),
    "train64": (64, 64, 56, 56, "bf16"),   # the reference's training batch per GPU (configs/M2D-T-ImageNet.yaml) at the stage-1 shape
    "cfg3": None,   # M2D-T backbone inference, handled by backbone_inference()
    "entry": None,  # wavefront_scan_cuda (projections + scan) at the cfg1 shape, handled by entry_point()
    "cfg2": None,   # the four M2D-T stage scans in sequence, handled by stage_sequence()
}
N = 16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, which this
# script cannot make from inside itself: `roofline.traffic` is null here, and the counter run of the same command is
# summarised, with its figure, in the file that `roofline.traffic_profile` names.
TRAFFIC_PROFILE = {"cfg1": "profiles/scan_cfg1_kernel_trace_and_traffic.txt"}
# Vector-ALU operations per (cell, channel, state) of the scan kernels, as (multiply-add class, v_exp_f32):
# forward: 2 exponent multiply-adds + 5 (input term, two gate terms, y), 2 gates;
# backward with a snapshot every 4 steps (m2d_bwd_kernel): the block recomputed (2 + 4, 2 gates), the adjoint (17,
#   the gates of three steps in four: 1.5 + 1.5), 4.5 for the lane-swap sums over the channels of a wave;
# backward with a snapshot every 2 steps (m2d_bwd2_kernel): one step in two recomputed (1 + 2, 1 gate), the adjoint
#   (17, the gates of one step in two: 1 + 1), 4.5 for the channel sums, 1 for unpacking the restored states.
UNIT_OPS = {"fwd": (7, 2), "bwd4": (29, 3.5), "bwd2": (26.5, 2)}
# nominal issue slots of the same (a v_exp_f32 takes two on gfx950)
FWD_SLOTS = 11
BWD_SLOTS = {"m2d_bwd_kernel": 36, "m2d_bwd2_kernel": 30.5}


def nominal_valu_slots_per_s():
    """fp32 lane-operations per second the device can issue at its nominal clock: compute units x 64 lanes
    x engine clock from the device properties.  Not measured here; under load the clock is lower."""
    import torch
    prop = torch.cuda.get_device_properties(0)
    return prop.multi_processor_count * 64 * getattr(prop, "clock_rate", 2400000) * 1e3   # kHz; MI355X: 2.4 GHz


def scan_roofline(name, B, E, H, W, s, bwd_kernel_ms, fwd_kernel_ms):
    """The `roofline` object for the backward scan kernel (the dominant kernel) of a scan workload."""
    from mamba2d_amd import cabi
    fb, bb = algorithmic_bytes(B, E, H, W, s)
    achieved = bb / (bwd_kernel_ms * 1e-3) / 1e9
    dts = "bf16" if s == 2 else "f32"
    plan_bwd = cabi.scan_plan(B, H, W, E, dts, cabi.M2D_PASS_BWD)
    plan_fwd = cabi.scan_plan(B, H, W, E, dts, cabi.M2D_PASS_FWD)
    return {
        "kernel": plan_bwd.split(":")[0], "schedule": plan_bwd, "fwd_schedule": plan_fwd, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None, "traffic_profile": TRAFFIC_PROFILE.get(name),
        "kernel_ms": round(bwd_kernel_ms, 4), "algorithmic_bytes": bb,
        "fwd_kernel_ms": round(fwd_kernel_ms, 4), "fwd_algorithmic_bytes": fb,
        "fwd_kernel_frac": round(fb / (fwd_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
    }


def measured_valu_rates():
    """Instruction rates of the device's vector ALUs from the library's probe kernel (m2d_valu_rate_probe), at the
    two waves per SIMD that the scan kernels run: lane-operations per second of v_fma_f32 and v_exp_f32 with 16
    independent chains per lane and with one dependent chain, and the forward scan's own mix in units per second."""
    from mamba2d_amd import cabi
    return {k: cabi.valu_rate_probe(k, 2) for k in ("fma", "exp", "fma_dependent", "exp_dependent", "scan_fwd_unit")}


def valu_ceiling(units, fwd_kernel_ms, bwd_kernel_ms, bwd_kernel_name, rates=None):
    """The `valu_ceiling` object: the scan is bound by instruction issue, not by HBM.  The measured ceiling of a
    kernel is units x (multiply-adds / measured multiply-add rate + gates / measured v_exp_f32 rate): the time its
    arithmetic alone would take at the rates the probe kernel reaches on this device in this process."""
    rates = rates or measured_valu_rates()
    peak_slots = nominal_valu_slots_per_s()
    bwd_ops = UNIT_OPS["bwd2" if bwd_kernel_name.startswith("m2d_bwd2") else "bwd4"]
    floor_ms = lambda ops: units * (ops[0] / rates["fma"] + ops[1] / rates["exp"]) * 1e3
    bwd_slots = BWD_SLOTS.get(bwd_kernel_name.split(":")[0], 36)
    return {
        "measured_lane_slots_per_s": round(rates["fma"]),   # v_fma_f32, independent chains, 2 waves per SIMD, whole device
        "measured_exp_per_s": round(rates["exp"]),
        "measured_fma_dependent_per_s": round(rates["fma_dependent"]),
        "measured_exp_dependent_per_s": round(rates["exp_dependent"]),
        "measured_scan_fwd_units_per_s": round(rates["scan_fwd_unit"]),   # the forward's arithmetic alone, as a kernel of its own
        "predicted_scan_fwd_units_per_s": round(1.0 / (UNIT_OPS["fwd"][0] / rates["fma"] + UNIT_OPS["fwd"][1] / rates["exp"])),
        "units": units, "fwd_ops_per_unit": UNIT_OPS["fwd"], "bwd_ops_per_unit": bwd_ops,
        "fwd_arithmetic_floor_ms": round(floor_ms(UNIT_OPS["fwd"]), 4), "bwd_arithmetic_floor_ms": round(floor_ms(bwd_ops), 4),
        "fwd_kernel_frac_of_measured": round(floor_ms(UNIT_OPS["fwd"]) / fwd_kernel_ms, 4),
        "bwd_kernel_frac_of_measured": round(floor_ms(bwd_ops) / bwd_kernel_ms, 4),
        "nominal_lane_slots_per_s": peak_slots,
        "note": "measured: m2d_valu_rate_probe in this process (16 independent chains per lane, 2 waves per SIMD); nominal: compute units x 64 lanes x engine clock from the device properties",
        "fwd_slots_per_unit": FWD_SLOTS, "bwd_slots_per_unit": bwd_slots,
        "fwd_kernel_frac": round(units * FWD_SLOTS / peak_slots / (fwd_kernel_ms * 1e-3), 4),
        "bwd_kernel_frac": round(units * bwd_slots / peak_slots / (bwd_kernel_ms * 1e-3), 4),
    }


def algorithmic_bytes(B, E, H, W, s):
    P = B * H * W
    fwd = s * (P * (4 * E + 3 * N) + 2 * E * N + E)
    bwd = s * (P * (7 * E + 6 * N) + 4 * E * N + 2 * E)
    return fwd, bwd


def cpu_baseline(B, E, H, W, budget_s=20.0):
    """fp32 C port of the reference recurrence (oracle/m2d_oracle.c), OpenMP over the batch,
    on a batch sample; scaled linearly to the full batch (the scan is independent per image)."""
    import numpy as np
    import torch
    from oracle import scan_oracle as so

    cs = so.CScan()
    cores = len(os.sched_getaffinity(0))   # host cores this process may run on
    threads = min(cores, 16)               # OpenMP threads of the oracle (one image per thread)
    cs.set_threads(threads)
    per_image_units = H * W * E * N
    # ~60 ns per state update forward+backward on one core is a safe guess for sizing the sample
    bs = max(1, min(B, int(budget_s * threads / (per_image_units * 60e-9 * 4)) // threads * threads or 1))
    inp = so.make_inputs(bs, H, W, E, N, seed=0, dtype=torch.float32)
    a = [inp[k] for k in so.INPUT_NAMES]
    t0 = time.perf_counter()
    cs.forward(*a, dtype=np.float32)
    t1 = time.perf_counter()
    cs.backward(*a, inp["dy"], dtype=np.float32)
    t2 = time.perf_counter()
    scale = B / bs
    return {
        "value": round(((t1 - t0) + (t2 - t1)) * 1e3 * scale, 1),
        "fwd_ms": round((t1 - t0) * 1e3 * scale, 1),
        "unit": "ms",
        "cores": cores,
        "threads": threads,
        "kind": "port",
        "sample": f"fp32 C/OpenMP oracle, {bs} of {B} images forward+backward, scaled x{scale:g}",
    }


def backbone_inference(args):
    """M2D-T backbone (blocks [3,3,9,3], channels [64,128,320,512], scan mixers with local path at
    stages 1-2, rotary attention at stages 3-4, odd blocks scanning from the bottom-right corner),
    random weights, B=128 images of 3x224x224, inference.  One step = one batch."""
    import torch
    from mamba2d_amd import cabi
    from mamba2d_amd.backbone import Mamba2DBackbone, M2D_T
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    B = 128
    net = Mamba2DBackbone(**M2D_T).to(dev).eval()
    x = torch.randn(B, 3, 224, 224, device=dev)
    cabi.profile_enable(False)   # (the library's event records stay out of the timed batches)

    def run(model, inp, autocast):
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            return model(inp)

    def timed(model, inp, autocast):
        for _ in range(args.warmup):
            run(model, inp, autocast)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            run(model, inp, autocast)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms_autocast = timed(net, x, True)                  # fp32 weights, bf16 autocast (the reference's bf16-mixed)
    cabi.profile_enable(True)
    run(net, x, True)
    torch.cuda.synchronize()
    scan_ms = cabi.profile_last_ms(cabi.M2D_PASS_FWD)  # last scan of the batch: stage 2, 28x28x128
    cabi.profile_enable(False)
    net16 = net.to(torch.bfloat16)
    ms_bf16 = timed(net16, x.to(torch.bfloat16), False)
    out = {
        "metric": "M2D-T backbone inference images/sec at 224x224, B=128",
        "value": round(B / (ms_bf16 * 1e-3), 1),
        "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_bf16, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3: M2D-T backbone, blocks [3,3,9,3], channels [64,128,320,512], B=128 x 3x224x224, "
                               "random init, 6 scans (3 at 56x56x64, 3 at 28x28x128, odd blocks bottom-right)"},
        "images_per_s_bf16_weights": round(B / (ms_bf16 * 1e-3), 1),
        "images_per_s_autocast_fp32_weights": round(B / (ms_autocast * 1e-3), 1),
        "last_scan_kernel_ms": round(scan_ms, 4),
        # the library's largest kernel inside the model: the forward scan (the last one of a batch is the
        # 28x28x128 scan of stage 2); the model's other time is spread over some 190 smaller launches
        "roofline": {"kernel": "m2d_fwd_kernel (stage 2 scan, B=128 E=128 28x28)", "bound": "hbm",
                     "achieved": round(algorithmic_bytes(128, 128, 28, 28, 2)[0] / (scan_ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(algorithmic_bytes(128, 128, 28, 28, 2)[0] / (scan_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "kernel_ms": round(scan_ms, 4),
                     "algorithmic_bytes": algorithmic_bytes(128, 128, 28, 28, 2)[0]},
        "cpu_baseline": None,
    }
    print(json.dumps(out))


def stage_sequence(args):
    """The four M2D-T stage scans one after the other, (E,H,W) = (64,56,56), (128,28,28), (320,14,14),
    (512,7,7) at B=128, bf16 tensors with fp32 state.  One step = forward + backward of all four."""
    import torch
    from mamba2d_amd import cabi, wavefront
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g)
    sp = torch.nn.functional.softplus
    stages, units, alg = [], 0, 0
    for name in ("cfg1", "stage2", "stage3", "stage4"):
        B, E, H, W, _ = WORKLOADS[name]
        host = [r(B, H, W, E), sp(r(B, H, W, E)), sp(r(B, H, W, E)), -torch.exp(-4 * torch.rand(E, N, generator=g)),
                -torch.exp(-4 * torch.rand(E, N, generator=g)), r(B, H, W, N), r(B, H, W, N), r(B, H, W, N), r(E)]
        leaves = [t.to(torch.bfloat16).to(dev).requires_grad_(True) for t in host]
        stages.append((leaves, [t.detach() for t in leaves], r(B, H, W, E).to(torch.bfloat16).to(dev)))
        units += B * H * W * E * N
        alg += sum(algorithmic_bytes(B, E, H, W, 2))

    def fwd_only():
        with torch.no_grad():
            for _, frozen, _ in stages:
                wavefront.wf_cuda_fn_pr.apply(*frozen)

    def fwd_bwd():
        for leaves, _, dy in stages:
            torch.autograd.grad(wavefront.wf_cuda_fn_pr.apply(*leaves), leaves, dy)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    fwd_ms, both_ms = timed(fwd_only), timed(fwd_bwd)
    # kernel durations per stage from the library's own events (a second, untimed pass)
    cabi.profile_enable(True)
    per_stage = {}
    for name, (leaves, _, dy) in zip(("cfg1", "stage2", "stage3", "stage4"), stages):
        ks = []
        for _ in range(5):
            torch.autograd.grad(wavefront.wf_cuda_fn_pr.apply(*leaves), leaves, dy)
            ks.append((cabi.profile_last_ms(cabi.M2D_PASS_FWD), cabi.profile_last_ms(cabi.M2D_PASS_BWD)))
        B, E, H, W, _ = WORKLOADS[name]
        f, b = sum(k[0] for k in ks) / len(ks), sum(k[1] for k in ks) / len(ks)
        per_stage[name] = scan_roofline(name, B, E, H, W, 2, b, f)
    dominant = max(per_stage, key=lambda k: per_stage[k]["kernel_ms"])
    roof = dict(per_stage[dominant])
    roof["kernel"] = f"m2d_bwd_kernel ({dominant} scan)"
    print(json.dumps({
        "metric": "four M2D-T stage scans in sequence, fwd+bwd ms at B=128 N=16", "value": round(both_ms, 4), "unit": "ms",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(both_ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 in/out, f32 state",
        "data": "synthetic",
        "config": {"workload": "cfg2: scans of (E,H,W) = (64,56,56), (128,28,28), (320,14,14), (512,7,7) in sequence, B=128 N=16"},
        "fwd_ms": round(fwd_ms, 4), "fwd_bwd_ms": round(both_ms, 4),
        "pct_hbm_roofline": {"fwd_bwd": round(100 * alg / (both_ms * 1e-3) / (HBM_PEAK_GBS * 1e9), 2)},
        "valu_ceiling_frac_nominal": round(units * (FWD_SLOTS + BWD_SLOTS["m2d_bwd2_kernel"]) / nominal_valu_slots_per_s() / (both_ms * 1e-3), 4),
        "roofline": roof,
        "per_stage_bwd_kernel": {k: {"kernel_ms": v["kernel_ms"], "frac": v["frac"], "fwd_kernel_ms": v["fwd_kernel_ms"]} for k, v in per_stage.items()},
        "cpu_baseline": None,
    }))


def entry_point(args):
    """The reference's entry point, wavefront_scan_cuda(x, A_logs, projection weights, D): projections
    (x_proj, two dt_proj + softplus), scan, and the backward of both, at the cfg1 shape with fp32
    parameters initialised like an M2D block and bf16 activations.  One step = forward + backward."""
    import math
    import torch
    from mamba2d_amd import cabi, wavefront as wf
    dev = torch.device("cuda:0")
    B, E, H, W = WORKLOADS["cfg1"][:4]
    R = math.ceil(E / 16)
    g = torch.Generator().manual_seed(0)
    dt = torch.exp(torch.rand(E, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
    inv_dt = dt + torch.log(-torch.expm1(-dt))
    params = [
        torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)),          # AT_log
        torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)),          # AL_log
        (torch.rand(2 * R + 3 * N, E, generator=g) * 2 - 1) / math.sqrt(E),           # x_proj_w
        (torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5, inv_dt.clone(),          # dt_projT w, b
        (torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5, inv_dt.clone(),          # dt_projL w, b
        torch.ones(E)]                                                                # D
    params = [p.to(dev).requires_grad_(True) for p in params]
    x = torch.randn(B, H, W, E, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    dy = torch.randn(B, H, W, E, generator=g).to(torch.bfloat16).to(dev)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    def fwd_bwd(recomp):
        y = wf.wavefront_scan_cuda(x, *params, recomp)
        torch.autograd.grad(y, [x] + params, dy)

    def fwd_only():
        with torch.no_grad():
            wf.wavefront_scan_cuda(x, *params)

    res = {}
    for own in (True, False):
        wf.FUSED_PROJECTIONS = own
        key = "own" if own else "torch"
        res[key] = {"fwd_ms": round(timed(fwd_only), 4), "fwd_bwd_ms": round(timed(lambda: fwd_bwd("partial")), 4),
                    "fwd_bwd_full_recompute_ms": round(timed(lambda: fwd_bwd("full")), 4)}
    wf.FUSED_PROJECTIONS = True

    # the projection passes alone, through the C ABI (they run on torch's current stream)
    w32 = [p.detach() for p in params[2:7]]
    xd = x.detach()
    outs = cabi.proj_fwd(xd, *w32, N, round_weights=True)
    ups = [torch.randn_like(t) for t in (outs[1], outs[2], outs[3], outs[4], outs[5])]
    dx = torch.zeros_like(xd)
    proj_fwd_ms = timed(lambda: cabi.proj_fwd(xd, *w32, N, round_weights=True))
    # as the entry point calls it: the scan hands over the gradients before the softplus, the deltas are not read
    proj_bwd_ms = timed(lambda: cabi.proj_bwd(xd, outs[0], None, None, w32[0], w32[1], w32[3], *ups, dx,
                                              round_weights=True, dpre=True))
    cabi.profile_enable(True)
    ks = []
    for _ in range(5):
        fwd_bwd("partial")
        ks.append((cabi.profile_last_ms(cabi.M2D_PASS_FWD), cabi.profile_last_ms(cabi.M2D_PASS_BWD)))
    scan_fwd_ms, scan_bwd_ms = sum(k[0] for k in ks) / len(ks), sum(k[1] for k in ks) / len(ks)
    P, s = B * H * W, 2
    nw = (2 * R + 3 * N) * E + 2 * E * R + 2 * E
    proj_fwd_bytes = s * P * (E + 2 * R + 2 * E + 3 * N) + 4 * nw
    proj_bwd_bytes = s * P * (E + 2 * R + 2 * E + 3 * N + 2 * E) + 8 * nw   # x, low-rank inputs, 2 dpre, dB_T dB_L dC, dx in and out
    out = {
        "metric": "wavefront_scan_cuda (projections + scan) fwd+bwd ms at B=128 D=64 56x56 N=16",
        "value": res["own"]["fwd_bwd_ms"], "unit": "ms",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["own"]["fwd_bwd_ms"],
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 activations, f32 parameters and state", "data": "synthetic",
        "config": {"workload": "entry: wavefront_scan_cuda fwd+bwd, B=128 E=64 56x56 N=16 dt_rank=4, recomp=partial"},
        "own_projection_kernels": res["own"], "stock_torch_projections": res["torch"],
        "projection_passes": {
            "fwd_ms": round(proj_fwd_ms, 4), "bwd_ms": round(proj_bwd_ms, 4),
            "fwd_algorithmic_bytes": proj_fwd_bytes, "bwd_algorithmic_bytes": proj_bwd_bytes,
            "fwd_frac_of_hbm_peak": round(proj_fwd_bytes / (proj_fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "bwd_frac_of_hbm_peak": round(proj_bwd_bytes / (proj_bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "roofline": scan_roofline("entry", B, E, H, W, 2, scan_bwd_ms, scan_fwd_ms),
        "cpu_baseline": None,
    }
    print(json.dumps(out))


def _timed(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def _device_scan_inputs(B, E, H, W, dtype, seed):
    """The synthetic inputs of a scan workload, drawn on the device (same distributions as the headline workload's)."""
    import torch
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, device=dev)
    sp = torch.nn.functional.softplus
    host = [r(B, H, W, E), sp(r(B, H, W, E)), sp(r(B, H, W, E)), -torch.exp(-4 * torch.rand(E, N, generator=g, device=dev)),
            -torch.exp(-4 * torch.rand(E, N, generator=g, device=dev)), r(B, H, W, N), r(B, H, W, N), r(B, H, W, N), r(E)]
    leaves = [t.to(dtype).requires_grad_(True) for t in host]
    return leaves, r(B, H, W, E).to(dtype)


def _short_scan(name, steps, warmup):
    """fwd and fwd+bwd of one scan workload in a few steps, with the kernel durations from the library's events."""
    import torch
    from mamba2d_amd import cabi, wavefront
    B, E, H, W, dts = WORKLOADS[name]
    dtype = torch.bfloat16 if dts == "bf16" else torch.float32
    s = 2 if dts == "bf16" else 4
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    leaves, dy = _device_scan_inputs(B, E, H, W, dtype, seed=1)
    frozen = [t.detach() for t in leaves]

    def fwd_only():
        with torch.no_grad():
            wavefront.wf_cuda_fn_pr.apply(*frozen)

    def fwd_bwd():
        torch.autograd.grad(wavefront.wf_cuda_fn_pr.apply(*leaves), leaves, dy)

    cabi.profile_enable(False)
    fwd_ms, both_ms = _timed(fwd_only, steps, warmup), _timed(fwd_bwd, steps, warmup)
    peak = torch.cuda.max_memory_allocated()
    cabi.profile_enable(True)
    ks = []
    for _ in range(3):
        fwd_bwd()
        torch.cuda.synchronize()
        ks.append((cabi.profile_last_ms(cabi.M2D_PASS_FWD), cabi.profile_last_ms(cabi.M2D_PASS_BWD)))
    cabi.profile_enable(False)
    fk, bk = sum(k[0] for k in ks) / len(ks), sum(k[1] for k in ks) / len(ks)
    fb, bb = algorithmic_bytes(B, E, H, W, s)
    roof = scan_roofline(name, B, E, H, W, s, bk, fk)
    del leaves, frozen, dy
    torch.cuda.empty_cache()
    return {"workload": f"B={B} E={E} {H}x{W} {dts}", "fwd_ms": round(fwd_ms, 4), "fwd_bwd_ms": round(both_ms, 4), "steps": steps,
            "peak_hbm_bytes": int(peak),
            "pct_hbm_roofline_fwd_bwd": round(100 * (fb + bb) / (both_ms * 1e-3) / (HBM_PEAK_GBS * 1e9), 2),
            "roofline": {k: roof[k] for k in ("kernel", "schedule", "bound", "achieved", "peak", "unit", "frac", "kernel_ms", "fwd_kernel_ms", "fwd_kernel_frac")}}


def also_workloads(args, rates, cfg1_fwd_bwd_ms):
    """Short measurements of the other configurations in the same process, after the timed region of the headline
    workload: the four stage scans in sequence (cfg2), one image of 256x256, 1024x1024 and 2048x2048 (cfg4, with the
    allocator's peak), the stage-1 scan at the reference's training batch of 64, and the entry point
    wavefront_scan_cuda with its projections at the headline shape."""
    import math
    import torch
    from mamba2d_amd import wavefront as wf
    out = {}
    stages = {k: _short_scan(k, 30, 5) for k in ("stage2", "stage3", "stage4")}
    # (the first stage is the headline workload itself; the stages run back to back on one stream, so the sum of their
    # steps is what `--workload cfg2` times as one step)
    out["cfg2"] = {"fwd_bwd_ms": round(cfg1_fwd_bwd_ms + sum(v["fwd_bwd_ms"] for v in stages.values()), 4), "stages": stages}
    out["cfg4_256"] = _short_scan("hires256", 30, 5)
    out["train64"] = _short_scan("train64", 30, 5)   # (not a configuration of the baseline: the batch the reference trains with)
    free, _ = torch.cuda.mem_get_info()
    if free > 40 * 2**30:
        out["cfg4_1024"] = _short_scan("hires1024", 10, 3)
        out["cfg4_2048"] = _short_scan("hires2048", 3, 1)
    # entry point: projections + scan, fp32 parameters initialised like an M2D block, bf16 activations
    B, E, H, W = WORKLOADS["cfg1"][:4]
    R = math.ceil(E / 16)
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    dt = torch.exp(torch.rand(E, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
    inv_dt = dt + torch.log(-torch.expm1(-dt))
    params = [torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)), torch.log(torch.arange(1, N + 1, dtype=torch.float32).repeat(E, 1)),
              (torch.rand(2 * R + 3 * N, E, generator=g) * 2 - 1) / math.sqrt(E),
              (torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5, inv_dt.clone(), (torch.rand(E, R, generator=g) * 2 - 1) * R ** -0.5, inv_dt.clone(), torch.ones(E)]
    params = [p.to(dev).requires_grad_(True) for p in params]
    gd = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn(B, H, W, E, generator=gd, device=dev).to(torch.bfloat16).requires_grad_(True)
    dy = torch.randn(B, H, W, E, generator=gd, device=dev).to(torch.bfloat16)

    def entry_fwd_bwd():
        torch.autograd.grad(wf.wavefront_scan_cuda(x, *params), [x] + params, dy)

    def entry_fwd():
        with torch.no_grad():
            wf.wavefront_scan_cuda(x, *params)

    out["entry"] = {"workload": "wavefront_scan_cuda (projections + scan), B=128 E=64 56x56 N=16 dt_rank=4, bf16 activations, recomp=partial",
                    "fwd_ms": round(_timed(entry_fwd, 30, 5), 4), "fwd_bwd_ms": round(_timed(entry_fwd_bwd, 30, 5), 4), "steps": 30}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-also", action="store_true", help="skip the short measurements of the other workloads that the default workload appends")
    ap.add_argument("--no-ckpt", action="store_true", help="rebuild checkpoints inside the backward")
    ap.add_argument("--ckpt-interval", type=int, default=0, choices=(0, 2, 4, 8, 16),
                    help="steps between the state snapshots the forward keeps (0: the library's choice, 2 where every "
                         "image or stack has a stream to itself and 4 elsewhere; 8, 16: fewer snapshots, and the backward "
                         "replays the forward in between)")
    ap.add_argument("--dtype", default=None, choices=("f32", "bf16"),
                    help="tensor type of a single-scan workload (default: the workload's own)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a known-size kernel to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE readings by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the scan shards over the batch with no "
              "exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from mamba2d_amd import cabi, wavefront
    cabi.CKPT_INTERVAL = args.ckpt_interval

    if args.workload == "cfg3":
        backbone_inference(args)
        return
    if args.workload == "entry":
        entry_point(args)
        return
    if args.workload == "cfg2":
        stage_sequence(args)
        return
    B, E, H, W, dts = WORKLOADS[args.workload]
    dts = args.dtype or dts
    dtype = torch.bfloat16 if dts == "bf16" else torch.float32
    if args.no_ckpt:
        wavefront.SAVE_CHECKPOINTS = False
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g)
    sp = torch.nn.functional.softplus
    host = [r(B, H, W, E), sp(r(B, H, W, E)), sp(r(B, H, W, E)), -torch.exp(-4 * torch.rand(E, N, generator=g)),
            -torch.exp(-4 * torch.rand(E, N, generator=g)), r(B, H, W, N), r(B, H, W, N), r(B, H, W, N), r(E)]
    leaves = [t.to(dtype).to(dev).requires_grad_(True) for t in host]
    dy = r(B, H, W, E).to(dtype).to(dev)

    # The library can bracket its scan kernel with a pair of HIP events on the stream it launches on (the kernel
    # durations below).  Each record is a packet of its own in the queue and costs the step a few microseconds, so
    # the steps behind `value` run without them and the same number of steps is then run again, timed, with them.
    cabi.profile_enable(False)
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    frozen = [t.detach() for t in leaves]   # inference: nothing requires grad, no checkpoints are kept

    def fwd_only():
        with torch.no_grad():
            return wavefront.wf_cuda_fn_pr.apply(*frozen)

    def fwd_bwd():
        y = wavefront.wf_cuda_fn_pr.apply(*leaves)
        return torch.autograd.grad(y, leaves, dy)

    for _ in range(args.warmup):
        fwd_only()
        fwd_bwd()
    torch.cuda.synchronize()

    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        fwd_only()
    e1.record()
    torch.cuda.synchronize()
    fwd_ms = e0.elapsed_time(e1) / args.steps

    torch.cuda.synchronize()
    t_wall0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fwd_bwd()
    e1.record()
    torch.cuda.synchronize()
    t_wall = (time.perf_counter() - t_wall0) / args.steps * 1e3
    step_ms = e0.elapsed_time(e1) / args.steps

    # kernel durations: the same steps again with the library's events on, each step's pair read after the step
    cabi.profile_enable(True)
    fwd_only()
    torch.cuda.synchronize()
    fwd_kernel_ms = cabi.profile_last_ms(cabi.M2D_PASS_FWD)
    ks, inst = [], 0.0
    for _ in range(args.steps):
        e0.record()
        fwd_bwd()
        e1.record()
        torch.cuda.synchronize()
        inst += e0.elapsed_time(e1)
        ks.append(cabi.profile_last_ms(cabi.M2D_PASS_BWD))
    bwd_kernel = sum(ks) / len(ks)
    instrumented_ms = inst / args.steps

    peak_mem = torch.cuda.max_memory_allocated()
    input_bytes = sum(t.numel() * t.element_size() for t in leaves) + dy.numel() * dy.element_size()
    s = 2 if dts == "bf16" else 4
    fb, bb = algorithmic_bytes(B, E, H, W, s)
    out = {
        # (the headline metric is quoted on cfg1; the other scan workloads say their own shape)
        "metric": f"2D-scan fwd & fwd+bwd ms at B={B} D={E} {H}x{W} N={N}; % of HBM roofline",
        "value": round(step_ms, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 in/out, f32 state" if dts == "bf16" else "f32",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: single scan fwd+bwd, B={B} E={E} {H}x{W} N={N}",
                   "checkpoints": ("saved by forward" if not args.no_ckpt else "rebuilt in backward") +
                                  (f", a snapshot every {args.ckpt_interval} steps" if args.ckpt_interval > 4 else "")},
        "fwd_ms": round(fwd_ms, 4),
        "fwd_bwd_ms": round(step_ms, 4),
        "wall_ms_per_step": round(t_wall, 4),
        "ms_per_step_with_kernel_events": round(instrumented_ms, 4),   # the steps that `roofline.kernel_ms` was read from
        "peak_hbm_bytes": int(peak_mem),          # torch allocator peak: inputs, outputs, gradients, checkpoints, scratch
        "input_bytes": int(input_bytes),
        "pct_hbm_roofline": {
            "fwd": round(100 * fb / (fwd_ms * 1e-3) / (HBM_PEAK_GBS * 1e9), 2),
            "fwd_bwd": round(100 * (fb + bb) / (step_ms * 1e-3) / (HBM_PEAK_GBS * 1e9), 2),
        },
        "roofline": scan_roofline(args.workload, B, E, H, W, s, bwd_kernel, fwd_kernel_ms),
    }
    # Second ceiling: the scan is bounded by instruction issue, not by HBM.  Measured on this device by the library's
    # probe kernel, outside the timed region.
    rates = measured_valu_rates()
    out["valu_ceiling"] = valu_ceiling(B * H * W * E * N, fwd_kernel_ms, bwd_kernel, out["roofline"]["schedule"], rates)
    if args.workload == "cfg1" and not args.no_also:
        out["also"] = also_workloads(args, rates, step_ms)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(B, E, H, W)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
