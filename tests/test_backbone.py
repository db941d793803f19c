"""Backbone around the scan: parameter names follow the reference's state-dict layout
(models/mamba2d.py:57-155,220-254,300-366; models/utils.py:99-105,207-233), bottom-right blocks
equal flipped top-left blocks, and the whole model runs on the GPU through the HIP scan."""
import re

import pytest
import torch


def say(msg):
    print(msg, flush=True)


def build(**kw):
    from mamba2d_amd.backbone import Mamba2DBackbone, M2D_T
    cfg = dict(M2D_T)
    cfg.update(kw)
    return Mamba2DBackbone(**cfg)


def test_state_dict_keys_follow_the_reference_layout():
    torch.manual_seed(0)
    net = build()
    keys = set(net.state_dict().keys())
    # stem and downsampling
    for name in ("stem", "ds1", "ds2", "ds3"):
        assert f"ds.{name}.conv.weight" in keys and f"ds.{name}.conv.bias" in keys
    assert "ds.stem.post_norm.norm.weight" in keys and "ds.stem.post_norm.norm.bias" in keys
    assert not any(k.startswith("ds.ds1.post_norm") for k in keys)
    n_blocks = (3, 3, 9, 3)
    for s, n in enumerate(n_blocks):
        assert f"stages.{s}.{n}.weight" in keys and f"stages.{s}.{n}.bias" in keys      # stage post-norm
        for k in range(n):
            pre = f"stages.{s}.{k}."
            for sub in ("norm1.weight", "norm2.bias", "MLP.fc1.weight", "MLP.fc2.bias", "res_scale1.scale", "res_scale2.scale"):
                assert pre + sub in keys, pre + sub
            if s < 2:   # scan stages with the local path
                for sub in ("in_proj.weight", "in_proj.bias", "x_proj.weight", "dt_projT.weight", "dt_projT.bias",
                            "dt_projL.weight", "dt_projL.bias", "AT_log", "AL_log", "D", "out_proj.weight",
                            "local_norm.weight", "local_path.pwconv1.weight", "local_path.dwconv.weight",
                            "local_path.pwconv2.weight", "local_path.act1.scale", "local_path.act1.bias",
                            "local_path.act2.scale", "local_path.act2.bias"):
                    assert pre + "token_mixer." + sub in keys, sub
                assert pre + "token_mixer.x_proj.bias" not in keys
                assert pre + "token_mixer.local_path.pwconv1.bias" not in keys
            else:       # attention stages
                for sub in ("qkv.weight", "proj.weight", "q_norm.weight", "q_norm.bias", "k_norm.weight", "k_norm.bias"):
                    assert pre + "token_mixer." + sub in keys, sub
                assert pre + "token_mixer.qkv.bias" not in keys and pre + "token_mixer.proj.bias" not in keys
    # nothing outside these families
    fam = re.compile(r"^(ds\.(stem|ds[123])\.(conv|post_norm\.norm)\.(weight|bias)|stages\.[0-3]\.\d+\..+)$")
    assert all(fam.match(k) for k in keys)


def test_shapes_and_initialisation_rules():
    torch.manual_seed(0)
    net = build()
    sd = net.state_dict()
    assert sd["ds.stem.conv.weight"].shape == (64, 3, 7, 7)
    assert sd["ds.ds2.conv.weight"].shape == (320, 128, 3, 3)
    tm = "stages.0.0.token_mixer."
    assert sd[tm + "x_proj.weight"].shape == (2 * 4 + 3 * 16, 64)          # dt_rank = ceil(64/16)
    assert sd[tm + "dt_projT.weight"].shape == (64, 4)
    assert sd[tm + "AT_log"].shape == (64, 16)
    assert torch.allclose(sd[tm + "AT_log"].exp()[5], torch.arange(1.0, 17.0))   # S4D-real: A = 1..N
    assert torch.all(sd[tm + "D"] == 1)
    dt = torch.nn.functional.softplus(sd[tm + "dt_projT.bias"])
    assert dt.min() >= 1e-3 * 0.999 and dt.max() <= 1e-1 * 1.001                 # log-uniform in [1e-3, 1e-1]
    assert torch.equal(sd[tm + "dt_projT.bias"], sd[tm + "dt_projL.bias"])
    assert sd["stages.1.0.token_mixer.local_path.dwconv.weight"].shape == (256, 1, 3, 3)
    assert sd["stages.2.0.token_mixer.qkv.weight"].shape == (3 * 320, 320)       # 10 heads of 32
    # interleaved scan directions: odd blocks of the scan stages start bottom-right
    assert [net.stages["0"][k].token_mixer.flip for k in range(3)] == [False, True, False]
    with pytest.raises(ValueError):
        build(token_mixer=("2D", "nope", "RopeAttention", "RopeAttention"))


def test_rotary_tables_match_a_direct_evaluation():
    from mamba2d_amd.backbone import RoPEAttention2D
    att = RoPEAttention2D(64, head_dim=32)
    H, W = 3, 5
    cos, sin = att._rope_tables(H, W, torch.device("cpu"), torch.float64)
    inv = 1.0 / (10000.0 ** (torch.arange(0, 8, dtype=torch.float64) / 8))
    for cell in (0, 7, 14):
        i, j = divmod(cell, W)
        for d in range(32):
            pos = i if d < 16 else j
            ang = pos * inv[(d % 16) // 2]
            assert abs(cos[cell, d] - torch.cos(ang)) < 1e-6 and abs(sin[cell, d] - torch.sin(ang)) < 1e-6
    t = torch.arange(8.0).view(1, 8)
    assert torch.equal(att._rotate_pairs(t), torch.tensor([[-1., 0., -3., 2., -5., 4., -7., 6.]]))


def test_training_checkpoint_of_the_reference_layout_loads(tmp_path):
    """A file shaped like the reference's Lightning checkpoints (state_dict with the backbone under
    'backbone.' next to head weights, downstream/Mamba2D/mamba2d.py:397-415) loads key by key."""
    from mamba2d_amd.backbone import load_backbone_checkpoint
    torch.manual_seed(3)
    src = build(n_blocks=(1, 1, 1, 1))
    sd = {"backbone." + k: v.clone() for k, v in src.state_dict().items()}
    sd["head.fc1.weight"] = torch.zeros(4, 4)          # classifier parts are ignored
    sd["norm.weight"] = torch.ones(512)
    path = tmp_path / "m2d.ckpt"
    torch.save({"state_dict": sd, "epoch": 3}, path)
    dst = build(n_blocks=(1, 1, 1, 1))
    assert not torch.equal(dst.state_dict()["stages.0.0.token_mixer.in_proj.weight"], src.state_dict()["stages.0.0.token_mixer.in_proj.weight"])
    load_backbone_checkpoint(dst, str(path))
    for k, v in src.state_dict().items():
        assert torch.equal(dst.state_dict()[k], v), k
    # a checkpoint of another depth does not load silently
    other = build(n_blocks=(2, 1, 1, 1))
    with pytest.raises(RuntimeError):
        load_backbone_checkpoint(other, str(path))
    with pytest.raises(FileNotFoundError):
        load_backbone_checkpoint(dst, str(tmp_path / "nope.ckpt"))


@pytest.mark.gpu
def test_bottom_right_block_equals_flipped_top_left_block():
    from mamba2d_amd.backbone import M2DBlock
    torch.manual_seed(1)
    dev = torch.device("cuda:0")
    tl = M2DBlock(32, local_path=True, scan_start="TL").to(dev)
    br = M2DBlock(32, local_path=True, scan_start="BR").to(dev)
    br.load_state_dict(tl.state_dict())
    x = torch.randn(2, 20, 17, 32, device=dev)
    say("\ncase backbone BR block vs flipped TL block")
    with torch.no_grad():
        # reference semantics (models/mamba2d.py:163-176): flip, scan path, flip back; the local path is not flipped
        local = tl.local_path(tl.local_norm(x))
        want = torch.flip(tl(torch.flip(x, (1, 2))) - tl.local_path(tl.local_norm(torch.flip(x, (1, 2)))), (1, 2)) + local
        got = br(x)
    err = (got - want).abs().max() / want.abs().max()
    say(f"  rel err {err:.3e}")
    assert err < 1e-5


@pytest.mark.gpu
def test_backbone_runs_and_backpropagates_on_gpu():
    torch.manual_seed(2)
    dev = torch.device("cuda:0")
    net = build(n_blocks=(2, 2, 1, 1), drop_path_rate=0.0).to(dev)
    x = torch.randn(2, 3, 64, 64, device=dev)
    say("\ncase backbone forward/backward 64x64")
    y = net(x)
    assert y.shape == (2, 512, 2, 2) and torch.isfinite(y).all()
    y.float().square().mean().backward()
    g = net.stages["0"][1].token_mixer.AT_log.grad
    assert g is not None and torch.isfinite(g).all() and g.abs().sum() > 0
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        yb = net(x)
    assert yb.shape == y.shape and torch.isfinite(yb.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 96, 64), (1, 224, 224), (3, 128, 160)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)], ids=["f32", "bf16"])
def test_inference_kernels_match_stock_operators(monkeypatch, dtype, tol, shape):
    """At inference LayerNorm and the local path's depthwise convolution run in the library's kernels; the
    backbone's output must agree with the one the stock operators give (same weights, same input)."""
    from mamba2d_amd import backbone as bb
    torch.manual_seed(3)
    dev = torch.device("cuda:0")
    net = build(n_blocks=(2, 1, 1, 1), drop_path_rate=0.0).to(dev).to(dtype).eval()
    with torch.no_grad():   # norms that are no identity
        for m in net.modules():
            if isinstance(m, torch.nn.LayerNorm):
                m.weight.uniform_(0.5, 1.5)
                m.bias.normal_(0, 0.3)
    x = torch.randn(shape[0], 3, shape[1], shape[2], device=dev, dtype=dtype)
    say(f"\ncase backbone inference kernels vs stock {dtype} {shape}")
    calls = {"n": 0}
    real, real_fused = bb.layernorm_fwd_op, bb.scale_residual_layernorm_fwd_op
    monkeypatch.setattr(bb, "layernorm_fwd_op", lambda *a: (calls.__setitem__("n", calls["n"] + 1), real(*a))[1])
    monkeypatch.setattr(bb, "scale_residual_layernorm_fwd_op",
                        lambda *a: (calls.__setitem__("n", calls["n"] + 1), real_fused(*a))[1])
    with torch.no_grad():
        got = net(x)
    assert calls["n"] > 10   # the library's kernels did run (LayerNorm alone or behind a residual update)
    monkeypatch.setattr(bb, "_inference", lambda *t: False)
    with torch.no_grad():
        want = net(x)
    err = so_rel(got, want)
    say(f"  rel err {err:.3e}")
    assert err < tol


def so_rel(a, b):
    return ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()
