"""CPU restatement of the reference's blocks around the scan -- TEST INFRASTRUCTURE ONLY.

Plain functions of a state dict (the reference's key layout) and an input tensor, in whatever
dtype they are handed (the tests use float64), written with elementary torch operators and
following the reference line by line.  Nothing here imports the package under test, and the
shipped package never imports this file.

What is restated (cocoalex00/Mamba2D):
  LayerNorm2D, StarReLU, Scale, MLP, SepConv, Downsampling      models/utils.py:9-19, 26-41, 46-55, 58-81, 83-118, 121-141
  rotate_half, rope_cos_sin_1d, apply_rope_1d, RoPEAttention2D  models/utils.py:144-172, 175-316
  M2DBlock.forward / .ssm (flip-copy formulation of BR scans)    models/mamba2d.py:157-188
  ResBlock.forward                                               models/mamba2d.py:256-261
  Mamba2DBackbone: stages, inter_flip, stage post-norm, forward  models/mamba2d.py:340-386
The scan itself is ``scan_oracle.wavefront_scan_ref`` (projections + differentiable recurrence).

Drop-path and dropout are identities at inference and are left out.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import scan_oracle as so

LN_EPS = 1e-5   # nn.LayerNorm default, used everywhere in the reference


def layer_norm(x, sd, prefix):
    """nn.LayerNorm over the last axis (biased variance)."""
    w, b = sd[prefix + "weight"], sd[prefix + "bias"]
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + LN_EPS) * w + b


def star_relu(x, sd, prefix):
    """models/utils.py:40-41: scale * relu(x)**2 + bias."""
    return sd[prefix + "scale"] * torch.clamp(x, min=0) ** 2 + sd[prefix + "bias"]


def linear(x, sd, prefix):
    y = x @ sd[prefix + "weight"].transpose(0, 1)
    return y + sd[prefix + "bias"] if prefix + "bias" in sd else y


def gelu(x):
    """nn.GELU() (exact form)."""
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def mlp(x, sd, prefix):
    """models/utils.py:73-80 (dropout 0)."""
    return linear(gelu(linear(x, sd, prefix + "fc1.")), sd, prefix + "fc2.")


def sep_conv(x, sd, prefix):
    """models/utils.py:103-118 as configured at models/mamba2d.py:57-60: expansion 2, both
    activations StarReLU, 3x3 depthwise, padding 1, no bias, no residual."""
    x = star_relu(linear(x, sd, prefix + "pwconv1."), sd, prefix + "act1.")
    w = sd[prefix + "dwconv.weight"]                       # (C, 1, 3, 3)
    x = F.conv2d(x.permute(0, 3, 1, 2), w, padding=1, groups=w.shape[0]).permute(0, 2, 3, 1)
    x = star_relu(x, sd, prefix + "act2.")
    return linear(x, sd, prefix + "pwconv2.")


def m2d_block(x, sd, prefix, scan_start):
    """models/mamba2d.py:157-178: local path on the unflipped input; for a BR block the input is
    flipped before in_proj and the result flipped back after out_proj; the local features are added last."""
    local = None
    if prefix + "local_norm.weight" in sd:
        local = sep_conv(layer_norm(x, sd, prefix + "local_norm."), sd, prefix + "local_path.")
    if scan_start == "BR":
        x = torch.flip(x, dims=(1, 2))
    x = gelu(linear(x, sd, prefix + "in_proj."))
    x = so.wavefront_scan_ref(x, sd[prefix + "AT_log"], sd[prefix + "AL_log"], sd[prefix + "x_proj.weight"],
                              sd[prefix + "dt_projT.weight"], sd[prefix + "dt_projT.bias"],
                              sd[prefix + "dt_projL.weight"], sd[prefix + "dt_projL.bias"], sd[prefix + "D"],
                              compute_dtype=x.dtype)
    x = linear(gelu(x), sd, prefix + "out_proj.")
    if scan_start == "BR":
        x = torch.flip(x, dims=(1, 2))
    return x if local is None else x + local


def _rotate_half(x):
    """models/utils.py:144-147."""
    x = x.reshape(*x.shape[:-1], -1, 2)
    x1, x2 = x.unbind(dim=-1)
    return torch.stack((-x2, x1), dim=-1).flatten(-2)


def _rope_cos_sin(pos, dim, base, dtype):
    """models/utils.py:150-162: angles in float32, cast at the end."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim // 2, dtype=torch.float32) / (dim // 2)))
    freqs = pos.to(torch.float32)[:, None] * inv_freq[None, :]
    return freqs.cos().repeat_interleave(2, dim=-1).to(dtype), freqs.sin().repeat_interleave(2, dim=-1).to(dtype)


def rope_attention(x, sd, prefix, head_dim=32, rope_base=10000.0):
    """models/utils.py:243-316 with the defaults the backbone uses (no CLS token, no biases, rope_ratio 1,
    not causal): rotary embedding of the first h_dim features by the row and the next w_dim by the column,
    LayerNorm of q and k per head after the rotation, softmax attention with scale head_dim**-0.5."""
    B, H, W, C = x.shape
    heads = max(C // head_dim, 1)
    N = H * W
    qkv = linear(x, sd, prefix + "qkv.").reshape(B, N, 3, heads, head_dim).permute(2, 0, 3, 1, 4)
    q, k, v = qkv.unbind(0)
    half = int(head_dim * 1.0) // 2
    h_dim = w_dim = (half // 2) * 2
    h_pos = torch.arange(H).repeat_interleave(W)
    w_pos = torch.arange(W).repeat(H)
    cos_h, sin_h = _rope_cos_sin(h_pos, h_dim, rope_base, x.dtype)
    cos_w, sin_w = _rope_cos_sin(w_pos, w_dim, rope_base, x.dtype)

    def rope(t):
        th = t[..., :h_dim]
        tw = t[..., h_dim:h_dim + w_dim]
        th = th * cos_h + _rotate_half(th) * sin_h
        tw = tw * cos_w + _rotate_half(tw) * sin_w
        return torch.cat([th, tw, t[..., h_dim + w_dim:]], dim=-1)

    q = layer_norm(rope(q), sd, prefix + "q_norm.")
    k = layer_norm(rope(k), sd, prefix + "k_norm.")
    attn = torch.softmax((q @ k.transpose(-2, -1)) * head_dim ** -0.5, dim=-1)
    out = (attn @ v).transpose(1, 2).reshape(B, H, W, heads * head_dim)
    return linear(out, sd, prefix + "proj.")


def res_block(x, sd, prefix, scan_start="TL"):
    """models/mamba2d.py:256-261; the residual scale is the identity where the block has none
    (res_scale_init_value None, :247-254)."""
    s1 = sd.get(prefix + "res_scale1.scale")
    s2 = sd.get(prefix + "res_scale2.scale")
    n1 = layer_norm(x, sd, prefix + "norm1.")
    if prefix + "token_mixer.qkv.weight" in sd:
        mixed = rope_attention(n1, sd, prefix + "token_mixer.")
    else:
        mixed = m2d_block(n1, sd, prefix + "token_mixer.", scan_start)
    x = (x if s1 is None else x * s1) + mixed
    x = (x if s2 is None else x * s2) + mlp(layer_norm(x, sd, prefix + "norm2."), sd, prefix + "MLP.")
    return x


def stage(x, sd, prefix, n_blocks, inter_flip):
    """models/mamba2d.py:347-366: odd blocks scan from the bottom-right corner when inter_flip is set; a
    LayerNorm ends the stage (module index n_blocks of the nn.Sequential)."""
    for n in range(n_blocks):
        x = res_block(x, sd, f"{prefix}{n}.", "BR" if inter_flip and n % 2 == 1 else "TL")
    return layer_norm(x, sd, f"{prefix}{n_blocks}.")


def downsampling(x, sd, prefix, stride, padding):
    """models/utils.py:121-141 on a channel-first tensor; the stem has a LayerNorm over channels behind the
    convolution (LayerNorm2D, models/utils.py:9-19)."""
    x = F.conv2d(x, sd[prefix + "conv.weight"], sd[prefix + "conv.bias"], stride=stride, padding=padding)
    if prefix + "post_norm.norm.weight" in sd:
        x = layer_norm(x.permute(0, 2, 3, 1), sd, prefix + "post_norm.norm.").permute(0, 3, 1, 2)
    return x


def backbone(x, sd, n_blocks, inter_flip):
    """models/mamba2d.py:372-386 with the M2D downsampling stages (stem: k7 s4 p2 + norm; then k3 s2 p1,
    :317-336).  x is (B, 3, H, W); returns the last stage's features, channel-first."""
    for i, n in enumerate(n_blocks):
        name = "stem" if i == 0 else f"ds{i}"
        x = downsampling(x, sd, f"ds.{name}.", 4 if i == 0 else 2, 2 if i == 0 else 1)
        x = stage(x.permute(0, 2, 3, 1), sd, f"stages.{i}.", n, inter_flip).permute(0, 3, 1, 2)
    return x
