"""M2D backbone around the MI355X scan, for measuring the scan inside a whole model.

The module tree and parameter names follow the reference backbone (``models/mamba2d.py:16-386``,
``models/utils.py:7-233``) so that a reference state dict maps onto it key by key:
``ds.{stem,ds1,ds2,ds3}.conv.*``, ``ds.stem.post_norm.norm.*``, ``stages.{s}.{k}.{norm1,norm2}.*``,
``stages.{s}.{k}.token_mixer.{in_proj,out_proj,x_proj,dt_projT,dt_projL,AT_log,AL_log,D,
local_norm,local_path.*}`` or ``.token_mixer.{qkv,proj,q_norm,k_norm}.*``,
``stages.{s}.{k}.res_scale{1,2}.scale``, ``stages.{s}.{k}.MLP.{fc1,fc2}.*`` and the stage
post-norm ``stages.{s}.{n_blocks}.*``.

Differences in how it runs (not in what it computes):
  * activations stay channel-last from stem to head; convolutions see them as NCHW views in
    ``torch.channels_last`` memory format, so there are no layout copies between stages;
  * a block that scans from the bottom-right corner passes ``flip=True`` to the scan instead of
    flipping its input and output (``models/mamba2d.py:163-173``): every other operator of the block
    acts per cell and commutes with the flip;
  * the rotary tables of the attention stages are built once per grid size.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .wavefront import (dwconv3x3_fwd_op, layernorm_fwd_op, layernorm_linear_act_fwd_op, linear_act_fwd_op, mlp_fwd_op,
                        rope_qknorm_fwd_op,
                        rope_attention_fwd_op, scale_residual_fwd_op, scale_residual_layernorm_fwd_op, starrelu_fwd_op,
                        wavefront_scan_cuda)

M2D_T = dict(n_blocks=(3, 3, 9, 3), embed_dim=(64, 128, 320, 512),
             token_mixer=("2D_local", "2D_local", "RopeAttention", "RopeAttention"),
             res_scale_init_values=(1.0, 1.0, 1.0, 1.0), inter_flip=True, drop_path_rate=0.175)


def _inference(*tensors):
    """No gradient will be asked of this call: the library's inference kernels may take it."""
    return not torch.is_grad_enabled() or not any(t.requires_grad for t in tensors)


ACT_NONE, ACT_GELU, ACT_STARRELU = 0, 1, 2


def _act(kind, star, t):
    if kind == ACT_GELU:
        return F.gelu(t)
    return star(t) if kind == ACT_STARRELU else t


def _norm_joins(norm, x, w):
    """The LayerNorm ``norm`` over x's last axis can run inside the kernel of the layer (weights ``w``) that reads it."""
    return (isinstance(norm, nn.LayerNorm) and norm.weight is not None and norm.bias is not None
            and tuple(norm.normalized_shape) == (x.shape[-1],) and norm.weight.dtype == w.dtype and norm.bias.dtype == w.dtype
            and _inference(norm.weight, norm.bias))


def linear_act(lin, x, pre=ACT_NONE, post=ACT_NONE, star=None, norm=None):
    """post(lin(pre(x))) for a narrow linear layer: pre / post are nothing, GELU, or the StarReLU module
    ``star``; with ``norm`` (a LayerNorm, and no ``pre``) the layer reads norm(x).  At inference on bf16 activations
    the product runs in the library's kernel together with its neighbouring activation, or norm, where the layer is
    narrow (up to 256 inputs and 512 outputs, the layers of the stages with 64 and 128 channels: there the kernel is
    bound by the activations' bytes; wider layers are faster in the stock library); otherwise stock operators."""
    w, b = lin.weight, lin.bias
    N, K = w.shape
    extra = [t for t in (b, *((star.scale, star.bias) if star is not None else ())) if t is not None]
    if (x.is_cuda and x.dtype == torch.bfloat16 and _inference(x, w, *extra) and w.dtype in (torch.float32, torch.bfloat16)
            and K % 32 == 0 and K <= 256 and N % 16 == 0 and N <= 512 and x.numel() > 0
            and (star is None or star.scale.dtype == w.dtype)):
        ps = (star.scale, star.bias) if pre == ACT_STARRELU else (None, None)
        qs = (star.scale, star.bias) if post == ACT_STARRELU else (None, None)
        if norm is not None and pre == ACT_NONE and K <= 128 and _norm_joins(norm, x, w):
            # the normalised rows go from registers into the product and are never written
            return layernorm_linear_act_fwd_op(x.contiguous(), norm.weight, norm.bias, norm.eps, w, b, post, *qs)
        if norm is not None:
            x = norm(x)
        return linear_act_fwd_op(x.contiguous(), w, b, pre, *ps, post, *qs)
    if norm is not None:
        x = norm(x)
    return _act(post, star, lin(_act(pre, star, x)))


class LayerNorm(nn.LayerNorm):
    """nn.LayerNorm over the channels of a channel-last tensor.  At inference on the GPU the library's
    kernel runs (stock LayerNorm spends a workgroup on every row of 32 to 512 values: 46 % of the
    backbone's inference time); training, the CPU and widths outside the kernel's range take the stock
    operator.  Same parameters and state-dict keys."""

    def forward(self, x):
        w, b = self.weight, self.bias
        if (x.is_cuda and w is not None and b is not None and len(self.normalized_shape) == 1 and _inference(x, w, b)
                and x.dtype in (torch.float32, torch.bfloat16) and w.dtype in (torch.float32, torch.bfloat16)
                and x.shape[-1] % (8 if x.dtype == torch.bfloat16 else 4) == 0 and x.shape[-1] <= 2048 and x.numel() > 0):
            return layernorm_fwd_op(x.contiguous(), w, b, self.eps)
        return super().forward(x)


class LayerNorm2D(nn.Module):
    """LayerNorm over channels of a channel-last tensor (kept as a module with a ``norm`` child for
    the parameter names, ``models/utils.py:7-18``)."""

    def __init__(self, dim):
        super().__init__()
        self.norm = LayerNorm(dim)

    def forward(self, x):           # (B, H, W, C)
        return self.norm(x)


class StarReLU(nn.Module):
    """scale * relu(x)^2 + bias with scalar parameters (``models/utils.py:22-37``)."""

    def __init__(self):
        super().__init__()
        self.scale = nn.Parameter(torch.ones(1))
        self.bias = nn.Parameter(torch.zeros(1))

    def forward(self, x):
        if (x.is_cuda and _inference(x, self.scale, self.bias) and x.is_contiguous() and x.dtype in (torch.float32, torch.bfloat16)
                and self.scale.dtype in (torch.float32, torch.bfloat16) and x.numel() % 8 == 0 and x.numel() > 0):
            return starrelu_fwd_op(x, self.scale, self.bias)      # one pass instead of three
        return torch.addcmul(self.bias, self.scale, F.relu(x).square())


class Scale(nn.Module):
    def __init__(self, dim, init_value=1.0):
        super().__init__()
        self.scale = nn.Parameter(init_value * torch.ones(dim))

    def forward(self, x):
        return x * self.scale


class MLP(nn.Module):
    def __init__(self, dim, expand=4):
        super().__init__()
        self.fc1 = nn.Linear(dim, dim * expand)
        self.fc2 = nn.Linear(dim * expand, dim)

    def forward(self, x, norm=None):
        """fc2(GELU(fc1 x)), of norm(x) with ``norm`` (the block's norm2, which only the MLP reads)."""
        w1, w2 = self.fc1.weight, self.fc2.weight
        if (x.is_cuda and x.dtype == torch.bfloat16 and x.numel() > 0 and x.shape[-1] in (32, 64) and w1.shape[0] == 4 * w1.shape[1]
                and _inference(x, w1, w2, self.fc1.bias, self.fc2.bias) and w1.dtype in (torch.float32, torch.bfloat16)
                and w2.dtype == w1.dtype):
            # both layers in one kernel: the hidden activations, four times x, never reach memory
            if norm is not None and _norm_joins(norm, x, w1):
                return mlp_fwd_op(x.contiguous(), w1, self.fc1.bias, w2, self.fc2.bias, norm.weight, norm.bias, norm.eps)
            return mlp_fwd_op((x if norm is None else norm(x)).contiguous(), w1, self.fc1.bias, w2, self.fc2.bias)
        return linear_act(self.fc2, linear_act(self.fc1, x, post=ACT_GELU, norm=norm))

    def takes_norm(self, x, norm):
        """norm(x) would not be written: the kernel of the first layer computes it."""
        w1 = self.fc1.weight
        return (x.is_cuda and x.dtype == torch.bfloat16 and x.numel() > 0
                and _inference(x, w1, self.fc2.weight, self.fc1.bias, self.fc2.bias)
                and w1.dtype in (torch.float32, torch.bfloat16) and self.fc2.weight.dtype == w1.dtype and _norm_joins(norm, x, w1)
                and w1.shape[1] % 32 == 0 and w1.shape[1] <= 128 and w1.shape[0] % 16 == 0 and w1.shape[0] <= 512)


def _conv_channel_last(conv, x):
    """conv on a (B, H, W, C) tensor without a layout copy: the NCHW view of a channel-last tensor
    is already in channels_last memory format; the result is handed back as (B, H', W', C')."""
    y = conv(x.permute(0, 3, 1, 2))
    return y.permute(0, 2, 3, 1)


class SepConv(nn.Module):
    """pointwise -> StarReLU -> depthwise 3x3 -> StarReLU -> pointwise, no bias
    (``models/utils.py:83-113`` as configured at ``models/mamba2d.py:57-60``)."""

    def __init__(self, dim, expansion=2, kernel_size=3, padding=1):
        super().__init__()
        med = int(expansion * dim)
        self.pwconv1 = nn.Linear(dim, med, bias=False)
        self.act1 = StarReLU()
        self.dwconv = nn.Conv2d(med, med, kernel_size, padding=padding, groups=med, bias=False)
        self.act2 = StarReLU()
        self.pwconv2 = nn.Linear(med, dim, bias=False)

    def forward(self, x, norm=None):
        x = linear_act(self.pwconv1, x, post=ACT_STARRELU, star=self.act1, norm=norm)
        w = self.dwconv.weight
        if (x.is_cuda and _inference(x, w) and self.dwconv.kernel_size == (3, 3) and self.dwconv.padding == (1, 1)
                and x.dtype in (torch.float32, torch.bfloat16) and w.dtype in (torch.float32, torch.bfloat16)
                and x.shape[-1] % (8 if x.dtype == torch.bfloat16 else 4) == 0 and x.numel() > 0):
            # the library's depthwise kernel (the stock library falls back to a generic direct
            # convolution for channel-last bf16 here, ten times slower than the memory traffic allows)
            x = dwconv3x3_fwd_op(x.contiguous(), w)
        else:
            x = _conv_channel_last(self.dwconv, x)
        return linear_act(self.pwconv2, x, pre=ACT_STARRELU, star=self.act2)


class Downsampling(nn.Module):
    """Strided convolution with an optional norm after it (``models/utils.py:116-136``)."""

    def __init__(self, cin, cout, kernel_size, stride, padding, post_norm=False):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, kernel_size, stride=stride, padding=padding)
        self.post_norm = LayerNorm2D(cout) if post_norm else nn.Identity()

    def forward(self, x):           # channel-last in, channel-last out
        return self.post_norm(_conv_channel_last(self.conv, x))


class M2DBlock(nn.Module):
    """Token mixer: in_proj -> GELU -> 2-D selective scan -> GELU -> out_proj, plus an optional local
    convolution path on the normalised input (``models/mamba2d.py:16-188``).  Parameter
    initialisation follows ``models/mamba2d.py:66-111``: dt log-uniform in [dt_min, dt_max] through
    the inverse softplus into the dt biases, A = 1..N (S4D-real), D = 1."""

    def __init__(self, d_model, d_state=16, dt_min=1e-3, dt_max=1e-1, dt_init_floor=1e-4,
                 local_path=False, scan_start="TL", recomp="partial"):
        super().__init__()
        if scan_start not in ("TL", "BR"):
            raise ValueError(f"Invalid Scan Direction, expected TL or BR and got {scan_start}")
        self.flip = scan_start == "BR"
        self.recomp = recomp
        self.dt_rank = math.ceil(d_model / 16)
        self.local_norm = LayerNorm(d_model) if local_path else None
        self.local_path = SepConv(d_model) if local_path else None
        self.in_proj = nn.Linear(d_model, d_model)
        self.x_proj = nn.Linear(d_model, 2 * self.dt_rank + 3 * d_state, bias=False)
        self.dt_projT = nn.Linear(self.dt_rank, d_model)
        self.dt_projL = nn.Linear(self.dt_rank, d_model)
        std = self.dt_rank ** -0.5
        nn.init.uniform_(self.dt_projT.weight, -std, std)
        nn.init.uniform_(self.dt_projL.weight, -std, std)
        dt = torch.exp(torch.rand(d_model) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min)).clamp(min=dt_init_floor)
        inv_softplus = dt + torch.log(-torch.expm1(-dt))
        with torch.no_grad():
            self.dt_projT.bias.copy_(inv_softplus)
            self.dt_projL.bias.copy_(inv_softplus)
        a = torch.log(torch.arange(1, d_state + 1, dtype=torch.float32)).repeat(d_model, 1)
        self.AT_log = nn.Parameter(a.clone())
        self.AL_log = nn.Parameter(a.clone())
        self.D = nn.Parameter(torch.ones(d_model))
        for prm in (self.AT_log, self.AL_log, self.D):
            prm._no_weight_decay = True
        self.out_proj = nn.Linear(d_model, d_model)

    def forward(self, x, split=False):           # (B, H, W, C)
        """The mixed tokens; with ``split`` and a local path, the two terms of the sum, for a caller that
        adds them in a pass of its own."""
        local = self.local_path(x, norm=self.local_norm) if self.local_path is not None else None
        u = linear_act(self.in_proj, x, post=ACT_GELU)
        y = wavefront_scan_cuda(u, self.AT_log, self.AL_log, self.x_proj.weight,
                                self.dt_projT.weight, self.dt_projT.bias,
                                self.dt_projL.weight, self.dt_projL.bias, self.D, self.recomp, flip=self.flip)
        y = linear_act(self.out_proj, y, pre=ACT_GELU)
        if split and local is not None:
            return y, local
        return y if local is None else y + local


class RoPEAttention2D(nn.Module):
    """Multi-head self-attention over the H*W cells with rotary embeddings on the two grid axes
    (``models/utils.py:165-316``): of every head, the first 2*floor(head_dim/4) dims
    rotate with the row index, the next as many with the column index (16 + 16 of a 32-wide head) and
    any remainder is left alone; q and k are layer-normed per head."""

    def __init__(self, dim, head_dim=32, rope_base=10000.0):
        super().__init__()
        self.head_dim = head_dim
        self.num_heads = max(dim // head_dim, 1)
        inner = self.num_heads * head_dim
        self.qkv = nn.Linear(dim, 3 * inner, bias=False)
        self.proj = nn.Linear(inner, dim, bias=False)
        self.q_norm = LayerNorm(head_dim)
        self.k_norm = LayerNorm(head_dim)
        self.axis_dim = (head_dim // 2 // 2) * 2        # rotated dims per axis
        self.rope_base = rope_base
        self._tables = {}

    def _rope_tables(self, H, W, device, dtype):
        key = (H, W, str(device), dtype)
        if key not in self._tables:
            # built outside inference mode (and without a graph): a table made under torch.inference_mode
            # could not be saved for the backward pass of a later training call
            with torch.inference_mode(False), torch.no_grad():
                d = self.axis_dim
                inv_freq = 1.0 / (self.rope_base ** (torch.arange(0, d // 2, device=device, dtype=torch.float32) / (d // 2)))
                rows = torch.arange(H, device=device, dtype=torch.float32).repeat_interleave(W)
                cols = torch.arange(W, device=device, dtype=torch.float32).repeat(H)
                ang = torch.cat([rows[:, None] * inv_freq, cols[:, None] * inv_freq], dim=-1)   # (HW, d)
                ang = ang.repeat_interleave(2, dim=-1)                                           # pairs share an angle
                # layout per head: [row-rotated d | column-rotated d | untouched]
                cos = torch.ones(H * W, self.head_dim, device=device)
                sin = torch.zeros(H * W, self.head_dim, device=device)
                cos[:, :2 * d] = torch.cat([ang[:, 0:d].cos(), ang[:, d:2 * d].cos()], dim=-1)
                sin[:, :2 * d] = torch.cat([ang[:, 0:d].sin(), ang[:, d:2 * d].sin()], dim=-1)
                self._tables[key] = (cos.to(dtype), sin.to(dtype))
        return self._tables[key]

    @staticmethod
    def _rotate_pairs(t):
        a, b = t.unflatten(-1, (-1, 2)).unbind(-1)
        return torch.stack((-b, a), dim=-1).flatten(-2)

    def forward(self, x):           # (B, H, W, C)
        B, H, W, _ = x.shape
        qkv = self.qkv(x).view(B, H * W, 3, self.num_heads, self.head_dim)
        cos, sin = self._rope_tables(H, W, x.device, qkv.dtype)
        qn, kn, hd = self.q_norm, self.k_norm, self.head_dim
        if (qkv.is_cuda and _inference(qkv, qn.weight, qn.bias, kn.weight, kn.bias) and qkv.dtype in (torch.float32, torch.bfloat16)
                and qn.weight.dtype in (torch.float32, torch.bfloat16) and qn.eps == kn.eps and hd & (hd - 1) == 0
                and 8 <= hd <= 128 and qkv.numel() > 0):
            if hd == 32 and H * W <= 256 and qkv.dtype == torch.bfloat16:
                # the whole attention in one kernel, a head per workgroup, answering in the projection's layout
                o = rope_attention_fwd_op(qkv, cos, sin, qn.weight, qn.bias, kn.weight, kn.bias, qn.eps, hd ** -0.5)
                return self.proj(o.view(B, H, W, self.num_heads * hd))
            # rotation and the two LayerNorms in one pass; q and k keep the projection's token-major layout,
            # like v, so the attention kernel answers in it and its output needs no transposing copy
            q, k = rope_qknorm_fwd_op(qkv, cos, sin, qn.weight, qn.bias, kn.weight, kn.bias, qn.eps, True)
            o = F.scaled_dot_product_attention(q, k, qkv[:, :, 2].permute(0, 2, 1, 3), scale=hd ** -0.5)
            return self.proj(o.transpose(1, 2).reshape(B, H, W, self.num_heads * hd))
        q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)     # (B, heads, HW, head_dim)
        q = q * cos + self._rotate_pairs(q) * sin      # sin is zero on the untouched dims
        k = k * cos + self._rotate_pairs(k) * sin
        q, k = self.q_norm(q), self.k_norm(k)
        o = F.scaled_dot_product_attention(q, k, v, scale=self.head_dim ** -0.5)
        return self.proj(o.transpose(1, 2).reshape(B, H, W, self.num_heads * self.head_dim))


def _drop_path(x, p, training):
    if p == 0.0 or not training:
        return x
    keep = torch.rand(x.shape[0], *([1] * (x.ndim - 1)), device=x.device) >= p
    return x * keep.to(x.dtype) / (1.0 - p)


class ResBlock(nn.Module):
    """x <- s1*x + mixer(norm1 x);  x <- s2*x + MLP(norm2 x)  (``models/mamba2d.py:191-254``)."""

    def __init__(self, dim, token_mixer="2D", mlp_expand_factor=4, drop_path=0.0, res_scale_init_value=None,
                 scan_start="TL", recomp="partial"):
        super().__init__()
        self.norm1 = LayerNorm(dim)
        if token_mixer == "2D":
            self.token_mixer = M2DBlock(dim, scan_start=scan_start, recomp=recomp)
        elif token_mixer == "2D_local":
            self.token_mixer = M2DBlock(dim, scan_start=scan_start, recomp=recomp, local_path=True)
        elif token_mixer == "RopeAttention":
            self.token_mixer = RoPEAttention2D(dim)
        else:
            raise ValueError(f"Invalid token mixer type: {token_mixer}")
        self.res_scale1 = Scale(dim, res_scale_init_value) if res_scale_init_value else nn.Identity()
        self.norm2 = LayerNorm(dim)
        self.MLP = MLP(dim, mlp_expand_factor)
        self.res_scale2 = Scale(dim, res_scale_init_value) if res_scale_init_value else nn.Identity()
        self.drop_path = float(drop_path)

    @staticmethod
    def _residual(x, scale, branch, branch2=None):
        """scale(x) + branch (+ branch2); with a learned scale, at inference on the GPU, in one pass."""
        terms = (branch,) if branch2 is None else (branch, branch2)
        if (isinstance(scale, Scale) and x.is_cuda and _inference(x, scale.scale, *terms) and x.is_contiguous()
                and all(t.is_contiguous() and t.dtype == x.dtype and t.shape == x.shape for t in terms)
                and x.dtype in (torch.float32, torch.bfloat16) and scale.scale.dtype in (torch.float32, torch.bfloat16)
                and x.shape[-1] % 8 == 0 and x.numel() > 0):
            return scale_residual_fwd_op(x, scale.scale, branch, branch2)
        return scale(x) + (branch if branch2 is None else branch + branch2)

    @staticmethod
    def _residual_norm(x, scale, terms, norm):
        """(y, norm(y)) for y = scale(x) + sum(terms); (y, None) without a norm.  At inference on the GPU the update
        and the LayerNorm behind it are one pass over the rows."""
        if (norm is not None and isinstance(scale, Scale) and x.is_cuda and x.is_contiguous() and x.numel() > 0
                and _inference(x, scale.scale, norm.weight, norm.bias, *terms)
                and all(t.is_contiguous() and t.dtype == x.dtype and t.shape == x.shape for t in terms)
                and x.dtype in (torch.float32, torch.bfloat16) and scale.scale.dtype in (torch.float32, torch.bfloat16)
                and norm.weight is not None and norm.bias is not None and norm.weight.dtype == scale.scale.dtype
                and norm.bias.dtype == scale.scale.dtype and tuple(norm.normalized_shape) == (x.shape[-1],)
                and x.shape[-1] % 8 == 0 and x.shape[-1] <= 2048):
            return scale_residual_layernorm_fwd_op(x, scale.scale, terms[0], terms[1] if len(terms) > 1 else None,
                                                   norm.weight, norm.bias, norm.eps)
        y = ResBlock._residual(x, scale, *terms)
        return y, (norm(y) if norm is not None else None)

    def forward_fused(self, x, normed=None, next_norm=None):
        """The block on x, with ``normed`` = norm1(x) where the caller has it already; returns the block's output
        and ``next_norm`` of it (None without ``next_norm``): the LayerNorm that follows the block, computed in
        the pass of the second residual update."""
        n1 = self.norm1(x) if normed is None else normed
        if isinstance(self.token_mixer, M2DBlock) and not self.training:
            mixed = self.token_mixer(n1, split=True)       # scan path and local path, summed in the update
            terms = mixed if isinstance(mixed, tuple) else (mixed,)
        else:
            terms = (_drop_path(self.token_mixer(n1), self.drop_path, self.training),)
        if self.MLP.takes_norm(x, self.norm2):      # norm2 inside the MLP's first kernel: nobody else reads it
            x = self._residual(x, self.res_scale1, *terms)
            branch = self.MLP(x, norm=self.norm2)
        else:
            x, n2 = self._residual_norm(x, self.res_scale1, terms, self.norm2)
            branch = self.MLP(n2)
        return self._residual_norm(x, self.res_scale2, (_drop_path(branch, self.drop_path, self.training),), next_norm)

    def forward(self, x):
        return self.forward_fused(x)[0]


class Mamba2DBackbone(nn.Module):
    """Stem (k7 s4 p2 + norm), then per stage a k3 s2 p1 downsampling (from the second stage on),
    ``n_blocks`` residual blocks and a LayerNorm (``models/mamba2d.py:256-386``).  Takes
    (B, 3, H, W) images, returns the last stage's features as (B, C, H/32, W/32)."""

    def __init__(self, in_channels=3, n_blocks=(3, 3, 9, 3), embed_dim=(64, 128, 320, 512),
                 token_mixer=("2D_local", "2D_local", "RopeAttention", "RopeAttention"),
                 drop_path_rate=0.1, res_scale_init_values=(None, None, 1.0, 1.0), inter_flip=False,
                 recomp="partial"):
        super().__init__()
        if not (len(n_blocks) == len(embed_dim) == len(token_mixer) == len(res_scale_init_values)):
            raise ValueError("Check backbone init_args are defined for each stage!")
        self.ds = nn.ModuleDict()
        for i, dim in enumerate(embed_dim):
            if i == 0:
                self.ds["stem"] = Downsampling(in_channels, dim, 7, 4, 2, post_norm=True)
            else:
                self.ds[f"ds{i}"] = Downsampling(embed_dim[i - 1], dim, 3, 2, 1)
        total = sum(n_blocks)
        rates = [drop_path_rate * k / max(total - 1, 1) for k in range(total)]
        self.stages = nn.ModuleDict()
        done = 0
        for i, (n, dim) in enumerate(zip(n_blocks, embed_dim)):
            blocks = [ResBlock(dim, token_mixer[i], drop_path=rates[done + k],
                               res_scale_init_value=res_scale_init_values[i],
                               scan_start="BR" if inter_flip and k % 2 == 1 else "TL", recomp=recomp)
                      for k in range(n)]
            blocks.append(LayerNorm(dim))
            self.stages[str(i)] = nn.Sequential(*blocks)
            done += n

    @staticmethod
    def _run_stage(stage, x):
        """The stage's modules in order; a block is handed the LayerNorm that follows it (the next block's norm1 or
        the norm that ends the stage) so that it can compute it together with its last residual update."""
        mods = list(stage)
        normed = None
        for i, m in enumerate(mods):
            if isinstance(m, ResBlock):
                nxt = mods[i + 1] if i + 1 < len(mods) else None
                follows = nxt.norm1 if isinstance(nxt, ResBlock) else nxt if isinstance(nxt, nn.LayerNorm) else None
                x, normed = m.forward_fused(x, normed, follows)
            elif isinstance(m, nn.LayerNorm) and normed is not None:
                x, normed = normed, None
            else:
                x, normed = m(x), None
        return x

    def forward(self, x):
        x = x.permute(0, 2, 3, 1)                      # channel-last view; the stem makes it real
        for ds, stage in zip(self.ds.values(), self.stages.values()):
            x = self._run_stage(stage, ds(x).contiguous())
        return x.permute(0, 3, 1, 2)


def load_backbone_checkpoint(model: Mamba2DBackbone, path: str, layers=("ds", "stages")) -> None:
    """Loads the backbone weights of a training checkpoint of the reference: a file whose
    ``["state_dict"]`` holds the backbone under the prefix ``backbone.`` next to the classifier head
    (the convention of ``downstream/Mamba2D/mamba2d.py:397-415``).  Only tensors are read
    (``weights_only=True``); keys outside ``layers`` are ignored; any key of ``layers`` that is missing
    on either side raises."""
    try:
        ckpt = torch.load(path, weights_only=True, mmap=True)
    except FileNotFoundError:
        raise FileNotFoundError(f"Pretrained checkpoint not found: {path}")
    wanted = lambda name: any(name.startswith(l + ".") for l in layers)
    sd = {}
    for name, tensor in ckpt["state_dict"].items():
        name = name[len("backbone."):] if name.startswith("backbone.") else name
        if wanted(name):
            sd[name] = tensor
    missing, unexpected = model.load_state_dict(sd, strict=False)
    missing = [k for k in missing if wanted(k)]
    unexpected = [k for k in unexpected if wanted(k)]
    if missing or unexpected:
        raise RuntimeError(f"Backbone/checkpoint key mismatch.\nmissing: {missing}\nunexpected: {unexpected}")
