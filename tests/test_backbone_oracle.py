"""The residual blocks and the backbone of mamba2d_amd.backbone against oracle/backbone_oracle.py, an
independent float64 restatement of the reference's modules (models/mamba2d.py:157-178, 256-261, 340-386;
models/utils.py:26-118, 144-316) as functions of a state dict: one state dict goes into both.

What this pins that the other backbone tests do not: the order of operations inside M2DBlock (local path
on the unflipped input, flip before in_proj and after out_proj for BR blocks -- here done by the scan's
flip flag), the residual scaling of ResBlock, the stage loop with interleaved scan directions and the norm
that ends a stage, the rotary embedding (which features rotate with which axis, pair layout) and the order
rotation -> q/k LayerNorm -> attention.

CPU: blocks without a scan (rotary attention) in float64 on the stock-operator path.
GPU: a TL block, a BR block, an attention block and a two-stage backbone with inter_flip, fp32 (1e-4) and
bf16 (3e-2; the library kernels of the inference path).
"""
import pytest
import torch

from oracle import backbone_oracle as bo
from oracle import scan_oracle as so


def randomize(module, seed):
    """Every parameter away from its initial value (norm weights and scales near 1, the rest small), so that
    no term of a block is an identity."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in module.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if name.endswith(("AT_log", "AL_log")):
                p.add_(0.3 * torch.randn(p.shape, generator=g))
            elif name.endswith("dt_projT.bias") or name.endswith("dt_projL.bias"):
                p.add_(0.2 * torch.randn(p.shape, generator=g))
            elif leaf in ("scale",) or "norm" in name and leaf == "weight":
                p.copy_(1.0 + 0.3 * torch.randn(p.shape, generator=g))
            elif leaf == "bias" or name.endswith(".D"):
                p.copy_(0.3 * torch.randn(p.shape, generator=g) + (1.0 if name.endswith(".D") else 0.0))
            else:
                p.mul_(1.0 + 0.2 * torch.randn(p.shape, generator=g))
    return module


def ref_state(module, dtype):
    """The module's parameters as the oracle sees them: the values the module computes with (rounded to
    ``dtype`` where the module holds them in it), in float64."""
    return {k: v.detach().to(dtype).double().cpu() for k, v in module.state_dict().items()}


def test_attention_block_cpu_float64():
    from mamba2d_amd.backbone import ResBlock
    blk = randomize(ResBlock(64, "RopeAttention", res_scale_init_value=1.0), 1).double().eval()
    x = torch.randn(2, 5, 7, 64, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    with torch.no_grad():
        got = blk(x)
    want = bo.res_block(x, ref_state(blk, torch.float64), "")
    assert so.rel_err(got, want) < 1e-12


def test_attention_block_without_residual_scale_cpu():
    from mamba2d_amd.backbone import ResBlock
    blk = randomize(ResBlock(32, "RopeAttention", res_scale_init_value=None), 3).double().eval()
    x = torch.randn(1, 4, 4, 32, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    with torch.no_grad():
        got = blk(x)
    assert so.rel_err(got, bo.res_block(x, ref_state(blk, torch.float64), "")) < 1e-12


def test_rope_rotates_rows_then_columns_in_pairs():
    """The oracle's rotary embedding against the textbook form: feature pair (2i, 2i+1) of the first h_dim
    features is the complex number rotated by row * base**(-i/(h_dim/2)), of the next w_dim by the column."""
    H, W, hd = 3, 5, 32
    g = torch.Generator().manual_seed(5)
    sd = {"qkv.weight": torch.randn(3 * hd, hd, generator=g, dtype=torch.float64), "proj.weight": torch.eye(hd, dtype=torch.float64),
          "q_norm.weight": torch.ones(hd, dtype=torch.float64), "q_norm.bias": torch.zeros(hd, dtype=torch.float64),
          "k_norm.weight": torch.ones(hd, dtype=torch.float64), "k_norm.bias": torch.zeros(hd, dtype=torch.float64)}
    x = torch.randn(1, H, W, hd, generator=g, dtype=torch.float64)
    got = bo.rope_attention(x, sd, "", head_dim=hd)
    qkv = (x.reshape(H * W, hd) @ sd["qkv.weight"].T).reshape(H * W, 3, hd)
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]

    def rot(t):
        out = t.clone()
        for n in range(H * W):
            i, j = divmod(n, W)
            for ax, pos in ((0, i), (1, j)):
                for m in range(8):   # of a 32-wide head, 16 features = 8 pairs per axis (models/utils.py:219-223)
                    ang = torch.tensor(pos * 10000.0 ** (-m / 8.0), dtype=torch.float32).double()
                    a, b = t[n, ax * 16 + 2 * m], t[n, ax * 16 + 2 * m + 1]
                    out[n, ax * 16 + 2 * m] = a * torch.cos(ang) - b * torch.sin(ang)
                    out[n, ax * 16 + 2 * m + 1] = b * torch.cos(ang) + a * torch.sin(ang)
        return out

    ln = lambda t: (t - t.mean(-1, keepdim=True)) / torch.sqrt(t.var(-1, unbiased=False, keepdim=True) + 1e-5)
    qr, kr = ln(rot(q)), ln(rot(k))
    want = torch.softmax(qr @ kr.T * hd ** -0.5, dim=-1) @ v
    assert so.rel_err(got.reshape(H * W, hd), want) < 1e-6    # angles are float32 in the reference (models/utils.py:156-159)


# ------------------------------------------------------------------------------------------- GPU
def on_gpu(module, x, dtype):
    m = module.to("cuda").to(dtype).eval()
    with torch.no_grad():
        return m(x.to("cuda").to(dtype)).float().cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("scan_start", ["TL", "BR"])
def test_scan_block_against_reference_composition(scan_start, dtype, tol):
    from mamba2d_amd.backbone import ResBlock
    print(f"\ncase scan block {scan_start} {dtype}", flush=True)
    blk = randomize(ResBlock(64, "2D_local", res_scale_init_value=1.0, scan_start=scan_start), 11)
    x = torch.randn(2, 17, 20, 64, generator=torch.Generator().manual_seed(12))
    got = on_gpu(blk, x, dtype)
    want = bo.res_block(x.to(dtype).double(), ref_state(blk, dtype), "", scan_start)
    e = so.rel_err(got, want)
    print(f"  rel_err {e:.3e}", flush=True)
    assert e < tol


@pytest.mark.gpu
def test_plain_scan_block_without_local_path_or_scale():
    from mamba2d_amd.backbone import ResBlock
    blk = randomize(ResBlock(32, "2D", res_scale_init_value=None, scan_start="BR"), 13)
    x = torch.randn(3, 9, 30, 32, generator=torch.Generator().manual_seed(14))
    e = so.rel_err(on_gpu(blk, x, torch.float32), bo.res_block(x.double(), ref_state(blk, torch.float32), "", "BR"))
    assert e < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("grid", [(14, 14), (7, 7), (9, 20)], ids=lambda g: f"{g[0]}x{g[1]}")
def test_attention_block_against_reference_composition(grid, dtype, tol):
    from mamba2d_amd.backbone import ResBlock
    print(f"\ncase attention block {grid} {dtype}", flush=True)
    blk = randomize(ResBlock(320, "RopeAttention", res_scale_init_value=1.0), 21)
    x = torch.randn(2, *grid, 320, generator=torch.Generator().manual_seed(22))
    e = so.rel_err(on_gpu(blk, x, dtype), bo.res_block(x.to(dtype).double(), ref_state(blk, dtype), ""))
    print(f"  rel_err {e:.3e}", flush=True)
    assert e < tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)], ids=["f32", "bf16"])
def test_two_stage_backbone_with_interleaved_directions(dtype, tol):
    """Stem, a scan stage of three blocks (TL, BR, TL), downsampling, an attention stage of two blocks, the
    norms that end the stages: the stage loop of models/mamba2d.py:340-386."""
    from mamba2d_amd.backbone import Mamba2DBackbone
    print(f"\ncase two-stage backbone {dtype}", flush=True)
    net = randomize(Mamba2DBackbone(n_blocks=(3, 2), embed_dim=(64, 128), token_mixer=("2D_local", "RopeAttention"),
                                    res_scale_init_values=(None, 1.0), inter_flip=True, drop_path_rate=0.1), 31)
    x = torch.randn(2, 3, 96, 64, generator=torch.Generator().manual_seed(32))
    got = on_gpu(net, x, dtype)
    want = bo.backbone(x.to(dtype).double(), ref_state(net, dtype), (3, 2), True)
    e = so.rel_err(got, want)
    print(f"  rel_err {e:.3e}", flush=True)
    assert got.shape == want.shape == (2, 128, 12, 8) and e < tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)], ids=["f32", "bf16"])
def test_m2d_t_full_depth_at_224(dtype, tol):
    """The M2D-T backbone as the benchmark configuration runs it -- blocks [3, 3, 9, 3], channels [64, 128, 320,
    512], scan mixers with the local path at stages 1-2 (odd blocks from the bottom-right corner), rotary attention
    at stages 3-4 -- on one 3x224x224 image, every parameter randomised, against the float64 restatement of
    models/mamba2d.py:340-386 fed the same state dict."""
    from mamba2d_amd.backbone import M2D_T, Mamba2DBackbone
    print(f"\ncase M2D-T [3,3,9,3] at 1x3x224x224 {dtype}", flush=True)
    net = randomize(Mamba2DBackbone(**M2D_T), 41)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(42))
    got = on_gpu(net, x, dtype)
    want = bo.backbone(x.to(dtype).double(), ref_state(net, dtype), M2D_T["n_blocks"], M2D_T["inter_flip"])
    e = so.rel_err(got, want)
    print(f"  rel_err {e:.3e}", flush=True)
    assert got.shape == want.shape == (1, 512, 7, 7) and e < tol
