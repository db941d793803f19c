"""GPU parity of the residual-block operators (m2d_layernorm_fwd, m2d_dwconv3x3_fwd, m2d_starrelu_fwd,
m2d_scale_residual_fwd, m2d_scale_residual_layernorm_fwd, m2d_rope_qknorm_fwd, m2d_rope_attention_fwd, m2d_linear_fwd, m2d_layernorm_linear_fwd, m2d_mlp_fwd) through the C ABI, against the stock torch operators the reference uses (nn.LayerNorm, models/mamba2d.py:220;
depthwise nn.Conv2d, models/utils.py:101) evaluated in fp64 on the CPU.  Tolerances: fp32 2e-5,
bf16 tensors 1e-2 (max error over max value; one bf16 rounding of the result is 4e-3)."""
import pytest
import torch

from oracle import scan_oracle as so

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def cabi():
    from mamba2d_amd import cabi
    return cabi


TOL = {torch.float32: 2e-5, torch.bfloat16: 1e-2}

# rows, channels: the block's widths (64 to 512), a head of the attention stages (32), one chunk, the largest row
LN_SHAPES = [(2 * 9 * 12, 64), (1000, 128), (777, 320), (129, 512), (4 * 6 * 49, 32), (5, 8), (3, 2048), (1, 64), (70, 72)]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", LN_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_layernorm_matches_torch(cabi, shape, dtype, wdtype):
    say(f"\ncase layernorm {shape} {dtype} {wdtype}")
    rows, C = shape
    g = torch.Generator().manual_seed(rows + C)
    # rows away from zero with different spreads (a variance from E[x^2] - mean^2 would lose digits on them)
    x = (torch.randn(rows, C, generator=g) * (torch.rand(rows, 1, generator=g) * 3 + 0.5) + torch.randn(rows, 1, generator=g) * 5).to(dtype)
    w = (torch.rand(C, generator=g) + 0.5).to(wdtype)
    b = torch.randn(C, generator=g).to(wdtype)
    want = torch.nn.functional.layer_norm(x.double(), (C,), w.double(), b.double(), 1e-5)
    got = cabi.layernorm_fwd(x.cuda(), w.cuda(), b.cuda(), 1e-5)
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == x.shape
    assert so.rel_err(got.float().cpu(), want) < TOL[dtype]


def test_layernorm_limits_are_reported(cabi):
    x = torch.zeros(4, 12, device="cuda")
    w = torch.ones(12, device="cuda")
    cabi.layernorm_fwd(x, w, w)                                   # 12 = 3 chunks of fp32
    with pytest.raises(cabi.M2DError):
        cabi.layernorm_fwd(x.bfloat16(), w, w)                    # 12 is no multiple of 8
    with pytest.raises(cabi.M2DError):
        cabi.layernorm_fwd(torch.zeros(2, 4100, device="cuda"), torch.ones(4100, device="cuda"), torch.ones(4100, device="cuda"))


# B, H, W, C: the local path's shapes scaled down, a strip that ends inside the row, one-cell images, one chunk
DW_SHAPES = [(2, 14, 14, 128), (1, 9, 13, 64), (3, 7, 7, 256), (2, 1, 1, 8), (1, 3, 1, 16), (1, 2, 20, 24), (1, 56, 56, 128)]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", DW_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_depthwise_conv_matches_torch(cabi, shape, dtype, wdtype):
    say(f"\ncase dwconv {shape} {dtype} {wdtype}")
    B, H, W, C = shape
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(B, H, W, C, generator=g).to(dtype)
    w = (torch.randn(C, 1, 3, 3, generator=g) / 3).to(wdtype)
    want = torch.nn.functional.conv2d(x.double().permute(0, 3, 1, 2), w.double(), padding=1, groups=C).permute(0, 2, 3, 1)
    got = cabi.dwconv3x3_fwd(x.cuda(), w.cuda())
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == x.shape
    assert so.rel_err(got.float().cpu(), want) < TOL[dtype]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(2, 9, 12, 64), (1, 5, 8), (3, 1000, 24), (128 * 56, 56, 128)], ids=lambda s: "x".join(map(str, s)))
def test_fused_elementwise_match_torch(cabi, shape, dtype, wdtype):
    say(f"\ncase starrelu / scale_residual {shape} {dtype} {wdtype}")
    g = torch.Generator().manual_seed(len(shape) + shape[-1])
    x = torch.randn(*shape, generator=g).to(dtype)
    r = torch.randn(*shape, generator=g).to(dtype)
    sc, bi = torch.tensor([0.8944]).to(wdtype), torch.tensor([-0.4472]).to(wdtype)
    chan = (torch.rand(shape[-1], generator=g) + 0.5).to(wdtype)
    xd, rd = x.cuda(), r.cuda()
    got = cabi.starrelu_fwd(xd, sc.cuda(), bi.cuda())
    want = sc.double() * torch.relu(x.double()) ** 2 + bi.double()
    assert got.dtype == dtype and so.rel_err(got.float().cpu(), want) < TOL[dtype]
    got = cabi.scale_residual_fwd(xd, chan.cuda(), rd)
    want = x.double() * chan.double() + r.double()
    assert got.dtype == dtype and so.rel_err(got.float().cpu(), want) < TOL[dtype]
    r2 = torch.randn(*shape, generator=g).to(dtype)
    got = cabi.scale_residual_fwd(xd, chan.cuda(), rd, r2.cuda())
    want = x.double() * chan.double() + r.double() + r2.double()
    assert got.dtype == dtype and so.rel_err(got.float().cpu(), want) < TOL[dtype]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("two", [False, True], ids=["one_term", "two_terms"])
@pytest.mark.parametrize("shape", [(2, 9, 12, 64), (3, 50, 128), (2, 14, 14, 320), (130, 512), (7, 24), (3, 1000, 2048)],
                         ids=lambda s: "x".join(map(str, s)))
def test_residual_update_with_layernorm_matches_the_two_kernels(cabi, shape, two, dtype, wdtype):
    """The fused pass writes the same x_out as m2d_scale_residual_fwd, bit for bit, and the LayerNorm of exactly
    that tensor as m2d_layernorm_fwd gives it; both are checked against torch elsewhere in this file."""
    say(f"\ncase scale_residual_layernorm {shape} two={two} {dtype} {wdtype}")
    g = torch.Generator().manual_seed(sum(shape) + two)
    C = shape[-1]
    x, r, r2 = (torch.randn(*shape, generator=g).to(dtype).cuda() for _ in range(3))
    sc = (torch.rand(C, generator=g) + 0.5).to(wdtype).cuda()
    w = (torch.rand(C, generator=g) + 0.5).to(wdtype).cuda()
    b = (torch.randn(C, generator=g) * 0.3).to(wdtype).cuda()
    xo, y = cabi.scale_residual_layernorm_fwd(x, sc, r, r2 if two else None, w, b, 1e-5)
    want_x = cabi.scale_residual_fwd(x, sc, r, r2 if two else None)
    want_y = cabi.layernorm_fwd(want_x, w, b, 1e-5)
    torch.cuda.synchronize()
    assert xo.dtype == dtype and y.dtype == dtype
    assert torch.equal(xo, want_x)
    assert torch.equal(y, want_y)


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(2, 7, 9, 10, 32), (1, 14, 14, 16, 32), (3, 5, 4, 3, 64), (1, 2, 3, 1, 8)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rope_and_qk_norm_match_the_module(cabi, shape, dtype, wdtype):
    """Against the attention module's own stock-operator path (mamba2d_amd.backbone.RoPEAttention2D, which
    restates models/utils.py:253-301) evaluated in fp64 on the CPU."""
    from mamba2d_amd.backbone import RoPEAttention2D
    say(f"\ncase rope_qknorm {shape} {dtype} {wdtype}")
    B, H, W, nh, hd = shape
    g = torch.Generator().manual_seed(sum(shape))
    att = RoPEAttention2D(nh * hd, head_dim=hd)
    with torch.no_grad():
        for m in (att.q_norm, att.k_norm):
            m.weight.copy_((torch.rand(hd, generator=g) + 0.5).to(wdtype).float())
            m.bias.copy_((torch.randn(hd, generator=g) * 0.3).to(wdtype).float())
    qkv = torch.randn(B, H * W, 3, nh, hd, generator=g).to(dtype)
    cos, sin = att._rope_tables(H, W, torch.device("cpu"), dtype)
    q64, k64, _ = qkv.double().permute(2, 0, 3, 1, 4).unbind(0)
    c64, s64 = cos.double(), sin.double()
    want = []
    for t, m in ((q64, att.q_norm), (k64, att.k_norm)):
        r = t * c64 + att._rotate_pairs(t) * s64
        want.append(torch.nn.functional.layer_norm(r, (hd,), m.weight.double(), m.bias.double(), m.eps))
    wts = [t.detach().to(wdtype).cuda() for t in (att.q_norm.weight, att.q_norm.bias, att.k_norm.weight, att.k_norm.bias)]
    q, k = cabi.rope_qknorm_fwd(qkv.cuda(), cos.cuda(), sin.cuda(), *wts, att.q_norm.eps)
    torch.cuda.synchronize()
    assert q.shape == (B, nh, H * W, hd) and q.dtype == dtype and q.is_contiguous()
    assert so.rel_err(q.float().cpu(), want[0]) < TOL[dtype]
    assert so.rel_err(k.float().cpu(), want[1]) < TOL[dtype]
    qt, kt = cabi.rope_qknorm_fwd(qkv.cuda(), cos.cuda(), sin.cuda(), *wts, att.q_norm.eps, token_major=True)
    assert qt.shape == q.shape and qt.permute(0, 2, 1, 3).is_contiguous()      # the same values in (B, L, heads, hd) memory
    assert torch.equal(qt, q) and torch.equal(kt, k)


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("shape", [(2, 14, 14, 10), (3, 7, 7, 16), (1, 1, 1, 1), (2, 16, 16, 2), (1, 37, 1, 3), (2, 10, 10, 5), (1, 3, 11, 4),
                                   (1, 8, 8, 1), (2, 13, 5, 2)], ids=lambda s: "x".join(map(str, s)))
def test_rotary_attention_matches_the_module(cabi, shape, wdtype):
    """The one-kernel attention (heads of 32, up to 256 cells) against the module's stock-operator path
    (mamba2d_amd.backbone.RoPEAttention2D, which restates models/utils.py:253-316) in fp64 on the CPU, from the
    same bf16 projection output."""
    from mamba2d_amd.backbone import RoPEAttention2D
    say(f"\ncase rope_attention {shape} {wdtype}")
    B, H, W, nh = shape
    hd, L = 32, H * W
    g = torch.Generator().manual_seed(sum(shape))
    att = RoPEAttention2D(nh * hd, head_dim=hd)
    with torch.no_grad():
        for m in (att.q_norm, att.k_norm):
            m.weight.copy_((torch.rand(hd, generator=g) + 0.5).to(wdtype).float())
            m.bias.copy_((torch.randn(hd, generator=g) * 0.3).to(wdtype).float())
    qkv = (torch.randn(B, L, 3, nh, hd, generator=g) * 1.5).bfloat16()
    cos, sin = att._rope_tables(H, W, torch.device("cpu"), torch.bfloat16)
    q64, k64, v64 = qkv.double().permute(2, 0, 3, 1, 4).unbind(0)
    c64, s64 = cos.double(), sin.double()
    qk = []
    for t, m in ((q64, att.q_norm), (k64, att.k_norm)):
        r = t * c64 + att._rotate_pairs(t) * s64
        qk.append(torch.nn.functional.layer_norm(r, (hd,), m.weight.double(), m.bias.double(), m.eps))
    p = torch.softmax(qk[0] @ qk[1].transpose(-1, -2) * hd ** -0.5, dim=-1)
    want = (p @ v64).transpose(1, 2)                      # (B, L, heads, hd)
    wts = [t.detach().to(wdtype).cuda() for t in (att.q_norm.weight, att.q_norm.bias, att.k_norm.weight, att.k_norm.bias)]
    got = cabi.rope_attention_fwd(qkv.cuda(), cos.cuda(), sin.cuda(), *wts, att.q_norm.eps)
    torch.cuda.synchronize()
    assert got.shape == (B, L, nh, hd) and got.dtype == torch.bfloat16 and got.is_contiguous()
    err = so.rel_err(got.float().cpu(), want)
    say(f"  rel err {err:.3e}")
    assert err < TOL[torch.bfloat16]


def test_rotary_attention_limits_are_reported(cabi):
    """Heads that are not 32 wide and grids of more than 256 cells are refused, not computed wrongly."""
    dev = torch.device("cuda:0")
    for L, hd in ((257, 32), (16, 64), (16, 16)):
        qkv = torch.zeros(1, L, 3, 2, hd, device=dev, dtype=torch.bfloat16)
        t = torch.zeros(L, hd, device=dev, dtype=torch.bfloat16)
        w = torch.ones(hd, device=dev)
        with pytest.raises(cabi.M2DError) as e:
            cabi.rope_attention_fwd(qkv, t, t, w, w, w, w)
        assert e.value.status == 3      # M2D_ERR_UNSUPPORTED


# rows, K, N: the narrow layers of the model at 64 and 128 channels, rows that end inside a tile of 64, one tile
LIN_SHAPES = [(2 * 9 * 12, 64, 64), (1000, 64, 128), (333, 128, 64), (77, 64, 256), (130, 256, 64), (64, 128, 128), (5, 32, 16),
              (200, 128, 512), (190, 512, 128), (70, 256, 128)]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("acts", [(0, 0), (0, 1), (1, 0), (0, 2), (2, 0), (2, 1)], ids=lambda a: f"pre{a[0]}_post{a[1]}")
@pytest.mark.parametrize("shape", LIN_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_small_linear_matches_torch(cabi, shape, acts, wdtype):
    """bf16 activations, weights rounded to bf16 (as a bf16 model or autocast would), fp64 reference."""
    say(f"\ncase linear {shape} pre/post {acts} {wdtype}")
    rows, K, N = shape
    pre, post = acts
    g = torch.Generator().manual_seed(rows + K + N)
    x = torch.randn(rows, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(wdtype)
    b = (torch.randn(N, generator=g) * 0.3).to(wdtype)
    sc, bi = torch.tensor([0.8944]).to(wdtype), torch.tensor([-0.4472]).to(wdtype)

    def ref_act(kind, t):
        if kind == 1:
            return torch.nn.functional.gelu(t)
        if kind == 2:
            return sc.double() * torch.relu(t) ** 2 + bi.double()
        return t

    a_in = ref_act(pre, x.double())
    if pre:
        a_in = a_in.bfloat16().double()       # the activated input is the bf16 operand of the product
    want = ref_act(post, a_in @ w.bfloat16().double().t() + b.double())
    params = (sc.cuda(), bi.cuda())
    got = cabi.linear_fwd(x.cuda(), w.cuda(), b.cuda(), pre, params if pre == 2 else None, post, params if post == 2 else None)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == (rows, N)
    assert so.rel_err(got.float().cpu(), want) < 1e-2
    nb = cabi.linear_fwd(x.cuda(), w.cuda(), None, pre, params if pre == 2 else None, post, params if post == 2 else None)
    want_nb = ref_act(post, a_in @ w.bfloat16().double().t())
    assert so.rel_err(nb.float().cpu(), want_nb) < 1e-2


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("bias", [True, False], ids=["bias", "no_bias"])
@pytest.mark.parametrize("shape", [(2 * 9 * 12, 64), (1000, 64), (333, 32), (64, 64), (5, 32), (70000, 64)], ids=lambda s: "x".join(map(str, s)))
def test_fused_mlp_matches_torch(cabi, shape, bias, wdtype):
    """fc2(GELU(fc1 x)) in one kernel against fp64 on the CPU with the hidden activations rounded to bf16 (as the
    kernel hands them to fc2 and as the stock path stores them); weights rounded to bf16 as the kernel holds them."""
    P, C = shape
    say(f"\ncase mlp {shape} bias={bias} {wdtype}")
    g = torch.Generator().manual_seed(P + C)
    x = torch.randn(P, C, generator=g).bfloat16()
    w1 = (torch.randn(4 * C, C, generator=g) / C ** 0.5).to(wdtype)
    w2 = (torch.randn(C, 4 * C, generator=g) / (4 * C) ** 0.5).to(wdtype)
    b1 = (torch.randn(4 * C, generator=g) * 0.5).to(wdtype) if bias else None
    b2 = (torch.randn(C, generator=g) * 0.5).to(wdtype) if bias else None
    h = x.double() @ w1.bfloat16().double().T + (b1.double() if bias else 0)
    h = torch.nn.functional.gelu(h).bfloat16().double()
    want = h @ w2.bfloat16().double().T + (b2.double() if bias else 0)
    dev = lambda t: None if t is None else t.cuda()
    got = cabi.mlp_fwd(x.cuda(), dev(w1), dev(b1), dev(w2), dev(b2))
    torch.cuda.synchronize()
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    err = so.rel_err(got.float().cpu(), want)
    say(f"  rel err {err:.3e}")
    assert err < TOL[torch.bfloat16]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("shape", [(2 * 9 * 12, 64, 128), (1000, 128, 256), (333, 128, 512), (77, 64, 64), (5, 32, 16), (70000, 64, 128)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("post", [0, 1, 2], ids=lambda a: f"post{a}")
def test_layernorm_in_front_of_a_linear_layer(cabi, shape, post, wdtype):
    """m2d_layernorm_linear_fwd against the two kernels it replaces (their results agree up to the order of the sums
    inside the norm, i.e. an occasional last bf16 bit of a normalised value) and against fp64."""
    P, K, N = shape
    say(f"\ncase layernorm+linear {shape} post={post} {wdtype}")
    g = torch.Generator().manual_seed(P + K + N)
    x = (torch.randn(P, K, generator=g) * 2 + 0.5).bfloat16().cuda()
    lw = (torch.rand(K, generator=g) + 0.5).to(wdtype).cuda()
    lb = (torch.randn(K, generator=g) * 0.3).to(wdtype).cuda()
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(wdtype).cuda()
    b = (torch.randn(N, generator=g) * 0.5).to(wdtype).cuda()
    star = (torch.tensor([0.8944]).to(wdtype).cuda(), torch.tensor([-0.4472]).to(wdtype).cuda())
    got = cabi.linear_fwd(x, w, b, post=post, post_params=star if post == 2 else None, ln=(lw, lb, 1e-5))
    two = cabi.linear_fwd(cabi.layernorm_fwd(x, lw, lb, 1e-5), w, b, post=post, post_params=star if post == 2 else None)
    n64 = torch.nn.functional.layer_norm(x.double().cpu(), (K,), lw.double().cpu(), lb.double().cpu(), 1e-5).bfloat16().double()
    want = n64 @ w.bfloat16().double().cpu().T + b.double().cpu()
    want = torch.nn.functional.gelu(want) if post == 1 else (star[0].double().cpu() * torch.relu(want) ** 2 + star[1].double().cpu()) if post == 2 else want
    torch.cuda.synchronize()
    assert got.shape == (P, N) and got.dtype == torch.bfloat16
    assert so.rel_err(got.float().cpu(), want) < TOL[torch.bfloat16]
    assert so.rel_err(got.float().cpu(), two.double().cpu()) < TOL[torch.bfloat16]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16], ids=["w_f32", "w_bf16"])
@pytest.mark.parametrize("shape", [(1000, 64), (333, 32), (70000, 64)], ids=lambda s: "x".join(map(str, s)))
def test_layernorm_in_front_of_the_fused_mlp(cabi, shape, wdtype):
    P, C = shape
    say(f"\ncase layernorm+mlp {shape} {wdtype}")
    g = torch.Generator().manual_seed(P + C + 1)
    x = (torch.randn(P, C, generator=g) * 2 + 0.5).bfloat16().cuda()
    lw = (torch.rand(C, generator=g) + 0.5).to(wdtype).cuda()
    lb = (torch.randn(C, generator=g) * 0.3).to(wdtype).cuda()
    w1 = (torch.randn(4 * C, C, generator=g) / C ** 0.5).to(wdtype).cuda()
    w2 = (torch.randn(C, 4 * C, generator=g) / (4 * C) ** 0.5).to(wdtype).cuda()
    b1 = (torch.randn(4 * C, generator=g) * 0.5).to(wdtype).cuda()
    b2 = (torch.randn(C, generator=g) * 0.5).to(wdtype).cuda()
    got = cabi.mlp_fwd(x, w1, b1, w2, b2, lw, lb, 1e-5)
    two = cabi.mlp_fwd(cabi.layernorm_fwd(x, lw, lb, 1e-5), w1, b1, w2, b2)
    torch.cuda.synchronize()
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    assert so.rel_err(got.float().cpu(), two.double().cpu()) < TOL[torch.bfloat16]


def test_layernorm_in_front_of_a_wide_layer_is_refused(cabi):
    x = torch.zeros(8, 256, device="cuda", dtype=torch.bfloat16)
    w = torch.ones(256, device="cuda")
    with pytest.raises(cabi.M2DError) as e:
        cabi.linear_fwd(x, torch.zeros(64, 256, device="cuda"), ln=(w, w, 1e-5))
    assert e.value.status == 3      # M2D_ERR_UNSUPPORTED: more than 128 inputs


def test_fused_mlp_limits_are_reported(cabi):
    for C, H in ((128, 512), (64, 128), (48, 192)):
        x = torch.zeros(8, C, device="cuda", dtype=torch.bfloat16)
        with pytest.raises(cabi.M2DError) as e:
            cabi.mlp_fwd(x, torch.zeros(H, C, device="cuda"), None, torch.zeros(C, H, device="cuda"), None)
        assert e.value.status == 3      # M2D_ERR_UNSUPPORTED


def test_small_linear_limits_are_reported(cabi):
    x = torch.zeros(8, 48, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(cabi.M2DError):
        cabi.linear_fwd(x, torch.zeros(16, 48, device="cuda"))            # K is no multiple of 32
    x = torch.zeros(8, 544, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(cabi.M2DError):
        cabi.linear_fwd(x, torch.zeros(16, 544, device="cuda"))           # more than 512 inputs
    with pytest.raises(cabi.M2DError):
        cabi.linear_fwd(torch.zeros(8, 64, device="cuda", dtype=torch.bfloat16), torch.zeros(24, 64, device="cuda"))   # N is no multiple of 16
