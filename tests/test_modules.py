"""Host-side module wrappers: what they accept, what they hold (no GPU needed) and, on the GPU,
their results against the CPU oracle."""
import pytest
import torch

from basedxl_amd import (BasedXLFusedKV, BasedXLLowPConv1x1, BasedXLLowPLinear, patch_linear_layers,
                         patch_pointwise_convs)
from basedxl_amd.modules import is_pointwise
from oracle import cascade as oc


class _Block(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.shortcut = torch.nn.Conv2d(8, 16, 1)
        self.conv3 = torch.nn.Conv2d(8, 16, 3, padding=1)
        self.strided = torch.nn.Conv2d(8, 16, 1, stride=2)
        self.inner = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.Conv2d(4, 4, 1, bias=False))


def test_pointwise_predicate_and_patcher():
    m = _Block()
    assert is_pointwise(m.shortcut) and not is_pointwise(m.conv3) and not is_pointwise(m.strided)
    assert not is_pointwise(torch.nn.Conv2d(8, 8, 1, groups=2)) and not is_pointwise(torch.nn.Linear(4, 4))
    patch_pointwise_convs(m, terms=3)
    assert isinstance(m.shortcut, BasedXLLowPConv1x1) and m.shortcut.terms == 3 and m.shortcut.lowp == "bf16"
    assert isinstance(m.inner[1], BasedXLLowPConv1x1) and m.inner[1].bias is None
    assert isinstance(m.conv3, torch.nn.Conv2d) and isinstance(m.strided, torch.nn.Conv2d)
    assert isinstance(m.inner[0], torch.nn.Linear)          # Linear layers are the other patcher's
    patch_linear_layers(m)
    assert isinstance(m.inner[0], BasedXLLowPLinear)
    with pytest.raises(ValueError):
        BasedXLLowPConv1x1(torch.nn.Conv2d(8, 16, 3))


def test_fused_qkv_weight_is_the_concatenation():
    """Self-attention: query, key and value read the same tokens, so the three weights stack into one."""
    from basedxl_amd.modules import BasedXLFusedQKV
    to_q, to_k, to_v = (torch.nn.Linear(12, 8, bias=False) for _ in range(3))
    mod = BasedXLFusedQKV(to_q, to_k, to_v)
    assert mod.to_qkv.weight.shape == (12, 24) and mod.to_qkv.bias is None
    for i, lin in enumerate((to_q, to_k, to_v)):
        assert torch.equal(mod.to_qkv.weight[:, 8 * i:8 * i + 8], lin.weight.detach().T)
    with pytest.raises(AssertionError):
        BasedXLFusedQKV(to_q, torch.nn.Linear(16, 8, bias=False), torch.nn.Linear(16, 8, bias=False))   # cross-attention


def test_pointwise_conv_holds_both_weight_layouts():
    conv = torch.nn.Conv2d(6, 10, 1)
    mod = BasedXLLowPConv1x1(conv)
    assert mod.weight.shape == (10, 6) and mod.weight_t.shape == (6, 10)
    assert torch.equal(mod.weight, conv.weight.detach().reshape(10, 6)) and torch.equal(mod.weight_t, mod.weight.T)
    assert mod.weight.is_contiguous() and mod.weight_t.is_contiguous()
    assert mod.weight.data_ptr() != conv.weight.data_ptr()   # a clone, like lowp_linear.py:12
    with pytest.raises(ValueError):
        mod(torch.zeros(2, 5, 4, 4))


def test_fused_kv_weight_is_the_concatenation():
    """attn.py:23-39: rows [0, out) of the fused weight are to_k's, rows [out, 2 out) to_v's."""
    to_k, to_v = torch.nn.Linear(12, 8), torch.nn.Linear(12, 8)
    mod = BasedXLFusedKV(to_k, to_v)
    assert mod.to_kv.weight.shape == (12, 16)                 # stored transposed, [in, 2 out]
    assert torch.equal(mod.to_kv.weight[:, :8], to_k.weight.detach().T)
    assert torch.equal(mod.to_kv.weight[:, 8:], to_v.weight.detach().T)
    assert torch.equal(mod.to_kv.bias, torch.cat([to_k.bias, to_v.bias]).detach())
    with pytest.raises(AssertionError):
        BasedXLFusedKV(to_k, torch.nn.Linear(12, 8, bias=False))
    with pytest.raises(AssertionError):
        BasedXLFusedKV(to_k, torch.nn.Linear(12, 4))


class _ForeignAttention(torch.nn.Module):
    """An attention module of somebody else's (like diffusers'): its forward reads to_q / to_k / to_v."""

    def __init__(self):
        super().__init__()
        self.to_q = torch.nn.Linear(8, 8, bias=False)
        self.to_k = torch.nn.Linear(8, 8, bias=False)
        self.to_v = torch.nn.Linear(8, 8, bias=False)

    def forward(self, x):
        return self.to_q(x) + self.to_k(x) + self.to_v(x)


def test_fusion_leaves_attention_modules_it_does_not_know_alone():
    """The key / value fusion replaces children that only the skeleton's own forward knows how to use;
    a foreign attention module must come out of patch_unet with to_q / to_k / to_v still there (routed
    one by one, as basedxl/unet.py:81-87 does) and a forward that still runs."""
    from basedxl_amd.unet import patch_unet
    from basedxl_amd.utils import BasedXLConfig
    from basedxl_amd.unet_skeleton import Attention, fuse_kv_projections

    model = torch.nn.ModuleDict({"foreign": _ForeignAttention(), "own_self": Attention(8, None, 2),
                                 "own_cross": Attention(8, 12, 2)})
    want = model["foreign"](torch.ones(3, 8))
    fuse_kv_projections(model, fuse_q=True)
    f = model["foreign"]
    assert all(isinstance(getattr(f, n), torch.nn.Linear) for n in ("to_q", "to_k", "to_v"))
    assert not hasattr(f, "to_kv") and not hasattr(f, "to_qkv")
    assert torch.equal(f(torch.ones(3, 8)), want)                       # its forward still finds its children
    assert hasattr(model["own_self"], "to_qkv") and not hasattr(model["own_self"], "to_k")
    assert hasattr(model["own_cross"], "to_kv") and hasattr(model["own_cross"], "to_q")
    # the install hook routes the foreign module's three projections through the plain Linear walk
    model2 = torch.nn.ModuleDict({"foreign": _ForeignAttention()})
    patch_unet(model2, BasedXLConfig(fp16_acc_matmul=True))
    assert all(isinstance(getattr(model2["foreign"], n), BasedXLLowPLinear) for n in ("to_q", "to_k", "to_v"))


# ---------------------------------------------------------------------------------- GPU


def _conv_oracle(x, conv):
    """1x1 convolution through the oracle's cascade: pixels as rows, channels as K."""
    B, C, H, W = x.shape
    w = conv.weight.detach().cpu().reshape(conv.out_channels, C).T.contiguous()
    y = oc.cascade_matmul_ref(x.cpu().permute(0, 2, 3, 1).reshape(-1, C).contiguous(), w)
    if conv.bias is not None:
        y = y + conv.bias.detach().cpu()
    return y.reshape(B, H, W, -1).permute(0, 3, 1, 2)


@pytest.mark.gpu
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_pointwise_conv_matches_oracle(gpu_device, channels_last, bias):
    torch.manual_seed(31)
    conv = torch.nn.Conv2d(320, 640, 1, bias=bias).to("cuda:0")
    mod = BasedXLLowPConv1x1(conv).to("cuda:0")
    x = torch.randn(2, 320, 24, 16, device="cuda:0")
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    y = mod(x)
    assert y.shape == (2, 640, 24, 16)
    assert y.is_contiguous(memory_format=torch.channels_last) if channels_last else y.is_contiguous()
    want = _conv_oracle(x, conv)
    # the two layouts sum the same products in different orders: tolerance of the accumulation
    torch.testing.assert_close(y.cpu(), want, rtol=0, atol=3e-5)
    exp = torch.nn.functional.conv2d(x.double().cpu(), conv.weight.detach().double().cpu(),
                                     None if conv.bias is None else conv.bias.detach().double().cpu())
    got, ref = oc.error_metrics(y.cpu(), exp), oc.error_metrics(want, exp)
    assert got["rel_fro"] <= 1.25 * ref["rel_fro"] and got["max_abs"] <= 1.25 * ref["max_abs"]


@pytest.mark.gpu
def test_pointwise_conv_integer_exact_and_batches_beyond_one_group(gpu_device):
    """Small-integer operands: every layout gives the integer convolution exactly; 11 images
    need two grouped launches."""
    g = torch.Generator().manual_seed(32)
    conv = torch.nn.Conv2d(64, 32, 1)
    with torch.no_grad():
        conv.weight.copy_(torch.randint(-8, 9, conv.weight.shape, generator=g).float())
        conv.bias.copy_(torch.randint(-8, 9, (32,), generator=g).float())
    x = torch.randint(-8, 9, (11, 64, 8, 8), generator=g).float()
    want = torch.nn.functional.conv2d(x.double(), conv.weight.detach().double(), conv.bias.detach().double()).float()
    mod = BasedXLLowPConv1x1(conv).to("cuda:0")
    assert torch.equal(mod(x.to("cuda:0")).cpu(), want)
    assert torch.equal(mod(x.to("cuda:0").contiguous(memory_format=torch.channels_last)).cpu(), want)


@pytest.mark.gpu
def test_fused_kv_equals_separate_projections_and_caches(gpu_device):
    torch.manual_seed(33)
    to_k, to_v = torch.nn.Linear(2048, 640).to("cuda:0"), torch.nn.Linear(2048, 640).to("cuda:0")
    ctx = torch.randn(2, 77, 2048, device="cuda:0")
    mod = BasedXLFusedKV(to_k, to_v, cache=True)
    k, v = mod(ctx)
    assert k.shape == (2, 77, 640) and v.shape == (2, 77, 640)
    for got, lin in ((k, to_k), (v, to_v)):
        want = oc.cascade_matmul_ref(ctx.cpu().reshape(-1, 2048), lin.weight.detach().cpu().T.contiguous()) + lin.bias.detach().cpu()
        torch.testing.assert_close(got.cpu().reshape(-1, 640), want, rtol=0, atol=3e-5)
    # attn.py:74-78: later steps get the cached tensor, whatever they pass, until asked to recompute
    k2, v2 = mod(torch.zeros_like(ctx))
    assert k2.data_ptr() == k.data_ptr() and torch.equal(k2, k) and torch.equal(v2, v)
    k3, _ = mod(torch.zeros_like(ctx), recompute=True)
    assert torch.equal(k3.cpu(), to_k.bias.detach().cpu().expand(2, 77, 640))
    mod.reset()
    assert mod.kv_cache is None
    k4, _ = BasedXLFusedKV(to_k, to_v)(ctx)
    assert torch.equal(k4, k)


@pytest.mark.gpu
@pytest.mark.parametrize("lowp,terms,atol", [("bf16", 2, 3e-5), ("fp8", 3, 3e-4)])
def test_fused_qkv_equals_the_oracle_of_each_projection(gpu_device, lowp, terms, atol):
    from basedxl_amd.modules import BasedXLFusedQKV
    torch.manual_seed(34)
    lins = [torch.nn.Linear(640, 640, bias=False).to("cuda:0") for _ in range(3)]
    x = torch.randn(2, 512, 640, device="cuda:0")
    mod = BasedXLFusedQKV(*lins, lowp=lowp, terms=terms)
    outs = mod(x)
    assert all(o.shape == (2, 512, 640) for o in outs)
    # the fp8 cascade scales the stacked weight as one tensor: the oracle gets that exponent
    kw = {}
    if lowp == "fp8":
        kw = {"b_exp": oc.tensor_scale_exp(torch.cat([l.weight.detach().cpu() for l in lins]), "fp8")}
    for got, lin in zip(outs, lins):
        want = oc.cascade_matmul_ref(x.cpu().reshape(-1, 640), lin.weight.detach().cpu().T.contiguous(), lowp, terms, "tri", **kw)
        torch.testing.assert_close(got.cpu().reshape(-1, 640), want, rtol=0, atol=atol)


# ---------------------------------------------------------------------------------- gated projection


def test_geglu_module_holds_the_transposed_weight():
    from basedxl_amd import BasedXLLowPGEGLU

    proj = torch.nn.Linear(64, 128)
    mod = BasedXLLowPGEGLU(proj)
    assert mod.inner == 64 and mod.weight.shape == (64, 128) and torch.equal(mod.weight, proj.weight.detach().T)
    with pytest.raises(ValueError):
        BasedXLLowPGEGLU(torch.nn.Linear(64, 127))


def _glu_variants():
    from basedxl_amd import _lib

    l = _lib.lib()
    return [i for i in range(l.cascmm_variant_count()) if l.cascmm_variant_name(i).decode().endswith("_tri_bpre")]


@pytest.mark.gpu
def test_gated_kernels_integer_exact_value_and_gate_pairing(gpu_device):
    """Small-integer operands: h is exact, so every kernel with the gated store must give
    value * gelu(gate) of the integer product up to the erf evaluation, on a shape with ragged row
    and column tiles; kernels without the gated store must refuse."""
    from basedxl_amd import PreparedWeight, _lib, cascaded_lowp_matmul

    g = torch.Generator().manual_seed(41)
    M, K, inner = 200, 128, 96
    a = torch.randint(-3, 4, (M, K), generator=g).float()
    w = torch.randint(-2, 3, (K, 2 * inner), generator=g).float()
    bias = torch.randint(-2, 3, (2 * inner,), generator=g).float()
    h = (a.long() @ w.long() + bias.long()).double()
    want = h[:, :inner] * torch.nn.functional.gelu(h[:, inner:])
    ran = 0
    for lowp, terms in (("bf16", 2), ("bf16", 3), ("fp16", 3), ("fp8", 3)):
        pw = PreparedWeight(w.to("cuda:0"), lowp=lowp, terms=terms, glu=True)
        for v in _glu_variants():
            name = _lib.lib().cascmm_variant_name(v).decode()
            if f"_{lowp}x{terms}_" not in name:
                continue
            try:
                y = cascaded_lowp_matmul(a.to("cuda:0"), pw, bias=bias.to("cuda:0"), variant=v)
            except RuntimeError as e:
                assert "variant" in str(e).lower(), (name, str(e))
                continue
            assert y.shape == (M, inner), name
            # fp32 gate: 1 + erf(g / sqrt 2) cancels for g << 0, an absolute error of about |value * g| * 2^-24
            torch.testing.assert_close(y.cpu().double(), want, rtol=1e-5, atol=2e-5, msg=lambda m: f"{name}: {m}")
            ran += 1
    assert ran >= 6


@pytest.mark.gpu
@pytest.mark.parametrize("with_bias", [True, False])
def test_large_tile_kernel_gated_store_raw_and_prepared_weight(gpu_device, with_bias):
    """The 256 x 320 kernel's gated store, on the raw weight (gate columns fetched from the second half)
    and on the prepared one (columns interleaved): small-integer operands make h exact, so both must
    give value * gelu(gate) of the integer product up to the erf evaluation, and the same bits as each
    other; 2 x 3 tiles, so every wave's pairs and the pair that crosses two waves land in two row tiles."""
    from basedxl_amd import PreparedWeight, _lib, cascaded_lowp_matmul
    from basedxl_amd.cascaded_lowp_matmul import cascaded_lowp_matmul_glu, gated_variant

    g = torch.Generator().manual_seed(43)
    M, K, inner = 512, 128, 480
    a = torch.randint(-3, 4, (M, K), generator=g).float()
    w = torch.randint(-2, 3, (K, 2 * inner), generator=g).float()
    bias = torch.randint(-2, 3, (2 * inner,), generator=g).float()
    h = (a.long() @ w.long() + (bias.long() if with_bias else 0)).double()
    want = h[:, :inner] * torch.nn.functional.gelu(h[:, inner:])
    ad, wd, bd = a.to("cuda:0"), w.to("cuda:0"), bias.to("cuda:0") if with_bias else None
    names = _lib.variant_names()
    # (the selection: the kernel where it fills the chip, the plain product plus a gate pass where it does not)
    big_a, big_w = torch.empty(2048, 1280, device="cuda:0"), torch.empty(1280, 10240, device="cuda:0")
    assert names[gated_variant(big_a, big_w)] == "t256x320x32_w512_bf16x2_tri"
    assert gated_variant(big_a[:1024], big_w) < 0 and gated_variant(ad, wd) < 0
    out = torch.full((M, inner + 8), -7.0, device="cuda:0")
    y = cascaded_lowp_matmul_glu(ad, wd, bias=bd, out=out[:, :inner])
    assert bool((out[:, inner:] == -7.0).all())                        # nothing written past the row
    torch.testing.assert_close(y.cpu().double(), want, rtol=1e-5, atol=2e-5)
    pw = PreparedWeight(wd, lowp="bf16", terms=2, glu=True)
    y2 = cascaded_lowp_matmul(ad, pw, bias=bd, variant=names.index("t256x320x32_w512_bf16x2_tri_bpre"))
    assert torch.equal(y2, y)
    # problems the kernel does not take are reported, not launched
    assert gated_variant(ad[:200], wd) < 0 and gated_variant(ad, wd[:, :704].contiguous()) < 0
    assert gated_variant(ad, wd, lowp="fp16", terms=3) < 0
    with pytest.raises(RuntimeError):
        cascaded_lowp_matmul_glu(ad[:200], wd)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,inner", [(2048, 1280, 5120), (8192, 640, 2560)])
def test_geglu_module_on_the_raw_weight_at_the_feed_forward_shape(gpu_device, M, K, inner):
    """`prepared=False`: no second copy of the weight; the feed-forward projections of the 32x32 and
    64x64 stages at full latent (2048 x 1280 x 10240: one tile per CU; 8192 x 640 x 5120: two) run the
    gate in the large-tile kernel's store.  Against the oracle's gated projection (1.25x bound) and
    against the plain product followed by torch's gate."""
    from basedxl_amd import BasedXLLowPGEGLU, BasedXLLowPLinear

    torch.manual_seed(44)
    proj = torch.nn.Linear(K, 2 * inner).to("cuda:0")
    with torch.no_grad():
        proj.weight.mul_(0.02 * K ** 0.5)
    x = torch.randn(2, M // 2, K, device="cuda:0")
    mod = BasedXLLowPGEGLU(proj, prepared=False)
    y = mod(x)
    assert y.shape == (2, M // 2, inner) and mod._prepared is None
    h = BasedXLLowPLinear(proj, prepared=False)(x)
    unfused = h[..., :inner] * torch.nn.functional.gelu(h[..., inner:])
    torch.testing.assert_close(y, unfused, rtol=2e-5, atol=2e-5)
    rows = torch.arange(0, M, 8)                                       # a row sample keeps the fp64 product short
    x2, wt, b = x.cpu().reshape(-1, K)[rows], proj.weight.detach().cpu().T.contiguous(), proj.bias.detach().cpu()
    want = oc.gated_projection_ref(x2, wt, b)
    h64 = oc.fp64_matmul(x2, wt) + b.double()
    exp = h64[:, :inner] * oc.gelu_erf(h64[:, inner:])
    got, ref = oc.error_metrics(y.cpu().reshape(-1, inner)[rows], exp), oc.error_metrics(want, exp)
    assert got["rel_fro"] <= 1.25 * ref["rel_fro"] and got["max_abs"] <= 1.25 * ref["max_abs"], (got, ref)
    # a shape the kernel does not take: the plain product and torch's gate, still without a prepared copy
    y3 = mod(x[:, :100])
    torch.testing.assert_close(y3, unfused[:, :100], rtol=2e-5, atol=2e-5)
    assert mod._prepared is None


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,inner", [(4096, 640, 2560), (1024, 1280, 5120), (77, 640, 2560)])
def test_geglu_module_matches_oracle_and_unfused_path(gpu_device, M, K, inner):
    from basedxl_amd import BasedXLLowPGEGLU, BasedXLLowPLinear

    torch.manual_seed(42)
    proj = torch.nn.Linear(K, 2 * inner).to("cuda:0")
    with torch.no_grad():
        proj.weight.mul_(0.02 * K ** 0.5)     # weights of std ~0.02 like the UNet's
    x = torch.randn(2, M // 2 if M % 2 == 0 else M, K, device="cuda:0")
    if M % 2:
        x = x[:1]
    y = BasedXLLowPGEGLU(proj)(x)
    assert y.shape == (*x.shape[:-1], inner)
    # same cascade through the plain prepared path, gate applied by torch: only the erf evaluation
    # and (when another tile is chosen) the accumulation order differ
    h = BasedXLLowPLinear(proj, prepared=True)(x)
    unfused = h[..., :inner] * torch.nn.functional.gelu(h[..., inner:])
    torch.testing.assert_close(y, unfused, rtol=2e-5, atol=2e-5)
    x2, wt, b = x.cpu().reshape(-1, K), proj.weight.detach().cpu().T.contiguous(), proj.bias.detach().cpu()
    want = oc.gated_projection_ref(x2, wt, b)
    h64 = oc.fp64_matmul(x2, wt) + b.double()
    exp = h64[:, :inner] * oc.gelu_erf(h64[:, inner:])
    got, ref = oc.error_metrics(y.cpu().reshape(-1, inner), exp), oc.error_metrics(want, exp)
    assert got["rel_fro"] <= 1.25 * ref["rel_fro"] and got["max_abs"] <= 1.25 * ref["max_abs"], (got, ref)


@pytest.mark.gpu
def test_geglu_module_falls_back_to_three_kernels(gpu_device):
    """Shapes the fused kernel does not take (inner not a multiple of 32) give the same function."""
    from basedxl_amd import BasedXLLowPGEGLU

    torch.manual_seed(43)
    proj = torch.nn.Linear(64, 2 * 40).to("cuda:0")
    x = torch.randn(50, 64, device="cuda:0")
    y = BasedXLLowPGEGLU(proj)(x)
    want = oc.gated_projection_ref(x.cpu(), proj.weight.detach().cpu().T.contiguous(), proj.bias.detach().cpu())
    torch.testing.assert_close(y.cpu(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_gate_function_against_double_precision(gpu_device):
    """The gate on its own: with A = I and value columns of ones, the kernel's output is
    gelu(w[r, inner + j]) for gates on a grid of 2^-6 steps over [-12, 12] (exact in two bf16
    terms).  Against 0.5 g erfc(-g / sqrt 2) in double precision: within one fp32 ulp of the gate
    (4e-7 + 2e-7 |g|), and with RELATIVE accuracy in the negative tail, where the textbook
    0.5 g (1 + erf) cancels."""
    import math

    from basedxl_amd import PreparedWeight, cascaded_lowp_matmul

    inner = 64
    gates = (torch.arange(64 * inner, dtype=torch.float64) * (1536.0 / (64 * inner - 1))).round() / 64.0 - 12.0
    w = torch.ones(64, 2 * inner)
    w[:, inner:] = gates.float().reshape(64, inner)
    y = cascaded_lowp_matmul(torch.eye(64, device="cuda:0"), PreparedWeight(w.to("cuda:0"), glu=True)).cpu().double()
    g = w[:, inner:].double()
    want = torch.tensor([0.5 * v * math.erfc(-v / math.sqrt(2.0)) for v in g.flatten().tolist()], dtype=torch.float64).reshape(64, inner)
    err = (y - want).abs()
    assert bool((err <= 4e-7 + 2e-7 * g.abs()).all()), float(err.max())
    neg = g < 0
    assert bool((err[neg] <= 1e-5 * want[neg].abs() + 5e-8).all()), float((err[neg] / want[neg].abs().clamp_min(1e-30)).max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,fmt,ulp", [(torch.float16, "fp16", 2.0 ** -10), (torch.bfloat16, "bf16", 2.0 ** -7)])
def test_geglu_module_sixteen_bit_tensors(gpu_device, dtype, fmt, ulp):
    """fp16 / bf16 tensors (what the reference runs its UNet in): the gate is applied in fp32 to the
    unrounded accumulators and the result rounded once, so it must sit within one unit in the last
    place of the oracle's fp32 result (the 16-bit operands as one exact term each)."""
    from basedxl_amd import BasedXLLowPGEGLU

    torch.manual_seed(44)
    M, K, inner = 384, 640, 1280
    proj = torch.nn.Linear(K, 2 * inner).to("cuda:0").to(dtype)
    x = torch.randn(M, K, device="cuda:0").to(dtype)
    mod = BasedXLLowPGEGLU(proj)
    y = mod(x)
    assert mod._prepared is not None and mod._prepared.glu        # the fused kernel ran, not the fallback
    assert y.dtype == dtype and y.shape == (M, inner)
    want = oc.gated_projection_ref(x.cpu().float(), proj.weight.detach().cpu().float().T.contiguous(),
                                   proj.bias.detach().cpu().float(), fmt, 1)
    err = (y.cpu().float() - want).abs()
    assert bool((err <= ulp * want.abs() + 1e-6).all()), float((err / want.abs().clamp_min(1e-6)).max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,fmt,ulp", [(torch.float16, "fp16", 2.0 ** -10), (torch.bfloat16, "bf16", 2.0 ** -7)])
def test_linear_wrapper_keeps_sixteen_bit_weights_prepared_by_default(gpu_device, dtype, fmt, ulp):
    """fp16 / bf16 modules (the dtype the reference runs in): the wrapper re-lays its weight once
    instead of in every call; fp32 modules split both operands in every call unless asked."""
    torch.manual_seed(45)
    lin = torch.nn.Linear(640, 320).to("cuda:0").to(dtype)
    mod = BasedXLLowPLinear(lin)
    assert mod.prepared and not BasedXLLowPLinear(torch.nn.Linear(64, 64)).prepared
    assert not BasedXLLowPLinear(lin, lowp="bf16", terms=2).prepared      # other cascades: raw weight
    x = torch.randn(2, 100, 640, device="cuda:0").to(dtype)
    y = mod(x)
    assert mod._prepared_weight is not None and y.dtype == dtype and y.shape == (2, 100, 320)
    want = oc.cascade_matmul_ref(x.cpu().float().reshape(-1, 640), lin.weight.detach().cpu().float().T.contiguous(), fmt, 1) \
        + lin.bias.detach().cpu().float()
    err = (y.cpu().float().reshape(-1, 320) - want).abs()
    assert bool((err <= ulp * want.abs() + 1e-3).all())
    assert torch.equal(BasedXLLowPLinear(lin, prepared=False)(x), y) or \
        bool(((BasedXLLowPLinear(lin, prepared=False)(x).float() - y.float()).abs() <= ulp * y.float().abs() + 1e-3).all())


# ---------------------------------------------------------------------------------- torch.compile


def test_custom_op_shapes_without_a_gpu():
    """The op's shape-only implementation, which is all a tracer runs (fake tensors: no data, no GPU)."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from basedxl_amd import compiled  # noqa: F401  (registers the op)

    with FakeTensorMode():
        x = torch.empty(2, 77, 640, device="cuda")
        w = torch.empty(640, 1280, device="cuda")
        assert torch.ops.basedxl_amd.cascade_linear(x, w, None, None, "bf16", 2, "tri", False, None).shape == (2, 77, 1280)
        assert torch.ops.basedxl_amd.cascade_linear(x, w, None, None, "bf16", 2, "tri", True, None).shape == (2, 77, 640)


class _FeedForward(torch.nn.Module):
    """The shape of a transformer block's feed-forward part: GEGLU projection, then the output Linear."""

    def __init__(self, d, dtype):
        super().__init__()
        self.proj = torch.nn.Linear(d, 8 * d, dtype=dtype)
        self.out = torch.nn.Linear(4 * d, d, dtype=dtype)

    def forward(self, x):
        return self.out(self.proj(x))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_patched_model_traces_under_torch_compile(gpu_device, dtype):
    """The reference compiles its UNet with fullgraph=True (unet.py:76-78): a model whose Linear
    layers were swapped must trace without a graph break and give the eager result.  (Backend
    "aot_eager": traces and functionalises like the default backend but generates no code.)"""
    from basedxl_amd import BasedXLLowPGEGLU, BasedXLLowPLinear

    torch.manual_seed(46)
    m = _FeedForward(128, dtype).to("cuda:0")
    m.proj = BasedXLLowPGEGLU(m.proj)
    m.out = BasedXLLowPLinear(m.out, prepared=True)
    x = torch.randn(2, 96, 128, device="cuda:0", dtype=dtype)
    with torch.no_grad():
        eager = m(x)                       # first eager call prepares the weights
        assert m.proj._prepared is not None and m.out._prepared_weight is not None
        compiled = torch.compile(m, backend="aot_eager", fullgraph=True)
        traced = compiled(x)
        assert torch.equal(traced, eager)
        assert torch.equal(compiled(x * 2), m(x * 2))
        # never run eagerly: prepare() does what the first eager call would have done
        m2 = _FeedForward(128, dtype).to("cuda:0")
        m2.proj, m2.out = BasedXLLowPGEGLU(m2.proj), BasedXLLowPLinear(m2.out, prepared=True)
        m2.proj.prepare()
        m2.out.prepare()
        assert torch.equal(torch.compile(m2, backend="aot_eager", fullgraph=True)(x), m2(x))


@pytest.mark.gpu
@pytest.mark.parametrize("channels_last", [False, True])
def test_pointwise_conv_traces_under_torch_compile(gpu_device, channels_last):
    torch.manual_seed(47)
    mod = BasedXLLowPConv1x1(torch.nn.Conv2d(64, 128, 1).to("cuda:0")).to("cuda:0")
    x = torch.randn(2, 64, 16, 8, device="cuda:0")
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    with torch.no_grad():
        eager = mod(x)
        traced = torch.compile(mod, backend="aot_eager", fullgraph=True)(x)
    torch.testing.assert_close(traced, eager, rtol=0, atol=2e-5)   # per-image launches may pick another tile than the grouped one
