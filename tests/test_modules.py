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
