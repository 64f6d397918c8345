"""An SDXL-UNet-shaped ``nn.Module`` tree with random weights, for running the patched Linear path
as one denoising step.

The reference patches a diffusers ``UNet2DConditionModel`` loaded by name (basedxl/model.py:17-23,
basedxl/unet.py:72-73,81-87).  diffusers and the checkpoint are not available offline, so this
module builds the same tree of layers itself (SDXL base: channels 320/640/1280, two resnets per
down block and three per up block, Transformer2D blocks of depth 2 at 640 channels and 10 at 1280,
heads of 64 channels, cross-attention width 2048, GEGLU feed-forward, 2816-wide added
conditioning) with the child names diffusers uses (``to_q``, ``to_k``, ``to_v``, ``to_out.0``,
``ff.net.0.proj``, ``ff.net.2``, ``proj_in``, ``proj_out``, ``time_emb_proj``, ``conv_shortcut``
...), so the patchers walk it exactly as they would walk the real model.  Everything that is not a
Linear layer or a 1x1 convolution (3x3 convolutions, normalisations, softmax attention, up- and
down-sampling) runs in plain torch: those layers are not on the path this package accelerates.

``latent_rows`` lets a forward pass run on one GPU's share of a patch-parallel split (the latent
split along H, basedxl/unet.py:140-176): the model simply sees a shorter image.
"""
from __future__ import annotations

import math
from collections import OrderedDict
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .modules.fused_kv import BasedXLFusedKV, BasedXLFusedQKV
from .modules.geglu import BasedXLLowPGEGLU

W_STD = 0.02   # every weight ~ N(0, 0.02); biases zero-mean with the same spread


class GEGLU(nn.Module):
    def __init__(self, dim: int, inner: int):
        super().__init__()
        self.proj = nn.Linear(dim, 2 * inner)

    def forward(self, x):
        value, gate = self.proj(x).chunk(2, dim=-1)
        return value * F.gelu(gate)


class FeedForward(nn.Module):
    def __init__(self, dim: int, mult: int = 4):
        super().__init__()
        self.net = nn.ModuleList([GEGLU(dim, dim * mult), nn.Dropout(0.0), nn.Linear(dim * mult, dim)])

    def forward(self, x):
        for m in self.net:
            x = m(x)
        return x


class Attention(nn.Module):
    """Multi-head attention with separate to_q / to_k / to_v Linear layers (no bias) and an output
    Linear; after :func:`fuse_kv_projections` the key and value come from one ``to_kv`` module, or
    (self-attention, ``fuse_q``) query, key and value from one ``to_qkv`` module."""

    #: this forward knows ``to_kv`` / ``to_qkv``: the mark :func:`fuse_kv_projections` looks for
    consumes_fused_projections = True

    def __init__(self, query_dim: int, cross_dim: Optional[int], heads: int):
        super().__init__()
        self.heads = heads
        self.is_cross = cross_dim is not None
        kv_dim = cross_dim if cross_dim is not None else query_dim
        self.to_q = nn.Linear(query_dim, query_dim, bias=False)
        self.to_k = nn.Linear(kv_dim, query_dim, bias=False)
        self.to_v = nn.Linear(kv_dim, query_dim, bias=False)
        self.to_out = nn.ModuleList([nn.Linear(query_dim, query_dim), nn.Dropout(0.0)])

    def forward(self, x, context=None):
        src = x if context is None else context
        if hasattr(self, "to_qkv"):
            q, k, v = self.to_qkv(x)
        else:
            q = self.to_q(x)
            if hasattr(self, "to_kv"):
                k, v = self.to_kv(src)
            else:
                k, v = self.to_k(src), self.to_v(src)
        B, T, C = q.shape
        h = self.heads

        def heads(t):
            return t.reshape(B, -1, h, C // h).transpose(1, 2)

        o = F.scaled_dot_product_attention(heads(q), heads(k), heads(v))
        o = o.transpose(1, 2).reshape(B, T, C)
        return self.to_out[1](self.to_out[0](o))


class BasicTransformerBlock(nn.Module):
    def __init__(self, dim: int, heads: int, cross_dim: int):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn1 = Attention(dim, None, heads)
        self.norm2 = nn.LayerNorm(dim)
        self.attn2 = Attention(dim, cross_dim, heads)
        self.norm3 = nn.LayerNorm(dim)
        self.ff = FeedForward(dim)

    def forward(self, x, context):
        x = x + self.attn1(self.norm1(x))
        x = x + self.attn2(self.norm2(x), context)
        return x + self.ff(self.norm3(x))


class Transformer2DModel(nn.Module):
    """GroupNorm, Linear proj_in over tokens (``use_linear_projection``), ``depth`` transformer
    blocks, Linear proj_out, residual."""

    def __init__(self, channels: int, heads: int, depth: int, cross_dim: int):
        super().__init__()
        self.norm = nn.GroupNorm(32, channels, eps=1e-6)
        self.proj_in = nn.Linear(channels, channels)
        self.transformer_blocks = nn.ModuleList([BasicTransformerBlock(channels, heads, cross_dim) for _ in range(depth)])
        self.proj_out = nn.Linear(channels, channels)

    def forward(self, x, context):
        B, C, H, W = x.shape
        t = self.norm(x).permute(0, 2, 3, 1).reshape(B, H * W, C)
        t = self.proj_in(t)
        for blk in self.transformer_blocks:
            t = blk(t, context)
        t = self.proj_out(t)
        return t.reshape(B, H, W, C).permute(0, 3, 1, 2) + x


class ResnetBlock2D(nn.Module):
    def __init__(self, cin: int, cout: int, temb: int):
        super().__init__()
        self.norm1 = nn.GroupNorm(32, cin, eps=1e-5)
        self.conv1 = nn.Conv2d(cin, cout, 3, padding=1)
        self.time_emb_proj = nn.Linear(temb, cout)
        self.norm2 = nn.GroupNorm(32, cout, eps=1e-5)
        self.conv2 = nn.Conv2d(cout, cout, 3, padding=1)
        self.conv_shortcut = nn.Conv2d(cin, cout, 1) if cin != cout else None

    def forward(self, x, emb):
        h = self.conv1(F.silu(self.norm1(x)))
        h = h + self.time_emb_proj(F.silu(emb))[:, :, None, None]
        h = self.conv2(F.silu(self.norm2(h)))
        return (x if self.conv_shortcut is None else self.conv_shortcut(x)) + h


class Downsample2D(nn.Module):
    def __init__(self, c: int):
        super().__init__()
        self.conv = nn.Conv2d(c, c, 3, stride=2, padding=1)

    def forward(self, x):
        return self.conv(x)


class Upsample2D(nn.Module):
    def __init__(self, c: int):
        super().__init__()
        self.conv = nn.Conv2d(c, c, 3, padding=1)

    def forward(self, x):
        return self.conv(F.interpolate(x, scale_factor=2.0, mode="nearest"))


class _Block(nn.Module):
    """A down / mid / up block: resnets, optionally each followed by a Transformer2D."""

    def __init__(self, resnets, attentions, sampler):
        super().__init__()
        self.resnets = nn.ModuleList(resnets)
        self.attentions = nn.ModuleList(attentions) if attentions else None
        if sampler is not None:
            name = "downsamplers" if isinstance(sampler, Downsample2D) else "upsamplers"
            setattr(self, name, nn.ModuleList([sampler]))

    def sampler(self):
        for name in ("downsamplers", "upsamplers"):
            if hasattr(self, name):
                return getattr(self, name)[0]
        return None


class TimestepEmbedding(nn.Module):
    def __init__(self, cin: int, dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(cin, dim)
        self.linear_2 = nn.Linear(dim, dim)

    def forward(self, x):
        return self.linear_2(F.silu(self.linear_1(x)))


def sinusoidal(t: torch.Tensor, dim: int) -> torch.Tensor:
    """[n] -> [n, dim] sinusoidal features (cos first: ``flip_sin_to_cos``, no frequency shift)."""
    half = dim // 2
    freqs = torch.exp(-math.log(10000.0) * torch.arange(half, dtype=torch.float32, device=t.device) / half)
    ang = t.float()[:, None] * freqs[None]
    return torch.cat([ang.cos(), ang.sin()], dim=-1)


class SDXLUNetSkeleton(nn.Module):
    """``forward(sample [B, 4, H, W], timestep, encoder_hidden_states [B, 77, 2048], added_cond_kwargs)``
    like the model the reference wraps (basedxl/unet.py:120-139).  The defaults are SDXL base; tests
    build small models by passing fewer channels (multiples of 32), a smaller head and shallower
    transformers."""

    def __init__(self, *, channels: Tuple[int, int, int] = (320, 640, 1280), head_dim: int = 64,
                 depths: Tuple[int, int] = (2, 10), cross_dim: int = 2048, add_time_dim: int = 256, seed: int = 0,
                 device=None):
        super().__init__()
        with torch.device(device if device is not None else "cpu"):   # build (and initialise) on the target device
            self._build(channels, head_dim, depths, cross_dim, add_time_dim)
        self.reset_parameters(seed)

    def _build(self, channels, head_dim, depths, cross_dim, add_time_dim):
        c = list(channels)
        temb = c[2]
        self.channels, self.cross_dim = c, cross_dim
        self.time_dim, self.add_time_dim = c[0], add_time_dim
        self.text_embed_dim = c[2]
        head = head_dim
        self.conv_in = nn.Conv2d(4, c[0], 3, padding=1)
        self.time_embedding = TimestepEmbedding(self.time_dim, temb)
        self.add_embedding = TimestepEmbedding(self.text_embed_dim + 6 * self.add_time_dim, temb)

        def t2d(ch, depth):
            return Transformer2DModel(ch, ch // head, depth, cross_dim)

        self.down_blocks = nn.ModuleList([
            _Block([ResnetBlock2D(c[0], c[0], temb), ResnetBlock2D(c[0], c[0], temb)], None, Downsample2D(c[0])),
            _Block([ResnetBlock2D(c[0], c[1], temb), ResnetBlock2D(c[1], c[1], temb)],
                   [t2d(c[1], depths[0]) for _ in range(2)], Downsample2D(c[1])),
            _Block([ResnetBlock2D(c[1], c[2], temb), ResnetBlock2D(c[2], c[2], temb)],
                   [t2d(c[2], depths[1]) for _ in range(2)], None),
        ])
        self.mid_block = _Block([ResnetBlock2D(c[2], c[2], temb), ResnetBlock2D(c[2], c[2], temb)], [t2d(c[2], depths[1])], None)
        self.up_blocks = nn.ModuleList([
            _Block([ResnetBlock2D(c[2] + c[2], c[2], temb), ResnetBlock2D(c[2] + c[2], c[2], temb), ResnetBlock2D(c[2] + c[1], c[2], temb)],
                   [t2d(c[2], depths[1]) for _ in range(3)], Upsample2D(c[2])),
            _Block([ResnetBlock2D(c[2] + c[1], c[1], temb), ResnetBlock2D(c[1] + c[1], c[1], temb), ResnetBlock2D(c[1] + c[0], c[1], temb)],
                   [t2d(c[1], depths[0]) for _ in range(3)], Upsample2D(c[1])),
            _Block([ResnetBlock2D(c[1] + c[0], c[0], temb), ResnetBlock2D(c[0] + c[0], c[0], temb), ResnetBlock2D(c[0] + c[0], c[0], temb)],
                   None, None),
        ])
        self.conv_norm_out = nn.GroupNorm(32, c[0], eps=1e-5)
        self.conv_out = nn.Conv2d(c[0], 4, 3, padding=1)

    @torch.no_grad()
    def reset_parameters(self, seed: int) -> None:
        """Weights and biases of every Linear and convolution ~ N(0, 0.02) from one seeded generator
        on the model's device (normalisation layers keep weight 1, bias 0)."""
        dev = self.conv_in.weight.device
        if dev.type == "meta":   # structure only (shape bookkeeping without memory)
            return
        g = torch.Generator(device=dev).manual_seed(seed)
        for m in self.modules():
            if isinstance(m, (nn.Linear, nn.Conv2d)):
                m.weight.normal_(0.0, W_STD, generator=g)
                if m.bias is not None:
                    m.bias.normal_(0.0, W_STD, generator=g)

    def forward(self, sample, timestep, encoder_hidden_states, added_cond_kwargs: Dict[str, torch.Tensor]):
        B = sample.shape[0]
        t = torch.as_tensor(timestep, device=sample.device).reshape(-1).expand(B)
        emb = self.time_embedding(sinusoidal(t, self.time_dim).to(sample.dtype))
        ids = sinusoidal(added_cond_kwargs["time_ids"].reshape(-1), self.add_time_dim).reshape(B, -1).to(sample.dtype)
        emb = emb + self.add_embedding(torch.cat([added_cond_kwargs["text_embeds"], ids], dim=-1))
        ctx = encoder_hidden_states

        x = self.conv_in(sample)
        skips = [x]
        for blk in self.down_blocks:
            for i, res in enumerate(blk.resnets):
                x = res(x, emb)
                if blk.attentions is not None:
                    x = blk.attentions[i](x, ctx)
                skips.append(x)
            if blk.sampler() is not None:
                x = blk.sampler()(x)
                skips.append(x)
        x = self.mid_block.resnets[0](x, emb)
        x = self.mid_block.attentions[0](x, ctx)
        x = self.mid_block.resnets[1](x, emb)
        for blk in self.up_blocks:
            for i, res in enumerate(blk.resnets):
                x = res(torch.cat([x, skips.pop()], dim=1), emb)
                if blk.attentions is not None:
                    x = blk.attentions[i](x, ctx)
            if blk.sampler() is not None:
                x = blk.sampler()(x)
        return self.conv_out(F.silu(self.conv_norm_out(x)))


def synthetic_inputs(model: SDXLUNetSkeleton, *, batch: int = 2, latent: int = 128, latent_rows: Optional[int] = None,
                     text_tokens: int = 77, seed: int = 1, device="cpu", dtype=torch.float32):
    """Seeded inputs of one denoising step: latent ~ N(0,1) [batch, 4, rows, latent], text context
    ~ N(0,1) [batch, text_tokens, cross_dim], pooled text embedding and the six SDXL size ids.
    ``latent_rows`` < latent: one GPU's share of a split along H."""
    g = torch.Generator().manual_seed(seed)
    rows = latent if latent_rows is None else latent_rows
    sample = torch.randn(batch, 4, rows, latent, generator=g)
    ctx = torch.randn(batch, text_tokens, model.cross_dim, generator=g)
    added = {"text_embeds": torch.randn(batch, model.text_embed_dim, generator=g),
             "time_ids": torch.tensor([[1024.0, 1024.0, 0.0, 0.0, 1024.0, 1024.0]] * batch)}
    mv = lambda t: t.to(device=device, dtype=dtype)   # noqa: E731
    return mv(sample), torch.tensor(500.0, device=device), mv(ctx), {k: mv(v) for k, v in added.items()}


# ---------------------------------------------------------------------------------------------
# patchers beyond the reference's Linear walk, and the record of what a forward pass routes
# ---------------------------------------------------------------------------------------------
def fuse_kv_projections(model: nn.Module, *, cache_cross: bool = False, fuse_q: bool = False, **cascade_kwargs) -> nn.Module:
    """Every attention module with ``to_k`` / ``to_v`` Linear children WHOSE FORWARD IS KNOWN TO READ
    THE FUSED MODULES (class attribute ``consumes_fused_projections``, as :class:`Attention` here has)
    gets one ``to_kv`` (:class:`BasedXLFusedKV`) instead, as basedxl/modules/attn.py:16-39 does by
    wrapping the attention module in one of its own.  Any other attention module (a diffusers
    ``Attention``, whose processor calls ``attn.to_k`` / ``attn.to_v``) keeps its three Linear children
    for the plain walk of patch_linear_layers: removing them would break its forward.  With ``cache_cross``
    the cross-attention modules (``is_cross``) keep their result like attn.py:57,74-78.  With
    ``fuse_q`` the self-attention modules (not ``is_cross``: query, key and value read the same tokens)
    get one ``to_qkv`` (:class:`BasedXLFusedQKV`) for all three.  Call it BEFORE patch_linear_layers
    (it takes the plain Linear layers)."""
    for module in list(model.modules()):
        to_q, to_k, to_v = getattr(module, "to_q", None), getattr(module, "to_k", None), getattr(module, "to_v", None)
        if not (isinstance(to_k, nn.Linear) and isinstance(to_v, nn.Linear)):
            continue
        if not getattr(module, "consumes_fused_projections", False):
            continue
        is_cross = bool(getattr(module, "is_cross", False))
        if (fuse_q and not is_cross and hasattr(module, "is_cross") and isinstance(to_q, nn.Linear)
                and to_q.in_features == to_k.in_features):
            module.to_qkv = BasedXLFusedQKV(to_q, to_k, to_v, **cascade_kwargs)
            del module.to_q, module.to_k, module.to_v
        else:
            module.to_kv = BasedXLFusedKV(to_k, to_v, cache=cache_cross and is_cross, **cascade_kwargs)
            del module.to_k, module.to_v
    return model


def fuse_geglu_layers(model: nn.Module, **cascade_kwargs) -> nn.Module:
    """Every GEGLU child (a module named GEGLU whose ``proj`` is still a plain Linear) is replaced by
    :class:`BasedXLLowPGEGLU`, which applies the gate in the GEMM's store.  Call it BEFORE
    patch_linear_layers."""
    for module in list(model.modules()):
        for name, child in list(module.named_children()):
            if type(child).__name__ == "GEGLU" and isinstance(getattr(child, "proj", None), nn.Linear):
                setattr(module, name, BasedXLLowPGEGLU(child.proj, **cascade_kwargs))
    return model


ROUTED_TYPES = ("BasedXLLowPLinear", "BasedXLLowPConv1x1", "BasedXLLowPGEGLU")


def is_routed(m: nn.Module) -> bool:
    return type(m).__name__ in ROUTED_TYPES


def routed_calls(model: nn.Module, *inputs) -> List[dict]:
    """Runs ``model(*inputs)`` once and returns, in call order, one record per call of a module that
    goes through the cascade GEMM: qualified name, module, input shape and the GEMM it is (M, K, N)."""
    calls: List[dict] = []
    hooks = []
    for name, m in model.named_modules():
        chained = type(m).__name__ == "BasedXLChainedFeedForward"
        if not is_routed(m) and not chained:
            continue

        def hook(mod, args, name=name):
            x = args[0]
            if type(mod).__name__ == "BasedXLChainedFeedForward":
                # a feed-forward block that runs as a chain is ONE record of two GEMMs (M x in x 2 inner, then
                # M x inner x out); where it falls back, its two inner modules are called and record themselves
                if not mod._chain_ok(x):
                    return
                M, K, N = x.numel() // x.shape[-1], mod.in_features, 2 * mod.inner
                calls.append({"name": name, "module": mod, "input_shape": tuple(x.shape), "M": M, "K": K, "N": N,
                              "extra_flops": 2.0 * M * mod.inner * mod.out_features})
                return
            if type(mod).__name__ == "BasedXLLowPConv1x1":
                M, K, N = x.shape[0] * x.shape[2] * x.shape[3], mod.in_channels, mod.out_channels
            elif type(mod).__name__ == "BasedXLLowPGEGLU":
                M, K, N = x.numel() // x.shape[-1], mod.in_features, 2 * mod.inner
            else:
                M, K, N = x.numel() // x.shape[-1], mod.in_features, mod.out_features
            calls.append({"name": name, "module": mod, "input_shape": tuple(x.shape), "M": M, "K": K, "N": N})

        hooks.append(m.register_forward_pre_hook(hook))
    try:
        with torch.no_grad():
            model(*inputs)
    finally:
        for h in hooks:
            h.remove()
    return calls


def distinct_shapes(calls: List[dict]) -> "OrderedDict[Tuple[str, int, int, int], dict]":
    """The calls grouped by (module type, M, K, N): first call of each, with its count."""
    out: "OrderedDict[Tuple[str, int, int, int], dict]" = OrderedDict()
    for c in calls:
        key = (type(c["module"]).__name__, c["M"], c["K"], c["N"])
        if key not in out:
            out[key] = dict(c, count=0)
        out[key]["count"] += 1
    return out
