"""The two Linear layers of a transformer block's feed-forward as one chain of two kernels.

diffusers' ``FeedForward`` (third-party; its ``net`` holds a ``GEGLU`` whose ``proj`` and a final
``nn.Linear`` that are two of the layers the reference routes, basedxl/unet.py:81-87, each through
basedxl/modules/lowp_linear.py:15-20) runs ``net[0]`` (projection + gate), a dropout and ``net[2]``.
Routed layer by layer, the gated activations are written as fp32, read back and split again by the
second GEMM.  Here the first GEMM's gated store writes them directly as the operand slots of the
second, which then multiplies slots by slots: no split, no second kernel for its K split.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ..cascaded_lowp_matmul import (ChainedWeight, PreparedWeight, cascaded_lowp_matmul_chained, cascaded_lowp_matmul_glu_chained,
                                    chained_supported, glu_chained_worthwhile)
from .geglu import BasedXLLowPGEGLU
from .lowp_linear import BasedXLLowPLinear


class BasedXLChainedFeedForward(nn.Module):
    """``out(value * gelu(gate))`` with ``value, gate = proj(x).chunk(2, -1)``: ``proj`` ([in] -> [2 inner])
    and ``out`` ([inner] -> [out]) are the two ``nn.Linear`` layers of the block.

    The chain runs for fp32 activations on the GPU, two bf16 terms, rows % 256 == 0, inner % 160 == 0,
    in % 32 == 0, and where the library's estimates favour the large-tile kernel with the gate in its store
    over a plain kernel plus a gate pass (few rows on many CUs: they do not); anything else goes through :class:`BasedXLLowPGEGLU` and :class:`BasedXLLowPLinear`,
    which this module also holds (same weights).  ``prepared=True`` keeps the first weight split as
    well (the second one always is: the chained GEMM has no other form)."""

    def __init__(self, proj: nn.Linear, out: nn.Linear, *, lowp: Optional[str] = None, terms: Optional[int] = None,
                 products: str = "tri", prepared: Optional[bool] = None):
        super().__init__()
        self.geglu = BasedXLLowPGEGLU(proj, lowp=lowp, terms=terms, products=products, prepared=bool(prepared))
        self.linear = BasedXLLowPLinear(out, lowp=lowp, terms=terms, products=products, prepared=prepared)
        self.in_features, self.inner, self.out_features = proj.in_features, proj.out_features // 2, out.out_features
        self.chainable = (self.geglu.lowp, self.geglu.terms, self.geglu.products) == ("bf16", 2, "tri") and \
            self.geglu.weight.dtype == torch.float32
        self.prepared = bool(prepared)
        self._chained_weight: Optional[ChainedWeight] = None
        self.chained_calls = 0     # how many forward passes took the chain (for tests and the bench's record)

    def _chain_ok(self, x: torch.Tensor) -> bool:
        if not (self.chainable and x.is_cuda and x.dtype == torch.float32) or torch.compiler.is_compiling():
            return False
        M = x.numel() // self.in_features
        return glu_chained_worthwhile(x, 2 * self.inner) and chained_supported(M, self.out_features, self.inner)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not self._chain_ok(x):
            return self.linear(self.geglu(x))
        dev = self.linear.weight.device
        if self._chained_weight is None or self._chained_weight.device != dev:
            self._chained_weight = ChainedWeight(self.linear.weight)
        w1 = self.geglu.weight
        if self.prepared:
            if self.geglu._prepared is None or self.geglu._prepared.device != w1.device:
                self.geglu._prepared = PreparedWeight(w1, lowp="bf16", terms=2, glu=True)
            w1 = self.geglu._prepared
        slots = cascaded_lowp_matmul_glu_chained(x, w1, bias=self.geglu.bias)
        self.chained_calls += 1
        return cascaded_lowp_matmul_chained(slots, self._chained_weight, bias=self.linear.bias)


def chain_feed_forward_layers(model: nn.Module, **cascade_kwargs) -> nn.Module:
    """Every feed-forward block whose ``net`` is ``[GEGLU(proj: nn.Linear), Dropout, nn.Linear]`` (diffusers'
    layout; the dropout inactive) gets ``net = [BasedXLChainedFeedForward, Identity, Identity]``: a forward
    that walks ``net`` in order, as diffusers' does, is unchanged.  Call it BEFORE the GEGLU fusion and
    patch_linear_layers (it takes the plain Linear layers)."""
    for module in list(model.modules()):
        net = getattr(module, "net", None)
        if not isinstance(net, (nn.ModuleList, nn.Sequential)) or len(net) != 3:
            continue
        g, d, o = net[0], net[1], net[2]
        if type(g).__name__ != "GEGLU" or not isinstance(getattr(g, "proj", None), nn.Linear) or not isinstance(o, nn.Linear):
            continue
        if not isinstance(d, nn.Dropout) or (d.p > 0 and d.training):
            continue
        if g.proj.out_features != 2 * o.in_features:
            continue
        net[0] = BasedXLChainedFeedForward(g.proj, o, **cascade_kwargs)
        net[1] = nn.Identity()
        net[2] = nn.Identity()
    return model
