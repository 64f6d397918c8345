"""The gated feed-forward projection of the UNet's transformer blocks in one kernel.

diffusers' ``GEGLU`` module (third-party, not part of the reference tree; its ``proj`` is one of
the ``nn.Linear`` layers the reference routes, basedxl/unet.py:81-87) computes
``h = proj(x); value, gate = h.chunk(2, dim=-1); return value * gelu(gate)``.  Routed through
:class:`BasedXLLowPLinear` that is a GEMM that writes ``h`` plus two elementwise kernels that read
it again; here the gate is applied in the GEMM's store and ``h`` never reaches memory.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..cascaded_lowp_matmul import PreparedWeight, cascaded_lowp_matmul, cascaded_lowp_matmul_glu, default_cascade, gated_variant


class BasedXLLowPGEGLU(nn.Module):
    """Wraps the ``proj`` Linear ([in] -> [2 * inner]) of a GEGLU block; ``forward(x)`` returns
    ``value * gelu(gate)`` ([..., inner]), gelu in its exact (erf) form.

    The fused kernels take fp32 activations (any cascade) or fp16 / bf16 activations (as one term of
    their own format) on the GPU with ``in % 64 == 0`` and ``inner % 32 == 0`` and read a prepared
    (pre-split, column-interleaved) copy of the weight, made on first use.  ``prepared=False`` keeps
    no such copy: the large-tile kernel applies the gate on the raw weight where it takes the problem
    (fp32, two bf16 terms, rows % 256 == 0, inner % 160 == 0).  Anything else runs the cascade GEMM on the
    raw weight followed by torch's gate (the same arithmetic in three kernels)."""

    def __init__(self, proj: nn.Linear, *, lowp: Optional[str] = None, terms: Optional[int] = None,
                 products: str = "tri", prepared: Optional[bool] = None):
        super().__init__()
        if proj.out_features % 2 != 0:
            raise ValueError("a gated projection has an even number of output features")
        self.in_features, self.inner = proj.in_features, proj.out_features // 2
        self.weight = proj.weight.detach().T.contiguous().clone()          # [in, 2 * inner], like lowp_linear.py:12
        self.bias = proj.bias.detach().clone() if proj.bias is not None else None
        d_lowp, d_terms = default_cascade(self.weight.dtype)
        self.lowp, self.terms, self.products = d_lowp if lowp is None else lowp, d_terms if terms is None else terms, products
        self.prepared = True if prepared is None else bool(prepared)
        self._prepared: Optional[PreparedWeight] = None

    def _fusable(self, x: torch.Tensor) -> bool:
        if not x.is_cuda or x.dtype != self.weight.dtype or self.in_features % 64 != 0 or self.inner % 32 != 0:
            return False
        # 16-bit tensors have prepared kernels only for one term of their own format
        return x.dtype == torch.float32 or (self.lowp, self.terms) == default_cascade(x.dtype)

    def prepare(self) -> None:
        """Prepare the gated weight now (needs the weight on the GPU); otherwise on the first eager call."""
        if self.prepared and self.weight.is_cuda and self.in_features % 64 == 0 and self.inner % 32 == 0 and (
                self._prepared is None or self._prepared.device != self.weight.device):
            self._prepared = PreparedWeight(self.weight, lowp=self.lowp, terms=self.terms, glu=True)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if torch.compiler.is_compiling() and self._prepared is not None and x.dtype == self.weight.dtype:
            from ..compiled import cascade_linear
            return cascade_linear(x, self.weight, self._prepared.slots, self.bias, self.lowp, self.terms, self.products,
                                  True, self._prepared.exp)
        if torch.compiler.is_compiling():
            from ..compiled import cascade_linear
            h = cascade_linear(x, self.weight, None, self.bias, self.lowp, self.terms, self.products, False, None)
            value, gate = h.chunk(2, dim=-1)
            return value * F.gelu(gate)
        if not self.prepared and x.is_cuda and x.dtype == self.weight.dtype and gated_variant(
                x, self.weight, lowp=self.lowp, terms=self.terms, products=self.products) >= 0:
            return cascaded_lowp_matmul_glu(x, self.weight, bias=self.bias, lowp=self.lowp, terms=self.terms, products=self.products)
        if self.prepared and self._fusable(x):
            if self._prepared is None or self._prepared.device != self.weight.device:
                self._prepared = PreparedWeight(self.weight, lowp=self.lowp, terms=self.terms, glu=True)
            x2 = x.reshape(-1, self.in_features)
            if self._prepared.usable_with(x2 if x2.stride(-1) == 1 else x2.contiguous(), self.products):
                return cascaded_lowp_matmul(x, self._prepared, bias=self.bias, products=self.products)
        h = cascaded_lowp_matmul(x, self.weight, bias=self.bias, lowp=self.lowp, terms=self.terms, products=self.products)
        value, gate = h.chunk(2, dim=-1)
        return value * F.gelu(gate)
