"""Drop-in for the reference's BasedXLLowPLinear (basedxl/modules/lowp_linear.py:7-20)."""
from __future__ import annotations

import torch
import torch.nn as nn

from typing import Optional

from ..cascaded_lowp_matmul import PreparedWeight, cascaded_lowp_matmul, default_cascade, tensor_scale_exp


class BasedXLLowPLinear(nn.Module):
    """Wraps an ``nn.Linear``: the weight is stored transposed as ``[in, out]``
    (lowp_linear.py:12) and the forward pass is one cascade GEMM with the bias add fused
    into its store (the reference adds it in a second kernel, lowp_linear.py:17-19)."""

    def __init__(self, submodule: nn.Linear, *, lowp: Optional[str] = None, terms: Optional[int] = None,
                 products: str = "tri", prepared: Optional[bool] = None):
        super().__init__()
        self.in_features = submodule.in_features
        self.out_features = submodule.out_features
        self.weight = submodule.weight.detach().T.contiguous().clone()
        self.bias = submodule.bias.detach().clone() if submodule.bias is not None else None
        d_lowp, d_terms = default_cascade(self.weight.dtype)   # fp32: bf16 x 2; fp16 / bf16: their own format x 1
        self.lowp, self.terms, self.products = d_lowp if lowp is None else lowp, d_terms if terms is None else terms, products
        self._weight_exp = None   # fp8: tensor-scale exponent of the weight, found on first use
        # prepared=True: the weight is also kept split (once, on first use on the GPU); inputs
        # the prepared kernels do not take (K not a multiple of 64, ...) use the raw weight.
        # Default: on for fp16 / bf16 weights multiplied as one term of their own format (there
        # "prepared" is only a re-layout of the weight, which the raw path would redo in every
        # call), off for fp32 weights (both operands are then split inside every GEMM)
        if prepared is None:
            prepared = self.weight.dtype != torch.float32 and (self.lowp, self.terms) == (d_lowp, d_terms)
        self.prepared = prepared
        self._prepared_weight = None

    def prepare(self) -> None:
        """Split / re-lay the weight now (needs the weight on the GPU); otherwise it happens on the
        first eager call.  A model that is compiled before it ever ran eagerly should call this."""
        if self.prepared and self.weight.is_cuda and (self._prepared_weight is None
                                                      or self._prepared_weight.device != self.weight.device):
            self._prepared_weight = PreparedWeight(self.weight, lowp=self.lowp, terms=self.terms)
        if self.lowp == "fp8" and self.weight.is_cuda and (self._weight_exp is None or self._weight_exp.device != self.weight.device):
            self._weight_exp = tensor_scale_exp(self.weight)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if torch.compiler.is_compiling():
            # traced by torch.compile: one opaque op (whatever was prepared before tracing is used)
            from ..compiled import cascade_linear
            pw = self._prepared_weight
            return cascade_linear(x, self.weight, None if pw is None else pw.slots, self.bias, self.lowp, self.terms,
                                  self.products, False, self._weight_exp if pw is None else pw.exp)
        if self.prepared and x.is_cuda:
            if self._prepared_weight is None or self._prepared_weight.device != self.weight.device:
                self._prepared_weight = PreparedWeight(self.weight, lowp=self.lowp, terms=self.terms)
            x2 = x.reshape(-1, self.in_features)
            # a handful of rows (time embeddings): the raw fp32 weight has split-K kernels that stream
            # it with every CU, the prepared path has none
            few_rows = x2.shape[0] < 32 and x2.dtype == torch.float32
            if not few_rows and self._prepared_weight.usable_with(x2 if x2.stride(-1) == 1 else x2.contiguous(), self.products):
                return cascaded_lowp_matmul(x, self._prepared_weight, bias=self.bias, products=self.products)
        if self.lowp == "fp8" and (self._weight_exp is None or self._weight_exp.device != self.weight.device):
            self._weight_exp = tensor_scale_exp(self.weight)
        return cascaded_lowp_matmul(x, self.weight, bias=self.bias, lowp=self.lowp, terms=self.terms,
                                    products=self.products, b_exp=self._weight_exp)


def patch_linear_layers(model: nn.Module, **cascade_kwargs) -> nn.Module:
    """Replace every ``nn.Linear`` child with :class:`BasedXLLowPLinear`
    (same walk as basedxl/unet.py:81-87)."""
    for _name, module in model.named_modules():
        for subname, submodule in module.named_children():
            if isinstance(submodule, nn.Linear):
                setattr(module, subname, BasedXLLowPLinear(submodule, **cascade_kwargs))
    return model
