"""1x1 convolutions as cascade GEMMs.

The reference swaps only ``nn.Linear`` children (basedxl/unet.py:81-87) and leaves 1x1
convolutions to cuDNN (its patch-parallel Conv2d skips them too, unet.py:98-99).  A 1x1
convolution is a GEMM over channels, so it can take the same cascade.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ..cascaded_lowp_matmul import cascaded_lowp_matmul, cascaded_lowp_matmul_grouped, default_cascade, tensor_scale_exp

MAX_GROUP = 8   # problems one grouped launch takes


def is_pointwise(conv: nn.Module) -> bool:
    """A Conv2d that is a plain GEMM over channels: 1x1, stride 1, no padding / dilation / groups."""
    return (isinstance(conv, nn.Conv2d) and tuple(conv.kernel_size) == (1, 1) and tuple(conv.stride) == (1, 1)
            and conv.padding in ((0, 0), 0, "valid") and tuple(conv.dilation) == (1, 1) and conv.groups == 1
            and conv.padding_mode == "zeros")


class BasedXLLowPConv1x1(nn.Module):
    """Wraps a 1x1 ``nn.Conv2d``.  Two layouts, no copy of the activations in either:

    * channels-last input (``[B, H, W, C]`` in memory): ``[B*H*W, C_in] x [C_in, C_out]`` with the
      bias fused into the store, result channels-last;
    * NCHW-contiguous input: per image ``[C_out, C_in] x [C_in, H*W]`` (the image is already the
      row-major right-hand operand), all images of the batch in one grouped launch; the bias
      runs along rows there and is added afterwards.
    """

    def __init__(self, conv: nn.Conv2d, *, lowp: Optional[str] = None, terms: Optional[int] = None,
                 products: str = "tri"):
        super().__init__()
        if not is_pointwise(conv):
            raise ValueError("BasedXLLowPConv1x1 takes 1x1 convolutions with stride 1 and no padding, dilation or groups")
        self.in_channels, self.out_channels = conv.in_channels, conv.out_channels
        w = conv.weight.detach().reshape(conv.out_channels, conv.in_channels)
        # buffers, so that .to() / .cuda() move them; not parameters: the path has no backward
        self.register_buffer("weight", w.contiguous().clone())       # [C_out, C_in]: left operand for NCHW input
        self.register_buffer("weight_t", w.T.contiguous().clone())   # [C_in, C_out]: right operand for channels-last input
        self.register_buffer("bias", conv.bias.detach().clone() if conv.bias is not None else None)
        d_lowp, d_terms = default_cascade(self.weight.dtype)
        self.lowp, self.terms, self.products = d_lowp if lowp is None else lowp, d_terms if terms is None else terms, products
        self._weight_exp = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dim() != 4 or x.shape[1] != self.in_channels:
            raise ValueError(f"expected [B, {self.in_channels}, H, W], got {tuple(x.shape)}")
        B, _, H, W = x.shape
        if torch.compiler.is_compiling():
            # traced by torch.compile: the GEMMs as opaque ops (one per image for NCHW input)
            from ..compiled import cascade_linear
            if x.is_contiguous(memory_format=torch.channels_last) and not x.is_contiguous():
                y = cascade_linear(x.permute(0, 2, 3, 1), self.weight_t, None, self.bias, self.lowp, self.terms,
                                   self.products, False, None)
                return y.permute(0, 3, 1, 2)
            xc = x.contiguous()
            ys = [cascade_linear(self.weight, xc[b].reshape(self.in_channels, H * W), None, None, self.lowp, self.terms,
                                 self.products, False, None) for b in range(B)]
            out = torch.stack(ys).reshape(B, self.out_channels, H, W)
            return out if self.bias is None else out + self.bias.view(1, -1, 1, 1)
        rows = x.permute(0, 2, 3, 1)
        if rows.is_contiguous() and not x.is_contiguous():
            if self.lowp == "fp8" and (self._weight_exp is None or self._weight_exp.device != x.device):
                self._weight_exp = tensor_scale_exp(self.weight_t)
            y = cascaded_lowp_matmul(rows, self.weight_t, bias=self.bias, lowp=self.lowp, terms=self.terms,
                                     products=self.products, b_exp=self._weight_exp)
            return y.permute(0, 3, 1, 2)                  # [B, C_out, H, W] view of channels-last memory
        x = x.contiguous()
        out = torch.empty((B, self.out_channels, H, W), device=x.device, dtype=x.dtype)
        for b0 in range(0, B, MAX_GROUP):
            n = min(MAX_GROUP, B - b0)
            cascaded_lowp_matmul_grouped([self.weight] * n, [x[b0 + i].reshape(self.in_channels, H * W) for i in range(n)],
                                         outs=[out[b0 + i].reshape(self.out_channels, H * W) for i in range(n)],
                                         lowp=self.lowp, terms=self.terms, products=self.products)
        if self.bias is not None:
            out += self.bias.view(1, -1, 1, 1)
        return out


def patch_pointwise_convs(model: nn.Module, **cascade_kwargs) -> nn.Module:
    """Replace every 1x1 ``nn.Conv2d`` child that is a plain GEMM with :class:`BasedXLLowPConv1x1`
    (the walk of basedxl/unet.py:81-87, for the layers it leaves out)."""
    for _name, module in model.named_modules():
        for subname, submodule in module.named_children():
            if is_pointwise(submodule):
                setattr(module, subname, BasedXLLowPConv1x1(submodule, **cascade_kwargs))
    return model
