"""The module wrappers' GEMM as a ``torch.library`` custom op, so that a model holding them can be
traced by ``torch.compile`` (the reference compiles its UNet, basedxl/unet.py:76-78, and its Triton
kernel is traced natively; a ctypes call is opaque to the tracer).  The op has a shape-only ("fake")
implementation for tracing and runs the ordinary wrapper when executed.  The modules go through it
only while ``torch.compiler.is_compiling()``: in eager mode they call the wrapper directly, which
saves the dispatcher's per-call overhead.
"""
from __future__ import annotations

from typing import Optional

import torch

from .cascaded_lowp_matmul import PreparedWeight, cascaded_lowp_matmul


@torch.library.custom_op("basedxl_amd::cascade_linear", mutates_args=(), device_types="cuda")
def cascade_linear(x: torch.Tensor, weight: torch.Tensor, slots: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                   lowp: str, terms: int, products: str, glu: bool, b_exp: Optional[torch.Tensor]) -> torch.Tensor:
    """``x @ weight (+ bias)`` through the cascade; with ``slots`` (the operand slots of a
    PreparedWeight of ``weight``) the prepared kernels run when they take ``x``.  ``glu``: the
    gated projection, ``slots`` required, result ``[..., weight.shape[1] // 2]``."""
    K, N = int(weight.shape[0]), int(weight.shape[1])
    if slots is not None:
        pw = PreparedWeight.from_slots(slots, K, N, weight.dtype, lowp, terms, glu, b_exp)
        x2 = x.reshape(-1, K)
        few_rows = x2.shape[0] < 32 and x2.dtype == torch.float32 and not glu
        if glu or (not few_rows and pw.usable_with(x2 if x2.stride(-1) == 1 else x2.contiguous(), products)):
            return cascaded_lowp_matmul(x, pw, bias=bias, products=products)
    return cascaded_lowp_matmul(x, weight, bias=bias, lowp=lowp, terms=terms, products=products, b_exp=b_exp)


@cascade_linear.register_fake
def _(x, weight, slots, bias, lowp, terms, products, glu, b_exp):
    n = weight.shape[1] // 2 if glu else weight.shape[1]
    return x.new_empty((*x.shape[:-1], n))
