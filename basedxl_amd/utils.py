"""The configuration switch of the Linear path.

Counterpart of the reference's ``BasedXLConfig`` (basedxl/utils.py:8-21), reduced to what reaches
the cascaded matmul: its ``fp16_acc_matmul`` flag (utils.py:12, read at basedxl/unet.py:72 and set from
the command line at sample.py:29,42) and the tensor ``dtype`` (utils.py:11).  The process-group,
patch-parallel and compile fields of the reference's dataclass belong to subsystems that are not
part of this package.  The remaining fields choose the cascade and the fusions this package adds.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class BasedXLConfig:
    dtype: torch.dtype = torch.float32
    #: the reference's switch: route every nn.Linear of the UNet through cascaded_lowp_matmul
    fp16_acc_matmul: bool = False
    #: cascade of the routed layers (None: the default for the tensors' dtype, two bf16 terms for fp32)
    lowp: Optional[str] = None
    terms: Optional[int] = None
    products: str = "tri"
    #: also route 1x1 convolutions (the reference leaves them to the vendor library, unet.py:85,98-99)
    route_pointwise_convs: bool = True
    #: to_k / to_v of every attention layer as one GEMM (basedxl/modules/attn.py:23-39) ...
    fuse_kv: bool = True
    #: ... whose cross-attention result is kept between denoising steps (attn.py:57,74-78)
    cache_cross_kv: bool = False
    #: with fuse_kv: in self-attention, where all three read the same tokens, to_q too (one GEMM instead of two)
    fuse_qkv: bool = True
    #: GEGLU gate applied in the store of the projection GEMM (weights kept split)
    fuse_geglu: bool = False
    #: the two Linear layers of every feed-forward block as a chain: the gated store of the first GEMM
    #: writes the operand slots of the second (fp32, two bf16 terms; other layers fall back by themselves)
    chain_ffn: bool = False
    #: keep the weights of the Linear layers split (None: the module's default for its dtype)
    prepared: Optional[bool] = None

    def cascade_kwargs(self) -> dict:
        return {"lowp": self.lowp, "terms": self.terms, "products": self.products}
