"""Key / value projection of an attention layer as one GEMM, with the reference's
cross-attention cache (basedxl/modules/attn.py:12-39 builds ``to_kv``; :42-45, :56-78 keep its
result while the text conditioning does not change); and, for self-attention, where the query is
projected from the same tokens, query / key / value as one GEMM."""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn

from .lowp_linear import BasedXLLowPLinear


class BasedXLFusedKV(nn.Module):
    """``to_k`` and ``to_v`` of one attention layer as a single ``[in, 2 * out]`` cascade GEMM.

    ``forward(states)`` returns ``(key, value)``, views of the halves of one ``[..., 2 * out]``
    result (attn.py:79).  With ``cache=True`` the result is kept and returned again until
    ``forward(..., recompute=True)`` or :meth:`reset`: the reference recomputes the
    cross-attention K/V only on the first denoising step (attn.py:57, 74-78), since the text
    conditioning is the same on every step.
    """

    def __init__(self, to_k: nn.Linear, to_v: nn.Linear, *, cache: bool = False, **cascade_kwargs):
        super().__init__()
        assert isinstance(to_k, nn.Linear) and isinstance(to_v, nn.Linear)
        assert (to_k.bias is None) == (to_v.bias is None)
        assert to_k.weight.shape == to_v.weight.shape
        fused = nn.Linear(to_k.in_features, 2 * to_k.out_features, bias=to_k.bias is not None,
                          device=to_k.weight.device, dtype=to_k.weight.dtype)
        with torch.no_grad():
            fused.weight.copy_(torch.cat([to_k.weight, to_v.weight], dim=0))
            if to_k.bias is not None:
                fused.bias.copy_(torch.cat([to_k.bias, to_v.bias], dim=0))
        self.out_features = to_k.out_features
        self.to_kv = BasedXLLowPLinear(fused, **cascade_kwargs)
        self.cache = cache
        self.kv_cache: Optional[torch.Tensor] = None

    def reset(self) -> None:
        self.kv_cache = None

    def forward(self, states: torch.Tensor, recompute: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        if not self.cache:
            kv = self.to_kv(states)
        else:
            if recompute or self.kv_cache is None:
                self.kv_cache = self.to_kv(states)
            kv = self.kv_cache
        return kv[..., : self.out_features], kv[..., self.out_features:]


class BasedXLFusedQKV(nn.Module):
    """``to_q``, ``to_k`` and ``to_v`` of a SELF-attention layer as a single ``[in, 3 * out]`` cascade
    GEMM: the step the reference takes for key and value (attn.py:23-39) taken once more, possible
    where all three read the same tokens.  One launch instead of two, and whatever a call does to
    its activations before multiplying (the fp8 cascade: find their scale, write their operand
    slots) is done once.  ``forward(states)`` returns ``(query, key, value)``, views of one result.
    """

    def __init__(self, to_q: nn.Linear, to_k: nn.Linear, to_v: nn.Linear, **cascade_kwargs):
        super().__init__()
        assert all(isinstance(m, nn.Linear) for m in (to_q, to_k, to_v))
        assert (to_q.bias is None) == (to_k.bias is None) == (to_v.bias is None)
        assert to_q.in_features == to_k.in_features == to_v.in_features, "query and key / value read different tokens"
        assert to_k.weight.shape == to_v.weight.shape
        outs = (to_q.out_features, to_k.out_features, to_v.out_features)
        fused = nn.Linear(to_q.in_features, sum(outs), bias=to_q.bias is not None, device=to_q.weight.device,
                          dtype=to_q.weight.dtype)
        with torch.no_grad():
            fused.weight.copy_(torch.cat([to_q.weight, to_k.weight, to_v.weight], dim=0))
            if to_q.bias is not None:
                fused.bias.copy_(torch.cat([to_q.bias, to_k.bias, to_v.bias], dim=0))
        self.splits = outs
        self.to_qkv = BasedXLLowPLinear(fused, **cascade_kwargs)

    def forward(self, states: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        q, k, v = self.to_qkv(states).split(self.splits, dim=-1)
        return q, k, v
