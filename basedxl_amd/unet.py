"""The install hook of the Linear path: counterpart of ``BasedXLUnet`` (basedxl/unet.py:65-87, 120-139)
for one GPU.

``BasedXLUnet(model, cfg)`` patches ``model`` in place when ``cfg.fp16_acc_matmul`` is set, exactly
where the reference calls ``patch_linear_layers`` (unet.py:72-73), and forwards calls to it
unchanged (the single-device branch, unet.py:132-139).  The patch-parallel surgery, the CFG batch
split and the output gather of the reference (unet.py:69-70, 89-114, 140-195) need more than one
GPU and are not part of this package.
"""
from __future__ import annotations

import torch.nn as nn

from .modules import chain_feed_forward_layers, patch_linear_layers, patch_pointwise_convs
from .unet_skeleton import fuse_geglu_layers, fuse_kv_projections
from .utils import BasedXLConfig


def patch_unet(model: nn.Module, cfg: BasedXLConfig) -> nn.Module:
    """Applies ``cfg`` to ``model`` in place: the fusions first (they take plain ``nn.Linear``
    children), then the reference's walk over the remaining ``nn.Linear`` layers (unet.py:81-87) and,
    if asked, the same walk over the 1x1 convolutions.  Does nothing unless ``cfg.fp16_acc_matmul``."""
    if not cfg.fp16_acc_matmul:
        return model
    kw = cfg.cascade_kwargs()
    lin_kw = dict(kw, prepared=cfg.prepared)
    if cfg.fuse_kv:
        fuse_kv_projections(model, cache_cross=cfg.cache_cross_kv, fuse_q=cfg.fuse_qkv, **lin_kw)
    if cfg.chain_ffn:
        chain_feed_forward_layers(model, **lin_kw)
    if cfg.fuse_geglu:
        fuse_geglu_layers(model, **lin_kw)
    patch_linear_layers(model, **lin_kw)
    if cfg.route_pointwise_convs:
        patch_pointwise_convs(model, **kw)
    return model


class BasedXLUnet(nn.Module):
    def __init__(self, model: nn.Module, basedxl_config: BasedXLConfig):
        super().__init__()
        self.model = patch_unet(model, basedxl_config)
        self.cfg = basedxl_config

    def reset_kv_cache(self) -> None:
        """Forget the kept cross-attention K/V (a new prompt); the reference recomputes them when its
        step counter is 0 (basedxl/modules/attn.py:57)."""
        for m in self.model.modules():
            if hasattr(m, "kv_cache"):
                m.reset()

    def forward(self, sample, timestep, encoder_hidden_states, added_cond_kwargs=None, **kwargs):
        return self.model(sample, timestep, encoder_hidden_states, added_cond_kwargs, **kwargs)
