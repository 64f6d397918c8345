"""MI355X-native cascaded low-precision matmul (the Linear-layer hot path of basedxl)."""
from .cascaded_lowp_matmul import (cascaded_lowp_matmul, cascaded_lowp_matmul_grouped,  # noqa: F401
                                   cascaded_lowp_matmul_prepared, PreparedWeight, tensor_scale_exp,
                                   LeftSlots, ChainedWeight, cascaded_lowp_matmul_chained, cascaded_lowp_matmul_glu_chained)
from .modules import (BasedXLFusedKV, BasedXLLowPConv1x1, BasedXLLowPGEGLU, BasedXLLowPLinear, patch_linear_layers,  # noqa: F401
                      patch_pointwise_convs, BasedXLChainedFeedForward, chain_feed_forward_layers)

__all__ = ["cascaded_lowp_matmul", "cascaded_lowp_matmul_grouped", "cascaded_lowp_matmul_prepared", "PreparedWeight", "tensor_scale_exp",
           "LeftSlots", "ChainedWeight", "cascaded_lowp_matmul_chained", "cascaded_lowp_matmul_glu_chained",
           "BasedXLChainedFeedForward", "chain_feed_forward_layers",
           "BasedXLLowPLinear", "BasedXLLowPConv1x1", "BasedXLLowPGEGLU", "BasedXLFusedKV",
           "patch_linear_layers", "patch_pointwise_convs"]
