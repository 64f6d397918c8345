from .fused_kv import BasedXLFusedKV, BasedXLFusedQKV  # noqa: F401
from .chained_ff import BasedXLChainedFeedForward, chain_feed_forward_layers  # noqa: F401
from .geglu import BasedXLLowPGEGLU  # noqa: F401
from .lowp_linear import BasedXLLowPLinear, patch_linear_layers  # noqa: F401
from .pointwise_conv import BasedXLLowPConv1x1, is_pointwise, patch_pointwise_convs  # noqa: F401
