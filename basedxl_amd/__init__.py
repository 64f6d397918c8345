"""MI355X-native cascaded low-precision matmul (the Linear-layer hot path of basedxl)."""
from .cascaded_lowp_matmul import (cascaded_lowp_matmul, cascaded_lowp_matmul_grouped,  # noqa: F401
                                   cascaded_lowp_matmul_prepared, PreparedWeight, tensor_scale_exp)
from .modules import (BasedXLFusedKV, BasedXLLowPConv1x1, BasedXLLowPGEGLU, BasedXLLowPLinear, patch_linear_layers,  # noqa: F401
                      patch_pointwise_convs)

__all__ = ["cascaded_lowp_matmul", "cascaded_lowp_matmul_grouped", "cascaded_lowp_matmul_prepared", "PreparedWeight", "tensor_scale_exp",
           "BasedXLLowPLinear", "BasedXLLowPConv1x1", "BasedXLLowPGEGLU", "BasedXLFusedKV",
           "patch_linear_layers", "patch_pointwise_convs"]
