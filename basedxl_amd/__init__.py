"""MI355X-native cascaded low-precision matmul (the Linear-layer hot path of basedxl)."""
from .cascaded_lowp_matmul import (cascaded_lowp_matmul, cascaded_lowp_matmul_grouped,  # noqa: F401
                                   cascaded_lowp_matmul_prepared, PreparedWeight, tensor_scale_exp)
from .modules.lowp_linear import BasedXLLowPLinear, patch_linear_layers  # noqa: F401

__all__ = ["cascaded_lowp_matmul", "cascaded_lowp_matmul_grouped", "cascaded_lowp_matmul_prepared", "PreparedWeight", "tensor_scale_exp",
           "BasedXLLowPLinear",
           "patch_linear_layers"]
