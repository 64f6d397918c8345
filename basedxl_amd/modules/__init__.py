from .lowp_linear import BasedXLLowPLinear, patch_linear_layers  # noqa: F401
