"""Same import path as the reference (basedxl/triton/cascaded_lowp_matmul.py); re-exports the
HIP-backed operator."""
from ..cascaded_lowp_matmul import cascaded_lowp_matmul  # noqa: F401
