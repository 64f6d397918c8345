"""Import-path compatibility only: the reference exposes its operator as
``basedxl.triton.cascaded_lowp_matmul.cascaded_lowp_matmul``; nothing here uses Triton."""
