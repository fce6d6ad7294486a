"""Kernels of the FP8 block-scaled GEMM path; importing this package registers them with the op registry
(the reference registers at import time too, dlblas/kernels/__init__.py:5-44)."""
from . import fp8, fp8_gemm, fp8_gemm_grouped  # noqa: F401
