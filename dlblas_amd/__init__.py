"""MI355X-native FP8 block-scaled GEMM behind DLBlas' entry points.

    from dlblas_amd.kernels.fp8_gemm import fp8_gemm            # dlblas.kernels.fp8_gemm.fp8_gemm
    from dlblas_amd import get_op                                # dlblas.get_op / dlblas.utils.get_op
    op = get_op('fp8_gemm', (a, b, a_s, b_s)); c = op(a, b, a_s, b_s)

``dlblas_amd.compat.install()`` additionally publishes the same modules under the ``dlblas`` and ``deep_gemm``
names for code that imports those.
"""
from . import kernels  # noqa: F401  (registers the ops)
from ._lib import prepare
from .kernels.fp8 import per_token_group_quant_fp8
from .kernels.fp8_gemm import fp8_gemm
from .kernels.fp8_gemm_grouped import (fp8_gemm_grouped_contiguous, fp8_gemm_grouped_masked,
                                       m_grouped_fp8_gemm_nt_contiguous, m_grouped_fp8_gemm_nt_masked)
from .utils import get_args_from_op_name, get_list_op_names, get_op, register_dlblas_op

__version__ = '0.1.0'

__all__ = [
    'fp8_gemm', 'prepare', 'per_token_group_quant_fp8', 'fp8_gemm_grouped_contiguous', 'fp8_gemm_grouped_masked', 'm_grouped_fp8_gemm_nt_contiguous',
    'm_grouped_fp8_gemm_nt_masked', 'get_op', 'get_list_op_names', 'get_args_from_op_name', 'register_dlblas_op'
]
