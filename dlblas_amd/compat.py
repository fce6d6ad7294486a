"""Publish this package under the module names the reference's callers import.

``install()`` makes ``import dlblas``, ``from dlblas.kernels.fp8_gemm import fp8_gemm``,
``from dlblas.utils import register_dlblas_op, get_op, SymVar, Tensor`` resolve to this package, and (optionally)
provides a ``deep_gemm`` module exposing the grouped GEMMs under the names probed with ``hasattr`` at
dlblas/kernels/fused_moe_v3.py:241-244 and dlblas/layers/moe/ep_moe.py:189-196.  Nothing is replaced when a real
module of that name is already imported.
"""
import sys
import types

_ALIASES = {
    'dlblas': 'dlblas_amd',
    'dlblas.kernels': 'dlblas_amd.kernels',
    'dlblas.kernels.fp8_gemm': 'dlblas_amd.kernels.fp8_gemm',
    'dlblas.kernels.fp8': 'dlblas_amd.kernels.fp8',
    'dlblas.kernels.moe': 'dlblas_amd.kernels.moe',
    'dlblas.kernels.fused_moe_v3': 'dlblas_amd.kernels.fused_moe_v3',
    'dlblas.kernels.quant_dequant': 'dlblas_amd.kernels.quant_dequant',
    'dlblas.layers.moe.kernels.activation': 'dlblas_amd.kernels.activation',
    'dlblas.utils': 'dlblas_amd.utils',
    'dlblas.utils.logger': 'dlblas_amd.utils.logger',
    'dlblas.op_registry': 'dlblas_amd.op_registry',
    'dlblas.op_struct': 'dlblas_amd.op_struct',
    'dlblas.cache': 'dlblas_amd.cache',
    'dlblas.symbolic_var': 'dlblas_amd.symbolic_var',
    'dlblas.autotune': 'dlblas_amd.autotune',
    'dlblas.autotune.space': 'dlblas_amd.autotune.space',
    'dlblas.autotune.configs': 'dlblas_amd.autotune.configs',
}


def ceil_div(x: int, y: int) -> int:
    return (x + y - 1) // y


def install(dlblas: bool = True, deep_gemm: bool = True) -> None:
    import importlib
    if dlblas:
        for alias, target in _ALIASES.items():
            # intermediate packages this package has no counterpart for (dlblas.layers, dlblas.layers.moe, ...)
            parts = alias.split('.')
            for i in range(1, len(parts)):
                parent = '.'.join(parts[:i])
                if parent not in sys.modules and parent not in _ALIASES:
                    pkg = types.ModuleType(parent)
                    pkg.__path__ = []
                    sys.modules[parent] = pkg
                    if i > 1:
                        setattr(sys.modules['.'.join(parts[:i - 1])], parts[i - 1], pkg)
            if alias not in sys.modules:
                sys.modules[alias] = importlib.import_module(target)
                if len(parts) > 1:
                    setattr(sys.modules['.'.join(parts[:-1])], parts[-1], sys.modules[alias])
    if deep_gemm and 'deep_gemm' not in sys.modules:
        from .kernels import fp8_gemm_grouped as grouped
        mod = types.ModuleType('deep_gemm')
        mod.__doc__ = 'deep_gemm-compatible entry points served by dlblas_amd'
        mod.m_grouped_fp8_gemm_nt_contiguous = grouped.m_grouped_fp8_gemm_nt_contiguous
        mod.m_grouped_fp8_gemm_nt_masked = grouped.m_grouped_fp8_gemm_nt_masked
        mod.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous = grouped.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous
        mod.m_grouped_gemm_fp8_fp8_bf16_nt_masked = grouped.m_grouped_gemm_fp8_fp8_bf16_nt_masked
        mod.ceil_div = ceil_div
        sys.modules['deep_gemm'] = mod
