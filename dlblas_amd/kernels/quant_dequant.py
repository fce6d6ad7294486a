"""Scale re-layout helpers of the reference (dlblas/kernels/quant_dequant.py:22-83).

``tma_align_input_scale`` exists in the reference because its grouped GEMM wants the activation scales column-major
with the row count padded to 16 bytes.  The GEMM entry points of this package read scales through strides and need no
such call; the function is provided so that callers written against the reference keep working, and returns the same
view (values unchanged, strides (1, padded rows)).
"""
import torch

from .. import _lib


def ceil_div(x: int, y: int) -> int:
    return (x + y - 1) // y


def get_tma_aligned_size(x: int, element_size: int) -> int:
    """Row count padded to a multiple of 16 bytes' worth of elements (dlblas/kernels/quant_dequant.py:22-39)."""
    tma_alignment_bytes = 16
    assert tma_alignment_bytes % element_size == 0
    alignment = tma_alignment_bytes // element_size
    return ceil_div(x, alignment) * alignment


@torch.library.custom_op('dlblas::tma_align_input_scale', mutates_args=('output', ), device_types='cuda')
def _relayout_op(input_scale: torch.Tensor, output: torch.Tensor) -> None:
    _lib.scale_relayout(input_scale, output, input_scale.shape[0], input_scale.shape[1], output.shape[1])


def tma_align_input_scale(input_scale: torch.Tensor) -> torch.Tensor:
    assert input_scale.dim() == 2
    m, k_div_block_size = input_scale.shape
    if input_scale.dtype != torch.float32:
        raise TypeError(f'input_scale must be float32, got {input_scale.dtype}')
    padd_m = get_tma_aligned_size(m, input_scale.element_size())
    output = torch.empty((k_div_block_size, padd_m), dtype=input_scale.dtype, device=input_scale.device)
    _relayout_op(input_scale, output)
    return output.t()[:m]
