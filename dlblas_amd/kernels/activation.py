"""``silu_and_mul`` of the reference (dlblas/layers/moe/kernels/activation.py:61-95; kernel :16-58) and its fusion with
the 1 x 128 quantiser that follows it between the two contiguous grouped GEMMs (dlblas/kernels/fused_moe_v3.py:325-334).
"""
from typing import Optional, Tuple

import torch

from .. import _lib


@torch.library.custom_op('dlblas::silu_and_mul', mutates_args=('out', ), device_types='cuda')
def _silu_op(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _lib.silu_mul(gate_up, out, gate_up.shape[0], out.shape[1])


@torch.library.custom_op('dlblas::silu_and_mul_post_quant', mutates_args=('q', 's'), device_types='cuda')
def _silu_quant_op(gate_up: torch.Tensor, q: torch.Tensor, s: torch.Tensor, eps: float) -> None:
    _lib.silu_mul_quant(gate_up, q, s, gate_up.shape[0], q.shape[1], s.stride(0), s.stride(1), eps)


def silu_and_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu and mul: gate_up [M, 2N] -> out [M, N] = silu(gate_up[:, :N]) * gate_up[:, N:] in the dtype of gate_up."""
    assert gate_up.dim() == 2
    M = gate_up.size(0)
    N = gate_up.size(-1) // 2
    if out is None:
        out = gate_up.new_empty((M, N))
    if gate_up.dtype not in _lib.IN_CODES:
        raise TypeError(f'gate_up must be bfloat16, float16 or float32, got {gate_up.dtype}')
    if out.dtype != gate_up.dtype or tuple(out.shape) != (M, N):
        raise ValueError('out must be [M, N] in the dtype of gate_up')
    if gate_up.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError('the last dimension of gate_up and out must be contiguous')
    _silu_op(gate_up, out)
    return out


def silu_and_mul_post_quant(gate_up: torch.Tensor, group_size: int = 128, eps: float = 1e-10,
                            column_major_scales: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """``per_token_group_quant_fp8(silu_and_mul(gate_up), group_size, eps, column_major_scales=...)`` in one pass over
    the data; bit-identical to the two calls.  Returns (q float8_e4m3fn [M, N], s float32 [M, N / 128])."""
    assert gate_up.dim() == 2
    M = gate_up.size(0)
    N = gate_up.size(-1) // 2
    assert N % group_size == 0, f'N {N} must be divisible by group_size {group_size}'
    if group_size != 128:
        raise NotImplementedError(f'only group_size 128 is implemented, got {group_size}')
    if gate_up.dtype not in _lib.IN_CODES:
        raise TypeError(f'gate_up must be bfloat16, float16 or float32, got {gate_up.dtype}')
    if gate_up.stride(1) != 1:
        raise ValueError('the last dimension of gate_up must be contiguous')
    q = torch.empty((M, N), device=gate_up.device, dtype=torch.float8_e4m3fn)
    if column_major_scales:
        s = torch.empty((N // group_size, M), device=gate_up.device, dtype=torch.float32).t()
    else:
        s = torch.empty((M, N // group_size), device=gate_up.device, dtype=torch.float32)
    _silu_quant_op(gate_up, q, s, float(eps))
    return q, s
