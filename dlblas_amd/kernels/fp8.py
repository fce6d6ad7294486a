"""Activation quantiser that produces the (a, a_s) operands of the FP8 block-scaled GEMM.

Drop-in for ``per_token_group_quant_fp8`` of the reference (dlblas/kernels/fp8.py:108-182): same signature, same
assertions, same output shapes (including the column-major scale view), computed by a hand-written gfx950 kernel
through the C ABI.  Any group size that divides the row length is taken, as in the reference (the block-scaled GEMM uses
128); only float8_e4m3fn is implemented, which is also all the reference supports (:124-125).
"""
from typing import Optional, Tuple

import torch

from .. import _lib
from ..utils import SymVar, Tensor, register_dlblas_op


@torch.library.custom_op('dlblas::per_token_group_quant_fp8', mutates_args=('x_q', 'x_s'), device_types='cuda')
def quant_op(x: torch.Tensor, x_q: torch.Tensor, x_s: torch.Tensor, eps: float, group_size: int = 128) -> None:
    K = x.shape[-1]
    rows = x.numel() // K
    row_stride = x.stride(-2) if x.dim() >= 2 else K
    _lib.quant_group(x, x_q, x_s, rows, K, group_size, row_stride, x_s.stride(-2) if x_s.dim() >= 2 else K // group_size,
                     x_s.stride(-1), eps)


def per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: Optional[torch.dtype] = torch.float8_e4m3fn,
    column_major_scales: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token-group quantisation of ``x`` [..., K] (ndim >= 2, last dim contiguous) to float8_e4m3fn.

    Returns ``(x_q, x_s)``: ``x_q`` like ``x`` in fp8, ``x_s`` fp32 ``[..., K / group_size]`` (a column-major view
    when ``column_major_scales``), with ``x_s = max(amax, eps) / 448`` per group.
    """
    assert (x.shape[-1] % group_size == 0), (
        f"the last dimension of 'x' {x.shape[-1]} must be divisible by 'group_size' {group_size}")
    assert x.stride(-1) == 1, f'{x} groups must be contiguous'
    if dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f'only float8_e4m3fn is implemented, got {dtype}')
    if x.dtype not in _lib.IN_CODES:
        raise TypeError(f'x must be bfloat16, float16 or float32, got {x.dtype}')
    if x.dim() < 2:
        raise ValueError('x must have at least two dimensions')
    K = x.shape[-1]
    if x.dim() > 2 and not x.is_contiguous():
        x = x.contiguous()
    x2d = x if x.dim() == 2 else x.reshape(-1, K)
    rows = x2d.shape[0]
    x_q = torch.empty(x.shape, device=x.device, dtype=dtype)
    if column_major_scales:
        # the reference's layout: a [K / group, rows...] buffer viewed with the group axis last
        buf = torch.empty((K // group_size, rows), device=x.device, dtype=torch.float32)
        s2d = buf.t()
        x_s = s2d if x.dim() == 2 else buf.reshape((K // group_size, ) + x.shape[:-1]).movedim(0, -1)
    else:
        x_s = torch.empty(x.shape[:-1] + (K // group_size, ), device=x.device, dtype=torch.float32)
        s2d = x_s.reshape(rows, K // group_size)
    quant_op(x2d, x_q.reshape(-1, K), s2d, float(eps), int(group_size))
    return x_q, x_s


@torch.library.custom_op('dlblas::per_block_quant_fp8', mutates_args=('w_q', 'w_s'), device_types='cuda')
def block_quant_op(w: torch.Tensor, w_q: torch.Tensor, w_s: torch.Tensor, eps: float) -> None:
    G = w.shape[0] if w.dim() == 3 else 1
    _lib.quant_128x128(w, w_q, w_s, G, w.shape[-2], w.shape[-1], eps)


def per_block_quant_fp8(w: torch.Tensor, block_size: int = 128, eps: float = 1e-10,
                        dtype: Optional[torch.dtype] = torch.float8_e4m3fn) -> Tuple[torch.Tensor, torch.Tensor]:
    """128 x 128 block quantisation of a weight ``w`` [N, K] or [G, N, K] to float8_e4m3fn: the (b, b_s) operands of
    fp8_gemm (dlblas/kernels/fp8_gemm.py:47,74-76) and of the grouped GEMMs.  The reference has no such function;
    the scheme is that of its test data builder (tests/kernels/test_fused_moe_v2.py:35-60).

    Returns ``(w_q, w_s)``: ``w_q`` like ``w`` in fp8, ``w_s`` fp32 ``[(G,) ceil(N/128), ceil(K/128)]``.
    """
    if block_size != 128:
        raise NotImplementedError(f'only block_size 128 is implemented, got {block_size}')
    if dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f'only float8_e4m3fn is implemented, got {dtype}')
    if w.dtype not in _lib.IN_CODES:
        raise TypeError(f'w must be bfloat16, float16 or float32, got {w.dtype}')
    if w.dim() not in (2, 3):
        raise ValueError('w must be [N, K] or [G, N, K]')
    assert w.stride(-1) == 1, 'the last dimension of w must be contiguous'
    if w.dim() == 3 and w.stride(0) != w.shape[1] * w.stride(1):
        w = w.contiguous()
    N, K = w.shape[-2], w.shape[-1]
    assert K % 8 == 0, f'K {K} must be a multiple of 8'
    w_q = torch.empty(w.shape, device=w.device, dtype=dtype)
    w_s = torch.empty(w.shape[:-2] + (-(-N // 128), -(-K // 128)), device=w.device, dtype=torch.float32)
    block_quant_op(w, w_q, w_s, float(eps))
    return w_q, w_s


def _bench(x, group_size, warmup: int = 3, rep: int = 10) -> float:
    for _ in range(warmup):
        per_token_group_quant_fp8(x, group_size)
    times = []
    for _ in range(rep):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        per_token_group_quant_fp8(x, group_size)
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    times.sort()
    return times[len(times) // 2]


def _register():
    m, k = SymVar('m'), SymVar('k')
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        register_dlblas_op('per_token_group_quant_fp8', None, (Tensor((m, k), dtype=dt, device='cuda'), torch.SymInt),
                           per_token_group_quant_fp8, _bench, per_token_group_quant_fp8)


_register()
