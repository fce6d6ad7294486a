"""Grouped FP8 block-scaled GEMMs for MoE experts: expert-contiguous rows and masked fixed-capacity buffers.

The reference does not implement these; it forwards to the third-party ``deep_gemm`` package
(dlblas/kernels/fused_moe_v3.py:235-245 and dlblas/layers/moe/ep_moe.py:180-197).  The functions here take the
positional arguments those call sites pass, under both generations of deep_gemm names the call sites probe,
write ``out`` in place and return None.
"""
from typing import Sequence

import torch

from .. import _lib
from ..utils import SymVar, Tensor, register_dlblas_op

BLOCK = 128


def _unpack(pair: Sequence[torch.Tensor], what: str):
    if not isinstance(pair, (tuple, list)) or len(pair) != 2:
        raise TypeError(f'{what} must be a (tensor, scales) pair')
    return pair[0], pair[1]


def _check_common(a, a_s, w, w_s, out):
    for name, t, dt in (('a', a, torch.float8_e4m3fn), ('w', w, torch.float8_e4m3fn), ('a_s', a_s, torch.float32),
                        ('w_s', w_s, torch.float32)):
        if t.dtype != dt:
            raise TypeError(f'{name} must be {dt}, got {t.dtype}')
    if out.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f'out must be bfloat16 or float32, got {out.dtype}')
    assert a.is_contiguous() and w.is_contiguous() and out.is_contiguous(), 'Input tensors must be contiguous'
    assert w_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    if w.dim() != 3:
        raise ValueError(f'weights must be [G, N, K], got {tuple(w.shape)}')
    G, N, K = w.shape
    if K % 16 != 0:
        raise ValueError(f'grouped fp8 gemm needs K % 16 == 0, got K={K}')
    if tuple(w_s.shape) != (G, -(-N // BLOCK), -(-K // BLOCK)):
        raise ValueError(f'w_s must be [{G}, {-(-N // BLOCK)}, {-(-K // BLOCK)}], got {tuple(w_s.shape)}')
    return G, N, K


@torch.library.custom_op('dlblas::fp8_gemm_grouped_contiguous', mutates_args=('out', ), device_types='cuda')
def grouped_contiguous_op(a: torch.Tensor, a_s: torch.Tensor, w: torch.Tensor, w_s: torch.Tensor,
                          out: torch.Tensor, m_indices: torch.Tensor) -> None:
    G, N, K = w.shape
    _lib.gemm_contiguous(a, w, a_s, w_s, out, m_indices, a.size(0), N, K, G, a_s.stride(0), a_s.stride(1))


@torch.library.custom_op('dlblas::fp8_gemm_grouped_masked', mutates_args=('out', ), device_types='cuda')
def grouped_masked_op(a: torch.Tensor, a_s: torch.Tensor, w: torch.Tensor, w_s: torch.Tensor, out: torch.Tensor,
                      masked_m: torch.Tensor, expected_m: int) -> None:
    G, N, K = w.shape
    _lib.gemm_masked(a, w, a_s, w_s, out, masked_m, expected_m, a.size(1), N, K, G, a_s.stride(0), a_s.stride(1),
                     a_s.stride(2))


def fp8_gemm_grouped_contiguous(a, a_s, w, w_s, out, m_indices):
    """``out[r] = (a[r] * a_s[r]) @ (w[g] * w_s[g]).T`` with ``g = m_indices[r]``; rows of an expert are
    contiguous, every expert's span is a multiple of 128 rows, a 128-row block whose first index is negative
    is skipped.  ``a_s`` may be any strided 2-D view (the reference passes a column-major one,
    dlblas/kernels/quant_dequant.py:65-83)."""
    G, N, K = _check_common(a, a_s, w, w_s, out)
    if a.dim() != 2 or a.size(1) != K:
        raise ValueError(f'a must be [M_sum, {K}], got {tuple(a.shape)}')
    M_sum = a.size(0)
    if tuple(a_s.shape) != (M_sum, -(-K // BLOCK)):
        raise ValueError(f'a_s must be [{M_sum}, {-(-K // BLOCK)}], got {tuple(a_s.shape)}')
    if tuple(out.shape) != (M_sum, N):
        raise ValueError(f'out must be [{M_sum}, {N}], got {tuple(out.shape)}')
    if m_indices.dtype != torch.int32 or tuple(m_indices.shape) != (M_sum, ) or not m_indices.is_contiguous():
        raise ValueError('m_indices must be a contiguous int32 vector with one entry per row of a')
    grouped_contiguous_op(a, a_s, w, w_s, out, m_indices)


@torch.library.custom_op('dlblas::fp8_gemm_grouped_contiguous_silu_quant', mutates_args=('out_q', 'out_s'), device_types='cuda')
def grouped_contiguous_silu_quant_op(a: torch.Tensor, a_s: torch.Tensor, w: torch.Tensor, w_s: torch.Tensor,
                                     out_q: torch.Tensor, out_s: torch.Tensor, m_indices: torch.Tensor, eps: float) -> bool:
    G, N, K = w.shape
    return _lib.gemm_contiguous_silu_quant(a, w, a_s, w_s, out_q, out_s, m_indices, a.size(0), N, K, G, a_s.stride(0),
                                           a_s.stride(1), eps)


@grouped_contiguous_silu_quant_op.register_fake
def _(a, a_s, w, w_s, out_q, out_s, m_indices, eps):
    return True


@torch.library.custom_op('dlblas::fp8_gemm_grouped_contiguous_gather_silu_quant', mutates_args=('out_q', 'out_s'),
                         device_types='cuda')
def grouped_contiguous_gather_silu_quant_op(a: torch.Tensor, a_s: torch.Tensor, w: torch.Tensor, w_s: torch.Tensor,
                                            out_q: torch.Tensor, out_s: torch.Tensor, m_indices: torch.Tensor,
                                            a_row_index: torch.Tensor, eps: float) -> bool:
    G, N, K = w.shape
    return _lib.gemm_contiguous_gather_silu_quant(a, w, a_s, w_s, out_q, out_s, m_indices, a_row_index, N, K, G, eps)


@grouped_contiguous_gather_silu_quant_op.register_fake
def _(a, a_s, w, w_s, out_q, out_s, m_indices, a_row_index, eps):
    return True


def fp8_gemm_grouped_contiguous_silu_quant(a, a_s, w13, w13_s, m_indices, eps: float = 1e-10, column_major_scales: bool = False,
                                           a_row_index=None):
    """The first half of an expert MLP in one kernel: ``gate_up = grouped_contiguous(a, w13)`` (bf16), ``silu_and_mul``,
    ``per_token_group_quant_fp8(.., 128)`` - the sequence of dlblas/kernels/fused_moe_v3.py:307-334 with the same bits and
    without the bf16 intermediate in memory.  ``w13`` is [G, 2 I, K] with the gate rows first.  Returns (q e4m3fn
    [M_sum, I], s float32 [M_sum, I / 128]), or None when the library has no fused kernel for the shape (K or I not a
    multiple of 128, ...): the caller then runs the three steps apart.

    ``a_row_index`` (int32 [M_sum], optional): row r of the GEMM is then row ``a_row_index[r]`` of ``a`` and ``a_s``, which
    hold the tokens in the order they were received (``ep_scatter_rows`` writes the table), so that no expert-sorted copy
    of the activations is needed."""
    for name, t, dt in (('a', a, torch.float8_e4m3fn), ('w13', w13, torch.float8_e4m3fn), ('a_s', a_s, torch.float32),
                        ('w13_s', w13_s, torch.float32)):
        if t.dtype != dt:
            raise TypeError(f'{name} must be {dt}, got {t.dtype}')
    assert a.is_contiguous() and w13.is_contiguous(), 'Input tensors must be contiguous'
    assert w13_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    if w13.dim() != 3 or a.dim() != 2 or a.size(1) != w13.size(2):
        raise ValueError(f'a must be [M_sum, K] and w13 [G, 2 I, K], got {tuple(a.shape)} and {tuple(w13.shape)}')
    G, N, K = w13.shape
    M_sum = a.size(0) if a_row_index is None else m_indices.numel()
    if N % (2 * BLOCK) != 0 or K % BLOCK != 0:
        return None
    if tuple(w13_s.shape) != (G, N // BLOCK, K // BLOCK) or tuple(a_s.shape) != (a.size(0), K // BLOCK):
        raise ValueError('a_s must be [rows of a, K / 128] and w13_s [G, 2 I / 128, K / 128]')
    if a_row_index is not None and (a_row_index.dtype != torch.int32 or tuple(a_row_index.shape) != (M_sum, ) or
                                    not a_row_index.is_contiguous()):
        raise ValueError('a_row_index must be a contiguous int32 vector with one entry per GEMM row')
    if m_indices.dtype != torch.int32 or tuple(m_indices.shape) != (M_sum, ) or not m_indices.is_contiguous():
        raise ValueError('m_indices must be a contiguous int32 vector with one entry per row of a')
    inter = N // 2
    q = torch.empty((M_sum, inter), device=a.device, dtype=torch.float8_e4m3fn)
    if column_major_scales:
        s = torch.empty((inter // BLOCK, M_sum), device=a.device, dtype=torch.float32).t()
    else:
        s = torch.empty((M_sum, inter // BLOCK), device=a.device, dtype=torch.float32)
    if M_sum == 0:
        return q, s
    if a_row_index is not None:
        if a.size(0) == 0 or not grouped_contiguous_gather_silu_quant_op(a, a_s, w13, w13_s, q, s, m_indices, a_row_index, float(eps)):
            return None
        return q, s
    if not grouped_contiguous_silu_quant_op(a, a_s, w13, w13_s, q, s, m_indices, float(eps)):
        return None
    return q, s


def fp8_gemm_grouped_masked(a, a_s, w, w_s, out, masked_m, expected_m=0):
    """For every expert g, rows ``[0, masked_m[g])`` of ``out[g]`` get ``(a[g] * a_s[g]) @ (w[g] * w_s[g]).T``;
    the other rows of ``out`` are left untouched and the matching rows of ``a`` are never used."""
    G, N, K = _check_common(a, a_s, w, w_s, out)
    if a.dim() != 3 or a.size(0) != G or a.size(2) != K:
        raise ValueError(f'a must be [{G}, M_max, {K}], got {tuple(a.shape)}')
    M_max = a.size(1)
    if tuple(a_s.shape) != (G, M_max, -(-K // BLOCK)):
        raise ValueError(f'a_s must be [{G}, {M_max}, {-(-K // BLOCK)}], got {tuple(a_s.shape)}')
    if tuple(out.shape) != (G, M_max, N):
        raise ValueError(f'out must be [{G}, {M_max}, {N}], got {tuple(out.shape)}')
    if masked_m.dtype != torch.int32 or tuple(masked_m.shape) != (G, ) or not masked_m.is_contiguous():
        raise ValueError('masked_m must be a contiguous int32 vector with one entry per expert')
    grouped_masked_op(a, a_s, w, w_s, out, masked_m, int(expected_m))


@torch.library.custom_op('dlblas::fp8_gemm_grouped_masked_silu_quant', mutates_args=('out_q', 'out_s'), device_types='cuda')
def grouped_masked_silu_quant_op(a: torch.Tensor, a_s: torch.Tensor, w: torch.Tensor, w_s: torch.Tensor, out_q: torch.Tensor,
                                 out_s: torch.Tensor, masked_m: torch.Tensor, expected_m: int, eps: float) -> bool:
    G, N, K = w.shape
    return _lib.gemm_masked_silu_quant(a, w, a_s, w_s, out_q, out_s, masked_m, expected_m, a.size(1), N, K, G, a_s.stride(0),
                                       a_s.stride(1), a_s.stride(2), eps)


@grouped_masked_silu_quant_op.register_fake
def _(a, a_s, w, w_s, out_q, out_s, masked_m, expected_m, eps):
    return True


def fp8_gemm_grouped_masked_silu_quant(a, a_s, w13, w13_s, out_q, out_s, masked_m, expected_m=0, eps: float = 1e-10) -> bool:
    """The first half of the masked (low-latency) expert MLP in one kernel: ``m_grouped_fp8_gemm_nt_masked`` into a
    bf16 buffer followed by ``silu_and_mul_masked_post_quant_fwd`` (dlblas/layers/moe/ep_moe.py:199-251), with the same
    bits and without the bf16 [G, M_max, 2 I] intermediate in memory.  ``w13`` is [G, 2 I, K] with the gate rows first;
    ``out_q`` e4m3fn [G, M_max, I] and ``out_s`` float32 [G, M_max, I / 128] (any strides) are written for the first
    ``masked_m[g]`` rows of every expert and keep their content elsewhere.  Returns False, with nothing written, when
    the library has no fused kernel for the shape: the caller then runs the two steps apart."""
    for name, t, dt in (('a', a, torch.float8_e4m3fn), ('w13', w13, torch.float8_e4m3fn), ('a_s', a_s, torch.float32),
                        ('w13_s', w13_s, torch.float32), ('out_q', out_q, torch.float8_e4m3fn), ('out_s', out_s, torch.float32)):
        if t.dtype != dt:
            raise TypeError(f'{name} must be {dt}, got {t.dtype}')
    assert a.is_contiguous() and w13.is_contiguous() and out_q.is_contiguous(), 'Input tensors must be contiguous'
    assert w13_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    if w13.dim() != 3 or a.dim() != 3 or a.size(0) != w13.size(0) or a.size(2) != w13.size(2):
        raise ValueError(f'a must be [G, M_max, K] and w13 [G, 2 I, K], got {tuple(a.shape)} and {tuple(w13.shape)}')
    G, N, K = w13.shape
    M_max = a.size(1)
    if N % (2 * BLOCK) != 0 or K % BLOCK != 0:
        return False
    inter = N // 2
    if tuple(w13_s.shape) != (G, N // BLOCK, K // BLOCK) or tuple(a_s.shape) != (G, M_max, K // BLOCK):
        raise ValueError('a_s must be [G, M_max, K / 128] and w13_s [G, 2 I / 128, K / 128]')
    if tuple(out_q.shape) != (G, M_max, inter) or tuple(out_s.shape) != (G, M_max, inter // BLOCK):
        raise ValueError(f'out_q must be [{G}, {M_max}, {inter}] and out_s [{G}, {M_max}, {inter // BLOCK}]')
    if masked_m.dtype != torch.int32 or tuple(masked_m.shape) != (G, ) or not masked_m.is_contiguous():
        raise ValueError('masked_m must be a contiguous int32 vector with one entry per expert')
    if G == 0 or M_max == 0:
        return True
    return grouped_masked_silu_quant_op(a, a_s, w13, w13_s, out_q, out_s, masked_m, int(expected_m), float(eps))


# --- deep_gemm-compatible positional entry points (what the reference's shims call) --------------------------


def m_grouped_fp8_gemm_nt_contiguous(input_tuple, w_tuple, out, m_indices, *unused, **unused_kw):
    a, a_s = _unpack(input_tuple, 'input_tuple')
    w, w_s = _unpack(w_tuple, 'w_tuple')
    fp8_gemm_grouped_contiguous(a, a_s, w, w_s, out, m_indices)


def m_grouped_fp8_gemm_nt_masked(input_tuple, w_tuple, out, masked_m, expected_m, *unused, **unused_kw):
    a, a_s = _unpack(input_tuple, 'input_tuple')
    w, w_s = _unpack(w_tuple, 'w_tuple')
    fp8_gemm_grouped_masked(a, a_s, w, w_s, out, masked_m, expected_m)


m_grouped_gemm_fp8_fp8_bf16_nt_contiguous = m_grouped_fp8_gemm_nt_contiguous
m_grouped_gemm_fp8_fp8_bf16_nt_masked = m_grouped_fp8_gemm_nt_masked


def _event_bench(fn, warmup=3, rep=10) -> float:
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(rep):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    times.sort()
    return times[len(times) // 2]


def _bench_contiguous(a, a_s, w, w_s, out, m_indices):
    return _event_bench(lambda: fp8_gemm_grouped_contiguous(a, a_s, w, w_s, out, m_indices))


def _bench_masked(a, a_s, w, w_s, out, masked_m, expected_m=0):
    return _event_bench(lambda: fp8_gemm_grouped_masked(a, a_s, w, w_s, out, masked_m, expected_m))


def _register():
    f8, f32, i32, dev = torch.float8_e4m3fn, torch.float32, torch.int32, 'cuda'
    g, m, n, k, kb, nb = (SymVar(s) for s in ('g', 'm', 'n', 'k', 'kb', 'nb'))
    for out_dtype in (torch.bfloat16, torch.float32):
        register_dlblas_op('fp8_gemm_grouped_contiguous', None, (
            Tensor((m, k), dtype=f8, device=dev),
            Tensor((m, kb), dtype=f32, device=dev),
            Tensor((g, n, k), dtype=f8, device=dev),
            Tensor((g, nb, kb), dtype=f32, device=dev),
            Tensor((m, n), dtype=out_dtype, device=dev),
            Tensor((m, ), dtype=i32, device=dev),
        ), fp8_gemm_grouped_contiguous, _bench_contiguous, fp8_gemm_grouped_contiguous)
        register_dlblas_op('fp8_gemm_grouped_masked', None, (
            Tensor((g, m, k), dtype=f8, device=dev),
            Tensor((g, m, kb), dtype=f32, device=dev),
            Tensor((g, n, k), dtype=f8, device=dev),
            Tensor((g, nb, kb), dtype=f32, device=dev),
            Tensor((g, m, n), dtype=out_dtype, device=dev),
            Tensor((g, ), dtype=i32, device=dev),
            torch.SymInt,
        ), fp8_gemm_grouped_masked, _bench_masked, fp8_gemm_grouped_masked)


_register()
