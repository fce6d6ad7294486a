"""FP8 block-scaled GEMM: the drop-in for dlblas/kernels/fp8_gemm.py of the reference.

``fp8_gemm(a, b, a_s, b_s)`` keeps the reference's signature, assertions and output rule
(dlblas/kernels/fp8_gemm.py:68-89) and runs the hand-written gfx950 kernels through the C ABI.  The op is
also exposed as ``torch.ops.dlblas.fp8_gemm`` and registered under the name ``'fp8_gemm'`` so that
``get_op('fp8_gemm', (a, b, a_s, b_s))`` selects and caches it (the reference file imports the registry but
never registers, dlblas/kernels/fp8_gemm.py:10).
"""
import torch

from .. import _lib
from ..utils import SymVar, Tensor, register_dlblas_op

BLOCK = 128  # K extent of one activation scale, K and N extent of one weight scale


def _launch_dense(a, b, a_s, b_s, c):
    K = a.size(-1)
    N = b.size(0)
    M = c.numel() // N if N else 0
    kb = a_s.size(-1)
    _lib.gemm_dense(a, b, a_s, b_s, c, M, N, K, kb, 1)


@torch.library.custom_op('dlblas::fp8_gemm', mutates_args=(), device_types='cuda')
def fp8_gemm_op(a: torch.Tensor, b: torch.Tensor, a_s: torch.Tensor, b_s: torch.Tensor,
                out_dtype: torch.dtype) -> torch.Tensor:
    N = b.size(0)
    kernel_dtype = out_dtype if out_dtype in (torch.bfloat16, torch.float32) else torch.float32
    c = a.new_empty(*a.size()[:-1], N, dtype=kernel_dtype)
    _launch_dense(a, b, a_s, b_s, c)
    return c if kernel_dtype == out_dtype else c.to(out_dtype)


@fp8_gemm_op.register_fake
def _(a, b, a_s, b_s, out_dtype):
    return a.new_empty(*a.size()[:-1], b.size(0), dtype=out_dtype)


def _check_dense(a, b, a_s, b_s):
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    if a.dtype != torch.float8_e4m3fn or b.dtype != torch.float8_e4m3fn:
        raise TypeError(f'fp8_gemm expects float8_e4m3fn operands, got {a.dtype} and {b.dtype}')
    if a_s.dtype != torch.float32 or b_s.dtype != torch.float32:
        raise TypeError(f'fp8_gemm expects float32 scales, got {a_s.dtype} and {b_s.dtype}')
    if b.dim() != 2 or a.dim() < 1 or a.size(-1) != b.size(1):
        raise ValueError(f'fp8_gemm shapes do not agree: a {tuple(a.shape)}, b {tuple(b.shape)}')
    K, N = b.size(1), b.size(0)
    kb, nb = -(-K // BLOCK), -(-N // BLOCK)
    rows = a.numel() // K if K else 0
    if a_s.numel() != rows * kb or (kb and a_s.size(-1) != kb):
        raise ValueError(f'a_s must hold one scale per row and 128-wide K block: expected {rows} x {kb}, '
                         f'got {tuple(a_s.shape)}')
    if tuple(b_s.shape) != (nb, kb):
        raise ValueError(f'b_s must be [{nb}, {kb}], got {tuple(b_s.shape)}')


def fp8_gemm(a: torch.Tensor, b: torch.Tensor, a_s: torch.Tensor, b_s: torch.Tensor):
    """
    Matrix product of block-scaled FP8 operands, ``(a * a_s) @ (b * b_s).T``.

    Args:
        a: activations ``[..., K]`` in float8_e4m3fn, contiguous; leading dimensions are flattened into M.
        b: weights ``[N, K]`` in float8_e4m3fn, contiguous.
        a_s: float32 ``[..., ceil(K/128)]``, one scale per row and 128-wide K block, contiguous.
        b_s: float32 ``[ceil(N/128), ceil(K/128)]``, one scale per 128 x 128 block of ``b``, contiguous.

    Returns:
        ``[..., N]`` in ``torch.get_default_dtype()``, newly allocated, enqueued on the current stream.
    """
    _check_dense(a, b, a_s, b_s)
    return fp8_gemm_op(a, b, a_s, b_s, torch.get_default_dtype())


def call(a, b, a_s, b_s):
    return fp8_gemm(a, b, a_s, b_s)


def bench_fn(a, b, a_s, b_s, warmup: int = 5, rep: int = 20) -> float:
    """Milliseconds per call (median of ``rep`` event-timed launches on the current stream)."""
    for _ in range(warmup):
        fp8_gemm(a, b, a_s, b_s)
    times = []
    for _ in range(rep):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fp8_gemm(a, b, a_s, b_s)
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    times.sort()
    return times[len(times) // 2]


def fp8_gemm_register_staged(a: torch.Tensor, b: torch.Tensor, a_s: torch.Tensor, b_s: torch.Tensor):
    """The same product on the register-staged tile kernels (global -> VGPR -> LDS double buffer, 16x16x128 MFMA) in
    place of the DMA-ring and decode kernels the planner would pick.  Registered as a second implementation of
    'fp8_gemm', the way the reference registers several implementations under one name
    (dlblas/kernels/matmul.py:381-402): get_op benchmarks both on the caller's shapes and caches the faster one."""
    _lib.force_variant('tile128x128')
    try:
        return fp8_gemm(a, b, a_s, b_s)
    finally:
        _lib.force_variant(None)


def _bench_of(fn):
    def bench(a, b, a_s, b_s, warmup: int = 5, rep: int = 20) -> float:
        for _ in range(warmup):
            fn(a, b, a_s, b_s)
        times = []
        for _ in range(rep):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            fn(a, b, a_s, b_s)
            stop.record()
            stop.synchronize()
            times.append(start.elapsed_time(stop))
        times.sort()
        return times[len(times) // 2]
    return bench


def _register():
    m, n, k, kb, nb = SymVar('m'), SymVar('n'), SymVar('k'), SymVar('kb'), SymVar('nb')
    f8, f32, dev = torch.float8_e4m3fn, torch.float32, 'cuda'
    args = (
        Tensor((m, k), dtype=f8, device=dev),
        Tensor((n, k), dtype=f8, device=dev),
        Tensor((m, kb), dtype=f32, device=dev),
        Tensor((nb, kb), dtype=f32, device=dev),
    )
    # spaces=None and kernel=call: the convention of the reference's non-Triton implementations
    # (dlblas/kernels/layer_norm/layernorm_torch.py:25)
    register_dlblas_op('fp8_gemm', None, args, call, bench_fn, call)
    register_dlblas_op('fp8_gemm', None, args, fp8_gemm_register_staged, _bench_of(fp8_gemm_register_staged),
                       fp8_gemm_register_staged)


_register()
