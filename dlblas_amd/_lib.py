"""ctypes binding of libdlblas_fp8_gemm.so (the C ABI declared in include/dlblas_fp8_gemm.h and dlblas_fp8_moe.h).

The library is the only implementation: when it has not been built, every op raises ImportError.  There is no
PyTorch or CPU fallback.  The calling convention (``c_void_p(tensor.data_ptr())`` operands, the stream handle as
``c_void_p``) is the one the reference uses for its native code, tests/kernels/cutlass/test_fp8_convert.py:8-39.
"""
import ctypes
import os
import threading

import torch

from ._build import LIB_PATH

ABI_VERSION = 7
OUT_BF16, OUT_F32 = 0, 1
WS_COUNTER_BYTES = 65536
WORKSPACE_BYTES = WS_COUNTER_BYTES + (32 << 20)
STATIC_SCRATCH_BYTES = 16 << 20  # DLB_STATIC_SCRATCH_BYTES: the array dlb_fp8_gemm_noalloc works in ...
STATIC_SCRATCH_SLICES = 4  # ... cut into this many slices, one per stream
STATIC_SCRATCH_SLICE_BYTES = STATIC_SCRATCH_BYTES // STATIC_SCRATCH_SLICES

ERR_NULL_POINTER, ERR_BAD_SHAPE, ERR_BAD_STRIDE, ERR_BAD_DTYPE, ERR_WORKSPACE, ERR_ALIGNMENT, ERR_LAUNCH = \
    -1, -2, -3, -4, -5, -6, -7

_c_i64, _c_i32, _c_vp, _c_sz = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol the headers under include/ declare
SYMBOLS = {
    'dlb_abi_version': (ctypes.c_int, []),
    'dlb_last_error': (ctypes.c_char_p, []),
    'dlb_fp8_gemm_workspace_bytes': (_c_sz, [_c_i64, _c_i64, _c_i64]),
    'dlb_fp8_gemm': (ctypes.c_int, [_c_vp] * 5 + [_c_i64] * 5 + [ctypes.c_int, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_gemm_noalloc': (ctypes.c_int, [_c_vp] * 5 + [_c_i64] * 5 + [ctypes.c_int, _c_vp]),
    'dlb_fp8_gemm_grouped_contiguous':
    (ctypes.c_int, [_c_vp] * 6 + [_c_i64] * 3 + [_c_i32] + [_c_i64] * 2 + [ctypes.c_int, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_gemm_grouped_contiguous_silu_quant':
    (ctypes.c_int, [_c_vp] * 7 + [_c_i64] * 3 + [_c_i32] + [_c_i64] * 4 + [ctypes.c_float, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_gemm_grouped_contiguous_gather_silu_quant':
    (ctypes.c_int, [_c_vp] * 8 + [_c_i64] * 4 + [_c_i32] + [_c_i64] * 4 + [ctypes.c_float, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_gemm_grouped_masked_silu_quant':
    (ctypes.c_int, [_c_vp] * 7 + [_c_i32] + [_c_i64] * 3 + [_c_i32] + [_c_i64] * 6 + [ctypes.c_float, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_gemm_grouped_masked':
    (ctypes.c_int, [_c_vp] * 6 + [_c_i32] + [_c_i64] * 3 + [_c_i32] + [_c_i64] * 3 + [ctypes.c_int, _c_vp, _c_sz, _c_vp]),
    'dlb_fp8_quant_1x128': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp, _c_vp] + [_c_i64] * 5 + [ctypes.c_float, _c_vp]),
    'dlb_fp8_quant_group': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp, _c_vp] + [_c_i64] * 6 + [ctypes.c_float, _c_vp]),
    'dlb_fp8_quant_128x128': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp, _c_vp] + [_c_i64] * 4 + [ctypes.c_float, _c_vp]),
    'dlb_fp8_gemm_force_variant': (ctypes.c_int, [ctypes.c_int]),
    'dlb_fp8_gemm_tune': (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    'dlb_fp8_gemm_variant_name': (ctypes.c_char_p, [ctypes.c_int]),
    'dlb_fp8_gemm_plan': (ctypes.c_int, [ctypes.c_int, _c_i64, _c_i64, _c_i64, _c_sz, ctypes.c_int] + [ctypes.POINTER(ctypes.c_int)] * 3 +
                          [ctypes.POINTER(_c_i64)]),
    'dlb_fp8_gemm_plan_grouped': (ctypes.c_int, [ctypes.c_int, _c_i64, _c_i64, _c_i64, ctypes.c_int32, ctypes.c_int32, _c_sz, ctypes.c_int,
                                                ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    'dlb_silu_mul': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp] + [_c_i64] * 4 + [_c_vp]),
    'dlb_silu_mul_quant': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp, _c_vp] + [_c_i64] * 5 + [ctypes.c_float, _c_vp]),
    'dlb_silu_mul_quant_masked': (ctypes.c_int, [_c_vp, ctypes.c_int, _c_vp, _c_vp, _c_vp] + [_c_i64] * 6 + [_c_vp]),
    'dlb_ep_scatter_workspace_bytes': (_c_sz, [_c_i64, _c_i64, _c_i64]),
    'dlb_ep_scatter':
    (ctypes.c_int, [_c_vp, _c_i64, _c_vp, _c_i64, _c_i64, _c_vp, ctypes.c_int, _c_i64, _c_i64, _c_vp, _c_vp, ctypes.c_int, _c_vp,
                    _c_i64, _c_vp, _c_i64, _c_i64, _c_vp, _c_i64, _c_vp, ctypes.c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
                    _c_i64, _c_vp, _c_sz, _c_vp]),
    'dlb_ep_scatter_rows':
    (ctypes.c_int, [_c_vp, ctypes.c_int, _c_i64, _c_i64, _c_vp, _c_vp, ctypes.c_int, _c_vp, _c_vp, _c_i64, _c_vp, ctypes.c_int,
                    _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_vp, _c_sz, _c_vp]),
    'dlb_ep_gather':
    (ctypes.c_int, [_c_vp, ctypes.c_int, _c_i64, _c_vp, ctypes.c_int, _c_i64, _c_i64, _c_vp, _c_i64, _c_i64, _c_vp, ctypes.c_int,
                    _c_i64, _c_i64, _c_vp, ctypes.c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_vp]),
    'dlb_scale_relayout': (ctypes.c_int, [_c_vp, _c_vp] + [_c_i64] * 5 + [_c_vp]),
}

_lock = threading.Lock()
_lib = None
_workspaces = {}


def library_path() -> str:
    return os.environ.get('DLBLAS_AMD_LIB', LIB_PATH)


def loaded() -> bool:
    """Whether load() has already brought the shared library in (never loads it)."""
    return _lib is not None


def load() -> ctypes.CDLL:
    """Load the shared library once; ImportError (never a silent fallback) when it is missing or stale."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise ImportError(f'{path} has not been built; run `python -m dlblas_amd._build` '
                              '(needs hipcc) - there is no fallback implementation')
        try:
            lib = ctypes.CDLL(path)
        except OSError as exc:
            raise ImportError(f'cannot load {path}: {exc}') from exc
        for name, (restype, argtypes) in SYMBOLS.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise ImportError(f'{path} does not export {name}; rebuild it') from None
            fn.restype, fn.argtypes = restype, argtypes
        if lib.dlb_abi_version() != ABI_VERSION:
            raise ImportError(f'{path} has ABI version {lib.dlb_abi_version()}, expected {ABI_VERSION}; rebuild it')
        _lib = lib
    return _lib


def last_error() -> str:
    return load().dlb_last_error().decode()


def check(rc: int) -> None:
    """Map a negative return code of the C ABI to a Python exception."""
    if rc == 0:
        return
    msg = f'dlblas fp8_gemm error {rc}: {last_error()}'
    if rc in (ERR_BAD_SHAPE, ERR_BAD_STRIDE, ERR_BAD_DTYPE, ERR_NULL_POINTER, ERR_ALIGNMENT):
        raise ValueError(msg)
    raise RuntimeError(msg)


def workspace(device: torch.device, stream_handle: int) -> torch.Tensor:
    """Zero-initialised scratch buffer, one per (device, stream): calls on one stream never overlap."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle)
    buf = _workspaces.get(key)
    if buf is None:
        buf = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def prepare(device=None, stream=None) -> None:
    """Do now, on (device, stream), everything a first call would do lazily: load the library, allocate the workspace
    of that (device, stream) pair and look up the device address of the static scratch of dlb_fp8_gemm_noalloc (one tiny
    GEMM through it).  Call it before capturing a HIP graph on `stream` or entering a loop that must not allocate; the
    calls captured or made afterwards allocate nothing in this package (torch still allocates outputs that the callee
    owns).  `stream` is a torch.cuda.Stream (default: the current one)."""
    lib = load()
    dev = torch.device('cuda', torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        st = torch.cuda.current_stream(dev) if stream is None else stream
        with torch.cuda.stream(st):
            workspace(dev, st.cuda_stream)
            a = torch.zeros(16, 128, dtype=torch.uint8, device=dev)
            s = torch.ones(16, 1, dtype=torch.float32, device=dev)
            c = torch.empty(16, 16, dtype=torch.float32, device=dev)
            check(lib.dlb_fp8_gemm_noalloc(_ptr(a), _ptr(a), _ptr(s), _ptr(s), _ptr(c), 16, 16, 128, 1, 1, OUT_F32,
                                           ctypes.c_void_p(st.cuda_stream)))
        st.synchronize()


_variant_names = None


def variant_names():
    global _variant_names
    if _variant_names is None:
        lib = load()
        names, i = [], 0
        while True:
            name = lib.dlb_fp8_gemm_variant_name(i)
            if name is None:
                break
            names.append(name.decode())
            i += 1
        _variant_names = names
    return list(_variant_names)


def plan(mode: int, rows: int, N: int, K: int, workspace_bytes: int = None, compute_units: int = 256):
    """(variant name, K slices, decode columns per workgroup) the library would use; touches no GPU."""
    return plan_full(mode, rows, N, K, workspace_bytes, compute_units)[:3]


def plan_full(mode: int, rows: int, N: int, K: int, workspace_bytes: int = None, compute_units: int = 256):
    """plan() plus the first column of the narrow tiles of the mixed-width prefill launch (N: all tiles equal)."""
    lib = load()
    v, s, c, n = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
    ws = WORKSPACE_BYTES if workspace_bytes is None else workspace_bytes
    check(lib.dlb_fp8_gemm_plan(mode, rows, N, K, ws, compute_units, ctypes.byref(v), ctypes.byref(s), ctypes.byref(c),
                                ctypes.byref(n)))
    return variant_names()[v.value], s.value, c.value, n.value


def plan_grouped(mode: int, rows: int, N: int, K: int, G: int, expected_m: int = -1, workspace_bytes: int = None,
                 compute_units: int = 256):
    """(variant name, tile lists used) of a grouped launch (mode 1 contiguous, 2 masked) with G experts and the masked
    layout's hint; touches no GPU."""
    lib = load()
    v, t = ctypes.c_int(), ctypes.c_int()
    ws = WORKSPACE_BYTES if workspace_bytes is None else workspace_bytes
    check(lib.dlb_fp8_gemm_plan_grouped(mode, rows, N, K, G, expected_m, ws, compute_units, ctypes.byref(v), ctypes.byref(t)))
    return variant_names()[v.value], bool(t.value)


def force_variant(name_or_id) -> None:
    """Pin the kernel variant used by later calls from this thread (None or -1: back to the heuristic)."""
    lib = load()
    if name_or_id is None:
        name_or_id = -1
    if isinstance(name_or_id, str):
        name_or_id = variant_names().index(name_or_id)
    check(lib.dlb_fp8_gemm_force_variant(int(name_or_id)))


KNOBS = {'splitk': 0, 'skinny_waves': 1, 'skinny_unroll': 2, 'skinny_nfrags': 3, 'group_m': 4, 'skinny_dma': 5, 'epilogue': 6, 'skinny_bn': 7,
         'splitk_mode': 8, 'spin_limit': 9, 'scale_table': 10, 'lds_oversize': 11, 'masked_grid': 12, 'tile_list': 13}


def tune(knob: str, value) -> None:
    """Set a tuning knob for later calls from this thread (None or 0: back to the heuristic)."""
    check(load().dlb_fp8_gemm_tune(KNOBS[knob], int(value or 0)))


def force_splitk(splitk) -> None:
    tune('splitk', splitk)


def out_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return OUT_BF16
    if dtype == torch.float32:
        return OUT_F32
    raise ValueError(f'fp8_gemm output dtype must be bfloat16 or float32, got {dtype}')


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def _stream_and_ws(t: torch.Tensor):
    stream = torch.cuda.current_stream(t.device).cuda_stream
    ws = workspace(t.device, stream)
    return stream, ws


def _require_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError('dlblas fp8_gemm runs on the GPU only; got a tensor on ' + str(t.device))


def gemm_dense(a, b, a_s, b_s, c, M, N, K, as_sm, as_sk):
    _require_gpu(a, b, a_s, b_s, c)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        check(lib.dlb_fp8_gemm(_ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(c), M, N, K, as_sm, as_sk,
                               out_code(c.dtype), _ptr(ws), ws.numel(), ctypes.c_void_p(stream)))


def gemm_contiguous(a, b, a_s, b_s, c, m_indices, M_sum, N, K, G, as_sm, as_sk):
    _require_gpu(a, b, a_s, b_s, c, m_indices)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        check(
            lib.dlb_fp8_gemm_grouped_contiguous(_ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(c), _ptr(m_indices),
                                                M_sum, N, K, G, as_sm, as_sk, out_code(c.dtype), _ptr(ws),
                                                ws.numel(), ctypes.c_void_p(stream)))


def gemm_contiguous_silu_quant(a, b, a_s, b_s, out_q, out_s, m_indices, M_sum, N, K, G, as_sm, as_sk, eps) -> bool:
    """The fused gate/up GEMM + silu * up + 1 x 128 quantiser.  False when the library has no fused kernel for the
    shape (ERR_BAD_SHAPE): nothing was enqueued and the caller runs the steps apart."""
    _require_gpu(a, b, a_s, b_s, out_q, out_s, m_indices)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        rc = lib.dlb_fp8_gemm_grouped_contiguous_silu_quant(_ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(out_q), _ptr(out_s),
                                                            _ptr(m_indices), M_sum, N, K, G, as_sm, as_sk, out_s.stride(0),
                                                            out_s.stride(1), float(eps), _ptr(ws), ws.numel(),
                                                            ctypes.c_void_p(stream))
        if rc == ERR_BAD_SHAPE:
            return False
        check(rc)
        return True


def gemm_contiguous_gather_silu_quant(a, b, a_s, b_s, out_q, out_s, m_indices, a_row_index, N, K, G, eps) -> bool:
    """gemm_contiguous_silu_quant whose row r is row a_row_index[r] of a / a_s.  False when the library declines the shape."""
    _require_gpu(a, b, a_s, b_s, out_q, out_s, m_indices, a_row_index)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        rc = lib.dlb_fp8_gemm_grouped_contiguous_gather_silu_quant(
            _ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(out_q), _ptr(out_s), _ptr(m_indices), _ptr(a_row_index), a.size(0),
            m_indices.numel(), N, K, G, a_s.stride(0), a_s.stride(1), out_s.stride(0), out_s.stride(1), float(eps), _ptr(ws),
            ws.numel(), ctypes.c_void_p(stream))
        if rc == ERR_BAD_SHAPE:
            return False
        check(rc)
        return True


def gemm_masked(a, b, a_s, b_s, c, masked_m, expected_m, M_max, N, K, G, as_sg, as_sm, as_sk):
    _require_gpu(a, b, a_s, b_s, c, masked_m)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        check(
            lib.dlb_fp8_gemm_grouped_masked(_ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(c), _ptr(masked_m),
                                            int(expected_m), M_max, N, K, G, as_sg, as_sm, as_sk,
                                            out_code(c.dtype), _ptr(ws), ws.numel(), ctypes.c_void_p(stream)))


def gemm_masked_silu_quant(a, b, a_s, b_s, out_q, out_s, masked_m, expected_m, M_max, N, K, G, as_sg, as_sm, as_sk, eps) -> bool:
    """The fused masked gate/up GEMM + up * silu(gate) + 1 x 128 quantiser.  False when the library has no fused kernel
    for the shape (ERR_BAD_SHAPE): nothing was enqueued and the caller runs the steps apart."""
    _require_gpu(a, b, a_s, b_s, out_q, out_s, masked_m)
    lib = load()
    with torch.cuda.device(a.device):
        stream, ws = _stream_and_ws(a)
        rc = lib.dlb_fp8_gemm_grouped_masked_silu_quant(_ptr(a), _ptr(b), _ptr(a_s), _ptr(b_s), _ptr(out_q), _ptr(out_s),
                                                        _ptr(masked_m), int(expected_m), M_max, N, K, G, as_sg, as_sm, as_sk,
                                                        out_s.stride(0), out_s.stride(1), out_s.stride(2), float(eps),
                                                        _ptr(ws), ws.numel(), ctypes.c_void_p(stream))
        if rc == ERR_BAD_SHAPE:
            return False
        check(rc)
        return True


IN_CODES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def quant_group(x2d, q, s, rows, K, group_size, x_row_stride, s_stride_m, s_stride_k, eps):
    _require_gpu(x2d, q, s)
    lib = load()
    with torch.cuda.device(x2d.device):
        stream = torch.cuda.current_stream(x2d.device).cuda_stream
        check(
            lib.dlb_fp8_quant_group(_ptr(x2d), IN_CODES[x2d.dtype], _ptr(q), _ptr(s), rows, K, group_size, x_row_stride, s_stride_m,
                                    s_stride_k, float(eps), ctypes.c_void_p(stream)))


def quant_1x128(x2d, q, s, rows, K, x_row_stride, s_stride_m, s_stride_k, eps):
    quant_group(x2d, q, s, rows, K, 128, x_row_stride, s_stride_m, s_stride_k, eps)


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def silu_mul(x2d, out2d, rows, N):
    lib = load()
    _require_gpu(x2d, out2d)
    with torch.cuda.device(x2d.device):
        check(lib.dlb_silu_mul(_ptr(x2d), IN_CODES[x2d.dtype], _ptr(out2d), rows, N, x2d.stride(0), out2d.stride(0), _stream(x2d)))


def silu_mul_quant(x2d, q, s, rows, N, s_stride_m, s_stride_k, eps):
    lib = load()
    _require_gpu(x2d, q, s)
    with torch.cuda.device(x2d.device):
        check(lib.dlb_silu_mul_quant(_ptr(x2d), IN_CODES[x2d.dtype], _ptr(q), _ptr(s), rows, N, x2d.stride(0), s_stride_m,
                                     s_stride_k, float(eps), _stream(x2d)))


def silu_mul_quant_masked(x, q, s, masked_m, G, M_max, N, s_strides):
    lib = load()
    _require_gpu(x, q, s, masked_m)
    with torch.cuda.device(x.device):
        check(lib.dlb_silu_mul_quant_masked(_ptr(x), IN_CODES[x.dtype], _ptr(q), _ptr(s), _ptr(masked_m), G, M_max, N,
                                            s_strides[0], s_strides[1], s_strides[2], _stream(x)))


IDX_CODES = {torch.int32: 0, torch.int64: 1}


def _idx_code(t: torch.Tensor) -> int:
    try:
        return IDX_CODES[t.dtype]
    except KeyError:
        raise TypeError(f'index tensors must be int32 or int64, got {t.dtype}') from None


def ep_scatter_args(recv_x, recv_x_scale, recv_topk, counts, expert_start_loc, out, out_scale, m_indices, output_index):
    """Marshalled argument tuple of dlb_ep_scatter on the current stream (kept by callers that launch repeatedly)."""
    lib = load()
    _require_gpu(recv_x, recv_x_scale, recv_topk, counts, expert_start_loc, out, out_scale, m_indices, output_index)
    T, H = recv_x.shape
    topk = recv_topk.shape[1]
    E = counts.shape[0]
    stream, ws = _stream_and_ws(recv_x)
    need = lib.dlb_ep_scatter_workspace_bytes(T, topk, E)
    if need > ws.numel():
        raise ValueError(f'ep_scatter needs {need} bytes of workspace, the per-stream buffer holds {ws.numel()}')
    return (_ptr(recv_x), recv_x.stride(0), _ptr(recv_x_scale), recv_x_scale.stride(0), recv_x_scale.stride(1), _ptr(recv_topk),
            _idx_code(recv_topk), recv_topk.stride(0), recv_topk.stride(1), _ptr(counts), _ptr(expert_start_loc),
            _idx_code(expert_start_loc), _ptr(out), out.stride(0), _ptr(out_scale), out_scale.stride(0), out_scale.stride(1),
            _ptr(m_indices), m_indices.numel(), _ptr(output_index), _idx_code(output_index), output_index.stride(0),
            output_index.stride(1), T, H, topk, E, _ptr(ws), ws.numel(), ctypes.c_void_p(stream))


def ep_scatter(recv_x, recv_x_scale, recv_topk, counts, expert_start_loc, out, out_scale, m_indices, output_index):
    with torch.cuda.device(recv_x.device):
        check(load().dlb_ep_scatter(*ep_scatter_args(recv_x, recv_x_scale, recv_topk, counts, expert_start_loc, out, out_scale,
                                                     m_indices, output_index)))


def ep_scatter_rows(recv_topk, counts, expert_start_loc, m_indices, src_row, output_index):
    """dlb_ep_scatter_rows: the tables of ep_scatter and the source token of every destination row; no row is moved."""
    lib = load()
    _require_gpu(recv_topk, counts, expert_start_loc, m_indices, src_row, output_index)
    T, topk = recv_topk.shape
    E = counts.shape[0]
    with torch.cuda.device(recv_topk.device):
        stream, ws = _stream_and_ws(recv_topk)
        need = lib.dlb_ep_scatter_workspace_bytes(T, topk, E)
        if need > ws.numel():
            raise ValueError(f'ep_scatter needs {need} bytes of workspace, the per-stream buffer holds {ws.numel()}')
        check(lib.dlb_ep_scatter_rows(_ptr(recv_topk), _idx_code(recv_topk), recv_topk.stride(0), recv_topk.stride(1), _ptr(counts),
                                      _ptr(expert_start_loc), _idx_code(expert_start_loc), _ptr(m_indices), _ptr(src_row),
                                      m_indices.numel(), _ptr(output_index), _idx_code(output_index), output_index.stride(0),
                                      output_index.stride(1), T, topk, E, _ptr(ws), ws.numel(), ctypes.c_void_p(stream)))


def ep_gather_args(inp, topk_ids, topk_weight, index, out):
    _require_gpu(inp, topk_ids, topk_weight, index, out)
    T, H = out.shape
    return (_ptr(inp), IN_CODES[inp.dtype], inp.stride(0), _ptr(topk_ids), _idx_code(topk_ids), topk_ids.stride(0),
            topk_ids.stride(1), _ptr(topk_weight), topk_weight.stride(0), topk_weight.stride(1), _ptr(index), _idx_code(index),
            index.stride(0), index.stride(1), _ptr(out), IN_CODES[out.dtype], out.stride(0), T, H, topk_ids.shape[1], _stream(inp))


def ep_gather(inp, topk_ids, topk_weight, index, out):
    with torch.cuda.device(inp.device):
        check(load().dlb_ep_gather(*ep_gather_args(inp, topk_ids, topk_weight, index, out)))


def scale_relayout(src, dst, rows, kblocks, rows_pad):
    lib = load()
    _require_gpu(src, dst)
    with torch.cuda.device(src.device):
        check(lib.dlb_scale_relayout(_ptr(src), _ptr(dst), rows, kblocks, rows_pad, src.stride(0), src.stride(1), _stream(src)))


def quant_128x128(w3d, q, s, G, N, K, eps):
    lib = load()
    _require_gpu(w3d, q, s)
    with torch.cuda.device(w3d.device):
        check(lib.dlb_fp8_quant_128x128(_ptr(w3d), IN_CODES[w3d.dtype], _ptr(q), _ptr(s), G, N, K, w3d.stride(-2), float(eps),
                                        _stream(w3d)))
