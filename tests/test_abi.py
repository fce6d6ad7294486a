"""The C ABI library loads on a machine without a GPU and exports exactly what the headers under include/ declare.
No compute entry point is called with real work here."""
import ctypes
import os
import re

import pytest

from dlblas_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'dlblas_fp8_gemm.h')


HEADERS = [HEADER, os.path.join(ROOT, 'include', 'dlblas_fp8_moe.h')]


def _declared_functions():
    text = ''.join(open(h).read() for h in HEADERS)
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(dlb_[a-z0-9_]+)\s*\(', text)))


def test_header_and_binding_table_agree():
    assert _declared_functions() == sorted(_lib.SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared_functions():
        assert hasattr(lib, name), name
    assert lib.dlb_abi_version() == _lib.ABI_VERSION
    header = open(HEADER).read()
    assert int(re.search(r'#define DLB_ABI_VERSION (\d+)', header).group(1)) == _lib.ABI_VERSION
    assert int(re.search(r'#define DLB_WS_COUNTER_BYTES (\d+)', header).group(1)) == _lib.WS_COUNTER_BYTES


def test_error_codes_match_header():
    header = open(HEADER).read()
    for name in ('NULL_POINTER', 'BAD_SHAPE', 'BAD_STRIDE', 'BAD_DTYPE', 'WORKSPACE', 'ALIGNMENT', 'LAUNCH'):
        value = int(re.search(rf'#define DLB_ERR_{name} \((-\d+)\)', header).group(1))
        assert getattr(_lib, f'ERR_{name}') == value


def test_knob_ids_match_header():
    header = open(HEADER).read()
    ids = {m.group(1).lower(): int(m.group(2)) for m in re.finditer(r'#define DLB_KNOB_([A-Z_]+) (\d+)', header)}
    assert ids == _lib.KNOBS
    lib = _lib.load()
    for knob in ids.values():
        assert lib.dlb_fp8_gemm_tune(knob, 0) == 0
    assert lib.dlb_fp8_gemm_tune(max(ids.values()) + 1, 0) == _lib.ERR_BAD_SHAPE and 'knob' in _lib.last_error()


def test_host_only_entry_points():
    lib = _lib.load()
    assert _lib.variant_names()[0] == 'exact' and 'tile128x128' in _lib.variant_names()
    assert lib.dlb_fp8_gemm_variant_name(10_000) is None
    assert lib.dlb_fp8_gemm_force_variant(10_000) == _lib.ERR_BAD_SHAPE and 'variant' in _lib.last_error()
    assert lib.dlb_fp8_gemm_force_variant(-1) == 0
    assert lib.dlb_fp8_gemm_workspace_bytes(0, 0, 0) == _lib.WS_COUNTER_BYTES
    for rows, n, k in ((16, 7168, 2048), (128, 2112, 7168), (4096, 7168, 18432), (1 << 20, 1 << 20, 128)):
        need = lib.dlb_fp8_gemm_workspace_bytes(rows, n, k)
        assert _lib.WS_COUNTER_BYTES <= need <= _lib.WORKSPACE_BYTES


def test_argument_validation_rejects_before_touching_the_device():
    """Bad arguments are refused on the host: nothing is launched, so this runs without a GPU."""
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(4096)
    rc = lib.dlb_fp8_gemm(fake, fake, fake, fake, fake, 8, 8, 128, 1, 1, 7, null, 0, null)
    assert rc == _lib.ERR_BAD_DTYPE and 'out_dtype' in _lib.last_error()
    rc = lib.dlb_fp8_gemm(fake, fake, fake, fake, fake, -1, 8, 128, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_BAD_SHAPE
    rc = lib.dlb_fp8_gemm(fake, fake, fake, fake, null, 8, 8, 128, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_NULL_POINTER
    rc = lib.dlb_fp8_gemm(null, fake, fake, fake, fake, 8, 8, 128, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_NULL_POINTER
    rc = lib.dlb_fp8_gemm(fake, fake, fake, fake, fake, 8, 8, 256, 0, 1, 0, null, 0, null)
    assert rc == _lib.ERR_BAD_STRIDE
    rc = lib.dlb_fp8_gemm(ctypes.c_void_p(4100), fake, fake, fake, fake, 8, 8, 128, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_ALIGNMENT
    rc = lib.dlb_fp8_gemm_grouped_contiguous(fake, fake, fake, fake, fake, null, 128, 8, 128, 2, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_NULL_POINTER and 'm_indices' in _lib.last_error()
    rc = lib.dlb_fp8_gemm_grouped_masked(fake, fake, fake, fake, fake, fake, 0, 128, 8, 100, 2, 1, 1, 1, 0, null, 0, null)
    assert rc == _lib.ERR_BAD_SHAPE and 'K % 16' in _lib.last_error()
    # empty problems succeed without work
    assert lib.dlb_fp8_gemm(null, null, null, null, null, 0, 8, 128, 1, 1, 0, null, 0, null) == 0
    with pytest.raises(ValueError):
        _lib.check(_lib.ERR_BAD_SHAPE)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.ERR_LAUNCH)


def test_moe_entry_points_validate_on_the_host():
    """The quantisers and the MoE steps refuse bad arguments before any launch (no GPU needed)."""
    lib = _lib.load()
    null, fake = ctypes.c_void_p(0), ctypes.c_void_p(4096)
    assert lib.dlb_fp8_quant_1x128(fake, 0, fake, fake, 4, 100, 100, 1, 1, 1e-10, null) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_quant_1x128(fake, 9, fake, fake, 4, 128, 128, 1, 1, 1e-10, null) == _lib.ERR_BAD_DTYPE
    assert lib.dlb_fp8_quant_128x128(fake, 0, fake, fake, 1, 128, 132, 132, 1e-10, null) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_quant_128x128(fake, 0, fake, null, 1, 128, 128, 128, 1e-10, null) == _lib.ERR_NULL_POINTER
    assert lib.dlb_fp8_quant_128x128(fake, 0, fake, fake, 1, 128, 128, 64, 1e-10, null) == _lib.ERR_BAD_STRIDE
    assert lib.dlb_fp8_quant_128x128(null, 0, null, null, 0, 128, 128, 128, 1e-10, null) == 0
    assert lib.dlb_silu_mul(fake, 3, fake, 4, 128, 256, 128, null) == _lib.ERR_BAD_DTYPE
    assert lib.dlb_silu_mul(fake, 0, fake, 4, 128, 128, 128, null) == _lib.ERR_BAD_STRIDE
    assert lib.dlb_silu_mul(fake, 0, null, 4, 128, 256, 128, null) == _lib.ERR_NULL_POINTER
    assert lib.dlb_silu_mul_quant(fake, 0, fake, fake, 4, 200, 400, 2, 1, 1e-10, null) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_silu_mul_quant(ctypes.c_void_p(4100), 0, fake, fake, 4, 128, 256, 1, 1, 1e-10, null) == _lib.ERR_ALIGNMENT
    assert lib.dlb_silu_mul_quant_masked(fake, 0, fake, fake, null, 2, 4, 128, 4, 1, 1, null) == _lib.ERR_NULL_POINTER
    assert lib.dlb_silu_mul_quant_masked(fake, 0, fake, fake, fake, -1, 4, 128, 4, 1, 1, null) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_silu_mul_quant_masked(fake, 0, fake, fake, fake, 2, 4, 128, 4, -1, 1, null) == _lib.ERR_BAD_STRIDE
    # ep_scatter: hidden % 128, topk limit, workspace size, index dtypes
    def scatter(hidden=256, topk=8, experts=4, ws=fake, ws_bytes=1 << 20, topk_dtype=0, x=fake):
        return lib.dlb_ep_scatter(x, hidden, fake, hidden // 128, 1, fake, topk_dtype, topk, 1, fake, fake, 0, fake, hidden, fake,
                                  hidden // 128, 1, fake, 512, fake, 0, topk, 1, 16, hidden, topk, experts, ws, ws_bytes, null)
    assert scatter(hidden=200) == _lib.ERR_BAD_SHAPE
    assert scatter(topk=65) == _lib.ERR_BAD_SHAPE and '64' in _lib.last_error()
    assert scatter(experts=5000) == _lib.ERR_BAD_SHAPE
    assert scatter(topk_dtype=2) == _lib.ERR_BAD_DTYPE
    assert scatter(ws=null) == _lib.ERR_WORKSPACE and scatter(ws_bytes=8) == _lib.ERR_WORKSPACE
    assert scatter(x=ctypes.c_void_p(4100)) == _lib.ERR_ALIGNMENT
    assert scatter(experts=0) == 0
    need = lib.dlb_ep_scatter_workspace_bytes(8192, 8, 32)
    assert need == (32 + 2) * 8 + 256 * 32 * 4
    # ep_gather
    def gather(hidden=1024, topk=8, in_dtype=0, out=fake):
        return lib.dlb_ep_gather(fake, in_dtype, hidden, fake, 0, topk, 1, fake, topk, 1, fake, 0, topk, 1, out, 0, hidden, 16,
                                 hidden, topk, null)
    assert gather(hidden=1020) == _lib.ERR_BAD_SHAPE
    assert gather(topk=100) == _lib.ERR_BAD_SHAPE
    assert gather(in_dtype=5) == _lib.ERR_BAD_DTYPE
    assert gather(out=null) == _lib.ERR_NULL_POINTER
    assert lib.dlb_scale_relayout(fake, fake, 8, 4, 4, 4, 1, null) == _lib.ERR_BAD_SHAPE      # rows_pad < rows
    assert lib.dlb_scale_relayout(fake, null, 8, 4, 8, 4, 1, null) == _lib.ERR_NULL_POINTER
    assert lib.dlb_scale_relayout(null, null, 0, 0, 0, 1, 1, null) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setenv('DLBLAS_AMD_LIB', str(tmp_path / 'nope.so'))
    with pytest.raises(ImportError, match='no fallback'):
        _lib.load()
