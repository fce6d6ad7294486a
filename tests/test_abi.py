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


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setenv('DLBLAS_AMD_LIB', str(tmp_path / 'nope.so'))
    with pytest.raises(ImportError, match='no fallback'):
        _lib.load()
