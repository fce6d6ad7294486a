"""The shape planner, queried on the host (dlb_fp8_gemm_plan launches nothing): invariants over a sweep of shapes and
the choices the design documents.  Runs without a GPU."""
import itertools

import pytest

from dlblas_amd import _lib

DENSE, CONTIGUOUS, MASKED = 0, 1, 2
RING = ('pipe256x128', 'pipe128x256', 'pipe256x256', 'pipe128x256w8', 'pipe256mix', 'pipe128x128', 'pipe128x64')
DECODE = {'skinny16': 16, 'skinny32': 32, 'skinny64': 64, 'skinny128': 128}


@pytest.fixture(autouse=True)
def _heuristic():
    _lib.force_variant(None)
    for knob in _lib.KNOBS:
        _lib.tune(knob, 0)
    yield


def test_documented_choices():
    assert _lib.plan(DENSE, 4096, 7168, 18432) == ('pipe256mix', 1, 0)
    assert _lib.plan(DENSE, 4096, 24576, 1536) == ('pipe256mix', 1, 0)
    assert _lib.plan(DENSE, 16, 7168, 2048) == ('skinny16', 1, 28)      # 256 workgroups of 28 columns on 256 CUs
    assert _lib.plan(DENSE, 1, 2112, 7168) == ('skinny16', 1, 12)
    assert _lib.plan(DENSE, 16, 1536, 7168)[2] == 8
    assert _lib.plan(DENSE, 128, 7168, 2048)[0] == 'skinny128'          # wide N, short K: streaming wins
    v, s, _ = _lib.plan(DENSE, 128, 2112, 7168)                          # narrow N, long K: K split over workgroups
    assert v in RING and s > 1
    v, s, _ = _lib.plan(DENSE, 256, 7168, 16384)
    assert v in RING and s > 1
    assert _lib.plan(DENSE, 256, 7168, 2048) == ('pipe128x64', 1, 0)
    assert _lib.plan(DENSE, 17, 64, 200)[0] == 'exact'                   # K % 16 != 0
    assert _lib.plan(DENSE, 300, 200, 400)[0] == 'tile128x128'           # K tail: the register-staged kernel
    assert _lib.plan(CONTIGUOUS, 9728, 4096, 7168) == ('pipe128x256w8', 1, 0)
    assert _lib.plan(MASKED, 256, 7168, 2048) == ('pipe128x256w8', 1, 0)


def test_invariants_over_a_sweep():
    Ms = (1, 15, 16, 17, 33, 64, 65, 100, 128, 129, 200, 256, 300, 512, 1000, 2048, 4096, 10000)
    Ns = (8, 100, 128, 392, 1000, 1536, 2112, 4096, 7168, 24576)
    Ks = (16, 128, 200, 256, 400, 1024, 2048, 7168, 18432)
    for M, N, K, cus in itertools.product(Ms, Ns, Ks, (256, 80)):
        v, s, c = _lib.plan(DENSE, M, N, K, compute_units=cus)
        what = f'{M}x{N}x{K} on {cus} CUs -> {v}, {s} slices, {c} columns'
        if v in RING:
            assert K % 128 == 0, what                                    # the DMA path moves whole K blocks
        if v in DECODE:
            assert M <= DECODE[v] and s == 1, what
            assert c % 4 == 0 and 4 <= c <= 32, what
        else:
            assert c == 0, what
        assert 1 <= s <= 32, what
        if s > 1:
            assert v != 'pipe256mix' and v != 'exact', what
            assert s <= (K + 127) // 128, what
            assert s * M * N * 4 <= _lib.WORKSPACE_BYTES, what           # the partial matrices fit the workspace
    for mode, M, N, K in itertools.product((CONTIGUOUS, MASKED), (128, 256, 1024, 9728), (128, 4096, 7168), (128, 400, 2048, 7168)):
        v, s, c = _lib.plan(mode, M, N, K)
        assert s == 1 and c == 0 and v not in DECODE and v != 'exact' and v != 'pipe256mix', (mode, M, N, K, v)
        if K % 128:
            assert v not in RING


def test_without_workspace_nothing_is_split():
    for M, N, K in ((128, 2112, 7168), (256, 7168, 16384), (200, 392, 2048)):
        assert _lib.plan(DENSE, M, N, K, workspace_bytes=0)[1] == 1
        assert _lib.plan(DENSE, M, N, K, workspace_bytes=_lib.WS_COUNTER_BYTES)[1] == 1


def test_plan_follows_the_hooks_and_rejects_nonsense():
    _lib.force_variant('tile128x128')
    _lib.tune('splitk', 4)
    try:
        assert _lib.plan(DENSE, 200, 392, 2048)[0] == 'tile128x128'
    finally:
        _lib.force_variant(None)
        _lib.tune('splitk', 0)
    lib = _lib.load()
    assert lib.dlb_fp8_gemm_plan(7, 1, 1, 1, 0, 256, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, -1, 1, 1, 0, 256, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, 1, 1, 1, 0, 0, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, 16, 7168, 2048, 0, 256, None, None, None) == 0
