"""The shape planner, queried on the host (dlb_fp8_gemm_plan launches nothing): invariants over a sweep of shapes and
the choices the design documents.  Runs without a GPU."""
import itertools

import pytest

from dlblas_amd import _lib

DENSE, CONTIGUOUS, MASKED = 0, 1, 2
RING = ('pipe256x256', 'pipe128x256w8', 'pipe256mix', 'pipe128x128', 'pipe128x64')
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
    v, s, _ = _lib.plan(DENSE, 64, 2112, 7168)                           # the same from 64 rows up ...
    assert v in RING and s > 1
    assert _lib.plan(DENSE, 33, 7168, 2048)[0] == 'skinny64'             # ... a wide weight matrix streams
    assert _lib.plan(DENSE, 64, 7168, 2048)[0] == 'skinny64'
    v, s, _ = _lib.plan(DENSE, 256, 7168, 16384)
    assert v in RING and s > 1
    assert _lib.plan(DENSE, 256, 7168, 2048) == ('pipe128x64', 1, 0)
    # prefill-sized: 256-row tiles unless their rows are mostly padding, they leave a round half empty or K is short
    assert _lib.plan(DENSE, 512, 18432, 7168) == ('pipe256mix', 1, 0)
    assert _lib.plan(DENSE, 384, 18432, 7168) == ('pipe128x256w8', 1, 0)  # two 256-row tiles, but three of 128 rows
    assert _lib.plan(DENSE, 2048, 4096, 7168) == ('pipe128x256w8', 1, 0)  # 128 tiles of 256 x 256 on 256 CUs
    assert _lib.plan(DENSE, 4096, 4096, 7168) == ('pipe256mix', 1, 0)
    assert _lib.plan(DENSE, 4096, 32768, 512) == ('pipe128x256w8', 1, 0)  # four K blocks: the tile's fixed part decides
    assert _lib.plan(DENSE, 48, 4096, 7168)[0] == 'skinny64'             # few rows stream even a narrow weight matrix
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
    assert lib.dlb_fp8_gemm_plan(7, 1, 1, 1, 0, 256, None, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, -1, 1, 1, 0, 256, None, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, 1, 1, 1, 0, 0, None, None, None, None) == _lib.ERR_BAD_SHAPE
    assert lib.dlb_fp8_gemm_plan(0, 16, 7168, 2048, 0, 256, None, None, None, None) == 0


def test_k_slices_are_what_a_launch_uses():
    """The plan query runs the code a launch runs: the slice-count knob, the no-empty-slice rule and the workspace
    clamp all show in its answer."""
    try:
        for want in (2, 3, 5, 7, 16):
            _lib.tune('splitk', want)
            v, s, _ = _lib.plan(DENSE, 200, 392, 2048)                       # 16 K blocks
            per = -(-16 // min(want, 16))
            assert s == -(-16 // per), (want, v, s)                          # slices of `per` blocks, none empty
            assert _lib.plan(DENSE, 200, 392, 2048, workspace_bytes=0)[1] == 1
            # a workspace that holds exactly two partial matrices (plus the re-laid scales of the ring kernels)
            tight = _lib.WS_COUNTER_BYTES + 2 * 200 * 392 * 4 + 16 * 200 * 4 + 512
            assert _lib.plan(DENSE, 200, 392, 2048, workspace_bytes=tight)[1] <= 2
        _lib.tune('splitk', 0)
        _lib.force_variant('pipe256mix')
        _lib.tune('splitk', 4)
        assert _lib.plan(DENSE, 4096, 7168, 2048)[1] == 1                    # the mixed-width launch never splits K
    finally:
        _lib.tune('splitk', 0)
        _lib.force_variant(None)


def test_mixed_width_split_matches_a_tile_by_tile_simulation():
    """The closed-form makespan behind the choice of the narrow-tile region against the obvious simulation: tiles handed
    out one by one to the worker that is free first."""
    import heapq

    def makespan(ta, tb, cb, workers):
        free = [0.0] * workers
        end = 0.0
        for t in range(ta + tb):
            done = heapq.heappop(free) + (1.0 if t < ta else cb)
            heapq.heappush(free, done)
            end = max(end, done)
        return end

    def pick(M, N, cus):
        tm = -(-M // 256)
        if tm * -(-N // 256) > 16 * cus:
            return N
        uniform = makespan(tm * -(-N // 256), 0, 0.78, cus)
        best, best_split = uniform, N
        for ca in range(N // 256, -1, -1):
            split = ca * 256
            if split >= N:
                continue
            t = makespan(tm * ca, tm * -(-(N - split) // 192), 0.78, cus)
            if t < best - 1e-6 and t < 0.96 * uniform:
                best, best_split = t, split
        return best_split

    _lib.force_variant('pipe256mix')
    try:
        for M, N, cus in [(4096, 7168, 256), (4096, 24576, 256), (2048, 7168, 256), (4096, 4096, 256), (1024, 2112, 80),
                          (300, 7168, 64), (8192, 1536, 256), (4000, 5000, 304), (512, 16384, 256), (256, 256, 256)]:
            assert _lib.plan_full(DENSE, M, N, 2048, compute_units=cus)[3] == pick(M, N, cus), (M, N, cus)
    finally:
        _lib.force_variant(None)
    assert _lib.plan_full(DENSE, 4096, 7168, 18432) == ('pipe256mix', 1, 0, 4096)
    assert _lib.plan_full(DENSE, 16, 7168, 2048)[3] == 7168


def test_planning_a_thousand_prefill_shapes_is_cheap():
    """A serving loop sees a new M with almost every prefill request: the planner keeps no per-shape state and has to
    answer in microseconds.  1000 distinct (M, N), each planned once; 20 us per plan on average including the ctypes
    call."""
    import ctypes
    import time
    shapes = [(257 + 37 * i, (1536, 2112, 4096, 7168, 18432, 24576)[i % 6] + 128 * (i % 7)) for i in range(1000)]
    assert len(set(shapes)) == 1000
    lib = _lib.load()
    v, s, c, n = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
    outs = (ctypes.byref(v), ctypes.byref(s), ctypes.byref(c), ctypes.byref(n))
    lib.dlb_fp8_gemm_plan(DENSE, 4096, 7168, 18432, _lib.WORKSPACE_BYTES, 256, *outs)
    best = 1.0
    for _ in range(3):  # best of three passes: the machine running the test is shared
        t0 = time.perf_counter()
        for M, N in shapes:
            lib.dlb_fp8_gemm_plan(DENSE, M, N, 7168, _lib.WORKSPACE_BYTES, 256, *outs)
        best = min(best, (time.perf_counter() - t0) / len(shapes))
    assert best < 20e-6, f'{best * 1e6:.1f} us per plan'


def test_shapes_beyond_32_bit_dma_offsets_take_the_64_bit_kernels():
    assert _lib.plan(DENSE, 4096, 4096, 1 << 24)[0] == 'tile128x128'
    assert _lib.plan(DENSE, 4096, 4096, (1 << 24) - 128)[0] in RING
    assert _lib.plan(CONTIGUOUS, 1024, 4096, 1 << 24)[0] == 'tile128x128'
    assert _lib.plan(DENSE, 16, 4096, 1 << 24)[0] == 'skinny16'              # its register-load form: 64-bit addressing
    lib = _lib.load()
    assert lib.dlb_fp8_gemm_plan(0, 1 << 31, 1, 1, 0, 256, None, None, None, None) == _lib.ERR_BAD_SHAPE


def test_decode_wave_count_is_clamped_to_the_lds():
    """16 waves x 16 fragments would need 256 KB for the partial sums of a 128-row decode launch: the knob is honoured
    only as far as the 160 KB of LDS allow (the launch itself is exercised on the GPU)."""
    try:
        _lib.tune('skinny_waves', 16)
        assert _lib.plan(DENSE, 128, 7168, 2048)[0] == 'skinny128'
    finally:
        _lib.tune('skinny_waves', 0)
