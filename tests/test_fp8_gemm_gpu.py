"""GPU parity of the HIP kernels (through the Python entry points -> C ABI) against the CPU oracle."""
import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def dev():
    import dlblas_amd  # noqa: F401
    from dlblas_amd import _lib
    _lib.load()
    return torch.device('cuda:0')


def _run_dense(dev, a_q, a_s, b_q, b_s, dtype=torch.bfloat16, variant=None):
    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        _lib.force_variant(variant)
        out = fp8_gemm(a_q.to(dev), b_q.to(dev), a_s.to(dev), b_s.to(dev))
        torch.cuda.synchronize()
    finally:
        _lib.force_variant(None)
        torch.set_default_dtype(prev)
    return out


DENSE_SHAPES = [
    (64, 512, 1024),      # the reference's CPU-runnable configuration
    (512, 512, 512),      # the shape of tests/kernels/test_fp8_gemm.py
    (1, 7168, 2048), (16, 7168, 2048), (64, 7168, 2048), (128, 7168, 2048),
    (1, 2112, 7168), (16, 2112, 7168), (64, 2112, 7168), (128, 2112, 7168),
    (16, 1000, 640), (1, 392, 896), (32, 520, 512),  # decode with 4 to 7 K blocks: 8 waves, some of them without a block
    (300, 2112, 1536),    # ragged M and N tiles
    (256, 7168, 2048), (384, 2112, 7168), (130, 7168, 16384),  # between decode and prefill: small tiles, K split over workgroups
    (129, 130, 384),      # N not a multiple of 4: scalar stores
    (33, 200, 400),       # K tail (400 = 3 * 128 + 16)
    (17, 64, 200),        # K not a multiple of 16: exact path
]


@pytest.mark.parametrize('M,N,K', DENSE_SHAPES)
def test_dense_bf16_matches_oracle(dev, M, N, K):
    print(f'case dense bf16 M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    out = _run_dense(dev, a_q, a_s, b_q, b_s)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
    helpers.tolerance_check(out, ref, f'dense {M}x{N}x{K}')


@pytest.mark.parametrize('variant', ['tile128x128', 'tile64x128', 'tile128x64', 'skinny16', 'skinny32', 'skinny64', 'skinny128', 'exact', 'pipe256x256', 'pipe128x256w8', 'pipe256mix', 'pipe128x128', 'pipe128x64'])
@pytest.mark.parametrize('M,N,K', [(16, 512, 1024), (30, 200, 400), (200, 392, 2048)])
def test_every_variant(dev, variant, M, N, K):
    print(f'case variant={variant} M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=7)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    out = _run_dense(dev, a_q, a_s, b_q, b_s, variant=variant)
    helpers.tolerance_check(out, ref, f'{variant} {M}x{N}x{K}')


@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('variant,splitk', [('tile128x128', 2), ('tile128x64', 5), ('tile64x128', 32), (None, 0), ('pipe128x256w8', 3),
                                            ('pipe128x128', 4), ('pipe128x64', 2), ('pipe256x256', 7)])
@pytest.mark.parametrize('M,N,K', [(128, 2112, 7168), (200, 392, 2048), (129, 130, 1040), (70, 131, 4096)])
def test_split_k_two_pass(dev, M, N, K, variant, splitk, out_dtype):
    """K split over workgroups: fp32 partial matrices in the workspace, a second kernel adds them in index order.
    (None, 0) is the library's own choice, which splits (128, 2112, 7168).  Two calls must agree bit for bit."""
    from dlblas_amd import _lib
    print(f'case split-K variant={variant} splitk={splitk} M={M} N={N} K={K} {out_dtype}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=11)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    try:
        _lib.force_splitk(splitk)
        out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=out_dtype, variant=variant)
        again = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=out_dtype, variant=variant)
    finally:
        _lib.force_splitk(0)
    assert out.dtype == out_dtype
    helpers.tolerance_check(out, ref, f'split-K {variant}/{splitk} {M}x{N}x{K}')
    assert torch.equal(out, again)


@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('variant,splitk', [('pipe128x64', 7), ('pipe128x64', 2), ('pipe128x128', 4), ('pipe128x128', 32), ('pipe128x256w8', 3),
                                            ('pipe256x256', 5)])
@pytest.mark.parametrize('M,N,K', [(128, 2112, 7168), (200, 392, 2048), (129, 130, 4096), (33, 64, 4096)])
def test_split_k_in_one_launch_equals_two_pass(dev, M, N, K, variant, splitk, out_dtype):
    """The K slices of a tile added by its own workgroups (arrival counter in the workspace head, bounded wait, slices
    summed in index order) give the bits of the two-pass path; so does the path in which nobody waits and the workgroup
    that completes a tile adds every share (spin limit 0).  Every call leaves the counter head all zero."""
    from dlblas_amd import _lib
    print(f'case one-launch split-K variant={variant} splitk={splitk} M={M} N={N} K={K} {out_dtype}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=13)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    head = _lib.workspace(dev, torch.cuda.current_stream().cuda_stream)[:_lib.WS_COUNTER_BYTES]
    outs = []
    try:
        _lib.force_splitk(splitk)
        for mode, spin in ((2, 0), (1, 0), (1, 1), (1, 0)):
            _lib.tune('splitk_mode', mode)
            _lib.tune('spin_limit', spin)
            outs.append(_run_dense(dev, a_q, a_s, b_q, b_s, dtype=out_dtype, variant=variant))
            assert int(head.count_nonzero()) == 0, f'counter head not zero after mode {mode} spin {spin}'
    finally:
        _lib.force_splitk(0)
        _lib.tune('splitk_mode', 0)
        _lib.tune('spin_limit', 0)
    helpers.tolerance_check(outs[0], ref, f'one-launch split-K {variant}/{splitk} {M}x{N}x{K}')
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


@pytest.mark.parametrize('variant,splitk', [('pipe128x64', 0), ('pipe128x64', 7), ('pipe128x128', 2), ('pipe128x128', 5)])
@pytest.mark.parametrize('M,N,K', [(128, 2112, 7168), (256, 520, 2048), (77, 200, 4096), (300, 392, 1024)])
def test_scale_table_equals_scales_per_stage(dev, M, N, K, variant, splitk):
    """Row-major activation scales fetched once per tile into the table in LDS (the default of the small ring kernels up
    to 32 K blocks per workgroup) against the same kernels fetching them stage by stage: the same values, the same bits.
    Column-major scales never take the table."""
    from dlblas_amd import _lib
    print(f'case scale table variant={variant} splitk={splitk} M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=19)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    try:
        _lib.force_splitk(splitk)
        with_table = _run_dense(dev, a_q, a_s, b_q, b_s, variant=variant)
        _lib.tune('scale_table', 2)
        per_stage = _run_dense(dev, a_q, a_s, b_q, b_s, variant=variant)
    finally:
        _lib.force_splitk(0)
        _lib.tune('scale_table', 0)
    helpers.tolerance_check(with_table, ref, f'scale table {variant}/{splitk} {M}x{N}x{K}')
    assert torch.equal(with_table, per_stage)


def test_refused_launch_enqueues_nothing(dev):
    """A call whose main kernel cannot be launched (here: a forced request for more LDS than the GPU has) returns
    DLB_ERR_LAUNCH before any pre-pass is enqueued: workspace and output keep their bytes."""
    import ctypes
    from dlblas_amd import _lib
    lib = _lib.load()
    M, N, K = 2048, 4096, 512  # row-major scales, 256-row tiles: the call starts with a scale re-layout pass
    a_q, a_s, b_q, b_s = (t.to(dev) for t in helpers.make_dense(M, N, K, seed=5))
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
    ws = torch.full((_lib.WORKSPACE_BYTES, ), 0x5a, dtype=torch.uint8, device=dev)
    ws[:_lib.WS_COUNTER_BYTES] = 0
    vp = ctypes.c_void_p
    args = (vp(a_q.data_ptr()), vp(b_q.data_ptr()), vp(a_s.data_ptr()), vp(b_s.data_ptr()), vp(out.data_ptr()), M, N, K, a_s.stride(0),
            a_s.stride(1), _lib.OUT_BF16, vp(ws.data_ptr()), ws.numel(), vp(torch.cuda.current_stream().cuda_stream))
    try:
        _lib.tune('lds_oversize', 1)
        rc = lib.dlb_fp8_gemm(*args)
    finally:
        _lib.tune('lds_oversize', 0)
    torch.cuda.synchronize()
    assert rc == _lib.ERR_LAUNCH and 'nothing enqueued' in _lib.last_error()
    assert bool((ws[_lib.WS_COUNTER_BYTES:] == 0x5a).all()) and bool((out == 7.0).all())
    assert lib.dlb_fp8_gemm(*args) == 0  # the same call goes through once the hook is off ...
    torch.cuda.synchronize()
    assert not bool((ws[_lib.WS_COUNTER_BYTES:] == 0x5a).all())  # ... and it does use the workspace
    helpers.tolerance_check(out, orc.dequant_ref(a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu()), 'after a refused launch')


@pytest.mark.parametrize('variant', ['pipe256x256', 'pipe128x256w8', 'pipe256mix', 'pipe128x128', 'pipe128x64'])
@pytest.mark.parametrize('M,N,K', [(200, 392, 2048), (513, 1032, 256)])
def test_epilogue_through_lds_equals_direct_stores(dev, variant, M, N, K):
    """bf16 results of the pipelined kernels leave through an LDS transpose (whole rows per store instruction) or, by
    knob, straight from the accumulator registers: the same fp32 values, the same rounding, the same bits."""
    from dlblas_amd import _lib
    print(f'case epilogue variant={variant} M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=23)
    try:
        _lib.tune('epilogue', 2)
        direct = _run_dense(dev, a_q, a_s, b_q, b_s, variant=variant)
    finally:
        _lib.tune('epilogue', 0)
    staged = _run_dense(dev, a_q, a_s, b_q, b_s, variant=variant)
    assert torch.equal(direct, staged)
    helpers.tolerance_check(staged, orc.dequant_ref(a_q, a_s, b_q, b_s), f'epilogue {variant}')


@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('bn', [0, 4, 12, 20, 28, 32])
@pytest.mark.parametrize('M,N,K', [(16, 1000, 1024), (5, 130, 256), (40, 2112, 1024), (100, 392, 512)])
def test_decode_column_split(dev, M, N, K, bn, out_dtype):
    """Decode kernels with every width of the per-workgroup column range: ranges that are no multiple of 16 straddle
    weight-scale blocks (128 columns) inside a fragment and end in partly owned fragments; N itself is ragged."""
    from dlblas_amd import _lib
    print(f'case decode column split M={M} N={N} K={K} bn={bn} {out_dtype}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=31)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    _lib.tune('skinny_bn', bn)
    try:
        out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=out_dtype)
    finally:
        _lib.tune('skinny_bn', 0)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    helpers.tolerance_check(out, ref, f'decode bn={bn} {M}x{N}x{K}')


@pytest.mark.parametrize('ws_bytes', [0, 65536 + 4096])
@pytest.mark.parametrize('M,N,K', [(128, 2112, 7168), (300, 2112, 1536), (16, 512, 1024)])
def test_c_abi_without_a_usable_workspace(dev, M, N, K, ws_bytes):
    """Straight through the C ABI with no workspace or one too small for anything: no re-laid scales, no K split,
    the same results."""
    import ctypes
    from dlblas_amd import _lib
    print(f'case no workspace M={M} N={N} K={K} ws_bytes={ws_bytes}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=17)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    a, b, sa, sb = a_q.to(dev), b_q.to(dev), a_s.to(dev), b_s.to(dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    vp = ctypes.c_void_p
    rc = _lib.load().dlb_fp8_gemm(vp(a.data_ptr()), vp(b.data_ptr()), vp(sa.data_ptr()), vp(sb.data_ptr()), vp(out.data_ptr()),
                                  M, N, K, sa.stride(0), sa.stride(1), _lib.OUT_BF16, vp(ws.data_ptr() if ws_bytes else 0), ws_bytes,
                                  vp(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    helpers.tolerance_check(out, ref, f'no workspace {M}x{N}x{K}')


@pytest.mark.parametrize('M,N,K', [(0, 512, 1024), (16, 0, 1024), (16, 512, 0), (300, 392, 0)])
def test_empty_dimensions(dev, M, N, K):
    """No rows or no columns: an empty result; no K: a sum over nothing, i.e. zeros."""
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    print(f'case empty M={M} N={N} K={K}', flush=True)
    a = torch.zeros(M, K, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    b = torch.zeros(N, K, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    a_s = torch.ones(M, (K + 127) // 128, device=dev)
    b_s = torch.ones((N + 127) // 128, (K + 127) // 128, device=dev)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        out = fp8_gemm(a, b, a_s, b_s)
    finally:
        torch.set_default_dtype(prev)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (M, N) and out.dtype == torch.bfloat16
    assert (out == 0).all()


def _random_shapes(n, seed):
    import random
    rng = random.Random(seed)
    shapes = []
    for _ in range(n):
        kind = rng.random()
        M = rng.choice([1, 2, 15, 16, 17, 31, 33, 64, 65, 127, 128, 129, 255, 257, 300, 511, 640])
        N = rng.choice([1, 7, 8, 24, 128, 130, 192, 200, 256, 264, 392, 520, 776, 1032])
        if kind < 0.6:
            K = 128 * rng.randint(1, 18)
        elif kind < 0.85:
            K = 16 * rng.randint(1, 60)
        else:
            K = rng.randint(1, 300)
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize('M,N,K', _random_shapes(40, 2024))
def test_dense_random_shapes_take_the_library_choice(dev, M, N, K):
    """Seeded random shapes across every branch of the shape heuristic (decode, split-K, pipelined, mixed, tiled with
    K tails, exact), bf16 and fp32 alternating."""
    out_dtype = torch.float32 if (M + N + K) % 2 else torch.bfloat16
    print(f'case random M={M} N={N} K={K} {out_dtype}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=M * 7 + N * 3 + K)
    out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    helpers.tolerance_check(out, orc.dequant_ref(a_q, a_s, b_q, b_s), f'random {M}x{N}x{K}')


def test_limits_of_the_launch_grid_and_of_the_lds(dev):
    """More rows than the second grid dimension holds on the exact path (rows run in a grid-stride loop), and a forced
    decode wave count that would not fit the LDS (clamped): both launch and give the right answer."""
    from dlblas_amd import _lib
    M, N, K = 262200, 8, 8
    g = helpers.gen(5)
    a_q = torch.randint(-4, 5, (M, K), generator=g).float().to(torch.float8_e4m3fn)
    b_q = torch.randint(-4, 5, (N, K), generator=g).float().to(torch.float8_e4m3fn)
    a_s, b_s = torch.rand(M, 1, generator=g) + 0.5, torch.rand(1, 1, generator=g) + 0.5
    print(f'case exact path M={M}', flush=True)
    out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=torch.float32)
    ref = (a_q.float() @ b_q.float().t()) * a_s * b_s
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-6, atol=0)
    try:
        _lib.tune('skinny_waves', 16)
        print('case skinny128 with 16 waves asked for', flush=True)
        a_q, a_s, b_q, b_s = helpers.make_dense(128, 512, 2048, seed=6)
        out = _run_dense(dev, a_q, a_s, b_q, b_s, variant='skinny128')
        helpers.tolerance_check(out, orc.dequant_ref(a_q, a_s, b_q, b_s), 'skinny128, 16 waves asked for')
    finally:
        _lib.tune('skinny_waves', 0)


def test_dense_f32_reference_test_construction(dev):
    """The reference's own test: randn e4m3 operands, randn (signed) scales, fp32 out, atol 1e-1
    (tests/kernels/test_fp8_gemm.py:8-31,70-72)."""
    print('case dense f32 reference construction', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_raw(512, 512, 512)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=torch.float32)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), ref, atol=1e-1, rtol=0)
    helpers.tolerance_check(out, ref, 'reference construction')


def test_dense_exact_small_integers(dev):
    """Operands holding small integers and unit scales: every partial sum is an integer below 2^24, so the fp32
    result is exact whatever the summation order - bit-exact comparison."""
    print('case dense exact integers', flush=True)
    g = helpers.gen(3)
    M, N, K = 48, 272, 640
    a = torch.randint(-4, 5, (M, K), generator=g).float()
    b = torch.randint(-4, 5, (N, K), generator=g).float()
    a_q, b_q = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    a_s, b_s = torch.ones(M, 5), torch.ones(3, 5)
    out = _run_dense(dev, a_q, a_s, b_q, b_s, dtype=torch.float32)
    assert torch.equal(out.cpu(), a @ b.t())


def test_leading_dims_are_flattened(dev):
    print('case leading dims', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(6 * 5, 256, 256, seed=11)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    out = _run_dense(dev, a_q.reshape(6, 5, 256), a_s.reshape(6, 5, 2), b_q, b_s)
    assert tuple(out.shape) == (6, 5, 256)
    helpers.tolerance_check(out.reshape(30, 256), ref, 'leading dims')


def test_contiguity_asserts(dev):
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    a_q, a_s, b_q, b_s = (t.to(dev) for t in helpers.make_dense(32, 256, 256))
    with pytest.raises(AssertionError, match='Input tensors must be contiguous'):
        fp8_gemm(a_q.t().contiguous().t(), b_q, a_s, b_s)
    with pytest.raises(AssertionError, match='Scaling factor tensors must be contiguous'):
        fp8_gemm(a_q, b_q, a_s.t().contiguous().t(), b_s)


def test_repeat_calls_are_deterministic(dev):
    """Split-K partials are added in split order by whichever workgroup arrives last: bit-identical reruns."""
    print('case determinism', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense(16, 2112, 7168, seed=5)
    outs = [_run_dense(dev, a_q, a_s, b_q, b_s) for _ in range(3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    a_q, a_s, b_q, b_s = helpers.make_dense(128, 1024, 4096, seed=5)
    outs = [_run_dense(dev, a_q, a_s, b_q, b_s) for _ in range(3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


# ----------------------------------------------------------------------------------------------------------------
# grouped
# ----------------------------------------------------------------------------------------------------------------
def _make_grouped_weights(G, N, K, seed):
    g = helpers.gen(seed)
    w = (torch.randn(G, N, K, generator=g) * 0.02).to(torch.bfloat16)
    qs = [orc.quant_weight_128x128(w[i]) for i in range(G)]
    return torch.stack([q for q, _ in qs]), torch.stack([s for _, s in qs])


@pytest.mark.parametrize('col_major_scales', [False, True])
@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
def test_grouped_contiguous(dev, col_major_scales, out_dtype):
    print(f'case contiguous col_major={col_major_scales} {out_dtype}', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_contiguous
    G, N, K = 4, 384, 512
    counts = [128, 0, 384, 256]  # padded per-expert spans, one expert empty
    M_sum = sum(counts)
    g = helpers.gen(9)
    a = torch.randn(M_sum, K, generator=g).to(torch.bfloat16)
    a_q, a_s = orc.quant_act_1x128(a)
    w_q, w_s = _make_grouped_weights(G, N, K, 10)
    m_indices = torch.cat([torch.full((c, ), e, dtype=torch.int32) for e, c in enumerate(counts)])
    m_indices[128:256] = -1  # one skipped block
    sentinel = 777.0
    ref = orc.grouped_contiguous_ref(a_q, a_s, w_q, w_s, torch.full((M_sum, N), sentinel), m_indices)

    a_s_dev = a_s.to(dev)
    if col_major_scales:  # the layout dlblas/kernels/quant_dequant.py:65-83 hands over
        pad = -(-M_sum // 4) * 4
        buf = torch.zeros(K // 128, pad, device=dev)
        buf[:, :M_sum] = a_s_dev.t()
        a_s_dev = buf.t()[:M_sum]
        assert not a_s_dev.is_contiguous()
    out = torch.full((M_sum, N), sentinel, dtype=out_dtype, device=dev)
    m_grouped_fp8_gemm_nt_contiguous([a_q.to(dev), a_s_dev], (w_q.to(dev), w_s.to(dev)), out, m_indices.to(dev))
    torch.cuda.synchronize()
    assert torch.all(out[128:256] == sentinel), 'skipped block was written'
    helpers.tolerance_check(out, ref, 'grouped contiguous')


@pytest.mark.parametrize('variant', [None, 'list', 'pipe128x256w8', 'tile128x128'])
def test_grouped_contiguous_run_lengths(dev, variant):
    """Runs of 1 to 5 blocks of 128 rows, skipped blocks between and inside runs, an expert that owns two separate
    runs, experts out of order.  'list' pairs blocks into 256-row tiles from a list built on the device (the library's
    own choice for batches of more than two rounds of tiles; a batch this small gets 128 x 128 tiles); forced variants
    take the uniform 128-row path.  All must agree with the oracle."""
    print(f'case contiguous run lengths variant={variant}', flush=True)
    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_contiguous
    G, N, K = 5, 520, 384
    blocks = [3, 3, -1, 0, 0, 0, 0, 0, 2, -1, -1, 4, 4, 4, 3, 1, 1, -1]   # expert of every 128-row block
    M_sum = 128 * len(blocks)
    g = helpers.gen(19)
    a_q, a_s = orc.quant_act_1x128(torch.randn(M_sum, K, generator=g).to(torch.bfloat16))
    w_q, w_s = _make_grouped_weights(G, N, K, 20)
    m_indices = torch.tensor(blocks, dtype=torch.int32).repeat_interleave(128)
    sentinel = 321.0
    ref = orc.grouped_contiguous_ref(a_q, a_s, w_q, w_s, torch.full((M_sum, N), sentinel), m_indices)
    out = torch.full((M_sum, N), sentinel, dtype=torch.bfloat16, device=dev)
    try:
        if variant == 'list':
            _lib.tune('tile_list', 1)
            assert _lib.plan(1, M_sum, N, K)[0] == 'pipe128x256w8'
        else:
            _lib.force_variant(variant)
        m_grouped_fp8_gemm_nt_contiguous((a_q.to(dev), a_s.to(dev)), (w_q.to(dev), w_s.to(dev)), out, m_indices.to(dev))
        torch.cuda.synchronize()
    finally:
        _lib.force_variant(None)
        _lib.tune('tile_list', 0)
    skipped = (m_indices < 0)
    assert torch.all(out.cpu()[skipped] == sentinel), 'a skipped block was written'
    helpers.tolerance_check(out, ref, f'contiguous run lengths {variant}')


def test_grouped_contiguous_many_blocks(dev):
    """700 blocks of 128 rows: the device-side tile list then works in chunks of several blocks per thread, and runs of
    1 to 7 blocks (256-row tiles, pairs of 192-row tiles for the odd ones, single 128-row tiles) cross the chunk
    boundaries in every way.  Skipped blocks in between; the last block is short."""
    print('case contiguous many blocks', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_contiguous
    G, N, K = 12, 256, 128
    g = helpers.gen(31)
    blocks = []
    while len(blocks) < 700:
        e = int(torch.randint(-1, G, (1, ), generator=g))
        blocks += [e] * int(torch.randint(1, 8, (1, ), generator=g))
    blocks = blocks[:700]
    M_sum = 128 * len(blocks) - 37
    a_q, a_s = orc.quant_act_1x128(torch.randn(M_sum, K, generator=g).to(torch.bfloat16))
    w_q, w_s = _make_grouped_weights(G, N, K, 32)
    m_indices = torch.tensor(blocks, dtype=torch.int32).repeat_interleave(128)[:M_sum].contiguous()
    sentinel = 99.0
    ref = orc.grouped_contiguous_ref(a_q, a_s, w_q, w_s, torch.full((M_sum, N), sentinel), m_indices)
    out = torch.full((M_sum, N), sentinel, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_contiguous((a_q.to(dev), a_s.to(dev)), (w_q.to(dev), w_s.to(dev)), out, m_indices.to(dev))
    torch.cuda.synchronize()
    assert torch.all(out.cpu()[m_indices < 0] == sentinel), 'a skipped block was written'
    helpers.tolerance_check(out, ref, 'contiguous many blocks')


def test_grouped_masked(dev):
    print('case masked', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    G, M_max, N, K = 6, 256, 512, 384
    g = helpers.gen(12)
    masked_m = torch.tensor([0, 1, 256, 130, 77, 128], dtype=torch.int32)
    a = torch.randn(G, M_max, K, generator=g).to(torch.bfloat16)
    a_q, a_s = orc.quant_act_1x128(a)
    w_q, w_s = _make_grouped_weights(G, N, K, 13)
    # rows at or beyond masked_m hold NaN codes and NaN scales: they must never reach a valid output
    a_bits = a_q.view(torch.uint8).clone()
    for e in range(G):
        a_bits[e, int(masked_m[e]):] = 0x7F
        a_s[e, int(masked_m[e]):] = float('nan')
    a_q = a_bits.view(torch.float8_e4m3fn)
    sentinel = -555.0
    ref = orc.grouped_masked_ref(a_q, a_s, w_q, w_s, torch.full((G, M_max, N), sentinel), masked_m)
    out = torch.full((G, M_max, N), sentinel, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_masked((a_q.to(dev), a_s.to(dev)), (w_q.to(dev), w_s.to(dev)), out, masked_m.to(dev), 0)
    torch.cuda.synchronize()
    for e in range(G):
        assert torch.all(out[e, int(masked_m[e]):] == sentinel), f'expert {e}: rows beyond masked_m were written'
    assert not torch.isnan(out.float()).any()
    helpers.tolerance_check(out, ref, 'grouped masked')


def test_grouped_masked_hint_picks_the_tile_shape(dev):
    """expected_m picks the tile shape - unknown: 128 x 256; a few short experts: 128 x 128; several hundred rows per
    expert: 256-row tiles - and never a result bit."""
    print('case masked expected_m', flush=True)
    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    G, M_max, N, K = 6, 512, 1536, 256
    g = helpers.gen(16)
    masked_m = torch.tensor([0, 1, 512, 130, 400, 257], dtype=torch.int32)
    a_q, a_s = orc.quant_act_1x128(torch.randn(G, M_max, K, generator=g).to(torch.bfloat16))
    w_q, w_s = _make_grouped_weights(G, N, K, 17)
    a_bits = a_q.view(torch.uint8).clone()
    for e in range(G):
        a_bits[e, int(masked_m[e]):] = 0x7F
        a_s[e, int(masked_m[e]):] = float('nan')
    a_q = a_bits.view(torch.float8_e4m3fn)
    sentinel = -555.0
    ref = orc.grouped_masked_ref(a_q, a_s, w_q, w_s, torch.full((G, M_max, N), sentinel), masked_m)
    outs, shapes = [], []
    for hint in (0, 16, 500):
        shapes.append(_lib.plan_grouped(2, M_max, N, K, G, hint)[0])
        out = torch.full((G, M_max, N), sentinel, dtype=torch.bfloat16, device=dev)
        m_grouped_fp8_gemm_nt_masked((a_q.to(dev), a_s.to(dev)), (w_q.to(dev), w_s.to(dev)), out, masked_m.to(dev), hint)
        torch.cuda.synchronize()
        for e in range(G):
            assert torch.all(out[e, int(masked_m[e]):] == sentinel), f'expected_m = {hint}, expert {e}: rows beyond masked_m were written'
        outs.append(out)
    assert shapes == ['pipe128x256w8', 'pipe128x128', 'pipe256x256'], shapes
    helpers.tolerance_check(outs[0], ref, 'masked expected_m')
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


@pytest.mark.parametrize('K', [384, 2048, 2176])
def test_grouped_masked_scale_table(dev, K):
    """The masked layout fetches a tile's row-major activation scales once, into a table in LDS, when K has at most 16
    blocks (no re-layout launch in front); longer K and the knob take the re-laid copy in the workspace.  Same bits
    either way, rows at or beyond masked_m (NaN codes, NaN scales) never read into a valid row nor written."""
    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    print(f'case masked scale table K={K}', flush=True)
    G, M_max, N = 5, 256, 512
    g = helpers.gen(14)
    masked_m = torch.tensor([3, 256, 0, 129, 200], dtype=torch.int32)
    a_q, a_s = orc.quant_act_1x128(torch.randn(G, M_max, K, generator=g).to(torch.bfloat16))
    w_q, w_s = _make_grouped_weights(G, N, K, 15)
    a_bits = a_q.view(torch.uint8).clone()
    for e in range(G):
        a_bits[e, int(masked_m[e]):] = 0x7F
        a_s[e, int(masked_m[e]):] = float('nan')
    a_q = a_bits.view(torch.float8_e4m3fn)
    sentinel = -555.0
    ref = orc.grouped_masked_ref(a_q, a_s, w_q, w_s, torch.full((G, M_max, N), sentinel), masked_m)
    outs = []
    for knob in (0, 2):
        out = torch.full((G, M_max, N), sentinel, dtype=torch.bfloat16, device=dev)
        _lib.tune('scale_table', knob)
        try:
            m_grouped_fp8_gemm_nt_masked((a_q.to(dev), a_s.to(dev)), (w_q.to(dev), w_s.to(dev)), out, masked_m.to(dev), 0)
            torch.cuda.synchronize()
        finally:
            _lib.tune('scale_table', 0)
        outs.append(out)
    for e in range(G):
        assert torch.all(outs[0][e, int(masked_m[e]):] == sentinel)
    helpers.tolerance_check(outs[0], ref, f'masked scale table K={K}')
    assert torch.equal(outs[0], outs[1])


def test_registry_selects_and_caches_on_gpu(dev):
    print('case registry', flush=True)
    from dlblas_amd import get_op
    a_q, a_s, b_q, b_s = (t.to(dev) for t in helpers.make_dense(64, 512, 1024))
    op = get_op('fp8_gemm', (a_q, b_q, a_s, b_s))
    assert get_op('fp8_gemm', (a_q, b_q, a_s, b_s)) is op
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        out = op(a_q, b_q, a_s, b_s)
    finally:
        torch.set_default_dtype(prev)
    ref = orc.dequant_ref(a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu())
    helpers.tolerance_check(out, ref, 'registry')


def test_registry_chooses_between_two_real_implementations(dev):
    """'fp8_gemm' has two registered implementations (the planner's kernels, the register-staged tile kernels): both
    match, both are benchmarked on the caller's tensors, the faster one is cached and returned, and both are right."""
    print('case registry selection', flush=True)
    from dlblas_amd import get_op
    from dlblas_amd.op_registry import op_registry
    from dlblas_amd.op_struct import match
    for (M, N, K) in ((16, 2112, 2048), (512, 1024, 2048)):
        a_q, a_s, b_q, b_s = (t.to(dev) for t in helpers.make_dense(M, N, K, seed=9))
        args = (a_q, b_q, a_s, b_s)
        cands = [impl for impl in op_registry.ops['fp8_gemm'] if match(args, impl.params)]
        assert len(cands) == 2 and cands[0].call is not cands[1].call
        ref = orc.dequant_ref(a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu())
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch.bfloat16)
        try:
            op = get_op('fp8_gemm', args)
            assert op in cands and get_op('fp8_gemm', args) is op
            times = [min(impl.bench(*args) for _ in range(3)) for impl in cands]
            other = cands[1 - cands.index(op)]
            # the cached choice is the faster one (25 % slack: the two benches ran at different moments)
            assert times[cands.index(op)] <= 1.25 * times[cands.index(other)], (M, N, K, times)
            for impl in cands:
                helpers.tolerance_check(impl(*args), ref, f'registry candidate {impl.call.__name__} {M}x{N}x{K}')
        finally:
            torch.set_default_dtype(prev)
