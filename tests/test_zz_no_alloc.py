"""dlb_fp8_gemm_noalloc (the entry point that works in the library's own static scratch) against dlb_fp8_gemm with a
caller-owned workspace of the size of one slice of that scratch, both called straight through the C ABI: two calls in a
row on the same stream, the second with a smaller input, so the second runs over what the first left in the slice."""
import ctypes

import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc

pytestmark = pytest.mark.gpu

vp = ctypes.c_void_p


def _both_entry_points(lib, dev, M, N, K, seed, out_dtype):
    from dlblas_amd import _lib
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=seed)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    a_q, a_s, b_q, b_s = (t.to(dev) for t in (a_q, a_s, b_q, b_s))
    ws = torch.empty(_lib.STATIC_SCRATCH_SLICE_BYTES, dtype=torch.uint8, device=dev).fill_(0xA5)
    ws[:_lib.WS_COUNTER_BYTES] = 0   # the counter head of a workspace starts at zero (and every call leaves it so)
    out_ws = torch.full((M, N), 7.0, dtype=out_dtype, device=dev)
    out_static = torch.full((M, N), -7.0, dtype=out_dtype, device=dev)
    stream = vp(torch.cuda.current_stream().cuda_stream)
    code = _lib.out_code(out_dtype)
    torch.cuda.synchronize()
    _lib.check(lib.dlb_fp8_gemm(vp(a_q.data_ptr()), vp(b_q.data_ptr()), vp(a_s.data_ptr()), vp(b_s.data_ptr()),
                                vp(out_ws.data_ptr()), M, N, K, a_s.stride(0), a_s.stride(1), code, vp(ws.data_ptr()),
                                ws.numel(), stream))
    _lib.check(lib.dlb_fp8_gemm_noalloc(vp(a_q.data_ptr()), vp(b_q.data_ptr()), vp(a_s.data_ptr()), vp(b_s.data_ptr()),
                                        vp(out_static.data_ptr()), M, N, K, a_s.stride(0), a_s.stride(1), code, stream))
    torch.cuda.synchronize()
    return out_ws, out_static, ref


# (first call, second smaller call): each pair runs back to back over the same slice of the static array
PAIRS = [
    ((512, 2112, 16384), (256, 2112, 2048)),   # ring kernels: re-laid scales + fp32 partial sums of K slices in the scratch
    ((4096, 1024, 2048), (300, 392, 1024)),    # mixed-width prefill launch (re-laid scales only), then a ragged small one
    ((128, 2112, 7168), (16, 512, 1024)),      # K split over workgroups, then a decode launch that needs no scratch
]


@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('first,second', PAIRS)
def test_noalloc_matches_workspace_entry_point(first, second, out_dtype):
    from dlblas_amd import _lib
    lib = _lib.load()
    dev = torch.device('cuda:0')
    for i, (M, N, K) in enumerate((first, second)):
        print(f'case noalloc call {i} M={M} N={N} K={K} {out_dtype}', flush=True)
        out_ws, out_static, ref = _both_entry_points(lib, dev, M, N, K, seed=31 + i, out_dtype=out_dtype)
        # same plan, same kernels, same summation order: bit for bit the existing entry point's result
        assert torch.equal(out_ws.view(torch.uint8), out_static.view(torch.uint8)), f'call {i}: {M}x{N}x{K} differs'
        helpers.tolerance_check(out_static, ref, f'noalloc {M}x{N}x{K}')


def test_noalloc_rejects_what_does_not_fit():
    """Beyond the static array's size the call is refused on the host (nothing is enqueued); bad arguments are refused
    as in dlb_fp8_gemm."""
    from dlblas_amd import _lib
    lib = _lib.load()
    fake, null = vp(4096), vp(0)
    M, K = 1 << 16, 128 * 128   # 65536 rows x 128 K blocks x 4 bytes = 32 MiB of re-laid scales
    rc = lib.dlb_fp8_gemm_noalloc(fake, fake, fake, fake, fake, M, 128, K, 128, 1, 0, null)
    assert rc == _lib.ERR_WORKSPACE and 'static scratch' in _lib.last_error()
    # the same problem with column-major scales keeps nothing in scratch: it passes the size check (and fails later,
    # on the fake pointers' alignment or not at all - never with DLB_ERR_WORKSPACE)
    assert lib.dlb_fp8_gemm_noalloc(fake, fake, fake, fake, fake, 8, 8, 128, 1, 1, 7, null) == _lib.ERR_BAD_DTYPE
    assert lib.dlb_fp8_gemm_noalloc(null, null, null, null, null, 0, 8, 128, 1, 1, 0, null) == 0


def test_noalloc_gives_every_stream_its_own_slice():
    """Calls on different streams work in different slices of the static array, so they may overlap in time; once every
    slice is bound to a stream, a call on yet another stream is refused.  (How many slices are still free depends on what
    ran in this process before, so the test makes one stream more than there are slices.)"""
    from dlblas_amd import _lib
    lib = _lib.load()
    dev = torch.device('cuda:0')
    M, N, K = 128, 2112, 7168  # K split over workgroups: fp32 partial sums in the slice
    a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=41)
    ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
    a_q, a_s, b_q, b_s = (t.to(dev) for t in (a_q, a_s, b_q, b_s))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=dev) for _ in range(_lib.STATIC_SCRATCH_SLICES + 1)]
    outs, rcs = [], []
    for st in streams:
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        outs.append(out)
        rc = [lib.dlb_fp8_gemm_noalloc(vp(a_q.data_ptr()), vp(b_q.data_ptr()), vp(a_s.data_ptr()), vp(b_s.data_ptr()),
                                       vp(out.data_ptr()), M, N, K, a_s.stride(0), a_s.stride(1), _lib.OUT_BF16, vp(st.cuda_stream))
              for _ in range(3)]  # several launches per stream, all streams in flight at once
        assert rc[0] == rc[1] == rc[2]
        rcs.append(rc[0])
    torch.cuda.synchronize()
    n_ok = rcs.count(0)
    assert 1 <= n_ok <= _lib.STATIC_SCRATCH_SLICES, rcs
    assert rcs == [0] * n_ok + [_lib.ERR_WORKSPACE] * (len(rcs) - n_ok), rcs
    assert 'slices' in _lib.last_error()
    for out in outs[:n_ok]:
        helpers.tolerance_check(out, ref, 'noalloc on a stream of its own')
        assert torch.equal(out, outs[0])
    # a stream that has its slice keeps it
    assert lib.dlb_fp8_gemm_noalloc(vp(a_q.data_ptr()), vp(b_q.data_ptr()), vp(a_s.data_ptr()), vp(b_s.data_ptr()), vp(outs[0].data_ptr()),
                                    M, N, K, a_s.stride(0), a_s.stride(1), _lib.OUT_BF16, vp(streams[0].cuda_stream)) == 0
    torch.cuda.synchronize()
