"""HIP graph capture of the decode GEMM and of the masked grouped GEMM on a side stream: after prepare() and one warm-up
call nothing in the launch path allocates, synchronises or records a memset, so the calls can be captured and replayed.
Every replay is checked against the eager result (bit for bit) and the CPU oracle, with the inputs rewritten and
ordinary eager work and synchronisations between the replays."""
import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc

pytestmark = pytest.mark.gpu


def test_decode_and_masked_gemm_replay_from_a_graph():
    import dlblas_amd
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    dev = torch.device('cuda:0')
    side = torch.cuda.Stream(device=dev)   # default priority
    dlblas_amd.prepare(dev, side)

    M, N, K = 16, 2112, 2048
    G, M_max, GN, GK = 4, 128, 512, 512
    inputs = []
    for seed in (51, 52, 53):
        a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=seed)
        g = helpers.gen(seed)
        x_q, x_s = orc.quant_act_1x128(torch.randn(G, M_max, GK, generator=g).to(torch.bfloat16))
        w = [orc.quant_weight_128x128((torch.randn(GN, GK, generator=g) * 0.02).to(torch.bfloat16)) for _ in range(G)]
        masked_m = torch.randint(0, M_max + 1, (G, ), generator=g, dtype=torch.int32)
        inputs.append(dict(a_q=a_q, a_s=a_s, b_q=b_q, b_s=b_s, x_q=x_q, x_s=x_s, w_q=torch.stack([q for q, _ in w]),
                           w_s=torch.stack([s for _, s in w]), masked_m=masked_m))
    static = {k: v.to(dev) for k, v in inputs[0].items()}
    gout = torch.full((G, M_max, GN), -7.0, dtype=torch.bfloat16, device=dev)

    import ctypes
    from dlblas_amd import _lib
    lib, vp = _lib.load(), ctypes.c_void_p
    na_out = torch.full((M, N), -3.0, dtype=torch.bfloat16, device=dev)

    def step():
        c = fp8_gemm(static['a_q'], static['b_q'], static['a_s'], static['b_s'])
        # the entry point that works in the library's static scratch (bound to this stream by prepare())
        _lib.check(lib.dlb_fp8_gemm_noalloc(vp(static['a_q'].data_ptr()), vp(static['b_q'].data_ptr()), vp(static['a_s'].data_ptr()),
                                            vp(static['b_s'].data_ptr()), vp(na_out.data_ptr()), M, N, K, static['a_s'].stride(0),
                                            static['a_s'].stride(1), _lib.OUT_BF16, vp(torch.cuda.current_stream().cuda_stream)))
        m_grouped_fp8_gemm_nt_masked((static['x_q'], static['x_s']), (static['w_q'], static['w_s']), gout,
                                     static['masked_m'], M_max // 2)
        return c

    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.cuda.stream(side):
            step()                                   # warm-up: kernel attributes are set on the first launch
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured_c = step()
        for rep, data in enumerate(inputs):
            print(f'case graph replay {rep}', flush=True)
            for k, v in data.items():
                static[k].copy_(v.to(dev))           # eager work between the replays
            gout.fill_(-7.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got_c, got_g, got_na = captured_c.clone(), gout.clone(), na_out.clone()
            gout.fill_(-7.0)
            na_out.fill_(-3.0)
            with torch.cuda.stream(side):
                eager_c = step()
            torch.cuda.synchronize()
            assert torch.equal(got_c, eager_c) and torch.equal(got_g, gout), f'replay {rep} differs from the eager call'
            assert torch.equal(got_na, eager_c) and torch.equal(na_out, eager_c), f'replay {rep}: the no-allocation entry point differs'
            helpers.tolerance_check(got_c, orc.dequant_ref(data['a_q'], data['a_s'], data['b_q'], data['b_s']), f'graph dense replay {rep}')
            ref = orc.grouped_masked_ref(data['x_q'], data['x_s'], data['w_q'], data['w_s'],
                                         torch.full((G, M_max, GN), -7.0, dtype=torch.float32), data['masked_m'])
            for e in range(G):
                m = int(data['masked_m'][e])
                assert torch.all(got_g[e, m:] == -7.0)
                if m:
                    helpers.tolerance_check(got_g[e, :m], ref[e, :m], f'graph masked replay {rep} expert {e}')
    finally:
        torch.set_default_dtype(prev)
