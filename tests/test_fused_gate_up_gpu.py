"""The gate/up GEMM with silu * up and the 1 x 128 quantiser in its epilogue against the three separate steps it
replaces (grouped GEMM -> silu_and_mul -> per_token_group_quant_fp8, dlblas/kernels/fused_moe_v3.py:307-334): the same
bytes and the same scale bits, since the epilogue rounds to bf16 where the separate kernels store bf16.  The separate
steps are themselves held against the CPU oracles elsewhere (test_fp8_gemm_gpu.py, test_moe_activation_gpu.py)."""
import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def dev():
    from dlblas_amd import _lib
    _lib.load()
    return torch.device('cuda:0')


def _both(dev, a_q, a_s, w_q, w_s, m_indices, column_major_scales=False):
    from dlblas_amd.kernels.activation import silu_and_mul_post_quant
    from dlblas_amd.kernels.fp8_gemm_grouped import (fp8_gemm_grouped_contiguous_silu_quant,
                                                     m_grouped_fp8_gemm_nt_contiguous)
    fused = fp8_gemm_grouped_contiguous_silu_quant(a_q, a_s, w_q, w_s, m_indices, column_major_scales=column_major_scales)
    gate_up = torch.zeros(a_q.size(0), w_q.size(1), dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_contiguous((a_q, a_s), (w_q, w_s), gate_up, m_indices)
    ref_q, ref_s = silu_and_mul_post_quant(gate_up, 128)
    torch.cuda.synchronize()
    return fused, (ref_q, ref_s)


@pytest.mark.parametrize('blocks,inter,K,col_major_in,col_major_out', [
    ([1], 128, 128, False, False),
    ([2, 1, 3], 256, 512, False, False),
    ([3, 0, 2, 1], 384, 1024, True, False),
    ([1, 4, 2], 512, 768, False, True),
    ([5], 128, 2048, True, True),
])
def test_fused_equals_the_three_steps(dev, blocks, inter, K, col_major_in, col_major_out):
    print(f'case fused gate/up blocks={blocks} I={inter} K={K}', flush=True)
    G = len(blocks)
    M_sum = 128 * sum(blocks)
    g = helpers.gen(300 + M_sum + inter + K)
    a_q, a_s = orc.quant_act_1x128((torch.randn(M_sum, K, generator=g) * 1.5).to(torch.bfloat16))
    ws = [orc.quant_weight_128x128((torch.randn(2 * inter, K, generator=g) * 0.05).to(torch.bfloat16)) for _ in range(G)]
    w_q, w_s = torch.stack([w[0] for w in ws]).to(dev), torch.stack([w[1] for w in ws]).to(dev)
    m_indices = torch.repeat_interleave(torch.arange(G, dtype=torch.int32), torch.tensor(blocks) * 128)
    if M_sum >= 384:
        m_indices[256:384] = -1  # a skipped block: its rows are not written
    a_s_d = a_s.to(dev)
    if col_major_in:
        a_s_d = a_s_d.t().contiguous().t()
    fused, (ref_q, ref_s) = _both(dev, a_q.to(dev), a_s_d, w_q, w_s, m_indices.to(dev), col_major_out)
    assert fused is not None
    q, s = fused
    assert q.dtype == torch.float8_e4m3fn and tuple(q.shape) == (M_sum, inter) and tuple(s.shape) == (M_sum, inter // 128)
    if col_major_out:
        assert s.stride(0) == 1
    keep = (m_indices >= 0).to(dev)
    assert torch.equal(q.view(torch.uint8)[keep], ref_q.view(torch.uint8)[keep]), 'quantised codes differ'
    assert torch.equal(s[keep], ref_s[keep]), 'scales differ'


def test_shapes_without_a_fused_kernel_are_declined(dev):
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous_silu_quant
    a_q = torch.zeros(128, 192, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)   # K % 128 != 0
    a_s = torch.ones(128, 2, device=dev)
    w_q = torch.zeros(1, 256, 192, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    w_s = torch.ones(1, 2, 2, device=dev)
    m_indices = torch.zeros(128, dtype=torch.int32, device=dev)
    assert fp8_gemm_grouped_contiguous_silu_quant(a_q, a_s, w_q, w_s, m_indices) is None


def test_fused_full_size(dev):
    """One GPU's share of the gate/up projection: 32 experts, 8192 tokens in 9728 padded rows, 2 x 2048 x 7168."""
    print('case fused gate/up full size', flush=True)
    G, inter, K, tokens = 32, 2048, 7168, 8192
    g = torch.Generator().manual_seed(20)
    assign = torch.multinomial(torch.full((G, ), 1.0 / G), tokens, replacement=True, generator=g)
    padded = (torch.bincount(assign, minlength=G) + 127) // 128 * 128
    M_sum = int(padded.sum())
    m_indices = torch.repeat_interleave(torch.arange(G, dtype=torch.int32), padded).to(dev)
    gd = torch.Generator(device=dev).manual_seed(21)
    a_q, a_s = helpers.quantise_act_device(torch.randn(M_sum, K, device=dev, generator=gd).to(torch.bfloat16))
    w_q, w_s = helpers.expert_weights_device(G, 2 * inter, K, dev, 22)
    fused, (ref_q, ref_s) = _both(dev, a_q, a_s, w_q, w_s, m_indices)
    assert fused is not None
    assert torch.equal(fused[0].view(torch.uint8), ref_q.view(torch.uint8))
    assert torch.equal(fused[1], ref_s)
