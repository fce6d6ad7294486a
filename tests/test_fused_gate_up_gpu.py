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


# --- masked (low-latency) layout: m_grouped_fp8_gemm_nt_masked -> silu_and_mul_masked_post_quant_fwd in one kernel ----


def _masked_both(dev, a_q, a_s, w_q, w_s, masked_m, col_major_out=False):
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_masked_silu_quant, m_grouped_fp8_gemm_nt_masked
    from dlblas_amd.kernels.moe import silu_and_mul_masked_post_quant_fwd
    G, M_max, _ = a_q.shape
    inter = w_q.size(1) // 2
    sentinel_q, sentinel_s = 0x5a, -7.0
    q = torch.full((G, M_max, inter), sentinel_q, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    if col_major_out:
        s = torch.full((G, inter // 128, M_max), sentinel_s, device=dev).transpose(1, 2)
    else:
        s = torch.full((G, M_max, inter // 128), sentinel_s, device=dev)
    ok = fp8_gemm_grouped_masked_silu_quant(a_q, a_s, w_q, w_s, q, s, masked_m, expected_m=int(masked_m.max()))
    gate_up = torch.zeros(G, M_max, 2 * inter, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_masked((a_q, a_s), (w_q, w_s), gate_up, masked_m, int(masked_m.max()))
    ref_q = torch.full((G, M_max, inter), sentinel_q, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    ref_s = torch.full((G, M_max, inter // 128), sentinel_s, device=dev)
    silu_and_mul_masked_post_quant_fwd(gate_up, ref_q, ref_s, 128, masked_m)
    torch.cuda.synchronize()
    return ok, (q, s), (ref_q, ref_s)


@pytest.mark.parametrize('masked,M_max,inter,K,col_major_out', [
    ([5], 128, 128, 128, False),
    ([0, 128, 77], 128, 256, 512, False),
    ([200, 1, 256, 129], 256, 384, 1024, True),
    ([300, 0, 45], 384, 128, 2048, False),
    ([64, 64, 64, 64, 64, 64, 64, 64, 3], 64, 512, 256, True),
])
def test_masked_fused_equals_the_two_steps(dev, masked, M_max, inter, K, col_major_out):
    print(f'case fused masked gate/up masked_m={masked} M_max={M_max} I={inter} K={K}', flush=True)
    G = len(masked)
    g = helpers.gen(700 + M_max + inter + K)
    qs = [orc.quant_act_1x128((torch.randn(M_max, K, generator=g) * 1.5).to(torch.bfloat16)) for _ in range(G)]
    a_q, a_s = torch.stack([x[0] for x in qs]).to(dev), torch.stack([x[1] for x in qs]).to(dev)
    ws = [orc.quant_weight_128x128((torch.randn(2 * inter, K, generator=g) * 0.05).to(torch.bfloat16)) for _ in range(G)]
    w_q, w_s = torch.stack([w[0] for w in ws]).to(dev), torch.stack([w[1] for w in ws]).to(dev)
    masked_m = torch.tensor(masked, dtype=torch.int32, device=dev)
    ok, (q, s), (ref_q, ref_s) = _masked_both(dev, a_q, a_s, w_q, w_s, masked_m, col_major_out)
    assert ok
    # every byte and every scale: valid rows equal the two-step result, rows beyond masked_m keep the sentinels
    assert torch.equal(q.view(torch.uint8), ref_q.view(torch.uint8)), 'quantised codes differ'
    assert torch.equal(s, ref_s), 'scales differ'
    valid = torch.arange(M_max, device=dev)[None, :] < masked_m[:, None]
    assert (ref_s[~valid] == -7.0).all() and (ref_s[valid] > 0).all()


def test_masked_shapes_without_a_fused_kernel_are_declined(dev):
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_masked_silu_quant
    a_q = torch.zeros(2, 128, 192, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)   # K % 128 != 0
    a_s = torch.ones(2, 128, 2, device=dev)
    w_q = torch.zeros(2, 256, 192, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    w_s = torch.ones(2, 2, 2, device=dev)
    q = torch.zeros(2, 128, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s = torch.zeros(2, 128, 1, device=dev)
    masked_m = torch.tensor([3, 4], dtype=torch.int32, device=dev)
    assert fp8_gemm_grouped_masked_silu_quant(a_q, a_s, w_q, w_s, q, s, masked_m) is False
    torch.cuda.synchronize()
    assert (s == 0).all()


def test_masked_fused_full_size_and_low_latency_experts(dev):
    """The decode MoE layer's compute on one GPU at the size of the masked benchmark row (32 experts x 256 slots,
    2 x 2048 x 7168 and 7168 x 2048): the fused first half equals the two steps bit for bit, and low_latency_experts,
    which uses it, equals the three-kernel sequence of the reference driver."""
    print('case fused masked gate/up full size', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    from dlblas_amd.kernels.moe import low_latency_experts
    G, M_max, inter, K = 32, 256, 2048, 7168
    gd = torch.Generator(device=dev).manual_seed(31)
    x = torch.randn(G * M_max, K, device=dev, generator=gd).to(torch.bfloat16)
    a_q, a_s = helpers.quantise_act_device(x)
    a_q, a_s = a_q.view(G, M_max, K), a_s.view(G, M_max, K // 128).contiguous()
    w13_q, w13_s = helpers.expert_weights_device(G, 2 * inter, K, dev, 32)
    w2_q, w2_s = helpers.expert_weights_device(G, K, inter, dev, 33)
    masked_m = torch.randint(0, M_max + 1, (G, ), generator=torch.Generator().manual_seed(34)).to(torch.int32).to(dev)
    ok, (q, s), (ref_q, ref_s) = _masked_both(dev, a_q, a_s, w13_q, w13_s, masked_m)
    assert ok
    assert torch.equal(q.view(torch.uint8), ref_q.view(torch.uint8))
    assert torch.equal(s, ref_s)
    out = low_latency_experts((a_q, a_s), w13_q, w13_s, w2_q, w2_s, masked_m, int(masked_m.max()))
    ref = torch.zeros(G, M_max, K, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_masked((ref_q, ref_s), (w2_q, w2_s), ref, masked_m, int(masked_m.max()))
    torch.cuda.synchronize()
    valid = torch.arange(M_max, device=dev)[None, :] < masked_m[:, None]
    assert torch.equal(out[valid], ref[valid])


# --- the fused kernel reading the tokens through the row table of ep_scatter_rows (no expert-sorted copy) ------------


@pytest.mark.parametrize('T,K,inter,E,topk,index_dtype', [
    (96, 512, 256, 4, 2, torch.int64),
    (700, 1024, 384, 8, 8, torch.int32),
    (2000, 256, 128, 40, 3, torch.int64),
    (900, 128, 128, 300, 4, torch.int32),   # more experts than threads in a table-only block
])
def test_gathered_rows_equal_the_copy(dev, T, K, inter, E, topk, index_dtype):
    """ep_scatter_rows leaves the tables ep_scatter leaves, names the token of every destination row, and the fused
    kernel that follows the table writes the bytes and scales of ep_scatter + the fused kernel on the copy."""
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous_silu_quant
    from dlblas_amd.kernels.fused_moe_v3 import ep_scatter, ep_scatter_rows
    print(f'case gathered fused gate/up T={T} K={K} I={inter} E={E} topk={topk}', flush=True)
    g = helpers.gen(900 + T + K + E)
    x_q, x_s = orc.quant_act_1x128((torch.randn(T, K, generator=g) * 1.5).to(torch.bfloat16))
    ws = [orc.quant_weight_128x128((torch.randn(2 * inter, K, generator=g) * 0.05).to(torch.bfloat16)) for _ in range(E)]
    w_q, w_s = torch.stack([w[0] for w in ws]).to(dev), torch.stack([w[1] for w in ws]).to(dev)
    ids = torch.randint(-1, E, (T, topk), generator=g).to(index_dtype)
    ids[torch.rand(T, topk, generator=g) < 0.3] = -1
    routed = torch.bincount(ids[ids >= 0].long(), minlength=E)
    counts = ((routed + 127) // 128 * 128).to(torch.int32).to(dev)
    rows = int(counts.sum())
    x_q, x_s, ids = x_q.to(dev), x_s.to(dev), ids.to(dev)

    sorted_q = torch.zeros(rows, K, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sorted_s = torch.ones(rows, K // 128, device=dev)
    m_ref = torch.empty(rows, dtype=torch.int32, device=dev)
    idx_ref = torch.full_like(ids, -1)
    start_ref = torch.empty(E, dtype=torch.int64, device=dev)
    ep_scatter(x_q, x_s, ids, counts, start_ref, sorted_q, sorted_s, m_ref, idx_ref)

    m_got = torch.full((rows, ), -9, dtype=torch.int32, device=dev)
    row_token = torch.full((rows, ), -9, dtype=torch.int32, device=dev)
    idx_got = torch.full_like(ids, -1)
    start_got = torch.empty(E, dtype=torch.int64, device=dev)
    ep_scatter_rows(ids, counts, start_got, m_got, row_token, idx_got)
    torch.cuda.synchronize()
    assert torch.equal(m_got, m_ref) and torch.equal(idx_got, idx_ref) and torch.equal(start_got, start_ref)
    valid = ids >= 0
    tok = torch.arange(T, device=dev).unsqueeze(1).expand(T, topk)[valid]
    assert torch.equal(row_token[idx_ref[valid]].long(), tok)
    used = torch.zeros(rows, dtype=torch.bool, device=dev)
    used[idx_ref[valid]] = True
    assert (row_token[~used] == 0).all()

    ref = fp8_gemm_grouped_contiguous_silu_quant(sorted_q, sorted_s, w_q, w_s, m_ref)
    got = fp8_gemm_grouped_contiguous_silu_quant(x_q, x_s, w_q, w_s, m_got, a_row_index=row_token, column_major_scales=True)
    torch.cuda.synchronize()
    assert ref is not None and got is not None
    assert torch.equal(got[0].view(torch.uint8)[used], ref[0].view(torch.uint8)[used]), 'quantised codes differ'
    assert torch.equal(got[1][used], ref[1][used]), 'scales differ'
