"""GPU parity at the full benchmark sizes: sampled rows against the CPU oracle plus size-independent properties
(exact power-of-two linearity in the scales, row-permutation equivariance, masked rows untouched)."""
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


def _gemm(a_q, b_q, a_s, b_s, dtype=torch.bfloat16):
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        return fp8_gemm(a_q, b_q, a_s, b_s)
    finally:
        torch.set_default_dtype(prev)


def _sample_rows(M, count, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randperm(M, generator=g)[:count].sort().values


@pytest.mark.parametrize('M,N,K', [(4096, 7168, 18432), (4096, 24576, 1536)])
def test_prefill_full_size(dev, M, N, K):
    print(f'case prefill full size M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense_device(M, N, K, dev)
    out = _gemm(a_q, b_q, a_s, b_s)
    torch.cuda.synchronize()
    rows = _sample_rows(M, 48, 1)
    ref = orc.dequant_ref(a_q[rows].cpu(), a_s[rows].cpu(), b_q.cpu(), b_s.cpu())
    helpers.tolerance_check(out[rows], ref, f'prefill {M}x{N}x{K} sampled rows')
    # doubling every activation scale doubles every output exactly (power of two: no rounding anywhere)
    out2 = _gemm(a_q, b_q, a_s * 2, b_s)
    assert torch.equal(out2, out * 2)
    # permuting the rows of a (and of a_s) permutes the rows of c bit for bit
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(2)).to(dev)
    out3 = _gemm(a_q[perm].contiguous(), b_q, a_s[perm].contiguous(), b_s)
    assert torch.equal(out3, out[perm])


@pytest.mark.parametrize('M,N,K,variant,slices', [
    (384, 18432, 7168, 'pipe128x256w8', 1),    # two 256-row tiles would be half padding: three rows of 128 x 256 tiles
    (2048, 4096, 7168, 'pipe128x256w8', 1),    # 128 tiles of 256 x 256 would leave half the CUs idle
    (4096, 32768, 512, 'pipe128x256w8', 1),    # four K blocks: 16 rounds of resident workgroups
    (512, 4096, 7168, 'pipe128x64', 1),        # the scale table at 56 K blocks
    (64, 1024, 16384, 'pipe128x64', 16),       # 16 K slices
    (16, 36864, 7168, 'skinny16', 1),          # six rounds of decode workgroups
])
def test_planner_choices_full_size(dev, M, N, K, variant, slices):
    """Shapes whose launch the planner's later rules decide, at their real size: sampled rows against the oracle,
    exact power-of-two linearity, row permutation."""
    from dlblas_amd import _lib
    print(f'case planner choice full size M={M} N={N} K={K}', flush=True)
    assert _lib.plan(0, M, N, K)[:2] == (variant, slices)
    a_q, a_s, b_q, b_s = helpers.make_dense_device(M, N, K, dev, seed=M + K)
    out = _gemm(a_q, b_q, a_s, b_s)
    torch.cuda.synchronize()
    rows = _sample_rows(M, min(M, 24), 3)
    ref = orc.dequant_ref(a_q[rows].cpu(), a_s[rows].cpu(), b_q.cpu(), b_s.cpu())
    helpers.tolerance_check(out[rows], ref, f'planner choice {M}x{N}x{K} sampled rows')
    assert torch.equal(_gemm(a_q, b_q, a_s * 4, b_s), out * 4)
    if variant != 'skinny16':  # (the decode kernels' summation order depends on the row fragment a row falls into)
        perm = torch.randperm(M, generator=torch.Generator().manual_seed(4)).to(dev)
        assert torch.equal(_gemm(a_q[perm].contiguous(), b_q, a_s[perm].contiguous(), b_s), out[perm])


@pytest.mark.parametrize('M', [1, 16, 64, 128])
@pytest.mark.parametrize('N,K', [(7168, 2048), (2112, 7168)])
def test_decode_full_size(dev, M, N, K):
    print(f'case decode full size M={M} N={N} K={K}', flush=True)
    a_q, a_s, b_q, b_s = helpers.make_dense_device(M, N, K, dev)
    out = _gemm(a_q, b_q, a_s, b_s)
    torch.cuda.synchronize()
    ref = orc.dequant_ref(a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu())
    helpers.tolerance_check(out, ref, f'decode {M}x{N}x{K}')
    assert torch.equal(_gemm(a_q, b_q, a_s * 0.5, b_s), out * 0.5)


def test_grouped_contiguous_full_size(dev):
    """32 experts, 8192 tokens drawn from a seeded multinomial, every expert's span padded to a multiple of 128
    (padding rows carry the expert id and zero data, the layout dlblas/kernels/fused_moe_v3.py:40-44 produces)."""
    print('case grouped contiguous full size', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_contiguous
    G, N, K, tokens = 32, 4096, 7168, 8192
    g = torch.Generator().manual_seed(20)
    assign = torch.multinomial(torch.full((G, ), 1.0 / G), tokens, replacement=True, generator=g)
    counts = torch.bincount(assign, minlength=G)
    padded = (counts + 127) // 128 * 128
    M_sum = int(padded.sum())
    m_indices = torch.repeat_interleave(torch.arange(G, dtype=torch.int32), padded)
    valid = torch.cat([torch.arange(int(p)) < int(c) for p, c in zip(padded, counts)])
    gd = torch.Generator(device=dev).manual_seed(21)
    a = torch.randn(M_sum, K, device=dev, generator=gd).to(torch.bfloat16)
    a[~valid.to(dev)] = 0
    a_q, a_s = helpers.quantise_act_device(a)
    w_q, w_s = helpers.expert_weights_device(G, N, K, dev, 22)
    out = torch.full((M_sum, N), 3.0, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_contiguous((a_q, a_s), (w_q, w_s), out, m_indices.to(dev))
    torch.cuda.synchronize()
    rows = _sample_rows(M_sum, 64, 3)
    for r in rows.tolist():
        e = int(m_indices[r])
        ref = orc.dequant_ref(a_q[r:r + 1].cpu(), a_s[r:r + 1].cpu(), w_q[e].cpu(), w_s[e].cpu())
        if bool(valid[r]):
            helpers.tolerance_check(out[r:r + 1], ref, f'contiguous row {r} expert {e}')
        else:
            assert torch.all(out[r] == 0), 'a zero padding row must give zeros'
    # column-major activation scales (the layout the reference hands over) give the same bits
    a_s_cm = a_s.t().contiguous().t()
    assert not a_s_cm.is_contiguous()
    out2 = torch.empty_like(out)
    m_grouped_fp8_gemm_nt_contiguous((a_q, a_s_cm), (w_q, w_s), out2, m_indices.to(dev))
    assert torch.equal(out2, out)


def test_grouped_masked_full_size(dev):
    print('case grouped masked full size', flush=True)
    from dlblas_amd.kernels.fp8_gemm_grouped import m_grouped_fp8_gemm_nt_masked
    G, M_max, N, K = 32, 256, 7168, 2048
    g = torch.Generator().manual_seed(20)
    masked_m = torch.randint(0, M_max + 1, (G, ), generator=g, dtype=torch.int32)
    gd = torch.Generator(device=dev).manual_seed(23)
    a = torch.randn(G * M_max, K, device=dev, generator=gd).to(torch.bfloat16)
    a_q, a_s = helpers.quantise_act_device(a)
    a_q, a_s = a_q.reshape(G, M_max, K), a_s.reshape(G, M_max, K // 128).clone()
    bits = a_q.view(torch.uint8).clone()
    garbage = torch.randint(0, 256, bits.shape, device=dev, generator=gd, dtype=torch.uint8)  # includes NaN codes
    beyond = (torch.arange(M_max, device=dev)[None, :] >= masked_m.to(dev)[:, None])
    bits[beyond] = garbage[beyond]
    a_s[beyond] = float('nan')
    a_q = bits.view(torch.float8_e4m3fn)
    w_q, w_s = helpers.expert_weights_device(G, N, K, dev, 24)
    sentinel = -7.0
    out = torch.full((G, M_max, N), sentinel, dtype=torch.bfloat16, device=dev)
    m_grouped_fp8_gemm_nt_masked((a_q, a_s), (w_q, w_s), out, masked_m.to(dev), int(masked_m.float().mean()))
    torch.cuda.synchronize()
    assert torch.all(out[beyond] == sentinel), 'rows at or beyond masked_m were written'
    assert not torch.isnan(out.float()).any()
    for e in (0, 7, 19, 31):
        m = int(masked_m[e])
        if m == 0:
            continue
        ref = orc.dequant_ref(a_q[e, :m].cpu(), a_s[e, :m].cpu(), w_q[e].cpu(), w_s[e].cpu())
        helpers.tolerance_check(out[e, :m], ref, f'masked expert {e} ({m} rows)')
