"""GPU parity of the per-token-group activation quantiser (1 x 128 and any other group size) and of the 128 x 128 weight
quantiser against the CPU oracle: byte-exact codes, bit-exact scales."""
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


def _check(x_cpu, dev, column_major=False):
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    q_ref, s_ref = orc.quant_act_1x128(x_cpu)
    q, s = per_token_group_quant_fp8(x_cpu.to(dev), 128, column_major_scales=column_major)
    torch.cuda.synchronize()
    assert q.dtype == torch.float8_e4m3fn and q.shape == x_cpu.shape
    assert s.dtype == torch.float32 and tuple(s.shape) == tuple(s_ref.shape)
    if column_major and x_cpu.dim() == 2:
        assert s.stride(0) == 1 and s.stride(1) == x_cpu.shape[0]
    assert torch.equal(s.cpu(), s_ref), 'scales differ'
    same = q.cpu().view(torch.uint8) == q_ref.view(torch.uint8)
    # +0 / -0 are the same value; everything else must be the same byte
    zero = (q_ref.view(torch.uint8) & 0x7F) == 0
    assert bool((same | (zero & ((q.cpu().view(torch.uint8) & 0x7F) == 0))).all()), \
        f'{int((~same).sum())} of {same.numel()} codes differ'
    return q, s


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('M,K', [(1, 128), (37, 512), (300, 7168), (4096, 2048)])
def test_quant_matches_oracle_bit_for_bit(dev, dtype, M, K):
    print(f'case quant {dtype} M={M} K={K}', flush=True)
    g = helpers.gen(31)
    x = (torch.randn(M, K, generator=g) * 3).to(dtype)
    _check(x, dev)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('group_size,M,K', [(32, 40, 256), (64, 300, 7168), (256, 33, 1024), (512, 20, 2048), (96, 50, 960), (8, 9, 64),
                                             (1024, 6, 2048), (100, 17, 700), (1, 5, 24), (2048, 3, 2048)])
def test_quant_any_group_size(dev, dtype, group_size, M, K):
    """The reference's signature takes any group size that divides the row (dlblas/kernels/fp8.py:35-36,147): multiples
    of 8 up to 512 run on the vector kernel (lanes past a group that is no power of two are masked), the rest on the
    element-wise kernel.  Byte-exact codes, bit-exact scales, row-major and column-major scale layouts."""
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    print(f'case quant group_size={group_size} {dtype} M={M} K={K}', flush=True)
    g = helpers.gen(35)
    x = (torch.randn(M, K, generator=g) * 2).to(dtype)
    x[0, :group_size] = 0   # an all-zero group takes the eps scale
    q_ref, s_ref = orc.quant_act_group(x, group_size)
    for column_major in (False, True):
        q, s = per_token_group_quant_fp8(x.to(dev), group_size, column_major_scales=column_major)
        torch.cuda.synchronize()
        assert tuple(s.shape) == (M, K // group_size) and torch.equal(s.cpu(), s_ref)
        if column_major:
            assert s.stride(0) == 1
        got, want = q.cpu().view(torch.uint8), q_ref.view(torch.uint8)
        assert bool(((got == want) | (((got | want) & 0x7F) == 0)).all()), f'{int((got != want).sum())} codes differ'


def test_quant_edge_values(dev):
    """Zero groups (eps scale), one huge outlier per group, values on e4m3 rounding ties, subnormal results."""
    print('case quant edges', flush=True)
    g = helpers.gen(32)
    x = torch.randn(64, 512, generator=g)
    x[0] = 0
    x[1, :128] = 0
    x[2, 5] = 1e4
    x[3, :128] = torch.linspace(-448, 448, 128)      # scale exactly 1: codes are the rounding of the inputs
    x[4, :128] = torch.tensor([17.0, 19.0, 21.0, 23.0] * 32) * (448.0 / 23.0) / (448.0 / 23.0)
    x[4, 0] = 448.0                                    # scale 1 again: 17, 19, 21, 23 are ties between e4m3 neighbours
    x[5, :128] = 1e-3 * torch.rand(128, generator=g)
    x[5, 0] = 448.0                                    # the rest of the group lands in the subnormal range
    _check(x.to(torch.float32), dev)
    _check(x.to(torch.bfloat16), dev)


def test_quant_column_major_scales_and_strided_rows(dev):
    print('case quant column major', flush=True)
    g = helpers.gen(33)
    x = torch.randn(200, 1024, generator=g).to(torch.bfloat16)
    q, s = _check(x, dev, column_major=True)
    # rows taken out of a wider buffer (row stride > K), as when quantising half of a gate-up output
    wide = torch.randn(50, 2048, generator=g).to(torch.bfloat16)
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    q2, s2 = per_token_group_quant_fp8(wide.to(dev)[:, :1024], 128)
    q_ref, s_ref = orc.quant_act_1x128(wide[:, :1024])
    assert torch.equal(s2.cpu(), s_ref) and torch.equal(q2.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_quant_3d_input_and_asserts(dev):
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    g = helpers.gen(34)
    x = torch.randn(4, 30, 256, generator=g).to(torch.bfloat16)
    _check(x, dev)
    with pytest.raises(AssertionError, match='must be divisible'):
        per_token_group_quant_fp8(torch.zeros(4, 100, device=dev), 128)
    with pytest.raises(AssertionError, match='groups must be contiguous'):
        per_token_group_quant_fp8(torch.zeros(256, 4, device=dev).t(), 128)


def test_quant_feeds_the_gemm(dev):
    """End to end on the device: quantise activations with the kernel, multiply, compare with the oracle fed by
    the oracle's own quantiser (identical bits in, so the usual GEMM tolerance applies)."""
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    g = helpers.gen(35)
    a = torch.randn(96, 1024, generator=g).to(torch.bfloat16)
    b_q, b_s = orc.quant_weight_128x128((torch.randn(384, 1024, generator=g) * 0.02).to(torch.bfloat16))
    a_q, a_s = per_token_group_quant_fp8(a.to(dev), 128)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        out = fp8_gemm(a_q, b_q.to(dev), a_s, b_s.to(dev))
    finally:
        torch.set_default_dtype(prev)
    a_q_ref, a_s_ref = orc.quant_act_1x128(a)
    helpers.tolerance_check(out, orc.dequant_ref(a_q_ref, a_s_ref, b_q, b_s), 'quant + gemm')


def _check_block(w_cpu, dev):
    from dlblas_amd.kernels.fp8 import per_block_quant_fp8
    if w_cpu.dim() == 2:
        q_ref, s_ref = orc.quant_weight_128x128(w_cpu)
    else:
        qs = [orc.quant_weight_128x128(w_cpu[i]) for i in range(w_cpu.shape[0])]
        q_ref, s_ref = torch.stack([q for q, _ in qs]), torch.stack([s for _, s in qs])
    q, s = per_block_quant_fp8(w_cpu.to(dev))
    torch.cuda.synchronize()
    assert q.dtype == torch.float8_e4m3fn and q.shape == w_cpu.shape and tuple(s.shape) == tuple(s_ref.shape)
    assert torch.equal(s.cpu(), s_ref), 'scales differ'
    qb, rb = q.cpu().view(torch.uint8), q_ref.view(torch.uint8)
    same = (qb == rb) | (((qb & 0x7F) == 0) & ((rb & 0x7F) == 0))
    assert bool(same.all()), f'{int((~same).sum())} of {same.numel()} codes differ'
    return q, s


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('shape', [(128, 128), (2112, 7168), (300, 392), (1, 8), (3, 200, 264), (4, 512, 1024)])
def test_block_quant_matches_oracle_bit_for_bit(dev, dtype, shape):
    """128 x 128 weight blocks, ragged at the N and K edges, 2-d and per-expert 3-d."""
    print(f'case block quant {dtype} {shape}', flush=True)
    g = helpers.gen(41)
    w = (torch.randn(*shape, generator=g) * 0.02).to(dtype)
    _check_block(w, dev)


def test_block_quant_edge_values_and_feeds_the_gemm(dev):
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    print('case block quant edges', flush=True)
    w = torch.zeros(256, 256, dtype=torch.bfloat16)
    w[:128, :128] = 0                      # all-zero block: eps scale, zero codes
    w[128:, :128] = 3.0                    # constant block: every code is 448
    w[:128, 128:] = torch.linspace(-1, 1, 128 * 128).reshape(128, 128).to(torch.bfloat16)
    w[128:, 128:] = 1e-30                  # far below eps
    q, s = _check_block(w, dev)
    assert s[0, 0] == torch.tensor(1e-10, dtype=torch.float32) / 448
    assert (orc.decode_e4m3fn(q[128:, :128].cpu()) == 448).all()
    # the quantised weight is a valid b / b_s operand
    g = helpers.gen(43)
    wb = (torch.randn(384, 1024, generator=g) * 0.02).to(torch.bfloat16)
    a_q, a_s = orc.quant_act_1x128(torch.randn(64, 1024, generator=g).to(torch.bfloat16))
    b_q, b_s = _check_block(wb, dev)
    out = fp8_gemm(a_q.to(dev), b_q, a_s.to(dev), b_s)
    torch.cuda.synchronize()
    helpers.tolerance_check(out, orc.dequant_ref(a_q, a_s, b_q.cpu(), b_s.cpu()), 'gemm on device-quantised weights')


def test_block_quant_asserts(dev):
    from dlblas_amd.kernels.fp8 import per_block_quant_fp8
    w = torch.zeros(128, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError):
        per_block_quant_fp8(w, 64)
    with pytest.raises(AssertionError):
        per_block_quant_fp8(torch.zeros(128, 132, dtype=torch.bfloat16, device=dev)[:, :4])
    with pytest.raises(ValueError):
        per_block_quant_fp8(torch.zeros(128, dtype=torch.bfloat16, device=dev))
