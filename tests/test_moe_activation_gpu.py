"""GPU parity of the activation kernels (Python entry points -> C ABI) against oracle/moe_activation.py.

Bar: the device evaluates silu with the hardware exponential and reciprocal (a few fp32 ulp from the correctly
rounded value the oracle uses; the reference's own kernels use fast exp and approximate division too), so a result can
differ from the oracle's only where the fp32 value lies within a few ulp of a rounding boundary of the bf16 / fp16
grid - about one element in 10^4.  Stated as: at most 2e-3 of the elements may differ (small samples: 3 groups), and
a differing element is at most one step of its grid away (one bf16 ulp; one e4m3 code where the group's scale
agrees; scales within 2^-7 relative).  The fused
contiguous entry point must equal the two-call sequence of this library bit for bit.
"""
import pytest
import torch

import helpers
from oracle import fp8_block_gemm as orc
from oracle import moe_activation as act

pytestmark = pytest.mark.gpu

MISMATCH_FRAC = 2e-3


@pytest.fixture(scope='module')
def dev():
    from dlblas_amd import _lib
    _lib.load()
    return torch.device('cuda:0')


def _gate_up(shape, seed, dtype=torch.bfloat16, std=2.0):
    g = helpers.gen(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def _check_codes(q_dev, s_dev, q_ref, s_ref, what):
    """codes / scales of the device against the oracle's under the bar of this file's docstring."""
    qd, qr = q_dev.cpu().view(torch.uint8), q_ref.view(torch.uint8)
    sd, sr = s_dev.cpu().float(), s_ref.float()
    assert (sd - sr).abs().max() <= sr.abs().max() * 2**-7, what
    bad_s = int((sd != sr).sum())
    bad_q = int((qd != qr).sum())
    print(f'{what}: scale mismatches {bad_s} of {sd.numel()}, code mismatches {bad_q} of {qd.numel()}', flush=True)
    # a differing scale re-codes its whole group of 128; small samples get an absolute allowance of 3 groups
    assert bad_s <= max(3, MISMATCH_FRAC * sd.numel()), (what, bad_s)
    assert bad_q <= max(3 * 128, 4 * MISMATCH_FRAC * qd.numel()), (what, bad_q)
    # a differing code is a neighbour on the e4m3 grid (codes are ordered by magnitude within a sign) unless its
    # group's scale differs too
    diff = (qd.int() - qr.int()).abs()
    group_ok = (sd == sr).repeat_interleave(128, -1).reshape(diff.shape)
    assert (diff[group_ok] <= 1).all(), what
    deq_d = orc.decode_e4m3fn(q_dev.cpu()) * sd.repeat_interleave(128, -1).reshape(diff.shape)
    deq_r = orc.decode_e4m3fn(q_ref) * sr.repeat_interleave(128, -1).reshape(diff.shape)
    assert (deq_d - deq_r).abs().max() <= deq_r.abs().max() * 2**-3, what


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('M,N', [(1, 128), (37, 256), (256, 2048), (64, 200), (5, 7)])
def test_silu_and_mul(dev, M, N, dtype):
    from dlblas_amd.kernels.activation import silu_and_mul
    print(f'case silu_and_mul M={M} N={N} {dtype}', flush=True)
    x = _gate_up((M, 2 * N), seed=M + N, dtype=dtype)
    ref = act.silu_and_mul_ref(x)
    out = silu_and_mul(x.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == dtype and tuple(out.shape) == (M, N)
    o, r = out.cpu().float(), ref.float()
    bad = int((o != r).sum())
    if dtype != torch.float32:  # fp32 results carry the few-ulp difference of the hardware exp() itself; only the bound below applies
        assert bad <= max(3, MISMATCH_FRAC * o.numel()), bad
    ulp = {torch.bfloat16: 2**-7, torch.float16: 2**-10, torch.float32: 2**-18}[dtype]
    assert ((o - r).abs() <= r.abs() * ulp + 1e-30).all()


def test_silu_and_mul_strided_rows_and_given_out(dev):
    from dlblas_amd.kernels.activation import silu_and_mul
    print('case silu_and_mul strided', flush=True)
    big = _gate_up((16, 3 * 512), seed=4).to(dev)
    x = big[:, :512]                    # row stride 1536, 2N = 512
    out_buf = torch.full((16, 384), 7.0, dtype=torch.bfloat16, device=dev)
    out = out_buf[:, :256]
    res = silu_and_mul(x, out)
    torch.cuda.synchronize()
    assert res.data_ptr() == out.data_ptr()
    ref = act.silu_and_mul_ref(x.cpu())
    assert (out.cpu() != ref).float().mean().item() <= MISMATCH_FRAC
    assert (out_buf[:, 256:] == 7).all()


@pytest.mark.parametrize('col_major', [False, True])
@pytest.mark.parametrize('M,N', [(1, 128), (100, 2048), (512, 1024)])
def test_silu_and_mul_post_quant_contiguous(dev, M, N, col_major):
    from dlblas_amd.kernels.activation import silu_and_mul, silu_and_mul_post_quant
    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    print(f'case silu_and_mul_post_quant M={M} N={N} col_major={col_major}', flush=True)
    x = _gate_up((M, 2 * N), seed=M * 3 + N)
    q_ref, s_ref = act.silu_and_mul_post_quant_ref(x)
    xd = x.to(dev)
    q, s = silu_and_mul_post_quant(xd, 128, column_major_scales=col_major)
    q2, s2 = per_token_group_quant_fp8(silu_and_mul(xd), 128, column_major_scales=col_major)
    torch.cuda.synchronize()
    assert q.dtype == torch.float8_e4m3fn and tuple(s.shape) == (M, N // 128)
    if col_major:
        assert s.stride() == (1, M)
    # fused == the two calls, bit for bit
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
    _check_codes(q, s, q_ref, s_ref, f'post_quant {M}x{N}')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_silu_and_mul_masked_post_quant(dev, dtype):
    from dlblas_amd.kernels.moe import silu_and_mul_masked_post_quant_fwd
    print(f'case masked post quant {dtype}', flush=True)
    E, M, N = 6, 40, 512
    x = _gate_up((E, M, 2 * N), seed=21, dtype=dtype)
    masked = torch.tensor([0, 1, 17, 40, 39, 1000], dtype=torch.int32)
    # rows beyond the mask hold NaN: they must not be read into anything that is written
    for e in range(E):
        x[e, min(int(masked[e]), M):] = float('nan')
    q_ref = torch.full((E, M, N), 0x5a, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s_ref = torch.full((E, M, N // 128), -3.0)
    act.silu_and_mul_masked_post_quant_ref(x, masked, q_ref, s_ref)
    q = torch.full((E, M, N), 0x5a, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s = torch.full((E, M, N // 128), -3.0, device=dev)
    silu_and_mul_masked_post_quant_fwd(x.to(dev), q, s, 128, masked.to(dev))
    torch.cuda.synchronize()
    for e in range(E):
        v = min(int(masked[e]), M)
        assert (q[e, v:].view(torch.uint8) == 0x5a).all() and (s[e, v:] == -3).all(), e   # untouched, bit for bit
    _check_codes(q, s, q_ref, s_ref, f'masked {dtype}')


def test_masked_post_quant_strided_scales_and_full_size(dev):
    """cfg5's second-GEMM input: 32 experts x 256 rows x N = 2048 (gate_up 4096 wide), scales written M-major
    (the layout the masked grouped GEMM reads through strides).  Size-independent properties at full size:
    every written group holds a +-448 code, and the output feeds dlb_fp8_gemm_grouped_masked unchanged."""
    from dlblas_amd.kernels.moe import silu_and_mul_masked_post_quant_fwd
    print('case masked post quant full size', flush=True)
    E, M, N = 32, 256, 2048
    g = helpers.gen(5)
    x = (torch.randn(E, M, 2 * N, generator=g) * 1.5).to(torch.bfloat16).to(dev)
    masked = torch.randint(0, M + 1, (E, ), generator=g, dtype=torch.int32)
    q = torch.zeros(E, M, N, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s_buf = torch.zeros(E, N // 128, M, device=dev)
    s = s_buf.transpose(1, 2)  # [E, M, N/128] with strides (.., 1, M)
    silu_and_mul_masked_post_quant_fwd(x, q, s, 128, masked.to(dev))
    torch.cuda.synchronize()
    # oracle on three experts
    for e in (0, 13, 31):
        v = int(masked[e])
        qr = torch.zeros(1, M, N, dtype=torch.float8_e4m3fn)
        sr = torch.zeros(1, M, N // 128)
        act.silu_and_mul_masked_post_quant_ref(x[e:e + 1].cpu(), masked[e:e + 1], qr, sr)
        _check_codes(q[e, :v], s[e, :v].contiguous(), qr[0, :v], sr[0, :v], f'full size expert {e}')
    codes = orc.decode_e4m3fn(q.cpu()).reshape(E, M, N // 128, 128).abs().amax(-1)
    for e in range(E):
        v = int(masked[e])
        assert (codes[e, :v] == 448).all() and (codes[e, v:] == 0).all()
        assert (s[e, :v] > 0).all() and (s[e, v:] == 0).all()


def test_activation_argument_validation(dev):
    from dlblas_amd.kernels.activation import silu_and_mul, silu_and_mul_post_quant
    from dlblas_amd.kernels.moe import silu_and_mul_masked_post_quant_fwd
    x = torch.zeros(4, 4, 512, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(4, 4, 256, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s = torch.zeros(4, 4, 2, device=dev)
    m = torch.zeros(4, dtype=torch.int32, device=dev)
    with pytest.raises(AssertionError):
        silu_and_mul_masked_post_quant_fwd(x[:, :, ::2], q, s, 128, m)           # not contiguous
    with pytest.raises(AssertionError):
        silu_and_mul_masked_post_quant_fwd(x, q, s, 128, m[:3])                  # expert count mismatch
    with pytest.raises(AssertionError):
        silu_and_mul_masked_post_quant_fwd(x, q, s, 96, m)                       # N % group != 0
    with pytest.raises(NotImplementedError):
        silu_and_mul_masked_post_quant_fwd(x, q, s, 64, m)
    with pytest.raises(AssertionError):
        silu_and_mul(x)                                                          # 3-d input
    with pytest.raises(AssertionError):
        silu_and_mul_post_quant(torch.zeros(4, 200, dtype=torch.bfloat16, device=dev))


@pytest.mark.parametrize('expected_m', [32, 0])
def test_low_latency_experts_end_to_end(dev, expected_m):
    """masked GEMM -> masked silu*up + quant -> masked GEMM (dlblas/layers/moe/ep_moe.py:199-261) against the same
    chain of oracles on the valid rows.  Bar as for the contiguous driver: the reference's similarity metric plus a
    bound on the largest deviation relative to the output's rms (the quantiser between the GEMMs can turn a GEMM
    difference within tolerance into a different fp8 code)."""
    from dlblas_amd import _lib
    from dlblas_amd.kernels.moe import low_latency_experts
    print(f'case low_latency_experts expected_m={expected_m}', flush=True)
    G, M, K, N = 4, 48, 512, 1024
    # a few short experts get 128 x 128 tiles and the steps apart; without the hint the fused gate/up kernel runs
    assert _lib.plan_grouped(2, M, N, K, G, expected_m)[0] == ('pipe128x128' if expected_m > 0 else 'pipe128x256w8')
    g = helpers.gen(91)
    masked = torch.tensor([0, 48, 17, 33], dtype=torch.int32)
    a_q, a_s = orc.quant_act_1x128(torch.randn(G, M, K, generator=g).to(torch.bfloat16))
    w13, w13_s, w2, w2_s = [], [], [], []
    for _ in range(G):
        q, s = orc.quant_weight_128x128((torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16))
        w13.append(q), w13_s.append(s)
        q, s = orc.quant_weight_128x128((torch.randn(K, N // 2, generator=g) * 0.05).to(torch.bfloat16))
        w2.append(q), w2_s.append(s)
    w13, w13_s, w2, w2_s = torch.stack(w13), torch.stack(w13_s), torch.stack(w2), torch.stack(w2_s)
    out = low_latency_experts((a_q.to(dev), a_s.to(dev)), w13.to(dev), w13_s.to(dev), w2.to(dev), w2_s.to(dev),
                              masked.to(dev), expected_m)
    torch.cuda.synchronize()
    gateup = torch.zeros(G, M, N, dtype=torch.bfloat16)
    orc.grouped_masked_ref(a_q, a_s, w13, w13_s, gateup, masked)
    d_q = torch.zeros(G, M, N // 2, dtype=torch.float8_e4m3fn)
    d_s = torch.zeros(G, M, N // 2 // 128)
    act.silu_and_mul_masked_post_quant_ref(gateup, masked, d_q, d_s)
    ref = torch.zeros(G, M, K, dtype=torch.bfloat16)
    orc.grouped_masked_ref(d_q, d_s, w2, w2_s, ref, masked)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (G, M, K)
    for e in range(G):
        v = int(masked[e])
        if v == 0:
            continue
        o, r = out[e, :v].cpu().float(), ref[e, :v].float()
        assert orc.similarity_gap(o, r) <= 1e-4, e
        assert (o - r).abs().max() <= 0.05 * r.pow(2).mean().sqrt(), e
