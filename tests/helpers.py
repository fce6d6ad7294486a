"""Seeded synthetic inputs shared by the tests (CPU tensors; the GPU tests copy them to the device)."""
import torch

from oracle import fp8_block_gemm as orc

SEED = 20  # the seed the reference's own core tests use (tests/test_kernels.py:14)


def gen(seed=SEED):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def make_dense(M, N, K, seed=SEED, a_std=1.0, b_std=0.02):
    """A ~ N(0, a_std) [M, K], B ~ N(0, b_std) [N, K], both bf16, quantised 1x128 / 128x128 (K padded to 128
    for the quantiser and cut back, so ragged K works)."""
    g = gen(seed)
    Kp = -(-K // 128) * 128
    a = (torch.randn(M, Kp, generator=g) * a_std).to(torch.bfloat16)
    b = (torch.randn(N, Kp, generator=g) * b_std).to(torch.bfloat16)
    a[:, K:] = 0
    b[:, K:] = 0
    a_q, a_s = orc.quant_act_1x128(a)
    b_q, b_s = orc.quant_weight_128x128(b)
    return a_q[:, :K].contiguous(), a_s, b_q[:, :K].contiguous(), b_s


def make_raw(M, N, K, seed=SEED, scale_kind='randn'):
    """The reference test's construction (tests/kernels/test_fp8_gemm.py:17-31): randn cast straight to e4m3fn,
    scales are unclamped normals (negative values included)."""
    g = gen(seed)
    a_q = torch.randn(M, K, generator=g).to(torch.float8_e4m3fn)
    b_q = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    kb, nb = -(-K // 128), -(-N // 128)
    if scale_kind == 'randn':
        a_s = torch.randn(M, kb, generator=g)
        b_s = torch.randn(nb, kb, generator=g)
    else:
        a_s = torch.ones(M, kb)
        b_s = torch.ones(nb, kb)
    return a_q, a_s, b_q, b_s


REL_TOL = 1e-2        # the stated bar: max relative error against the fp32 oracle, after bf16 rounding
FLOOR_FRAC = 5e-2     # |ref| below 5 % of rms(ref) is judged against 5 % of rms(ref) instead of against itself
F32_ABS_FRAC = 3e-4   # fp32 outputs: max |out - ref| <= 3e-4 * rms(ref)


def tolerance_check(out, ref_f32, what=''):
    """Parity bar of the GPU tests.

    bf16 outputs: max |out - ref| / max(|ref|, 0.05 rms(ref)) <= 1e-2.  The floor is what the hardware sets: the
    gfx950 f8f6f4 MFMA aligns the 8 products of each 8-byte K group to the group's largest exponent and keeps
    about 14 bits below it (measured on the device: a product 2^-14 of its group's largest is dropped), which
    leaves an absolute error of up to ~1e-4 rms(ref) per element; bf16 rounding adds up to 2^-8 |ref|.
    fp32 outputs are held to the absolute part alone, 3e-4 rms(ref).
    Both also have to meet the reference's global similarity metric (dlblas/utils/utils.py:113-170).
    Returns the error against the stricter floor of 1e-3 rms(ref) for reporting.
    """
    o = out.float().cpu()
    gap = orc.similarity_gap(o, ref_f32)
    assert gap <= 1e-5, f'{what}: similarity gap {gap:.3e}'
    if out.dtype == torch.float32:
        rms = float(ref_f32.double().pow(2).mean().sqrt())
        worst = float((o.double() - ref_f32.double()).abs().max())
        assert worst <= F32_ABS_FRAC * rms, f'{what}: max abs error {worst:.3e} > {F32_ABS_FRAC} * rms ({rms:.3e})'
    else:
        err = orc.max_rel_err(o, ref_f32, FLOOR_FRAC)
        assert err <= REL_TOL, f'{what}: max relative error {err:.3e} > {REL_TOL} (similarity gap {gap:.3e})'
    return orc.max_rel_err(o, ref_f32, 1e-3)
