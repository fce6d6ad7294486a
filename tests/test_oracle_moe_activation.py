"""Pins of oracle/moe_activation.py that do not retype its formulas: library routines, closed forms, constructed
inputs where a plausible mistake (halves swapped, single instead of double rounding, mask off by one) changes the
answer."""
import torch

import helpers
from oracle import fp8_block_gemm as orc
from oracle import moe_activation as act


def _gate_up(M, N, seed=3, dtype=torch.bfloat16, std=2.0):
    g = helpers.gen(seed)
    return (torch.randn(M, 2 * N, generator=g) * std).to(dtype)


def test_silu_matches_library_routine_and_identities():
    x = torch.arange(-2000, 2001).float() * 0.015  # symmetric grid on [-30, 30], exact zero in the middle
    ones = torch.ones_like(x)
    got = act.silu_and_mul_ref(torch.cat([x, ones]).reshape(1, -1).float(), torch.float32)[0]
    torch.testing.assert_close(got, torch.nn.functional.silu(x), rtol=2e-6, atol=1e-30)
    # closed forms: silu(0) = 0, silu(x) - silu(-x) = x, silu(x) -> x and silu(-x) -> 0 for large x
    assert got[2000] == 0
    torch.testing.assert_close(got - got.flip(0), x, rtol=1e-5, atol=1e-5)
    assert got[-1] == 30.0 and abs(got[0]) < 1e-11


def test_gate_is_first_half_up_is_second_half():
    M, N = 5, 256
    x = _gate_up(M, N)
    x[:, :N] = 0                     # gate half zero -> output zero whatever the up half holds
    assert torch.count_nonzero(act.silu_and_mul_ref(x)) == 0
    y = _gate_up(M, N)
    y[:, N:] = 1                     # up half one -> output = silu(gate)
    ref = torch.nn.functional.silu(y[:, :N].float()).to(torch.bfloat16)
    assert (act.silu_and_mul_ref(y).float() - ref.float()).abs().max() <= 2**-7 * ref.float().abs().max()
    z = torch.zeros(1, 4, dtype=torch.float32)
    z[0] = torch.tensor([20.0, -20.0, 3.0, 5.0])  # N = 2: gate (20, -20), up (3, 5)
    out = act.silu_and_mul_ref(z)
    torch.testing.assert_close(out, torch.tensor([[60.0, -20.0 * 5.0 / (1 + 4.851652e8)]]), rtol=1e-6, atol=0)


def test_single_rounding_of_the_unfused_variant():
    # silu(g) * u is rounded ONCE to bf16: compare with an fp64 evaluation rounded once
    x = _gate_up(64, 128, seed=5)
    g, u = x[:, :128].double(), x[:, 128:].double()
    exact = (g / (1 + torch.exp(-g)) * u)
    got = act.silu_and_mul_ref(x).double()
    # one bf16 rounding of a value computed in fp32: within half a bf16 ulp (<= 2^-8 relative, + fp32 noise) of the
    # exact value; a second rounding would reach 2^-7
    assert ((got - exact).abs() <= exact.abs() * (2**-8 + 2**-20) + 1e-38).all()


def test_masked_variant_rounds_twice_in_the_input_dtype():
    E, M, N = 2, 8, 128
    x = _gate_up(E * M, N, seed=9).reshape(E, M, 2 * N)
    masked = torch.tensor([M, M], dtype=torch.int32)
    q = torch.zeros(E, M, N, dtype=torch.float8_e4m3fn)
    s = torch.zeros(E, M, 1)
    act.silu_and_mul_masked_post_quant_ref(x, masked, q, s)
    # independent construction with torch's own bf16 arithmetic for the second rounding
    gate = torch.nn.functional.silu(x[..., :N].float()).to(torch.bfloat16)
    gate_up = x[..., N:] * gate  # bf16 * bf16 -> bf16 multiply of the library
    q2, s2 = orc.quant_act_1x128(gate_up)
    # torch's silu may differ from the oracle's in the last fp32 bit; that flips a bf16 rounding only rarely
    same = (q.view(torch.uint8) == q2.view(torch.uint8)).float().mean().item()
    assert same > 0.999, same
    assert (s.squeeze(-1) == s2.squeeze(-1)).float().mean().item() > 0.9
    # and the double rounding is observable: some products differ from the singly rounded ones
    once = act.silu_and_mul_ref(x)
    twice = (x[..., N:].float() * act._silu_f32(x[..., :N]).to(torch.bfloat16).float()).to(torch.bfloat16)
    assert (once != twice).any()


def test_masked_rows_are_untouched_and_mask_is_exclusive():
    E, M, N = 3, 6, 256
    x = _gate_up(E * M, N, seed=11).reshape(E, M, 2 * N)
    masked = torch.tensor([0, 4, 9], dtype=torch.int32)  # empty, partial, beyond M (clamped)
    q = torch.full((E, M, N), 0x55, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s = torch.full((E, M, N // 128), -7.0)
    act.silu_and_mul_masked_post_quant_ref(x, masked, q, s)
    qb = q.view(torch.uint8)
    assert (qb[0] == 0x55).all() and (s[0] == -7).all()
    assert (qb[1, 4:] == 0x55).all() and (s[1, 4:] == -7).all() and (s[1, :4] > 0).all()
    assert (s[2] > 0).all()
    # row 3 of expert 1 (the last valid one) is written: its amax element maps to +-448
    deq = orc.decode_e4m3fn(q[1, 3]).reshape(N // 128, 128).abs().amax(-1)
    assert (deq == 448).all()


def test_quantised_output_reconstructs_the_activation():
    x = _gate_up(32, 512, seed=13)
    q, s = act.silu_and_mul_post_quant_ref(x)
    y = act.silu_and_mul_ref(x).float()
    deq = orc.decode_e4m3fn(q).reshape(32, 4, 128) * s.unsqueeze(-1)
    err = (deq.reshape(32, 512) - y).abs()
    # e4m3 has 3 mantissa bits: half an ulp is at most 2^-4 of the value, subnormal step 2^-9 of the scale unit
    bound = y.abs() * 2**-4 + s.repeat_interleave(128, -1) * 2**-10 + 1e-30
    assert (err <= bound).all()
    assert (orc.decode_e4m3fn(q).abs() <= 448).all()
