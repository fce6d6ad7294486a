"""TEST INFRASTRUCTURE ONLY - CPU oracle of the activation step between the two grouped GEMMs of an expert MLP.

Restates (paths relative to the DLBlas tree):

  silu_and_mul_ref                     dlblas/layers/moe/kernels/activation.py:16-95 (``silu_and_mul``): gate and up
                                       halves of a [M, 2N] matrix, both widened to fp32, ``gate / (1 + exp(-gate)) *
                                       up``, ONE rounding to the output dtype (:44-52).  Called between the two
                                       contiguous grouped GEMMs at dlblas/kernels/fused_moe_v3.py:325, followed by
                                       per_token_group_quant_fp8 (:331-334).
  silu_and_mul_post_quant_ref          that sequence as one function: silu_and_mul in the input dtype, then the
                                       1 x 128 quantiser of oracle/fp8_block_gemm.py (dlblas/kernels/fp8.py:44-51).
  silu_and_mul_masked_post_quant_ref   dlblas/kernels/moe.py:204-319 (``silu_and_mul_masked_post_quant_fwd``): per
                                       expert e and token < masked_m[e]; the gate is widened to fp32, ``gate / (1 +
                                       exp(-gate))`` is rounded to the INPUT dtype (:256), multiplied with ``up`` in
                                       the input dtype (:257, a second rounding), then ``s = max(amax, 1e-10) / 448``
                                       and ``q = clamp(x / s, -448, 448)`` cast to e4m3fn (:258-260).  Tokens at or
                                       beyond masked_m[e] are neither read nor written (:244).

Arithmetic that is NOT fixed bit for bit by the reference and how it is taken here: the reference evaluates ``exp``
with Triton's fast exponential and ``/`` with the GPU's approximate division; this oracle uses correctly rounded fp32
``exp`` (evaluated in fp64, rounded to fp32) and IEEE division.  A device result may therefore differ from the oracle
where the fp32 value sits within an ulp of a rounding boundary of the input dtype; tests/helpers.py states the
tolerance that follows from it.  The 1e-10 floor of the masked variant is taken as an fp32 constant (it only decides
the scale that is stored for an all-zero group, whose codes are all zero either way).

How these are pinned (tests/test_oracle_moe_activation.py): the silu formula against torch.nn.functional.silu (library
routine) and its closed-form identities (silu(0) = 0, silu(x) - silu(-x) = x, silu(x) -> x for large x); the gate/up
order by inputs whose gate half is zero (output zero whatever the up half holds) and whose up half is one (output =
silu(gate)); the double rounding of the masked variant against torch's own bf16 multiply and by a constructed input
where single and double rounding differ; the quantisation through the invariants of the 1 x 128 quantiser (amax ->
+-448, |q| <= 448, half-ulp reconstruction); masking by sentinel rows.
"""
import torch

from oracle.fp8_block_gemm import quant_act_1x128


def _silu_f32(g: torch.Tensor) -> torch.Tensor:
    """gate / (1 + exp(-gate)) with every operation rounded to fp32 (exp correctly rounded via fp64)."""
    g = g.float()
    e = torch.exp(-g.double()).float()
    return g / (1.0 + e)


def silu_and_mul_ref(gate_up: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """gate_up [..., 2N] -> [..., N]: silu(gate_up[..., :N]) * gate_up[..., N:] in fp32, one rounding to out_dtype."""
    n = gate_up.shape[-1] // 2
    gate, up = gate_up[..., :n], gate_up[..., n:]
    out = _silu_f32(gate) * up.float()
    return out.to(out_dtype or gate_up.dtype)


def silu_and_mul_post_quant_ref(gate_up: torch.Tensor, eps: float = 1e-10):
    """silu_and_mul in the input dtype followed by the 1 x 128 quantiser.  Returns (q e4m3fn [..., N], s [..., N/128])."""
    return quant_act_1x128(silu_and_mul_ref(gate_up), eps)


def silu_and_mul_masked_post_quant_ref(inp: torch.Tensor, masked_m: torch.Tensor, q: torch.Tensor, s: torch.Tensor):
    """inp [E, M, 2N]; writes q [E, M, N] (e4m3fn) and s [E, M, N/128] for tokens < masked_m[e] only; returns (q, s)."""
    E, M, two_n = inp.shape
    n = two_n // 2
    for e in range(E):
        rows = int(min(max(int(masked_m[e]), 0), M))
        if rows == 0:
            continue
        gate = _silu_f32(inp[e, :rows, :n]).to(inp.dtype)
        # the product of two bf16 / fp16 values is exact in fp32, so this is the input dtype's own multiply
        gate_up = (inp[e, :rows, n:].float() * gate.float()).to(inp.dtype)
        qe, se = quant_act_1x128(gate_up.float(), 1e-10)
        q[e, :rows] = qe
        s[e, :rows] = se
    return q, s
