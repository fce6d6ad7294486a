"""MoE kernels of the FP8 expert MLP that sit next to the grouped GEMMs.

``silu_and_mul_masked_post_quant_fwd`` is a drop-in for the reference function of the same name
(dlblas/kernels/moe.py:264-319; kernel :204-261): same positional signature, same assertions, results written into
the caller's ``output`` / ``output_scale``.  It runs between the two masked grouped GEMMs
(dlblas/layers/moe/ep_moe.py:245-251).  Only quant_group_size 128 and float8_e4m3fn outputs are implemented.
"""
import torch

from .. import _lib


@torch.library.custom_op('dlblas::silu_and_mul_masked_post_quant', mutates_args=('output', 'output_scale'), device_types='cuda')
def _masked_op(input: torch.Tensor, output: torch.Tensor, output_scale: torch.Tensor, masked_m: torch.Tensor) -> None:
    G, M_max, two_n = input.shape
    _lib.silu_mul_quant_masked(input, output, output_scale, masked_m, G, M_max, two_n // 2, output_scale.stride())


def silu_and_mul_masked_post_quant_fwd(
    input: torch.Tensor,
    output: torch.Tensor,
    output_scale: torch.Tensor,
    quant_group_size: int,
    masked_m: torch.Tensor,
):
    """input [E, M_max, 2N] (bf16 / fp16 / fp32) -> output [E, M_max, N] fp8 and output_scale [E, M_max, N / 128] fp32
    for the first masked_m[e] tokens of every expert; other rows of both outputs keep their content."""
    assert input.is_contiguous()
    assert output.is_contiguous()
    assert len(input.shape) == 3
    assert input.shape[0] == masked_m.shape[0]
    assert input.shape[-1] % 2 == 0
    size_n = input.shape[-1] // 2
    assert size_n % quant_group_size == 0
    if quant_group_size != 128:
        raise NotImplementedError(f'only quant_group_size 128 is implemented, got {quant_group_size}')
    if output.dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f'only float8_e4m3fn output is implemented, got {output.dtype}')
    if input.dtype not in _lib.IN_CODES:
        raise TypeError(f'input must be bfloat16, float16 or float32, got {input.dtype}')
    if tuple(output.shape) != (input.shape[0], input.shape[1], size_n):
        raise ValueError(f'output shape {tuple(output.shape)} does not match input {tuple(input.shape)}')
    if tuple(output_scale.shape) != (input.shape[0], input.shape[1], size_n // 128) or output_scale.dtype != torch.float32:
        raise ValueError('output_scale must be float32 [E, M_max, N / 128]')
    if masked_m.dtype != torch.int32:
        masked_m = masked_m.to(torch.int32)
    _masked_op(input, output, output_scale, masked_m.contiguous())


def low_latency_experts(
    hidden_states_fp8,
    gate_up_weight: torch.Tensor,
    gate_up_scale: torch.Tensor,
    gate_down_weight: torch.Tensor,
    gate_down_scale: torch.Tensor,
    masked_m: torch.Tensor,
    expected_m: int,
    out_dtype: torch.dtype = torch.bfloat16,
    block_size: int = 128,
):
    """The per-GPU compute of the decode MoE layer, ``FusedMoELowLatency.experts`` of the reference
    (dlblas/layers/moe/ep_moe.py:199-261) without its dispatch / combine: masked grouped GEMM (gate and up) ->
    silu * up + 1 x 128 quantisation of the valid rows -> masked grouped GEMM (down).

    hidden_states_fp8 = (a [G, M_max, K] fp8, a_s [G, M_max, K / 128] fp32); weights [G, N, K] / [G, K, N / 2] fp8 with
    128 x 128 block scales; masked_m [G] int32.  Returns down_output [G, M_max, K] in out_dtype; rows at or beyond
    masked_m[g] are not written (they hold whatever the allocation held, as in the reference).
    """
    from .fp8_gemm_grouped import fp8_gemm_grouped_masked_silu_quant, m_grouped_fp8_gemm_nt_masked
    a, a_s = hidden_states_fp8
    num_groups, m, k = a.shape
    n = gate_up_weight.size(1)
    expected_m = min(expected_m, m)
    down_input = torch.empty((num_groups, m, n // 2), device=a.device, dtype=gate_down_weight.dtype)
    fused = False
    # The fused kernel exists for the 128 x 256 tiles only; where expected_m makes the library pick other tiles for the
    # plain GEMM (a few short experts, or several hundred rows per expert) the steps apart are faster (8 experts x up to
    # 128 rows: 60 against 78 us; 32 experts x ~520 rows: 619 against 678 us).
    from .. import _lib
    want_fused = _lib.plan_grouped(2, m, n, k, num_groups, expected_m)[0] == 'pipe128x256w8'
    if want_fused and out_dtype == torch.bfloat16 and block_size == 128 and n % 256 == 0 and masked_m.dtype == torch.int32:
        # one kernel for GEMM + activation + quantiser, same bits; its scales go out with the rows of a K block
        # contiguous, the layout the second GEMM reads without a re-layout pass
        down_input_scale = torch.empty((num_groups, n // 2 // block_size, m), device=a.device, dtype=torch.float32).transpose(1, 2)
        fused = fp8_gemm_grouped_masked_silu_quant(a, a_s, gate_up_weight, gate_up_scale, down_input, down_input_scale,
                                                   masked_m, expected_m)
    if not fused:
        gateup_output = torch.empty((num_groups, m, n), device=a.device, dtype=out_dtype)
        m_grouped_fp8_gemm_nt_masked((a, a_s), (gate_up_weight, gate_up_scale), gateup_output, masked_m, expected_m)
        down_input_scale = torch.empty((num_groups, m, n // 2 // block_size), device=a.device, dtype=torch.float32)
        silu_and_mul_masked_post_quant_fwd(gateup_output, down_input, down_input_scale, block_size, masked_m)
        del gateup_output
    down_output = torch.empty((num_groups, m, gate_down_weight.size(1)), device=a.device, dtype=out_dtype)
    m_grouped_fp8_gemm_nt_masked((down_input, down_input_scale), (gate_down_weight, gate_down_scale), down_output, masked_m,
                                 expected_m)
    return down_output
