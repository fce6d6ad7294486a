"""Expert-contiguous FP8 MoE forward of the reference (dlblas/kernels/fused_moe_v3.py), on the gfx950 kernels of this
package: ``ep_scatter`` (:95-158), ``ep_gather`` (:199-233) and the driver ``fused_moe_v3`` (:246-343) with the same
positional signatures.  Differences a caller can observe: destination rows are handed out in token-major order instead
of atomic order (both satisfy the contract that ``output_index`` names the row each slot was copied to), and the
driver runs the gate/up GEMM, silu_and_mul and the quantiser as one kernel (same bits as the three steps) that reads the
tokens through the row table of ``ep_scatter_rows`` instead of an expert-sorted copy, and skips the scale re-layout the
reference needs for its GEMM.
"""
from typing import List, Optional, Tuple

import torch

from .. import _lib
from .activation import silu_and_mul_post_quant
from .fp8_gemm_grouped import fp8_gemm_grouped_contiguous_silu_quant, m_grouped_fp8_gemm_nt_contiguous


@torch.library.custom_op('dlblas::ep_scatter', mutates_args=('expert_start_loc', 'output_tensor', 'output_tensor_scale',
                                                             'm_indices', 'output_index'), device_types='cuda')
def _scatter_op(recv_x: torch.Tensor, recv_x_scale: torch.Tensor, recv_topk: torch.Tensor,
                num_recv_tokens_per_expert: torch.Tensor, expert_start_loc: torch.Tensor, output_tensor: torch.Tensor,
                output_tensor_scale: torch.Tensor, m_indices: torch.Tensor, output_index: torch.Tensor) -> None:
    _lib.ep_scatter(recv_x, recv_x_scale, recv_topk, num_recv_tokens_per_expert, expert_start_loc, output_tensor,
                    output_tensor_scale, m_indices, output_index)


@torch.library.custom_op('dlblas::ep_scatter_rows', mutates_args=('expert_start_loc', 'm_indices', 'src_row', 'output_index'),
                         device_types='cuda')
def _scatter_rows_op(recv_topk: torch.Tensor, num_recv_tokens_per_expert: torch.Tensor, expert_start_loc: torch.Tensor,
                     m_indices: torch.Tensor, src_row: torch.Tensor, output_index: torch.Tensor) -> None:
    _lib.ep_scatter_rows(recv_topk, num_recv_tokens_per_expert, expert_start_loc, m_indices, src_row, output_index)


@torch.library.custom_op('dlblas::ep_gather', mutates_args=('output_tensor', ), device_types='cuda')
def _gather_op(input_tensor: torch.Tensor, recv_topk_ids: torch.Tensor, recv_topk_weight: torch.Tensor,
               input_index: torch.Tensor, output_tensor: torch.Tensor) -> None:
    _lib.ep_gather(input_tensor, recv_topk_ids, recv_topk_weight, input_index, output_tensor)


@torch.no_grad()
def ep_scatter(
    recv_x: torch.Tensor,
    recv_x_scale: torch.Tensor,
    recv_topk: torch.Tensor,
    num_recv_tokens_per_expert: torch.Tensor,
    expert_start_loc: torch.Tensor,
    output_tensor: torch.Tensor,
    output_tensor_scale: torch.Tensor,
    m_indices: torch.Tensor,
    output_index: torch.Tensor,
):
    """recv_x [T, H] fp8 and recv_x_scale [T, H / 128] are copied to output_tensor / output_tensor_scale so that the
    rows of each expert are adjacent; m_indices [rows] gets the expert of every reserved row, output_index [T, topk]
    the destination row of every routed slot, expert_start_loc [E] the first free row of every expert."""
    assert m_indices.shape[0] % 128 == 0, 'every expert span is a whole number of 128-row GEMM blocks'
    assert recv_x.dim() == 2 and recv_topk.dim() == 2 and recv_x.shape[0] == recv_topk.shape[0]
    assert recv_x.stride(1) == 1 and output_tensor.stride(1) == 1, 'rows must be contiguous'
    if recv_x.dtype != torch.float8_e4m3fn or output_tensor.dtype != torch.float8_e4m3fn:
        raise TypeError('recv_x and output_tensor must be float8_e4m3fn')
    if recv_x_scale.dtype != torch.float32 or output_tensor_scale.dtype != torch.float32:
        raise TypeError('scales must be float32')
    if num_recv_tokens_per_expert.dtype != torch.int32 or m_indices.dtype != torch.int32:
        raise TypeError('num_recv_tokens_per_expert and m_indices must be int32')
    if not (num_recv_tokens_per_expert.is_contiguous() and expert_start_loc.is_contiguous() and m_indices.is_contiguous()):
        raise ValueError('num_recv_tokens_per_expert, expert_start_loc and m_indices must be contiguous')
    _scatter_op(recv_x, recv_x_scale, recv_topk, num_recv_tokens_per_expert, expert_start_loc, output_tensor,
                output_tensor_scale, m_indices, output_index)
    return


@torch.no_grad()
def ep_scatter_rows(recv_topk: torch.Tensor, num_recv_tokens_per_expert: torch.Tensor, expert_start_loc: torch.Tensor,
                    m_indices: torch.Tensor, src_row: torch.Tensor, output_index: torch.Tensor):
    """The tables of ``ep_scatter`` without its copy: ``m_indices``, ``expert_start_loc`` and ``output_index`` as that call
    leaves them, and ``src_row`` [rows] int32 = the token ``ep_scatter`` would have copied to every destination row (0 for
    rows of an expert's span that stay empty).  ``fp8_gemm_grouped_contiguous_silu_quant(..., a_row_index=src_row)`` then
    reads the tokens where they lie."""
    assert m_indices.shape[0] % 128 == 0, 'every expert span is a whole number of 128-row GEMM blocks'
    if num_recv_tokens_per_expert.dtype != torch.int32 or m_indices.dtype != torch.int32 or src_row.dtype != torch.int32:
        raise TypeError('num_recv_tokens_per_expert, m_indices and src_row must be int32')
    if not (num_recv_tokens_per_expert.is_contiguous() and expert_start_loc.is_contiguous() and m_indices.is_contiguous() and
            src_row.is_contiguous()) or src_row.shape != m_indices.shape:
        raise ValueError('num_recv_tokens_per_expert, expert_start_loc, m_indices and src_row must be contiguous, '
                         'src_row as long as m_indices')
    _scatter_rows_op(recv_topk, num_recv_tokens_per_expert, expert_start_loc, m_indices, src_row, output_index)
    return


@torch.no_grad()
def ep_gather(
    input_tensor: torch.Tensor,
    recv_topk_ids: torch.Tensor,
    recv_topk_weight: torch.Tensor,
    input_index: torch.Tensor,
    output_tensor: torch.Tensor,
):
    """output_tensor[t] = sum_j input_tensor[input_index[t, j]] * recv_topk_weight[t, j] over slots with an expert."""
    hidden_size = input_tensor.shape[1]
    assert hidden_size % 8 == 0
    assert input_tensor.stride(1) == 1 and output_tensor.stride(1) == 1, 'rows must be contiguous'
    if recv_topk_weight.dtype != torch.float32:
        raise TypeError('recv_topk_weight must be float32')
    _gather_op(input_tensor, recv_topk_ids, recv_topk_weight, input_index, output_tensor)
    return


def fused_moe_v3(
    hidden_states_fp8: Tuple[torch.Tensor, torch.Tensor],
    topk_idx,
    topk_weights,
    w13_weight_fp8: Tuple[torch.Tensor, torch.Tensor],
    w2_weight_fp8: Tuple[torch.Tensor, torch.Tensor],
    num_recv_tokens_per_expert: Optional[List[int]],
):
    """One expert-parallel MLP over the tokens this GPU received: rows are sorted by expert (ep_scatter), pass through
    gate/up GEMM -> silu(gate) * up with 1 x 128 re-quantisation -> down GEMM as expert-contiguous grouped GEMMs, and
    come back to token order as the routing-weighted sum of each token's slots (ep_gather).  Signature and early
    returns of the reference driver (dlblas/kernels/fused_moe_v3.py:246-343); every intermediate is allocated here,
    per call, as there."""
    tokens_q, tokens_scale = hidden_states_fp8
    rows_total = 0 if num_recv_tokens_per_expert is None else sum(num_recv_tokens_per_expert)
    if rows_total <= 0:
        return tokens_q.to(torch.bfloat16)  # nothing routed to a local expert: the caller gets its input back in bf16
    n_tokens, hidden = tokens_q.shape
    inter2 = w13_weight_fp8[0].size(1)  # gate and up halves side by side
    dev = tokens_q.device

    def buf(shape, dtype):
        return torch.empty(shape, device=dev, dtype=dtype)

    row_expert = buf((rows_total, ), torch.int32)
    slot_row = torch.empty_like(topk_idx)
    per_expert = torch.tensor(num_recv_tokens_per_expert, dtype=torch.int32, pin_memory=True).to(dev, non_blocking=True)
    first_row = torch.empty_like(per_expert)

    # gate/up projection, silu(gate) * up and the 1 x 128 quantiser as one kernel that reads the tokens where they lie:
    # ep_scatter_rows only fills the tables (which expert and which token each sorted row stands for), the kernel
    # follows them, and neither the expert-sorted copy of the activations nor the bf16 [rows, 2 I] intermediate reaches
    # memory.  Same bits as the steps of the reference (:288-334).
    # (A batch of at most a round or two of tiles runs faster on uniform 128-row tiles, which have no fused epilogue:
    # the library's planner says which, and such a batch takes the three steps below.)
    fused = None
    want_fused = _lib.plan_grouped(1, rows_total, inter2, hidden, w13_weight_fp8[0].size(0))[1]
    if want_fused and tokens_q.is_contiguous() and hidden % 128 == 0 and inter2 % 256 == 0 and n_tokens * hidden < (1 << 32):
        row_token = buf((rows_total, ), torch.int32)
        ep_scatter_rows(topk_idx, per_expert, first_row, row_expert, row_token, slot_row)
        fused = fp8_gemm_grouped_contiguous_silu_quant(tokens_q, tokens_scale, w13_weight_fp8[0], w13_weight_fp8[1], row_expert,
                                                       column_major_scales=True,  # the layout the down GEMM reads in place
                                                       a_row_index=row_token)
    if fused is not None:
        act_q, act_scale = fused
    else:
        # Expert-sorted activations.  The spans are padded to 128 rows per expert; the padding rows keep whatever the
        # allocator hands out, as in the reference driver (:269-278).  The GEMMs and the quantiser treat every row on its
        # own, so what those rows turn into (NaN included) stays in rows that ep_gather never reads.
        sorted_q = buf((rows_total, hidden), torch.uint8).view(tokens_q.dtype)
        sorted_scale = buf((rows_total, hidden // 128), torch.float32)
        ep_scatter(tokens_q, tokens_scale, topk_idx, per_expert, first_row, sorted_q, sorted_scale, row_expert, slot_row)
        if want_fused:
            fused = fp8_gemm_grouped_contiguous_silu_quant(sorted_q, sorted_scale, w13_weight_fp8[0], w13_weight_fp8[1], row_expert,
                                                           column_major_scales=True)
        if fused is not None:
            act_q, act_scale = fused
        else:  # the three steps of the reference (:307-334)
            gate_up = buf((rows_total, inter2), torch.bfloat16)
            m_grouped_fp8_gemm_nt_contiguous((sorted_q, sorted_scale), w13_weight_fp8, gate_up, row_expert)
            act_q, act_scale = silu_and_mul_post_quant(gate_up, 128)
            del gate_up
    down = buf((rows_total, hidden), torch.bfloat16)
    m_grouped_fp8_gemm_nt_contiguous((act_q, act_scale), w2_weight_fp8, down, row_expert)

    combined = buf((n_tokens, hidden), torch.bfloat16)
    ep_gather(down, topk_idx, topk_weights, slot_row, combined)
    return combined
