"""Expert-contiguous FP8 MoE forward of the reference (dlblas/kernels/fused_moe_v3.py), on the gfx950 kernels of this
package: ``ep_scatter`` (:95-158), ``ep_gather`` (:199-233) and the driver ``fused_moe_v3`` (:246-343) with the same
positional signatures.  Differences a caller can observe: destination rows are handed out in token-major order instead
of atomic order (both satisfy the contract that ``output_index`` names the row each slot was copied to), and the
driver fuses silu_and_mul with the quantiser and skips the scale re-layout the reference needs for its GEMM.
"""
from typing import List, Optional, Tuple

import torch

from .. import _lib
from .activation import silu_and_mul_post_quant
from .fp8_gemm_grouped import m_grouped_fp8_gemm_nt_contiguous


@torch.library.custom_op('dlblas::ep_scatter', mutates_args=('expert_start_loc', 'output_tensor', 'output_tensor_scale',
                                                             'm_indices', 'output_index'), device_types='cuda')
def _scatter_op(recv_x: torch.Tensor, recv_x_scale: torch.Tensor, recv_topk: torch.Tensor,
                num_recv_tokens_per_expert: torch.Tensor, expert_start_loc: torch.Tensor, output_tensor: torch.Tensor,
                output_tensor_scale: torch.Tensor, m_indices: torch.Tensor, output_index: torch.Tensor) -> None:
    _lib.ep_scatter(recv_x, recv_x_scale, recv_topk, num_recv_tokens_per_expert, expert_start_loc, output_tensor,
                    output_tensor_scale, m_indices, output_index)


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
    BLOCK_E = 128  # token num of per expert is aligned to 128
    assert m_indices.shape[0] % BLOCK_E == 0
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
    """scatter -> grouped GEMM (gate/up) -> silu * up + quantise -> grouped GEMM (down) -> weighted gather."""
    hidden_states_fp8, hidden_states_scale = hidden_states_fp8
    if num_recv_tokens_per_expert is None:
        return hidden_states_fp8.to(torch.bfloat16)
    all_tokens = sum(num_recv_tokens_per_expert)
    if all_tokens <= 0:
        return hidden_states_fp8.to(torch.bfloat16)
    M, K = hidden_states_fp8.size()
    N = w13_weight_fp8[0].size(1)
    dev = hidden_states_fp8.device
    gather_out = torch.empty((M, K), device=dev, dtype=torch.bfloat16)
    # padding rows are computed by the GEMMs like any other row; zero them so that no NaN pattern left in the
    # allocation reaches the quantiser between the two GEMMs
    input_tensor = torch.zeros((all_tokens, K), device=dev, dtype=torch.uint8).view(hidden_states_fp8.dtype)
    input_tensor_scale = torch.zeros((all_tokens, K // 128), device=dev, dtype=torch.float32)
    m_indices = torch.empty(all_tokens, device=dev, dtype=torch.int32)
    output_index = torch.empty_like(topk_idx)
    num_recv_tokens_per_expert_gpu = torch.tensor(num_recv_tokens_per_expert, dtype=torch.int32, pin_memory=True,
                                                  device='cpu').to(dev, non_blocking=True)
    expert_start_loc = torch.empty_like(num_recv_tokens_per_expert_gpu)
    ep_scatter(hidden_states_fp8, hidden_states_scale, topk_idx, num_recv_tokens_per_expert_gpu, expert_start_loc,
               input_tensor, input_tensor_scale, m_indices, output_index)
    gateup_output = torch.empty((all_tokens, N), device=dev, dtype=torch.bfloat16)
    m_grouped_fp8_gemm_nt_contiguous((input_tensor, input_tensor_scale), w13_weight_fp8, gateup_output, m_indices)
    down_input_fp8, down_input_scale = silu_and_mul_post_quant(gateup_output, 128)
    down_output = torch.empty((all_tokens, K), device=dev, dtype=torch.bfloat16)
    m_grouped_fp8_gemm_nt_contiguous((down_input_fp8, down_input_scale), w2_weight_fp8, down_output, m_indices)
    ep_gather(down_output, topk_idx, topk_weights, output_index, gather_out)
    return gather_out
