"""TEST INFRASTRUCTURE ONLY - CPU oracle of the permutation steps around the contiguous grouped GEMMs.

Restates (paths relative to the DLBlas tree):

  ep_scatter_ref             ``ep_scatter``, dlblas/kernels/fused_moe_v3.py:18-158.  Kernel 1 (:18-45) writes the
                             exclusive prefix sum of the padded per-expert row counts to ``expert_start_loc`` and
                             fills ``m_indices[start_e : start_e + count_e] = e``.  Kernel 2 (:48-92) visits every
                             (token, top-k slot) whose expert id is >= 0, takes the next free row of that expert
                             (``atomic_add(expert_start_loc[e], 1)``), records it in ``output_index[token, slot]`` and
                             copies the token's fp8 row and its scales there.  The reference hands out rows in
                             whatever order its atomics resolve; its Ascend twin runs kernel 2 as ONE program
                             (dlblas/kernels/ascend/fused_moe_v3.py:137), i.e. in token-major, slot-minor order.  That
                             order is what this oracle (and the HIP implementation) produces.  Rows of the padding
                             and everything else in the outputs keep their previous content; ``expert_start_loc``
                             ends as start_e + (rows handed out), as the atomics leave it.
  ep_gather_ref              ``ep_gather``, dlblas/kernels/fused_moe_v3.py:161-233: out[t] = sum over the slots with
                             expert id >= 0, in slot order, of input[input_index[t, slot]] * weight[t, slot], fp32
                             accumulator (:178-186), one cast to the output dtype.  A token with no valid slot gets 0.
  tma_align_input_scale_ref  ``tma_align_input_scale``, dlblas/kernels/quant_dequant.py:42-83: scales [m, k] copied
                             into a [k, pad4(m)] buffer and returned as its transposed view cut to m rows (values
                             unchanged, strides (1, pad4(m))).

How these are pinned (tests/test_oracle_moe_scatter_gather.py): the reference's own test constructions
(tests/kernels/test_scatter_gather.py:10-76 and :79-107) are run against the oracle: m_indices equals the
repeat-interleaved expert ids, every valid (token, slot) finds its row and scales at output_index, and the gather
equals the reference test's accumulation loop.  Beyond those: output_index is a bijection onto
[start_e, start_e + n_e) per expert, in token-major order (brute force on small inputs); the gather equals a dense
matrix product with the scattered weight matrix (independent formulation); the re-layout is checked against
torch's own transpose.
"""
import torch


def ep_scatter_ref(recv_x, recv_x_scale, recv_topk, num_recv_tokens_per_expert, expert_start_loc, output_tensor,
                   output_tensor_scale, m_indices, output_index):
    """In-place on expert_start_loc, output_tensor, output_tensor_scale, m_indices, output_index (CPU tensors)."""
    E = num_recv_tokens_per_expert.shape[0]
    counts = [int(c) for c in num_recv_tokens_per_expert]
    start = [0] * E
    for e in range(1, E):
        start[e] = start[e - 1] + counts[e - 1]
    for e in range(E):
        m_indices[start[e]:start[e] + counts[e]] = e
    nxt = list(start)
    T, topk = recv_topk.shape
    for t in range(T):
        for j in range(topk):
            e = int(recv_topk[t, j])
            if e < 0 or e >= E:  # ids beyond the expert table index out of bounds in the reference; skipped here
                continue
            dst = nxt[e]
            nxt[e] += 1
            output_index[t, j] = dst
            output_tensor.view(torch.uint8)[dst] = recv_x.view(torch.uint8)[t]
            output_tensor_scale[dst] = recv_x_scale[t]
    for e in range(E):
        expert_start_loc[e] = nxt[e]


def ep_gather_ref(input_tensor, recv_topk_ids, recv_topk_weight, input_index, output_tensor):
    """In-place on output_tensor.  fp32 accumulation in slot order with fused multiply-add (evaluated in fp64 and
    rounded to fp32 after every step)."""
    T, topk = recv_topk_ids.shape
    x = input_tensor.double()
    for t in range(T):
        acc = torch.zeros(input_tensor.shape[1], dtype=torch.float32)
        for j in range(topk):
            if int(recv_topk_ids[t, j]) < 0:
                continue
            row = x[int(input_index[t, j])]
            acc = (row * float(recv_topk_weight[t, j]) + acc.double()).float()
        output_tensor[t] = acc.to(output_tensor.dtype)


def tma_align_input_scale_ref(input_scale: torch.Tensor) -> torch.Tensor:
    m, k = input_scale.shape
    pad_m = (m + 3) // 4 * 4
    out = torch.zeros(k, pad_m, dtype=input_scale.dtype)
    out[:, :m] = input_scale.t()
    return out.t()[:m]
