/*
 * C ABI of the steps that sit on either side of the FP8 grouped GEMMs in an expert MLP (MI355X / gfx950).
 * Same library (libdlblas_fp8_gemm.so), same conventions as include/dlblas_fp8_gemm.h: device pointers and sizes
 * only, nothing is allocated or synchronised, work is enqueued on `stream`, 0 = enqueued, negative DLB_ERR_* =
 * rejected with a reason in dlb_last_error().
 *
 * Reference interfaces these replace (paths relative to the DLBlas source tree):
 *   - dlb_silu_mul               : silu_and_mul, dlblas/layers/moe/kernels/activation.py:16-95
 *   - dlb_silu_mul_quant         : silu_and_mul followed by per_token_group_quant_fp8 as called between the two
 *                                  contiguous grouped GEMMs, dlblas/kernels/fused_moe_v3.py:325-334
 *   - dlb_silu_mul_quant_masked  : silu_and_mul_masked_post_quant_fwd, dlblas/kernels/moe.py:204-319, called
 *                                  between the two masked grouped GEMMs at dlblas/layers/moe/ep_moe.py:245-251
 *   - dlb_ep_scatter             : ep_scatter, dlblas/kernels/fused_moe_v3.py:18-158
 *   - dlb_ep_gather              : ep_gather, dlblas/kernels/fused_moe_v3.py:161-233
 *   - dlb_scale_relayout         : tma_align_input_scale, dlblas/kernels/quant_dequant.py:42-83
 */
#ifndef DLBLAS_FP8_MOE_H_
#define DLBLAS_FP8_MOE_H_

#include "dlblas_fp8_gemm.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * out[m, n] = silu(x[m, n]) * x[m, N + n], evaluated in fp32 and rounded once to the element type.
 *
 *   x    [rows, 2N]  bf16 / fp16 / fp32 (dtype = DLB_IN_*), last dimension contiguous, row stride x_row_stride elements
 *   out  [rows, N]   same element type, last dimension contiguous, row stride out_row_stride elements
 */
int dlb_silu_mul(const void* x, int dtype, void* out, int64_t rows, int64_t N, int64_t x_row_stride,
                 int64_t out_row_stride, void* stream);

/*
 * The two calls the reference makes between its contiguous grouped GEMMs, in one pass: y = silu_mul(x) rounded to
 * the element type of x, then the 1 x 128 quantiser of dlb_fp8_quant_1x128 on y.  Bit-identical to running the two
 * entry points one after the other; y is never written.
 *
 *   x  [rows, 2N]     bf16 / fp16 / fp32, row stride x_row_stride elements, rows 16-byte aligned, N % 128 == 0
 *   q  [rows, N]      e4m3fn, contiguous
 *   s  [rows, N/128]  fp32, element (m, g) at s[m * s_stride_m + g * s_stride_k]
 */
int dlb_silu_mul_quant(const void* x, int dtype, void* q, float* s, int64_t rows, int64_t N, int64_t x_row_stride,
                       int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream);

/*
 * Masked variant over fixed-capacity per-expert buffers.  For expert g and token m < masked_m[g]:
 *   gate = round_to_dtype(silu(x[g, m, n])),  y = round_to_dtype(x[g, m, N + n] * gate)      (two roundings)
 *   s[g, m, k] = max(max |y| over the 128 group, 1e-10) / 448,   q = e4m3(clamp(y / s, -448, 448))
 * Tokens at or beyond masked_m[g] are neither read nor written.
 *
 *   x         [G, M_max, 2N]     bf16 / fp16 / fp32, contiguous, N % 128 == 0
 *   q         [G, M_max, N]      e4m3fn, contiguous
 *   s         [G, M_max, N/128]  fp32, element (g, m, k) at s[g * s_stride_g + m * s_stride_m + k * s_stride_k]
 *   masked_m  [G]                int32 on the device; values are clamped to [0, M_max]
 */
int dlb_silu_mul_quant_masked(const void* x, int dtype, void* q, float* s, const int32_t* masked_m, int64_t G,
                              int64_t M_max, int64_t N, int64_t s_stride_g, int64_t s_stride_m, int64_t s_stride_k,
                              void* stream);

/* element type of index tensors (expert ids, row indices, expert_start_loc) */
#define DLB_IDX_I32 0
#define DLB_IDX_I64 1

/* Bytes of workspace dlb_ep_scatter needs for `tokens` tokens with `topk` slots each and `experts` experts. */
size_t dlb_ep_scatter_workspace_bytes(int64_t tokens, int64_t topk, int64_t experts);

/*
 * Copies every token's fp8 row and scales next to the other rows of each expert it is routed to (the layout the
 * contiguous grouped GEMM reads) and fills the tables that describe it.  Replaces ep_scatter
 * (dlblas/kernels/fused_moe_v3.py:95-158; kernels :18-92).
 *
 *   recv_x             [tokens, hidden]        e4m3fn, row stride x_row_stride bytes, rows 16-byte aligned
 *   recv_x_scale       [tokens, hidden/128]    fp32, element (t, k) at [t * xs_stride_m + k * xs_stride_k]
 *   recv_topk          [tokens, topk]          int32 / int64 (topk_dtype): expert id per slot; < 0 or >= experts = none
 *   num_recv_tokens_per_expert [experts]       int32: rows reserved per expert (padded to the GEMM's 128-row blocks)
 *   expert_start_loc   [experts]               int32 / int64 (start_dtype), OUT: first free row of each expert after
 *                                              the call = exclusive prefix sum of the reserved rows + rows handed out
 *   output_tensor      [rows, hidden]          e4m3fn, OUT, row stride out_row_stride bytes; only handed-out rows are written
 *   output_tensor_scale [rows, hidden/128]     fp32, OUT, through os_stride_m / os_stride_k
 *   m_indices          [m_indices_len]         int32, OUT: expert of every reserved row
 *   output_index       [tokens, topk]          int32 / int64 (index_dtype), OUT: destination row of every routed slot;
 *                                              other slots keep their content
 *
 * Rows are handed out in token-major, slot-minor order (the reference's atomics give an arbitrary order; its
 * single-program Ascend variant, dlblas/kernels/ascend/fused_moe_v3.py:137, gives this one), so the result is
 * reproducible.  hidden % 128 == 0, topk <= 64.  Three launches, no global atomics.
 */
int dlb_ep_scatter(const void* recv_x, int64_t x_row_stride, const float* recv_x_scale, int64_t xs_stride_m,
                   int64_t xs_stride_k, const void* recv_topk, int topk_dtype, int64_t topk_stride_m,
                   int64_t topk_stride_k, const int32_t* num_recv_tokens_per_expert, void* expert_start_loc,
                   int start_dtype, void* output_tensor, int64_t out_row_stride, float* output_tensor_scale,
                   int64_t os_stride_m, int64_t os_stride_k, int32_t* m_indices, int64_t m_indices_len,
                   void* output_index, int index_dtype, int64_t oi_stride_m, int64_t oi_stride_k, int64_t tokens,
                   int64_t hidden, int64_t topk, int64_t experts, void* workspace, size_t workspace_bytes,
                   void* stream);

/*
 * The tables of dlb_ep_scatter without the copy: m_indices, expert_start_loc and output_index exactly as that call
 * leaves them, plus src_row [m_indices_len] int32 = the token whose row dlb_ep_scatter would have copied to each
 * destination row (0 for the rows of an expert's span that no slot is copied to).  No row of recv_x is read or written:
 * dlb_fp8_gemm_grouped_contiguous_gather_silu_quant reads the tokens through src_row.  No counterpart in the
 * reference, whose ep_scatter always copies (dlblas/kernels/fused_moe_v3.py:95-158).  Workspace as dlb_ep_scatter.
 */
int dlb_ep_scatter_rows(const void* recv_topk, int topk_dtype, int64_t topk_stride_m, int64_t topk_stride_k,
                        const int32_t* num_recv_tokens_per_expert, void* expert_start_loc, int start_dtype,
                        int32_t* m_indices, int32_t* src_row, int64_t m_indices_len, void* output_index, int index_dtype,
                        int64_t oi_stride_m, int64_t oi_stride_k, int64_t tokens, int64_t topk, int64_t experts,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * out[t, :] = sum over the slots j with recv_topk_ids[t, j] >= 0, in slot order, of
 * input[input_index[t, j], :] * recv_topk_weight[t, j]; fp32 fused multiply-add chain, one cast at the end; a token
 * without a routed slot gets zeros.  Replaces ep_gather (dlblas/kernels/fused_moe_v3.py:199-233; kernel :161-196).
 *
 *   input   [rows, hidden]    bf16 / fp16 / fp32 (in_dtype = DLB_IN_*), row stride in_row_stride elements
 *   output  [tokens, hidden]  bf16 / fp16 / fp32 (out_dtype), row stride out_row_stride elements
 *   ids / weights / index     [tokens, topk] through their two strides; ids and index int32 / int64
 *
 * hidden % 8 == 0 (the reference asserts % 1024), rows 16-byte aligned, topk <= 64.
 */
int dlb_ep_gather(const void* input, int in_dtype, int64_t in_row_stride, const void* recv_topk_ids, int topk_dtype,
                  int64_t topk_stride_m, int64_t topk_stride_k, const float* recv_topk_weight, int64_t w_stride_m,
                  int64_t w_stride_k, const void* input_index, int index_dtype, int64_t idx_stride_m,
                  int64_t idx_stride_k, void* output, int out_dtype, int64_t out_row_stride, int64_t tokens,
                  int64_t hidden, int64_t topk, void* stream);

/*
 * dst[k * rows_pad + m] = src[m * src_stride_m + k * src_stride_k] for m < rows, 0 for rows <= m < rows_pad: the
 * activation scales re-laid "column-major" with the row count padded.  Replaces the kernel behind
 * tma_align_input_scale (dlblas/kernels/quant_dequant.py:42-83), whose result is the view dst.t()[:rows].  The GEMM
 * entry points of this library read scales through strides, so they accept either layout.
 */
int dlb_scale_relayout(const float* src, float* dst, int64_t rows, int64_t kblocks, int64_t rows_pad,
                       int64_t src_stride_m, int64_t src_stride_k, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* DLBLAS_FP8_MOE_H_ */
