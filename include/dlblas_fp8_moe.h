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

#ifdef __cplusplus
}
#endif

#endif /* DLBLAS_FP8_MOE_H_ */
