/*
 * dlblas_fp8_gemm.h -- C ABI of the MI355X (gfx950) FP8 block-scaled GEMM library.
 *
 * All three GEMM entry points compute, for every output element,
 *
 *     C[m, n] = sum_kb ( sum_{k in block kb} A[m, k] * B[n, k] ) * a_s[m, kb] * b_s[n / 128, kb]
 *
 * with A, B in OCP float8 e4m3fn, one fp32 activation scale per (row, 128-wide K block),
 * one fp32 weight scale per (128 x 128) block of B, fp32 accumulation, and a single cast to the
 * output type at the end.  "NT" layout: A is [M, K] and B is [N, K], both K-contiguous.
 *
 * Conventions shared by every function here
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless stated otherwise;
 *   - the library never allocates, frees or synchronises; work is enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the null stream) and the call returns at once;
 *   - return value 0 = enqueued, negative = rejected (see DLB_ERR_*), nothing was enqueued (every
 *     check, and the one launch attribute that can be refused, comes before the first kernel of a call);
 *     dlb_last_error() gives a thread-local human-readable reason for the last failure;
 *   - no C++ exception ever crosses this boundary;
 *   - `workspace` is caller-owned device memory of at least dlb_fp8_gemm_workspace_bytes()
 *     bytes, 16-byte aligned.  Its first DLB_WS_COUNTER_BYTES bytes hold the counters of the
 *     one-launch split-K path (DLB_KNOB_SPLITK_MODE): they must be ZERO before the first call
 *     that uses the buffer, and every call leaves them zero.  The rest is scratch that a call
 *     overwrites: re-laid activation scales, fp32 partial sums of the split-K path, the tile
 *     list of the expert-contiguous path; nothing there has to be initialised or to survive
 *     between calls, so one buffer serves any number of calls that do not overlap in time.
 *     Two calls that may run concurrently (different streams) need separate workspaces.
 *
 * Reference interfaces these replace (paths relative to the DLBlas source tree):
 *   - dlb_fp8_gemm                     : dlblas/kernels/fp8_gemm.py:15-65 (kernel) and :68-89 (host wrapper)
 *   - dlb_fp8_gemm_grouped_contiguous  : deep_gemm.m_grouped_fp8_gemm_nt_contiguous as called from
 *                                        dlblas/kernels/fused_moe_v3.py:235-245
 *   - dlb_fp8_gemm_grouped_masked      : deep_gemm.m_grouped_fp8_gemm_nt_masked as called from
 *                                        dlblas/layers/moe/ep_moe.py:180-197
 *   - the ctypes calling convention (void* data pointers, void* stream) follows the reference's only
 *     native entry point, dlblas/kernels/cutlass/fp8_convert.cu:8 and its loader
 *     tests/kernels/cutlass/test_fp8_convert.py:8-39.
 */
#ifndef DLBLAS_FP8_GEMM_H_
#define DLBLAS_FP8_GEMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLB_ABI_VERSION 7

/* output element type of C */
#define DLB_OUT_BF16 0
#define DLB_OUT_F32 1

/* error codes (all negative) */
#define DLB_OK 0
#define DLB_ERR_NULL_POINTER (-1)   /* a required pointer is NULL                                  */
#define DLB_ERR_BAD_SHAPE (-2)      /* a dimension is negative / too large / violates a constraint */
#define DLB_ERR_BAD_STRIDE (-3)     /* a stride cannot address the stated shape                    */
#define DLB_ERR_BAD_DTYPE (-4)      /* out_dtype is not DLB_OUT_BF16 / DLB_OUT_F32                  */
#define DLB_ERR_WORKSPACE (-5)      /* workspace is NULL or smaller than required                  */
#define DLB_ERR_ALIGNMENT (-6)      /* a pointer is not 16-byte aligned where the kernels need it  */
#define DLB_ERR_LAUNCH (-7)         /* the HIP runtime refused the launch                          */

/* reserved bytes at the head of every workspace */
#define DLB_WS_COUNTER_BYTES 65536

/* Version of this ABI (DLB_ABI_VERSION of the library that was loaded). */
int dlb_abi_version(void);

/* Thread-local description of the last failure on the calling thread ("" if none). */
const char* dlb_last_error(void);

/*
 * Upper bound of the workspace any of the three GEMM entry points can need for a problem with
 * `rows` activation rows in total (M, M_sum, or G * M_max), N outputs per row and contraction
 * length K.  Never fails; returns at least DLB_WS_COUNTER_BYTES.
 */
size_t dlb_fp8_gemm_workspace_bytes(int64_t rows, int64_t N, int64_t K);

/*
 * Dense block-scaled GEMM.   Replaces fp8_gemm_kernel / fp8_gemm (dlblas/kernels/fp8_gemm.py:15-89).
 *
 *   a    [M, K]                     e4m3fn, row-major, row stride K
 *   b    [N, K]                     e4m3fn, row-major, row stride K
 *   a_s  [M, ceil(K/128)]           fp32, element (m, kb) at a_s[m * as_stride_m + kb * as_stride_k]
 *   b_s  [ceil(N/128), ceil(K/128)] fp32, row-major
 *   c    [M, N]                     bf16 or fp32 (out_dtype), row-major, row stride N
 *
 * M, N, K >= 0 (M == 0 or N == 0 enqueues nothing; K == 0 stores zeros).  Any M, N, K below 2^31 - 1024 are accepted;
 * K % 16 == 0 takes the MFMA path, other K a slower exact path.  K >= 2^24 (or an a_s row stride >= 2^21 floats) is
 * beyond the 32-bit offsets of the DMA kernels and runs on the register-staged kernels instead.
 */
int dlb_fp8_gemm(const void* a, const void* b, const float* a_s, const float* b_s, void* c,
                 int64_t M, int64_t N, int64_t K,
                 int64_t as_stride_m, int64_t as_stride_k,
                 int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * dlb_fp8_gemm for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its Triton launch
 * needs no scratch).  Same operands, same kernels and same results as dlb_fp8_gemm called with a workspace of
 * DLB_STATIC_SCRATCH_SLICE_BYTES bytes; the scratch (re-laid activation scales, fp32 partial sums of the split-K
 * plans) is a fixed array inside the library's code object, DLB_STATIC_SCRATCH_BYTES per GPU, held by every GPU the
 * library runs on until the process ends.  The call allocates and frees nothing and does not synchronise.
 *
 *   - The array is cut into DLB_STATIC_SCRATCH_SLICES slices.  A stream is bound to the first free slice of its GPU at
 *     its first call and keeps it until the process ends: calls on different streams never share scratch memory, calls
 *     on one stream are ordered by the stream.  A call on one more stream than there are slices is rejected with
 *     DLB_ERR_WORKSPACE (use dlb_fp8_gemm with a workspace of its own for that stream).
 *   - Limit: what the plan keeps in scratch besides the partial sums (which adapt to the room there is) has to fit a
 *     slice minus its 64 KiB head: the re-laid activation scales, 4 * ceil(K/128) * M bytes (M rounded up to a multiple
 *     of 4), when M > 128 and a_s is row-major and the plan is not one of the small-tile ones that read a_s in place.
 *     Larger problems are rejected with DLB_ERR_WORKSPACE and nothing is enqueued.
 *   - A call overwrites what the previous call on its stream left in the slice; nothing in it has to be initialised
 *     (the array is zero when the library is loaded and every call leaves the slice's head zero).
 *   - The first call on a device looks up the array's device address (hipGetSymbolAddress); make that call outside
 *     a graph capture.
 */
#define DLB_STATIC_SCRATCH_BYTES (16u << 20)
#define DLB_STATIC_SCRATCH_SLICES 4
#define DLB_STATIC_SCRATCH_SLICE_BYTES (DLB_STATIC_SCRATCH_BYTES / DLB_STATIC_SCRATCH_SLICES)
int dlb_fp8_gemm_noalloc(const void* a, const void* b, const float* a_s, const float* b_s, void* c,
                         int64_t M, int64_t N, int64_t K,
                         int64_t as_stride_m, int64_t as_stride_k,
                         int out_dtype, void* stream);

/*
 * Grouped GEMM, expert-contiguous rows.  Replaces deep_gemm.m_grouped_fp8_gemm_nt_contiguous
 * (call site dlblas/kernels/fused_moe_v3.py:235-245, buffers built at :262-308).
 *
 *   a         [M_sum, K]                      e4m3fn, row stride K
 *   a_s       [M_sum, ceil(K/128)]            fp32, addressed through as_stride_m / as_stride_k
 *                                             (the reference hands over a column-major view)
 *   b         [G, N, K]                       e4m3fn, contiguous
 *   b_s       [G, ceil(N/128), ceil(K/128)]   fp32, contiguous
 *   c         [M_sum, N]                      bf16 or fp32, row stride N, caller allocated
 *   m_indices [M_sum]                         int32: expert of each row.  Rows of one expert are
 *                                             contiguous and every expert's span is a multiple of 128
 *                                             rows, so the expert is read once per aligned 128-row
 *                                             block (from its first row); a negative value skips the
 *                                             block and leaves its rows of c untouched.
 *
 * M_sum need not be a multiple of 128 (the last block may be short).  K % 16 == 0 is required.
 */
int dlb_fp8_gemm_grouped_contiguous(const void* a, const void* b, const float* a_s, const float* b_s,
                                    void* c, const int32_t* m_indices,
                                    int64_t M_sum, int64_t N, int64_t K, int32_t G,
                                    int64_t as_stride_m, int64_t as_stride_k,
                                    int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The gate/up projection of an expert MLP with its activation and the quantiser of the result fused into the GEMM:
 * one kernel instead of the sequence grouped GEMM -> silu_and_mul -> per_token_group_quant_fp8 of
 * dlblas/kernels/fused_moe_v3.py:307-334, with the same bits (the bf16 rounding of the GEMM output, the activation
 * in bf16 and the 1 x 128 quantiser are reproduced in the epilogue).  The bf16 [M_sum, N] intermediate never reaches
 * memory.
 *
 *   a, a_s, m_indices, G, as_stride_*   as dlb_fp8_gemm_grouped_contiguous
 *   b      [G, N, K]                    e4m3fn; N = 2 I weight rows per expert, the I gate rows first, then the I up rows
 *   b_s    [G, N/128, K/128]            fp32
 *   out_q  [M_sum, I]                   e4m3fn, row stride I:  quant(silu(gate) * up)
 *   out_s  [M_sum, I/128]               fp32, element (m, j) at [m * os_stride_m + j * os_stride_k]
 *   eps                                 lower bound of a group's amax (the reference passes 1e-10)
 *
 * Needs K % 128 == 0, N % 256 == 0, N * K < 2^32 and a workspace (the tile list of the expert-contiguous path lives
 * there); otherwise DLB_ERR_BAD_SHAPE is returned, nothing is enqueued, and the caller runs the three steps apart.
 * Rows of blocks whose m_indices entry is negative are not written.
 */
int dlb_fp8_gemm_grouped_contiguous_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s,
                                               void* out_q, float* out_s, const int32_t* m_indices,
                                               int64_t M_sum, int64_t N, int64_t K, int32_t G,
                                               int64_t as_stride_m, int64_t as_stride_k,
                                               int64_t os_stride_m, int64_t os_stride_k, float eps,
                                               void* workspace, size_t workspace_bytes, void* stream);

/*
 * dlb_fp8_gemm_grouped_contiguous_silu_quant reading its activation rows where the tokens lie instead of from a copy
 * sorted by expert: row r of the GEMM is row a_row_index[r] of a, and its scales are row a_row_index[r] of a_s.  With
 * dlb_ep_scatter_rows (include/dlblas_fp8_moe.h), which fills m_indices, a_row_index and the slot table without moving
 * a row, this replaces ep_scatter + the three steps of dlblas/kernels/fused_moe_v3.py:288-334; out_q / out_s hold the
 * same bits as after the copy.
 *
 *   a            [a_rows, K]            e4m3fn, contiguous (the received tokens)
 *   a_s          [a_rows, K/128]        fp32, element (t, kb) at a_s[t * as_stride_m + kb * as_stride_k]
 *   a_row_index  [M_sum]                int32 on the device: source row of every GEMM row, 0 <= . < a_rows (rows of the
 *                                       padding of an expert's span name any valid row; negative values are read as 0)
 *   the other arguments as dlb_fp8_gemm_grouped_contiguous_silu_quant
 *
 * Needs what that entry point needs and a_rows * K < 2^32; otherwise DLB_ERR_BAD_SHAPE, nothing is enqueued.
 */
int dlb_fp8_gemm_grouped_contiguous_gather_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s,
                                                      void* out_q, float* out_s, const int32_t* m_indices,
                                                      const int32_t* a_row_index, int64_t a_rows,
                                                      int64_t M_sum, int64_t N, int64_t K, int32_t G,
                                                      int64_t as_stride_m, int64_t as_stride_k,
                                                      int64_t os_stride_m, int64_t os_stride_k, float eps,
                                                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * Grouped GEMM, fixed-capacity buffers with a valid-row count per expert.  Replaces
 * deep_gemm.m_grouped_fp8_gemm_nt_masked (call site dlblas/layers/moe/ep_moe.py:180-197,
 * buffers built at :199-261).
 *
 *   a         [G, M_max, K]                   e4m3fn, contiguous
 *   a_s       [G, M_max, ceil(K/128)]         fp32, element (g, m, kb) at
 *                                             a_s[g * as_stride_g + m * as_stride_m + kb * as_stride_k]
 *   b         [G, N, K]                       e4m3fn, contiguous
 *   b_s       [G, ceil(N/128), ceil(K/128)]   fp32, contiguous
 *   c         [G, M_max, N]                   bf16 or fp32, contiguous, caller allocated
 *   masked_m  [G]                             int32 on the device: rows [0, masked_m[g]) of expert g
 *                                             are computed; rows at or beyond it are neither read
 *                                             into a valid result nor written.  Values are clamped
 *                                             to [0, M_max].
 *   expected_m                                scheduling hint only (typical masked_m); <= 0 = unknown.
 *                                             It picks the tile shape (128 x 128 for a few short experts,
 *                                             256-row tiles from several hundred rows per expert on) and
 *                                             never changes a result bit.
 *
 * The tile schedule is built on the device from masked_m: no host synchronisation and no tiles
 * for empty row ranges.  K % 16 == 0 is required.
 */
int dlb_fp8_gemm_grouped_masked(const void* a, const void* b, const float* a_s, const float* b_s,
                                void* c, const int32_t* masked_m, int32_t expected_m,
                                int64_t M_max, int64_t N, int64_t K, int32_t G,
                                int64_t as_stride_g, int64_t as_stride_m, int64_t as_stride_k,
                                int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The gate/up projection of the masked (low-latency) expert MLP with its activation and the quantiser of the result
 * fused into the GEMM: one kernel instead of m_grouped_fp8_gemm_nt_masked -> silu_and_mul_masked_post_quant_fwd
 * (dlblas/layers/moe/ep_moe.py:199-251), with the same bits (the bf16 rounding of the GEMM output, the two bf16
 * roundings of the masked activation, dlblas/kernels/moe.py:256-257, and the 1 x 128 quantiser are reproduced in the
 * epilogue).  The bf16 [G, M_max, N] intermediate never reaches memory.
 *
 *   a, a_s, masked_m, expected_m, G, as_stride_*   as dlb_fp8_gemm_grouped_masked
 *   b      [G, N, K]                    e4m3fn; N = 2 I weight rows per expert, the I gate rows first, then the I up rows
 *   b_s    [G, N/128, K/128]            fp32
 *   out_q  [G, M_max, I]                e4m3fn, contiguous:  quant(up * silu(gate))
 *   out_s  [G, M_max, I/128]            fp32, element (g, m, j) at [g * os_stride_g + m * os_stride_m + j * os_stride_k]
 *   eps                                 lower bound of a group's amax (the reference uses 1e-10)
 *
 * Rows at or beyond masked_m[g] of out_q and out_s are not written.  Needs K % 128 == 0, N % 256 == 0 and
 * N * K < 2^32; otherwise DLB_ERR_BAD_SHAPE is returned, nothing is enqueued, and the caller runs the two steps apart.
 */
int dlb_fp8_gemm_grouped_masked_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s,
                                           void* out_q, float* out_s, const int32_t* masked_m, int32_t expected_m,
                                           int64_t M_max, int64_t N, int64_t K, int32_t G,
                                           int64_t as_stride_g, int64_t as_stride_m, int64_t as_stride_k,
                                           int64_t os_stride_g, int64_t os_stride_m, int64_t os_stride_k, float eps,
                                           void* workspace, size_t workspace_bytes, void* stream);

/* element type of the quantiser input */
#define DLB_IN_BF16 0
#define DLB_IN_F16 1
#define DLB_IN_F32 2

/*
 * 1 x 128 activation quantiser, the producer of (a, a_s).  Replaces _per_token_group_quant_fp8 and
 * _per_token_group_quant_fp8_colmajor behind per_token_group_quant_fp8 (dlblas/kernels/fp8.py:8-182) for
 * group_size 128 and dtype float8_e4m3fn:
 *     s[m, g] = max(max_k |x[m, 128 g + k]|, eps) / 448,   q = round_to_nearest_even_e4m3(clamp(x / s, -448, 448))
 *
 *   x  [rows, K]      bf16 / fp16 / fp32 (x_dtype), K contiguous, row stride x_row_stride elements, rows 16-byte aligned
 *   q  [rows, K]      e4m3fn, contiguous
 *   s  [rows, K/128]  fp32, element (m, g) at s[m * s_stride_m + g * s_stride_k]  (row- or column-major)
 *
 * K % 128 == 0 is required (the reference asserts divisibility by the group size).
 */
int dlb_fp8_quant_1x128(const void* x, int x_dtype, void* q, float* s, int64_t rows, int64_t K, int64_t x_row_stride,
                        int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream);

/*
 * The same quantiser for any group size, as per_token_group_quant_fp8 takes it (dlblas/kernels/fp8.py:108-182:
 * group_size is any divisor of the row length, BLOCK = next_power_of_2(group_size)):
 *     s[m, j] = max(max |x[m, group_size j ..]|, eps) / 448,   q = round_to_nearest_even_e4m3(clamp(x / s, -448, 448))
 * with s [rows, K / group_size] addressed through (s_stride_m, s_stride_k).  K % group_size == 0 is required.  Group
 * sizes that are a multiple of 8 up to 512 on 16-byte aligned rows run at memory speed (dlb_fp8_quant_1x128 is this
 * function at group_size 128); anything else takes a slower element-wise kernel with the same arithmetic.
 */
int dlb_fp8_quant_group(const void* x, int x_dtype, void* q, float* s, int64_t rows, int64_t K, int64_t group_size,
                        int64_t x_row_stride, int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream);

/*
 * 128 x 128 block quantiser, the producer of (b, b_s): one scale per block of the weight matrix, blocks at the N and
 * K edges ragged.  The reference has no such function in the package; the scheme (block amax / 448) is that of its
 * test data builder (tests/kernels/test_fused_moe_v2.py:35-60) and of the b_s operand of fp8_gemm
 * (dlblas/kernels/fp8_gemm.py:47):
 *     s[g, i, j] = max(max |w[g, 128 i .., 128 j ..]|, eps) / 448,   q = round_to_nearest_even_e4m3(clamp(w / s, -448, 448))
 *
 *   w  [G, N, K]                        bf16 / fp16 / fp32 (w_dtype), K contiguous, row stride w_row_stride elements,
 *                                       experts N * w_row_stride apart, rows 16-byte aligned, K % 8 == 0
 *   q  [G, N, K]                        e4m3fn, contiguous
 *   s  [G, ceil(N/128), ceil(K/128)]    fp32, contiguous
 */
int dlb_fp8_quant_128x128(const void* w, int w_dtype, void* q, float* s, int64_t G, int64_t N, int64_t K,
                          int64_t w_row_stride, float eps, void* stream);

/*
 * Host-only query: what the library would launch for a problem, without launching anything (no GPU is touched).
 * mode 0 = dlb_fp8_gemm, 1 = grouped contiguous (rows = M_sum), 2 = grouped masked (rows = M_max); `compute_units`
 * is the CU count to plan for (256 on MI355X); activation scales are taken to be row-major.  Outputs (each may be
 * NULL): the kernel variant id (dlb_fp8_gemm_variant_name); the number of K slices summed in a second pass (1 = none),
 * exactly as a launch with this workspace size would use it; the output columns per workgroup of the decode kernels
 * (0 for other variants); the first column of the 192-wide tiles of the mixed-width prefill launch (N when all tiles
 * are equal).  Honours the calling thread's forced variant and knobs, as a launch does (both run the same code).
 * Costs a few microseconds at most and keeps no state.  No counterpart in the reference, whose single Triton
 * configuration needs no plan.
 */
int dlb_fp8_gemm_plan(int mode, int64_t rows, int64_t N, int64_t K, size_t workspace_bytes, int compute_units, int* variant,
                      int* k_slices, int* decode_columns, int64_t* narrow_from);

/*
 * The same query for the grouped layouts with what their choice depends on besides the shape: the expert count and, for
 * the masked layout (mode 2), the caller's expected_m (<= 0: unknown).  mode 1 = contiguous (rows = M_sum), 2 = masked
 * (rows = M_max).  Outputs (each may be NULL): the kernel variant id; whether a contiguous launch of this size pairs
 * blocks into taller tiles from lists built on the device (1) or runs uniform 128-row tiles (0).  The fused gate/up
 * entry points always take the lists, so a caller that can also run GEMM and activation apart does that where this
 * says 0 (a batch of at most a round or two of tiles, where the uniform tiles are faster).  No counterpart in the
 * reference.
 */
int dlb_fp8_gemm_plan_grouped(int mode, int64_t rows, int64_t N, int64_t K, int32_t G, int32_t expected_m, size_t workspace_bytes,
                              int compute_units, int* variant, int* tile_lists);

/*
 * Tuning / test hook: force the kernel variant the next calls FROM THIS THREAD use.
 * variant < 0 restores the built-in shape heuristic.  Returns DLB_ERR_BAD_SHAPE for an unknown id.
 * Variant ids are listed by dlb_fp8_gemm_variant_name().
 */
int dlb_fp8_gemm_force_variant(int variant);

/*
 * Tuning / test hook: set knob `knob` for the next calls FROM THIS THREAD; value 0 restores the heuristic.
 *   DLB_KNOB_SPLITK         K slices of the dense tile kernels (all but the decode kernels and the mixed-width launch), each summed
 *                           into its own fp32 matrix in the workspace and added by a second kernel in slice order (clamped to
 *                           what workspace and K allow)
 *   DLB_KNOB_SKINNY_WAVES   waves per workgroup of the decode kernels (4, 8 or 16)
 *   DLB_KNOB_SKINNY_UNROLL  K blocks a decode-kernel wave loads before its first MFMA (1, 2 or 4)
 *   DLB_KNOB_SKINNY_NFRAGS  16-row weight fragments per decode workgroup (1 or 2)
 *   DLB_KNOB_GROUP_M        m-tiles per L2 swizzle group of the tiled kernels
 *   DLB_KNOB_SKINNY_DMA     2 = decode kernels load operands through registers instead of the LDS DMA path
 *   DLB_KNOB_EPILOGUE       2 = the pipelined kernels store bf16 results straight from registers (no LDS transpose)
 *   DLB_KNOB_SKINNY_BN      output columns per workgroup of the DMA-staged decode kernels (multiple of 4, at most 32)
 *   DLB_KNOB_SPLITK_MODE    1 = the K slices of the DMA-ring kernels are added inside the launch (one launch per call: the
 *                           workgroups of a tile count themselves in on a counter in the workspace head and add the
 *                           slices in index order, the same bits as the second pass); 0 / 2 = by a second launch, which
 *                           is the faster of the two on MI355X
 *   DLB_KNOB_SPIN_LIMIT     one-launch split-K: value - 1 = polls a workgroup waits for the other slices of its tile
 *                           (1 = none: the workgroup that completes a tile adds all of it)
 *   DLB_KNOB_SCALE_TABLE    2 = the small DMA-ring kernels fetch row-major activation scales stage by stage instead of
 *                           once per tile into a table in LDS
 *   DLB_KNOB_MASKED_GRID    workgroups per CU of the persistent grid of the masked layout (default 1)
 *   DLB_KNOB_TILE_LIST      expert-contiguous rows: 1 = 256- / 192- / 128-row tiles from lists built on the device
 *                           whenever a workspace allows it, 2 = uniform 128-row tiles (default: lists from more than two
 *                           rounds of 128 x 256 tiles on)
 *   DLB_KNOB_LDS_OVERSIZE   test hook: 1 = every kernel asks for more LDS than the GPU has, so the call is refused
 *                           (DLB_ERR_LAUNCH) before anything is enqueued
 */
#define DLB_KNOB_SPLITK 0
#define DLB_KNOB_SKINNY_WAVES 1
#define DLB_KNOB_SKINNY_UNROLL 2
#define DLB_KNOB_SKINNY_NFRAGS 3
#define DLB_KNOB_GROUP_M 4
#define DLB_KNOB_SKINNY_DMA 5
#define DLB_KNOB_EPILOGUE 6
#define DLB_KNOB_SKINNY_BN 7
#define DLB_KNOB_SPLITK_MODE 8
#define DLB_KNOB_SPIN_LIMIT 9
#define DLB_KNOB_SCALE_TABLE 10
#define DLB_KNOB_LDS_OVERSIZE 11
#define DLB_KNOB_MASKED_GRID 12
#define DLB_KNOB_TILE_LIST 13
int dlb_fp8_gemm_tune(int knob, int value);

/* Name of kernel variant `variant`, or NULL beyond the last one. */
const char* dlb_fp8_gemm_variant_name(int variant);

#ifdef __cplusplus
}
#endif
#endif /* DLBLAS_FP8_GEMM_H_ */
