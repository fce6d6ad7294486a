// C ABI of the MoE steps around the grouped GEMMs: argument validation and launches.
// The declarations and the contract of every entry point are in include/dlblas_fp8_moe.h.
#include "../../include/dlblas_fp8_moe.h"

#include <atomic>
#include <cstring>

#include "host_common.h"
#include "moe_activation.h"
#include "moe_permute.h"

namespace dlb {
namespace {

// Row blocks of the activation grid: 4 rows (one per wave) per workgroup, capped so that the grid (x G) is a few
// workgroups per CU; longer inputs are covered by the grid-stride loop over rows.
int64_t act_row_blocks(int64_t rows, int64_t G, int cus) {
  int64_t blocks = ceil_div(rows, 4);
  const int64_t cap = ceil_div(static_cast<int64_t>(cus) * 16, G);
  return blocks > cap ? cap : (blocks < 1 ? 1 : blocks);
}

template <int MODE>
void launch_act(int dtype, const ActArgs& a, int cus, hipStream_t st) {
  const dim3 grid(static_cast<unsigned>(act_row_blocks(a.rows, a.G, cus)), static_cast<unsigned>(a.G)), block(256);
  if (dtype == kInBf16)
    hipLaunchKernelGGL((moe_activation_kernel<kInBf16, MODE>), grid, block, 0, st, a);
  else if (dtype == kInF16)
    hipLaunchKernelGGL((moe_activation_kernel<kInF16, MODE>), grid, block, 0, st, a);
  else
    hipLaunchKernelGGL((moe_activation_kernel<kInF32, MODE>), grid, block, 0, st, a);
}

int check_common(const void* x, int dtype, const void* out, int64_t rows, int64_t N) {
  if (dtype < kInBf16 || dtype > kInF32) return fail(DLB_ERR_BAD_DTYPE, "dtype %d is not DLB_IN_BF16 / F16 / F32", dtype);
  if (rows < 0 || N < 0) return fail(DLB_ERR_BAD_SHAPE, "negative dimension (rows=%lld N=%lld)", (long long)rows, (long long)N);
  if (rows > 0 && N > 0 && (!x || !out)) return fail(DLB_ERR_NULL_POINTER, "x or the output is NULL");
  return DLB_OK;
}

int finish(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "%s launch failed: %s", what, hipGetErrorString(e));
  return DLB_OK;
}

int scatter_blocks(int64_t tokens, int64_t topk, int* tokens_per_block) {
  const int tpb = topk >= kPermuteThreads ? 1 : static_cast<int>(kPermuteThreads / topk);
  *tokens_per_block = tpb;
  const int64_t nb = ceil_div(tokens, tpb);
  return static_cast<int>(nb < 1 ? 1 : nb);
}

size_t scatter_ws_bytes(int64_t tokens, int64_t topk, int64_t experts) {
  if (tokens < 0 || topk <= 0 || experts <= 0) return 0;
  int tpb = 1;
  const int64_t nb = scatter_blocks(tokens, topk, &tpb);
  return static_cast<size_t>((experts + 2) * 8 + nb * experts * 4);
}

bool bad_index_dtype(int d) { return d != DLB_IDX_I32 && d != DLB_IDX_I64; }

template <int IN>
void launch_gather_out(int out_dtype, const GatherArgs& a, dim3 grid, hipStream_t st) {
  if (out_dtype == kInBf16)
    hipLaunchKernelGGL((ep_gather_kernel<IN, kInBf16>), grid, dim3(64), 0, st, a);
  else if (out_dtype == kInF16)
    hipLaunchKernelGGL((ep_gather_kernel<IN, kInF16>), grid, dim3(64), 0, st, a);
  else
    hipLaunchKernelGGL((ep_gather_kernel<IN, kInF32>), grid, dim3(64), 0, st, a);
}

}  // namespace
}  // namespace dlb

extern "C" {

int dlb_silu_mul(const void* x, int dtype, void* out, int64_t rows, int64_t N, int64_t x_row_stride,
                 int64_t out_row_stride, void* stream) {
  using namespace dlb;
  clear_error();
  if (int rc = check_common(x, dtype, out, rows, N)) return rc;
  if (rows == 0 || N == 0) return DLB_OK;
  if (x_row_stride < 2 * N || out_row_stride < N)
    return fail(DLB_ERR_BAD_STRIDE, "row strides (%lld, %lld) are smaller than the rows (2N=%lld, N=%lld)",
                (long long)x_row_stride, (long long)out_row_stride, (long long)(2 * N), (long long)N);
  const int64_t esz = dtype == kInF32 ? 4 : 2;
  if (misaligned(x, esz) || misaligned(out, esz)) return fail(DLB_ERR_ALIGNMENT, "x / out are not aligned to their element size");
  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  ActArgs a{x, out, nullptr, nullptr, 1, rows, N, 0, x_row_stride, 0, out_row_stride, 0, 0, 0, 0.f};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = N % 128 == 0 && !misaligned(x, 16) && !misaligned(out, 16) && (x_row_stride * esz) % 16 == 0 &&
                   (out_row_stride * esz) % 16 == 0;
  if (vec) {
    launch_act<kSiluMul>(dtype, a, cus, st);
  } else {
    int64_t blocks = ceil_div(rows * N, 256);
    const int64_t cap = static_cast<int64_t>(cus) * 32;
    if (blocks > cap) blocks = cap;
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (dtype == kInBf16)
      hipLaunchKernelGGL(silu_mul_scalar_kernel<kInBf16>, grid, block, 0, st, a);
    else if (dtype == kInF16)
      hipLaunchKernelGGL(silu_mul_scalar_kernel<kInF16>, grid, block, 0, st, a);
    else
      hipLaunchKernelGGL(silu_mul_scalar_kernel<kInF32>, grid, block, 0, st, a);
  }
  return finish("silu_mul");
}

int dlb_silu_mul_quant(const void* x, int dtype, void* q, float* s, int64_t rows, int64_t N, int64_t x_row_stride,
                       int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream) {
  using namespace dlb;
  clear_error();
  if (int rc = check_common(x, dtype, q, rows, N)) return rc;
  if (N % kScaleBlock != 0) return fail(DLB_ERR_BAD_SHAPE, "N=%lld is not a multiple of the group size 128", (long long)N);
  if (rows == 0 || N == 0) return DLB_OK;
  if (!s) return fail(DLB_ERR_NULL_POINTER, "s is NULL");
  if (x_row_stride < 2 * N) return fail(DLB_ERR_BAD_STRIDE, "x row stride %lld < 2N", (long long)x_row_stride);
  if (s_stride_m < 0 || s_stride_k < 0) return fail(DLB_ERR_BAD_STRIDE, "negative scale stride");
  const int64_t esz = dtype == kInF32 ? 4 : 2;
  if (misaligned(x, 16) || (x_row_stride * esz) % 16 != 0 || misaligned(q, 8) || misaligned(s, 4))
    return fail(DLB_ERR_ALIGNMENT, "x rows must be 16-byte aligned, q 8-byte aligned");
  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  ActArgs a{x, q, s, nullptr, 1, rows, N, 0, x_row_stride, 0, N, 0, s_stride_m, s_stride_k, eps};
  launch_act<kSiluMulQuant>(dtype, a, cus, static_cast<hipStream_t>(stream));
  return finish("silu_mul_quant");
}

int dlb_silu_mul_quant_masked(const void* x, int dtype, void* q, float* s, const int32_t* masked_m, int64_t G,
                              int64_t M_max, int64_t N, int64_t s_stride_g, int64_t s_stride_m, int64_t s_stride_k,
                              void* stream) {
  using namespace dlb;
  clear_error();
  if (G < 0) return fail(DLB_ERR_BAD_SHAPE, "negative group count %lld", (long long)G);
  if (int rc = check_common(x, dtype, q, M_max, N)) return rc;
  if (N % kScaleBlock != 0) return fail(DLB_ERR_BAD_SHAPE, "N=%lld is not a multiple of the group size 128", (long long)N);
  if (G == 0 || M_max == 0 || N == 0) return DLB_OK;
  if (!s || !masked_m) return fail(DLB_ERR_NULL_POINTER, "s or masked_m is NULL");
  if (s_stride_g < 0 || s_stride_m < 0 || s_stride_k < 0) return fail(DLB_ERR_BAD_STRIDE, "negative scale stride");
  if (misaligned(x, 16) || misaligned(q, 8) || misaligned(s, 4) || misaligned(masked_m, 4))
    return fail(DLB_ERR_ALIGNMENT, "x must be 16-byte aligned, q 8-byte aligned");
  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  ActArgs a{x, q, s, masked_m, G, M_max, N, M_max * 2 * N, 2 * N, M_max * N, N, s_stride_g, s_stride_m, s_stride_k, 1e-10f};
  if (G > 65535) return fail(DLB_ERR_BAD_SHAPE, "more than 65535 experts (%lld)", (long long)G);
  launch_act<kSiluMulQuantMasked>(dtype, a, cus, static_cast<hipStream_t>(stream));
  return finish("silu_mul_quant_masked");
}

size_t dlb_ep_scatter_workspace_bytes(int64_t tokens, int64_t topk, int64_t experts) {
  return dlb::scatter_ws_bytes(tokens, topk, experts);
}

namespace {

// ep_scatter with its tables only (index_only: no row is moved, src_row names every destination row's token) or in full
int scatter_impl(const void* recv_x, int64_t x_row_stride, const float* recv_x_scale, int64_t xs_stride_m,
                 int64_t xs_stride_k, const void* recv_topk, int topk_dtype, int64_t topk_stride_m,
                 int64_t topk_stride_k, const int32_t* num_recv_tokens_per_expert, void* expert_start_loc,
                 int start_dtype, void* output_tensor, int64_t out_row_stride, float* output_tensor_scale,
                 int64_t os_stride_m, int64_t os_stride_k, int32_t* m_indices, int64_t m_indices_len,
                 void* output_index, int index_dtype, int64_t oi_stride_m, int64_t oi_stride_k, int64_t tokens,
                 int64_t hidden, int64_t topk, int64_t experts, void* workspace, size_t workspace_bytes,
                 void* stream, int32_t* src_row, bool index_only) {
  using namespace dlb;
  clear_error();
  if (bad_index_dtype(topk_dtype) || bad_index_dtype(start_dtype) || bad_index_dtype(index_dtype))
    return fail(DLB_ERR_BAD_DTYPE, "index dtypes must be DLB_IDX_I32 or DLB_IDX_I64 (%d, %d, %d)", topk_dtype, start_dtype, index_dtype);
  if (tokens < 0 || hidden < 0 || topk < 0 || experts < 0 || m_indices_len < 0)
    return fail(DLB_ERR_BAD_SHAPE, "negative dimension (tokens=%lld hidden=%lld topk=%lld experts=%lld)", (long long)tokens,
                (long long)hidden, (long long)topk, (long long)experts);
  if (experts == 0) return DLB_OK;
  if (hidden % kScaleBlock != 0) return fail(DLB_ERR_BAD_SHAPE, "hidden=%lld is not a multiple of 128", (long long)hidden);
  if (topk > kMaxTopk) return fail(DLB_ERR_BAD_SHAPE, "topk=%lld exceeds %d", (long long)topk, kMaxTopk);
  if (experts > kScanMaxExperts || hidden > (1ll << 30) || tokens > (1ll << 40))
    return fail(DLB_ERR_BAD_SHAPE, "experts=%lld / hidden=%lld / tokens=%lld beyond the supported range", (long long)experts,
                (long long)hidden, (long long)tokens);
  if (!num_recv_tokens_per_expert || !expert_start_loc || (m_indices_len > 0 && !m_indices))
    return fail(DLB_ERR_NULL_POINTER, "num_recv_tokens_per_expert, expert_start_loc or m_indices is NULL");
  const bool has_entries = tokens > 0 && topk > 0;
  if (has_entries && (!recv_topk || !output_index)) return fail(DLB_ERR_NULL_POINTER, "recv_topk or output_index is NULL");
  if (index_only) {
    if (m_indices_len > 0 && !src_row) return fail(DLB_ERR_NULL_POINTER, "src_row is NULL");
    if (tokens > (1ll << 31) - 1) return fail(DLB_ERR_BAD_SHAPE, "tokens=%lld does not fit the int32 row table", (long long)tokens);
  } else {
    if (has_entries && hidden > 0 && (!recv_x || !recv_x_scale || !output_tensor || !output_tensor_scale))
      return fail(DLB_ERR_NULL_POINTER, "recv_x, recv_x_scale, output_tensor or output_tensor_scale is NULL");
    if (x_row_stride < hidden || out_row_stride < hidden)
      return fail(DLB_ERR_BAD_STRIDE, "row strides (%lld, %lld) are smaller than hidden=%lld", (long long)x_row_stride,
                  (long long)out_row_stride, (long long)hidden);
    if (has_entries && hidden > 0 &&
        (misaligned(recv_x, 16) || misaligned(output_tensor, 16) || x_row_stride % 16 != 0 || out_row_stride % 16 != 0))
      return fail(DLB_ERR_ALIGNMENT, "recv_x / output_tensor rows must be 16-byte aligned");
  }
  const size_t need = scatter_ws_bytes(tokens, topk > 0 ? topk : 1, experts);
  if (!workspace || workspace_bytes < need)
    return fail(DLB_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace ? workspace_bytes : (size_t)0);
  if (misaligned(workspace, 8)) return fail(DLB_ERR_ALIGNMENT, "workspace must be 8-byte aligned");

  ScatterArgs a;
  memset(&a, 0, sizeof(a));
  a.x = static_cast<const uint8_t*>(recv_x);
  a.xs = recv_x_scale;
  a.topk = recv_topk;
  a.counts = num_recv_tokens_per_expert;
  a.start_loc = expert_start_loc;
  a.out = static_cast<uint8_t*>(output_tensor);
  a.out_s = output_tensor_scale;
  a.m_indices = m_indices;
  a.out_index = output_index;
  a.start_excl = static_cast<int64_t*>(workspace);
  a.block_hist = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + (experts + 2) * 8);
  a.x_row_stride = x_row_stride, a.xs_sm = xs_stride_m, a.xs_sk = xs_stride_k;
  a.topk_s0 = topk_stride_m, a.topk_s1 = topk_stride_k;
  a.out_row_stride = out_row_stride, a.os_sm = os_stride_m, a.os_sk = os_stride_k;
  a.oi_s0 = oi_stride_m, a.oi_s1 = oi_stride_k;
  a.T = topk > 0 ? tokens : 0;
  a.m_len = m_indices_len;
  a.H = static_cast<int>(hidden), a.E = static_cast<int>(experts), a.topk_n = static_cast<int>(topk > 0 ? topk : 1);
  a.nblocks = scatter_blocks(a.T, a.topk_n, &a.tokens_per_block);
  a.topk_is64 = topk_dtype == DLB_IDX_I64, a.start_is64 = start_dtype == DLB_IDX_I64, a.oi_is64 = index_dtype == DLB_IDX_I64;
  a.src_row = src_row;
  a.index_only = index_only;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(a.nblocks)), block(kPermuteThreads);
  a.fused_scan = static_cast<int64_t>(a.nblocks) * a.E <= kFusedScanMaxInts;
  hipLaunchKernelGGL(ep_scatter_count_kernel, grid, block, static_cast<size_t>(a.E) * sizeof(int), st, a);
  if (int rc = finish("ep_scatter (count)")) return rc;
  if (!a.fused_scan) {
    static std::atomic<unsigned long long> lds_done{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
    const unsigned long long bit = 1ull << (dev & 63);
    if (!(lds_done.load(std::memory_order_acquire) & bit)) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(ep_scatter_scan_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kScanTileInts * 4) != hipSuccess)
        return fail(DLB_ERR_LAUNCH, "cannot raise the LDS limit of the scan kernel");
      lds_done.fetch_or(bit, std::memory_order_release);
    }
    hipLaunchKernelGGL(ep_scatter_scan_kernel, dim3(1), dim3(kScanThreads), kScanTileInts * 4, st, a);
    if (int rc = finish("ep_scatter (scan)")) return rc;
  }
  hipLaunchKernelGGL(ep_scatter_copy_kernel, grid, dim3(index_only ? kPermuteThreads : kCopyThreads), 0, st, a);
  return finish("ep_scatter (copy)");
}

}  // namespace

int dlb_ep_scatter(const void* recv_x, int64_t x_row_stride, const float* recv_x_scale, int64_t xs_stride_m,
                   int64_t xs_stride_k, const void* recv_topk, int topk_dtype, int64_t topk_stride_m,
                   int64_t topk_stride_k, const int32_t* num_recv_tokens_per_expert, void* expert_start_loc,
                   int start_dtype, void* output_tensor, int64_t out_row_stride, float* output_tensor_scale,
                   int64_t os_stride_m, int64_t os_stride_k, int32_t* m_indices, int64_t m_indices_len,
                   void* output_index, int index_dtype, int64_t oi_stride_m, int64_t oi_stride_k, int64_t tokens,
                   int64_t hidden, int64_t topk, int64_t experts, void* workspace, size_t workspace_bytes,
                   void* stream) {
  return scatter_impl(recv_x, x_row_stride, recv_x_scale, xs_stride_m, xs_stride_k, recv_topk, topk_dtype, topk_stride_m,
                      topk_stride_k, num_recv_tokens_per_expert, expert_start_loc, start_dtype, output_tensor, out_row_stride,
                      output_tensor_scale, os_stride_m, os_stride_k, m_indices, m_indices_len, output_index, index_dtype,
                      oi_stride_m, oi_stride_k, tokens, hidden, topk, experts, workspace, workspace_bytes, stream, nullptr, false);
}

int dlb_ep_scatter_rows(const void* recv_topk, int topk_dtype, int64_t topk_stride_m, int64_t topk_stride_k,
                        const int32_t* num_recv_tokens_per_expert, void* expert_start_loc, int start_dtype,
                        int32_t* m_indices, int32_t* src_row, int64_t m_indices_len, void* output_index, int index_dtype,
                        int64_t oi_stride_m, int64_t oi_stride_k, int64_t tokens, int64_t topk, int64_t experts,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return scatter_impl(nullptr, 0, nullptr, 0, 0, recv_topk, topk_dtype, topk_stride_m, topk_stride_k, num_recv_tokens_per_expert,
                      expert_start_loc, start_dtype, nullptr, 0, nullptr, 0, 0, m_indices, m_indices_len, output_index, index_dtype,
                      oi_stride_m, oi_stride_k, tokens, 0, topk, experts, workspace, workspace_bytes, stream, src_row, true);
}

int dlb_ep_gather(const void* input, int in_dtype, int64_t in_row_stride, const void* recv_topk_ids, int topk_dtype,
                  int64_t topk_stride_m, int64_t topk_stride_k, const float* recv_topk_weight, int64_t w_stride_m,
                  int64_t w_stride_k, const void* input_index, int index_dtype, int64_t idx_stride_m,
                  int64_t idx_stride_k, void* output, int out_dtype, int64_t out_row_stride, int64_t tokens,
                  int64_t hidden, int64_t topk, void* stream) {
  using namespace dlb;
  clear_error();
  if (in_dtype < kInBf16 || in_dtype > kInF32 || out_dtype < kInBf16 || out_dtype > kInF32)
    return fail(DLB_ERR_BAD_DTYPE, "in_dtype %d / out_dtype %d is not DLB_IN_BF16 / F16 / F32", in_dtype, out_dtype);
  if (bad_index_dtype(topk_dtype) || bad_index_dtype(index_dtype))
    return fail(DLB_ERR_BAD_DTYPE, "index dtypes must be DLB_IDX_I32 or DLB_IDX_I64 (%d, %d)", topk_dtype, index_dtype);
  if (tokens < 0 || hidden < 0 || topk < 0)
    return fail(DLB_ERR_BAD_SHAPE, "negative dimension (tokens=%lld hidden=%lld topk=%lld)", (long long)tokens, (long long)hidden,
                (long long)topk);
  if (tokens == 0 || hidden == 0) return DLB_OK;
  if (hidden % 8 != 0) return fail(DLB_ERR_BAD_SHAPE, "hidden=%lld is not a multiple of 8", (long long)hidden);
  if (topk > kMaxTopk) return fail(DLB_ERR_BAD_SHAPE, "topk=%lld exceeds %d", (long long)topk, kMaxTopk);
  if (tokens > (1ll << 31) - 1 || hidden > (1ll << 30)) return fail(DLB_ERR_BAD_SHAPE, "tokens / hidden beyond the supported range");
  if (!output || (topk > 0 && (!input || !recv_topk_ids || !recv_topk_weight || !input_index)))
    return fail(DLB_ERR_NULL_POINTER, "a tensor pointer is NULL");
  if (in_row_stride < hidden || out_row_stride < hidden) return fail(DLB_ERR_BAD_STRIDE, "row stride smaller than hidden");
  const int64_t in_esz = in_dtype == kInF32 ? 4 : 2, out_esz = out_dtype == kInF32 ? 4 : 2;
  if ((topk > 0 && (misaligned(input, 16) || (in_row_stride * in_esz) % 16 != 0)) || misaligned(output, 16) ||
      (out_row_stride * out_esz) % 16 != 0)
    return fail(DLB_ERR_ALIGNMENT, "input / output rows must be 16-byte aligned");
  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  GatherArgs a{input, recv_topk_ids, recv_topk_weight, input_index, output, in_row_stride, topk_stride_m, topk_stride_k,
               w_stride_m, w_stride_k, idx_stride_m, idx_stride_k, out_row_stride, tokens, static_cast<int>(hidden),
               static_cast<int>(topk), topk_dtype == DLB_IDX_I64, index_dtype == DLB_IDX_I64};
  // column parts: enough single-wave blocks to cover the chip a few times over, at least 64 chunks of 8 per part
  const int64_t chunks = hidden / 8;
  int64_t parts = ceil_div(static_cast<int64_t>(cus) * 16, tokens);
  const int64_t max_parts = chunks / 64 > 0 ? chunks / 64 : 1;
  if (parts > max_parts) parts = max_parts;
  if (parts < 1) parts = 1;
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(parts));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (in_dtype == kInBf16)
    launch_gather_out<kInBf16>(out_dtype, a, grid, st);
  else if (in_dtype == kInF16)
    launch_gather_out<kInF16>(out_dtype, a, grid, st);
  else
    launch_gather_out<kInF32>(out_dtype, a, grid, st);
  return finish("ep_gather");
}

}  // extern "C"
