// C ABI of the MoE steps around the grouped GEMMs: argument validation and launches.
// The declarations and the contract of every entry point are in include/dlblas_fp8_moe.h.
#include "../../include/dlblas_fp8_moe.h"

#include "host_common.h"
#include "moe_activation.h"

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

}  // extern "C"
