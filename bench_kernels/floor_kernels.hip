// Bench-only kernels (not part of the library): what a launch of the decode GEMM's shape costs on this GPU when it
// computes nothing.  bench.py times them back to back on the same rotating weight buffers as the decode workloads:
//   floor_empty  a kernel with the decode kernel's grid and block that returns at once: the per-launch cost of the
//                queue (dependent launches on one stream)
//   floor_read   every byte of the weight matrix read once with 16-byte loads, nothing else: launch cost + the time the
//                memory system needs to deliver the bytes to 256 workgroups
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(512) floor_empty_kernel(int* sink) {
  if (sink == reinterpret_cast<int*>(1)) *sink = 0;  // never true: keeps the argument alive
}

// grid-stride over 16-byte words, U loads in flight per thread; the xor of everything read is stored only if it equals
// a value it cannot take, so the loads stay and nothing is written
template <int U>
__global__ void __launch_bounds__(512) floor_read_kernel(const v4i* src, int64_t words, int* sink) {
  v4i acc = {0, 0, 0, 0};
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + (U - 1) * stride < words; i += U * stride) {
    v4i v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  for (; i < words; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5a5a5a5a && sink == reinterpret_cast<int*>(1)) *sink = acc.x;
}

extern "C" {

int floor_empty(int workgroups, void* stream) {
  hipLaunchKernelGGL(floor_empty_kernel, dim3(workgroups), dim3(512), 0, static_cast<hipStream_t>(stream), nullptr);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// loads_in_flight: 16-byte loads each thread issues before it uses the first (2, 4 or 8)
int floor_read(const void* src, int64_t bytes, int workgroups, int loads_in_flight, void* stream) {
  const dim3 grid(workgroups), block(512);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const v4i* p = static_cast<const v4i*>(src);
  if (loads_in_flight >= 8)
    hipLaunchKernelGGL(floor_read_kernel<8>, grid, block, 0, st, p, bytes / 16, nullptr);
  else if (loads_in_flight >= 4)
    hipLaunchKernelGGL(floor_read_kernel<4>, grid, block, 0, st, p, bytes / 16, nullptr);
  else
    hipLaunchKernelGGL(floor_read_kernel<2>, grid, block, 0, st, p, bytes / 16, nullptr);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
