// Bench-only kernels (not part of the library): what this GPU allows the GEMM kernels' instruction mix and access
// patterns when everything else is taken away.  bench.py times them (--decode-floor, --ceilings):
//   floor_empty  a kernel with the decode kernel's grid and block that returns at once: the per-launch cost of the
//                queue (dependent launches on one stream)
//   floor_read   every byte of the weight matrix read once with 16-byte loads, nothing else: launch cost + the time the
//                memory system needs to deliver the bytes to 256 workgroups
//   floor_mfma   the prefill kernel's arithmetic from registers only: pairs of v_mfma_f32_32x32x64_f8f6f4 (first of a
//                pair on a zero accumulator) + 16 scale FMAs per pair, two waves per SIMD, optionally with the kernel's
//                rate of LDS fragment reads (3 ds_read_b128 per pair) whose data nobody waits for.  The operands come
//                from the caller, so the same loop runs on constant and on random e4m3 codes
//   floor_panel_stream  one workgroup per CU streams 256-row panels of a row-major byte matrix through the LDS DMA path
//                (global_load_lds_dwordx4, 8 rows x 128 bytes per wave instruction, K step by K step, S steps in
//                flight) and does nothing with them: the rate at which a CU can pull a weight tile's rows from HBM
//   floor_l2_stream  one workgroup per CU pulls the SAME 512 rows of a row-major byte matrix, 128 bytes per row and K
//                step (the 64 KB a 256 x 256 GEMM tile needs per K step), so that after the first touch every request
//                hits the L2: what the path from the L2 into a CU delivers, through the LDS DMA (S steps in flight) or
//                through 16-byte register loads
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

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

// The same reads, then what any GEMM of that shape also has to do at its end: one exchange between the waves of a
// workgroup through LDS (a barrier) and the store of the workgroup's share of `out_bytes` of output.
template <int U>
__global__ void __launch_bounds__(512) floor_read_store_kernel(const v4i* src, int64_t words, int* out, int64_t out_bytes) {
  __shared__ int xch[512];
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
  xch[threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
  __syncthreads();
  const int mixed = xch[threadIdx.x] ^ xch[(threadIdx.x + 64) & 511] ^ xch[(threadIdx.x + 192) & 511];
  const int64_t per_wg = out_bytes / 4 / gridDim.x;  // dwords of output per workgroup
  for (int64_t t = threadIdx.x; t < per_wg; t += 512) out[static_cast<int64_t>(blockIdx.x) * per_wg + t] = mixed;
}

// R = ds_read_b128 per MFMA pair (0 or 3).  in: 6 x 64 x 32 bytes of e4m3 codes (4 "A" + 2 "B" operand registers per lane).
template <int R>
__global__ void __launch_bounds__(512) floor_mfma_kernel(const v8i* in, float* out, int iters, float scale) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<int*>(lds)[i] = 0x38383838;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = lane & 31, half = lane >> 5, swz = (row & 7) ^ ((row >> 3) & 1);
  int addr[3];
  for (int i = 0; i < 3; ++i) addr[i] = wave * 8192 + row * 128 + ((((i >> 1) * 4 + 2 * half + (i & 1)) ^ swz) << 4);
  v8i a[4], b[2];
  for (int i = 0; i < 4; ++i) a[i] = in[lane + 64 * i];
  for (int i = 0; i < 2; ++i) b[i] = in[lane + 64 * (4 + i)];
  v16f acc[4], part[2];
  for (int j = 0; j < 16; ++j) acc[0][j] = acc[1][j] = acc[2][j] = acc[3][j] = part[0][j] = part[1][j] = 0.0f;
  v4i d[3] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      if (t == 4) asm volatile("" : "+v"(a[0][0]), "+v"(a[1][0]), "+v"(a[2][0]), "+v"(a[3][0]));  // pairs 4..7 are not copies of 0..3
      __builtin_amdgcn_sched_barrier(0);
      v16f z;
      for (int j = 0; j < 16; ++j) z[j] = 0.0f;
      z = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[t & 3], b[0], z, 0, 0, 0, 0, 0, 0);
      part[t & 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[(t + 1) & 3], b[1], z, 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < R; ++r) asm volatile("ds_read_b128 %0, %1" : "=v"(d[r]) : "v"(addr[r] + (t & 1) * 4096));
      __builtin_amdgcn_sched_barrier(0);
      acc[(t + 3) & 3] += part[(t + 1) & 1] * scale;  // the scale FMAs of the previous pair
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // fold the (constant) LDS data in and move the operands a little, so that no iteration is a copy of another
    a[0][0] ^= it ^ (d[0].x ^ d[1].y ^ d[2].z ^ 0x38383838 ^ (R == 0 ? 0x38383838 : 0));
    b[0][1] += 0x01010101;
  }
  float r = 0.0f;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 16; ++j) r += acc[i][j];
  out[blockIdx.x * 512 + threadIdx.x] = r;
}

// S = K steps a wave keeps in flight.  Matrix [panels * 256][row_bytes]; workgroup b takes panels b, b + grid, ...
// POLICY = cache-policy operand of the loads of src (0, or 2 = the non-temporal bit); the shared panel always uses 0
template <int S, int POLICY>
__global__ void __launch_bounds__(512) floor_panel_stream_kernel(const char* src, int panels, int64_t row_bytes, const char* hot,
                                                                 int hot_panels) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ksteps = static_cast<int>(row_bytes / 128);
  for (int p = blockIdx.x; p < panels; p += gridDim.x) {
    // lane -> (row of the wave's 32, 16-byte chunk of the row's 128-byte line)
    const char* base = src + (static_cast<int64_t>(p) * 256 + wave * 32 + (lane >> 3)) * row_bytes + (lane & 7) * 16;
    for (int k = 0; k < ksteps; ++k) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(base + static_cast<int64_t>(u) * 8 * row_bytes + k * 128),
                                         (lds_ptr_t)(lds + ((k % S) * 32 + wave * 4 + u) * 1024), 16, 0, POLICY);
      if (hot != nullptr) {
        // a second 256-row panel per K step that many workgroups share (the activation strip of a GEMM tile: L2 hits)
        const char* hbase = hot + (static_cast<int64_t>((p / 16) % hot_panels) * 256 + wave * 32 + (lane >> 3)) * row_bytes + (lane & 7) * 16;
#pragma unroll
        for (int u = 0; u < 4; ++u)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(hbase + static_cast<int64_t>(u) * 8 * row_bytes + k * 128),
                                           (lds_ptr_t)(lds + ((k % S) * 32 + wave * 4 + u) * 1024), 16, 0, 0);
        if (S == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (S == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        if (S == 4) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
        continue;
      }
      if (S == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (S == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      if (S == 4) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// MODE 0: global_load_lds_dwordx4 into a ring of S stages of 64 KB; MODE 1: global_load_dwordx4 into registers, the
// loads of S K steps (8 per wave and step) in flight.  Workgroup b starts its walk over K at step 7 b (mod ksteps).
template <int MODE, int S>
__global__ void __launch_bounds__(512) floor_l2_stream_kernel(const char* src, int64_t row_bytes, int iters, int* sink) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ksteps = static_cast<int>(row_bytes / 128);
  const char* base = src + (static_cast<int64_t>(wave) * 64 + (lane >> 3)) * row_bytes + (lane & 7) * 16;
  int k = static_cast<int>((blockIdx.x * 7u) % static_cast<unsigned>(ksteps));
  v4i acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(base + static_cast<int64_t>(u) * 8 * row_bytes + k * 128),
                                         (lds_ptr_t)(lds + ((it % S) * 64 + wave * 8 + u) * 1024), 16, 0, 0);
      if (S == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (S == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else {
      v4i v[S][8];
#pragma unroll
      for (int s2 = 0; s2 < S; ++s2) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[s2][u] = *reinterpret_cast<const v4i*>(base + static_cast<int64_t>(u) * 8 * row_bytes + k * 128);
        k = k + 1 == ksteps ? 0 : k + 1;
      }
#pragma unroll
      for (int s2 = 0; s2 < S; ++s2)
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[s2][u];
      it += S - 1;
      continue;
    }
    k = k + 1 == ksteps ? 0 : k + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5a5a5a5a && sink == reinterpret_cast<int*>(1)) *sink = acc.x;
}

extern "C" {

// src: [512][row_bytes] bytes; K steps of 64 KB per workgroup = iters; mode 0 = LDS DMA, 1 = register loads; depth = K
// steps in flight (1 or 2)
int floor_l2_stream(const void* src, int64_t row_bytes, int workgroups, int iters, int mode, int depth, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* p = static_cast<const char*>(src);
  if (row_bytes <= 0 || row_bytes % 128 != 0) return -1;
  auto launch = [&](auto kernel, int lds_bytes) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) return;
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(512), lds_bytes, st, p, row_bytes, iters, nullptr);
  };
  if (mode == 0 && depth >= 2) launch(floor_l2_stream_kernel<0, 2>, 131072);
  if (mode == 0 && depth < 2) launch(floor_l2_stream_kernel<0, 1>, 65536);
  if (mode != 0 && depth >= 2) launch(floor_l2_stream_kernel<1, 2>, 0);
  if (mode != 0 && depth < 2) launch(floor_l2_stream_kernel<1, 1>, 0);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

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

int floor_read_store(const void* src, int64_t bytes, int workgroups, int loads_in_flight, void* out, int64_t out_bytes, void* stream) {
  const dim3 grid(workgroups), block(512);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const v4i* p = static_cast<const v4i*>(src);
  int* o = static_cast<int*>(out);
  if (loads_in_flight >= 8)
    hipLaunchKernelGGL(floor_read_store_kernel<8>, grid, block, 0, st, p, bytes / 16, o, out_bytes);
  else if (loads_in_flight >= 4)
    hipLaunchKernelGGL(floor_read_store_kernel<4>, grid, block, 0, st, p, bytes / 16, o, out_bytes);
  else
    hipLaunchKernelGGL(floor_read_store_kernel<2>, grid, block, 0, st, p, bytes / 16, o, out_bytes);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// operands: 12288 bytes of e4m3 codes on the device; out: workgroups * 512 floats.  FLOP per launch =
// workgroups * 8 waves * iters * 16 MFMAs * 131072.
int floor_mfma(const void* operands, float* out, int workgroups, int iters, int lds_reads, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const v8i* in = static_cast<const v8i*>(operands);
  hipFuncSetAttribute(reinterpret_cast<const void*>(floor_mfma_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  hipFuncSetAttribute(reinterpret_cast<const void*>(floor_mfma_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  if (lds_reads > 0)
    hipLaunchKernelGGL(floor_mfma_kernel<3>, dim3(workgroups), dim3(512), 65536, st, in, out, iters, 1.5f);
  else
    hipLaunchKernelGGL(floor_mfma_kernel<0>, dim3(workgroups), dim3(512), 65536, st, in, out, iters, 1.5f);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// src: [panels * 256][row_bytes] bytes, row_bytes a multiple of 128; steps_in_flight 1, 2 or 4; non_temporal: the loads
// of src carry the non-temporal bit; hot: nullptr, or
// [hot_panels * 256][row_bytes] bytes of which every workgroup also pulls one panel per panel of src (16 consecutive
// panels of src share one)
int floor_panel_stream(const void* src, int panels, int64_t row_bytes, int workgroups, int steps_in_flight, const void* hot,
                       int hot_panels, int non_temporal, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* p = static_cast<const char*>(src);
  const char* h = static_cast<const char*>(hot);
  if (hot != nullptr && hot_panels <= 0) return -1;
  if (row_bytes <= 0 || row_bytes % 128 != 0 || panels <= 0) return -1;
  const dim3 grid(workgroups), block(512);
  const int s = steps_in_flight >= 4 ? 4 : (steps_in_flight >= 2 ? 2 : 1);
  auto launch = [&](auto kernel) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) return;
    hipLaunchKernelGGL(kernel, grid, block, s * 32768, st, p, panels, row_bytes, h, hot_panels);
  };
  if (non_temporal) {
    if (s == 4) launch(floor_panel_stream_kernel<4, 2>);
    if (s == 2) launch(floor_panel_stream_kernel<2, 2>);
    if (s == 1) launch(floor_panel_stream_kernel<1, 2>);
  } else {
    if (s == 4) launch(floor_panel_stream_kernel<4, 0>);
    if (s == 2) launch(floor_panel_stream_kernel<2, 0>);
    if (s == 1) launch(floor_panel_stream_kernel<1, 0>);
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
