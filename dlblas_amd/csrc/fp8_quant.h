// Per-token-group activation quantiser for gfx950: per row and group of `group_size` consecutive elements,
// s = max(amax, eps) / 448 and q = clamp(x / s, -448, 448) rounded to nearest-even e4m3fn.  Restates
// _per_token_group_quant_fp8 and its column-major-scale twin (dlblas/kernels/fp8.py:8-105), whose group size is any
// divisor of the row length (:35-36, BLOCK = next_power_of_2(group_size), lanes past the group masked).  HBM-bound:
// every element is read once (16-byte loads, 8 elements per lane) and written once (8-byte stores); LANES lanes
// (the power of two at or above group_size / 8) share a group and reduce its amax with DPP-style shuffles, so a wave
// handles 64 / LANES groups per step: 16 lanes and 4 groups for the 128-wide groups of the block-scaled GEMM.  Group
// sizes that are no multiple of 8, or beyond 512, take fp8_quant_group_generic_kernel (a wave per group, element loads).
#pragma once

#include "fp8_gemm_common.h"

namespace dlb {

struct QuantArgs {
  const void* x;
  uint8_t* q;
  float* s;
  int64_t rows;
  int64_t groups_per_row;  // K / group_size
  int64_t group_size;
  int64_t x_row_stride;    // elements
  int64_t s_stride_m;      // floats
  int64_t s_stride_k;
  float eps;
};

enum QuantIn : int { kInBf16 = 0, kInF16 = 1, kInF32 = 2 };

// Eight consecutive input elements of one lane as loaded (one 16-byte load, two for fp32) and their fp32 values.
// Loading and unpacking are separate so that a kernel can issue the loads of several groups before it touches the
// first value.
struct Raw8 {
  v4i a, b;
};

template <int IN>
__device__ __forceinline__ Raw8 quant_load_raw(const void* x, int64_t elem) {
  Raw8 r;
  if (IN == kInF32) {
    const v4i* p = reinterpret_cast<const v4i*>(static_cast<const float*>(x) + elem);
    r.a = p[0], r.b = p[1];
  } else {
    r.a = *reinterpret_cast<const v4i*>(static_cast<const uint16_t*>(x) + elem);
    r.b = r.a;
  }
  return r;
}

template <int IN>
__device__ __forceinline__ void quant_unpack8(const Raw8& r, float (&v)[8]) {
  if (IN == kInF32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __int_as_float(r.a[i]), v[4 + i] = __int_as_float(r.b[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = static_cast<uint32_t>(r.a[i]);
      if (IN == kInBf16) {
        v[2 * i] = __uint_as_float(w << 16);
        v[2 * i + 1] = __uint_as_float(w & 0xffff0000u);
      } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 hv = __builtin_bit_cast(h2, w);
        v[2 * i] = static_cast<float>(hv.x);
        v[2 * i + 1] = static_cast<float>(hv.y);
      }
    }
  }
}

template <int IN>
__device__ __forceinline__ void quant_load8(const void* x, int64_t elem, float (&v)[8]) {
  quant_unpack8<IN>(quant_load_raw<IN>(x, elem), v);
}

// v / s with the IEEE division hoisted out of the per-element work: r = 1 / s correctly rounded (once per group),
// q0 = v r, then one correction with the exact remainder, q = fma(fma(-q0, s, v), r, q0).  The value before the last
// rounding is within 2^-47 of v / s, so q is the correctly rounded quotient unless v / s lies that close to a
// midpoint between two floats; 3 instructions instead of the 10 of a full division, which made the quantisers
// ALU-bound.
__device__ __forceinline__ float div_by_scale(float v, float s, float r) { return act_div_by_scale(v, s, r); }

template <int IN, int LANES>
__global__ void __launch_bounds__(256) fp8_quant_group_kernel(const QuantArgs p) {
  constexpr int kPerWave = 64 / LANES;  // groups per wave and step
  const int lane = threadIdx.x & 63;
  const int sub = lane & (LANES - 1);  // position inside the group: elements 8 sub .. 8 sub + 7
  const int64_t total = p.rows * p.groups_per_row;
  const int64_t wave_id = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) >> 6;
  const int64_t n_waves = (static_cast<int64_t>(gridDim.x) * 256) >> 6;
  const bool in_group = sub * 8 < p.group_size;  // lanes past a group that is no power of two take no part
  for (int64_t g0 = wave_id * kPerWave; g0 < total; g0 += n_waves * kPerWave) {
    const int64_t g = g0 + lane / LANES;
    const bool live = g < total && in_group;
    const int64_t gc = g < total ? g : total - 1;
    // 32-bit division where it fits: the 64-bit one costs more than the rest of the loop body
    const int64_t row = total < (1ll << 31) ? static_cast<int64_t>(static_cast<uint32_t>(gc) / static_cast<uint32_t>(p.groups_per_row))
                                            : gc / p.groups_per_row;
    const int64_t kg = gc - row * p.groups_per_row;
    float v[8];
    if (in_group) {
      quant_load8<IN>(p.x, row * p.x_row_stride + kg * p.group_size + sub * 8, v);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = 0.f;
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, LANES));
    const float scale = fmaxf(amax, p.eps) / 448.0f;
    const float inv_scale = 1.0f / scale;
    int packed[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float c[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = fminf(fmaxf(div_by_scale(v[4 * i + j], scale, inv_scale), -448.0f), 448.0f);
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w, true);
      packed[i] = w;
    }
    if (live) {
      *reinterpret_cast<v2i*>(p.q + (row * p.groups_per_row + kg) * p.group_size + sub * 8) = v2i{packed[0], packed[1]};
      if (sub == 0) p.s[row * p.s_stride_m + kg * p.s_stride_k] = scale;
    }
  }
}

// Any group size: a wave per group, lane l takes elements l, l + 64, ... with element-sized loads and byte stores, the
// same arithmetic (correctly rounded quotient, hardware e4m3 cast).  Slow next to the kernel above; it is the general
// case of the reference's signature, not a path of the GEMM.
template <int IN>
__global__ void __launch_bounds__(256) fp8_quant_group_generic_kernel(const QuantArgs p) {
  const int lane = threadIdx.x & 63;
  const int64_t total = p.rows * p.groups_per_row;
  const int64_t n_waves = (static_cast<int64_t>(gridDim.x) * 256) >> 6;
  auto element = [&](int64_t idx) -> float {
    if (IN == kInF32) return static_cast<const float*>(p.x)[idx];
    const uint32_t w = static_cast<const uint16_t*>(p.x)[idx];
    if (IN == kInBf16) return __uint_as_float(w << 16);
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w)));
  };
  for (int64_t g = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) >> 6; g < total; g += n_waves) {
    const int64_t row = g / p.groups_per_row, kg = g - row * p.groups_per_row;
    const int64_t x0 = row * p.x_row_stride + kg * p.group_size;
    float amax = 0.f;
    for (int64_t e = lane; e < p.group_size; e += 64) amax = fmaxf(amax, fabsf(element(x0 + e)));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = fmaxf(amax, p.eps) / 448.0f;
    const float inv_scale = 1.0f / scale;
    uint8_t* q0 = p.q + g * p.group_size;
    for (int64_t e = lane; e < p.group_size; e += 64) {
      const float c = fminf(fmaxf(div_by_scale(element(x0 + e), scale, inv_scale), -448.0f), 448.0f);
      q0[e] = static_cast<uint8_t>(__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xff);
    }
    if (lane == 0) p.s[row * p.s_stride_m + kg * p.s_stride_k] = scale;
  }
}

// 128 x 128 block quantiser for weights: one scale per block, s = max(amax, eps) / 448, same cast as above.  The
// reference ships no such function; the scheme is that of its test data builder
// (tests/kernels/test_fused_moe_v2.py:35-60) and of the b_s operand of fp8_gemm (dlblas/kernels/fp8_gemm.py:47).
// One workgroup per block: 8 chunks of 8 elements per thread stay in registers between the amax reduction and the
// cast, so every element is read once.  Blocks at the N and K edges are ragged; K % 8 == 0, rows 16-byte aligned.
struct BlockQuantArgs {
  const void* w;  // [G][N][K], row stride w_row_stride, group stride N * w_row_stride (elements)
  uint8_t* q;     // [G][N][K] contiguous
  float* s;       // [G][ceil(N/128)][ceil(K/128)] contiguous
  int64_t N, K, w_row_stride;
  int nblocks_n, nblocks_k;
  float eps;
};

template <int IN>
__global__ void __launch_bounds__(256) fp8_quant_128x128_kernel(const BlockQuantArgs p) {
  __shared__ float wave_max[4];
  const int tid = threadIdx.x;
  const int64_t blk = blockIdx.x;
  const int kb = static_cast<int>(blk % p.nblocks_k);
  const int64_t rest = blk / p.nblocks_k;
  const int nb = static_cast<int>(rest % p.nblocks_n);
  const int64_t g = rest / p.nblocks_n;
  const void* w_g = static_cast<const char*>(p.w) + g * p.N * p.w_row_stride * (IN == kInF32 ? 4 : 2);
  uint8_t* q_g = p.q + g * p.N * p.K;
  float v[8][8];
  bool live[8];
  float amax = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int i = tid + 256 * k;  // chunk of the block: row i / 16, columns 8 (i % 16) ..
    const int64_t row = static_cast<int64_t>(nb) * 128 + (i >> 4);
    const int64_t col = static_cast<int64_t>(kb) * 128 + (i & 15) * 8;
    live[k] = row < p.N && col < p.K;
    if (live[k]) {
      quant_load8<IN>(w_g, row * p.w_row_stride + col, v[k]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[k][j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[k][j]));
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  const float scale = fmaxf(amax, p.eps) / 448.0f;
  const float inv_scale = 1.0f / scale;
  if (tid == 0) p.s[(g * p.nblocks_n + nb) * p.nblocks_k + kb] = scale;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    if (!live[k]) continue;
    const int i = tid + 256 * k;
    const int64_t row = static_cast<int64_t>(nb) * 128 + (i >> 4);
    const int64_t col = static_cast<int64_t>(kb) * 128 + (i & 15) * 8;
    int packed[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float c[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = fminf(fmaxf(div_by_scale(v[k][4 * h + j], scale, inv_scale), -448.0f), 448.0f);
      int wd = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
      wd = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], wd, true);
      packed[h] = wd;
    }
    *reinterpret_cast<v2i*>(q_g + row * p.K + col) = v2i{packed[0], packed[1]};
  }
}

}  // namespace dlb
