// Activation step between the two grouped GEMMs of an expert MLP, for gfx950: silu(gate) * up of a [.., 2N] matrix,
// optionally followed by the 1 x 128 e4m3fn quantiser in the same pass.  Restates
//   silu_and_mul                          dlblas/layers/moe/kernels/activation.py:16-95     (kSiluMul)
//   silu_and_mul + per_token_group_quant  dlblas/kernels/fused_moe_v3.py:325-334            (kSiluMulQuant)
//   silu_and_mul_masked_post_quant_fwd    dlblas/kernels/moe.py:204-319                     (kSiluMulQuantMasked)
// HBM-bound: 4 bytes read per output element (bf16 gate + up), 2 (bf16) or 1 + 4/128 (fp8 + scale) written.
// 16 lanes share a 128-wide group (8 elements = one 16-byte load of each half per lane), amax by four xor-shuffles.
#pragma once

#include <math.h>

#include "fp8_quant.h"

namespace dlb {

enum ActMode : int { kSiluMul = 0, kSiluMulQuant = 1, kSiluMulQuantMasked = 2 };

struct ActArgs {
  const void* x;            // [G][rows][2N], row stride x_row_stride, group stride x_g_stride (elements)
  void* out;                // kSiluMul: [rows][N] in the input dtype; else e4m3fn codes [G][rows][N]
  float* s;                 // scales [G][rows][N / 128] through strides (floats)
  const int32_t* masked_m;  // kSiluMulQuantMasked: valid rows per group
  int64_t G, rows, N;
  int64_t x_g_stride, x_row_stride;
  int64_t out_g_stride, out_row_stride;
  int64_t s_g_stride, s_m_stride, s_k_stride;
  float eps;
};

// fp32 -> input dtype -> fp32 (round to nearest even), the identity for fp32 inputs
template <int IN>
__device__ __forceinline__ float round_to_input(float v) {
  if (IN == kInBf16) return static_cast<float>(static_cast<__bf16>(v));
  if (IN == kInF16) return static_cast<float>(static_cast<_Float16>(v));
  return v;
}

// gate / (1 + exp(-gate)) with the hardware exponential and reciprocal (about 2 ulp each), as the reference's kernels
// do (fast exp and approximate division of the Triton build).  The result is rounded to a 8- or 11-bit significand
// right after, so the choice shows in about one result in 10^4; the correctly rounded forms cost 3x the instructions
// and made this HBM-bound kernel ALU-bound.
__device__ __forceinline__ float silu_f32(float g) { return act_silu_f32(g); }

template <int IN>
__device__ __forceinline__ void act_store8(void* out, int64_t elem, const float (&v)[8]) {
  if (IN == kInF32) {
    v4f* p = reinterpret_cast<v4f*>(static_cast<float*>(out) + elem);
    p[0] = v4f{v[0], v[1], v[2], v[3]};
    p[1] = v4f{v[4], v[5], v[6], v[7]};
  } else {
    v4i raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t lo, hi;
      if (IN == kInBf16) {
        lo = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v[2 * i]));
        hi = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v[2 * i + 1]));
      } else {
        lo = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v[2 * i]));
        hi = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v[2 * i + 1]));
      }
      raw[i] = static_cast<int>(lo | (hi << 16));
    }
    *reinterpret_cast<v4i*>(static_cast<uint16_t*>(out) + elem) = raw;
  }
}

// grid = (row blocks, G).  A wave owns whole rows of its expert (grid-stride over the rows below masked_m[g], so no
// wave ever visits a masked row) and walks a row 8 groups of 128 at a time: 16 lanes per group, 4 groups per
// 64-lane step, 2 steps in flight.  Row addressing is wave-uniform (scalar unit); a lane adds a 32-bit column
// offset.  N % 128 == 0; rows 16-byte aligned.
template <int IN, int MODE>
__global__ void __launch_bounds__(256) moe_activation_kernel(const ActArgs p) {
  constexpr int U = 2;
  const int lane = threadIdx.x & 63;
  const int sub = lane & 15;
  const int gpr = static_cast<int>(p.N / 128);  // groups per row
  const int g = blockIdx.y;
  int64_t rows = p.rows;
  if (MODE == kSiluMulQuantMasked) rows = min(static_cast<int64_t>(max(p.masked_m[g], 0)), rows);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int64_t first_row = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  const int64_t row_step = static_cast<int64_t>(gridDim.x) * 4;
  const size_t in_esz = IN == kInF32 ? 4 : 2;
  for (int64_t row = first_row; row < rows; row += row_step) {
    const char* x_row = static_cast<const char*>(p.x) + (g * p.x_g_stride + row * p.x_row_stride) * in_esz;
    char* out_row = static_cast<char*>(p.out) +
                    (g * p.out_g_stride + row * p.out_row_stride) * (MODE == kSiluMul ? in_esz : 1);
    float* s_row = p.s + g * p.s_g_stride + row * p.s_m_stride;
    for (int kg0 = 0; kg0 < gpr; kg0 += 4 * U) {
      bool live[U];
      int col[U];
      Raw8 raw_gate[U], raw_up[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kg = kg0 + u * 4 + (lane >> 4);
        live[u] = kg < gpr;
        col[u] = min(kg, gpr - 1) * 128 + sub * 8;
        raw_gate[u] = quant_load_raw<IN>(x_row, col[u]);
        raw_up[u] = quant_load_raw<IN>(x_row, col[u] + p.N);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float gate[8], up[8], v[8];
        quant_unpack8<IN>(raw_gate[u], gate);
        quant_unpack8<IN>(raw_up[u], up);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (MODE == kSiluMulQuantMasked)
            v[i] = round_to_input<IN>(up[i] * round_to_input<IN>(silu_f32(gate[i])));  // two roundings (moe.py:256-257)
          else
            v[i] = round_to_input<IN>(silu_f32(gate[i]) * up[i]);                       // one (activation.py:50-52)
        }
        if (MODE == kSiluMul) {
          if (live[u]) act_store8<IN>(out_row, col[u], v);
          continue;
        }
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 16));
        const float scale = fmaxf(amax, p.eps) / 448.0f;
        const float inv_scale = 1.0f / scale;
        int packed[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          float c[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) c[j] = fminf(fmaxf(div_by_scale(v[4 * i + j], scale, inv_scale), -448.0f), 448.0f);
          int wd = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
          wd = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], wd, true);
          packed[i] = wd;
        }
        if (live[u]) {
          *reinterpret_cast<v2i*>(out_row + col[u]) = v2i{packed[0], packed[1]};
          if (sub == 0) s_row[static_cast<int64_t>(col[u] >> 7) * p.s_k_stride] = scale;
        }
      }
    }
  }
}

// silu_and_mul for widths that are not a multiple of 128 or rows that are not 16-byte aligned: one element per thread.
template <int IN>
__global__ void __launch_bounds__(256) silu_mul_scalar_kernel(const ActArgs p) {
  const int64_t total = p.rows * p.N;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t row = i / p.N, col = i - row * p.N;
    const int64_t src = row * p.x_row_stride + col;
    float g, u;
    if (IN == kInBf16) {
      const __bf16* x = static_cast<const __bf16*>(p.x);
      g = static_cast<float>(x[src]), u = static_cast<float>(x[src + p.N]);
      static_cast<__bf16*>(p.out)[row * p.out_row_stride + col] = static_cast<__bf16>(silu_f32(g) * u);
    } else if (IN == kInF16) {
      const _Float16* x = static_cast<const _Float16*>(p.x);
      g = static_cast<float>(x[src]), u = static_cast<float>(x[src + p.N]);
      static_cast<_Float16*>(p.out)[row * p.out_row_stride + col] = static_cast<_Float16>(silu_f32(g) * u);
    } else {
      const float* x = static_cast<const float*>(p.x);
      g = x[src], u = x[src + p.N];
      static_cast<float*>(p.out)[row * p.out_row_stride + col] = silu_f32(g) * u;
    }
  }
}

}  // namespace dlb
