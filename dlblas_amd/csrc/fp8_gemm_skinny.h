// Weight-streaming FP8 block-scaled GEMM for decode-sized M (M <= 16 * MF) on gfx950.
//
// The problem is bound by reading B once from HBM, so the kernel is organised around keeping as many
// 16-byte weight loads in flight as possible and never staging through LDS: a workgroup owns 16 rows of B
// (one MFMA operand), its waves take interleaved 128-byte K blocks, every lane loads its own MFMA operand
// bytes straight from global memory, and the per-wave partial sums meet in LDS at the end.  K can further
// be split across workgroups; those partials meet in the workspace and the last workgroup to arrive adds
// them in split order, so results do not depend on scheduling.
//
// Arithmetic is that of fp8_gemm_kernel (dlblas/kernels/fp8_gemm.py:49-60): one scale FMA per K block.
#pragma once

#include "fp8_gemm_common.h"

namespace dlb {

template <int MF_, int WAVES_>
struct SkinnyCfg {
  static constexpr int MF = MF_;        // 16-row activation fragments (M <= 16 * MF)
  static constexpr int WAVES = WAVES_;  // waves per workgroup, each taking every WAVES-th K block
  static constexpr int NT = WAVES * 64;
  static constexpr int BN = 16;         // rows of B per workgroup
  static constexpr int UNROLL = 4;      // K blocks whose loads are issued before the first MFMA
};

// 32 operand bytes of one lane for K block `kb`: bytes [16 q, 16 q + 16) and [64 + 16 q, 64 + 16 q + 16) of the
// block.  Any assignment of K bytes to lanes is valid as long as both MFMA operands use the same one; this
// one makes each of the two load instructions of a wave cover 64 contiguous bytes per row.
__device__ __forceinline__ v8i skinny_load_frag(const uint8_t* row, int kb, int q, int K, bool valid) {
  const int k_lo = kb * kScaleBlock + q * 16;
  const int k_hi = k_lo + 64;
  v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
  if (valid && k_lo < K) lo = *reinterpret_cast<const v4i*>(row + k_lo);
  if (valid && k_hi < K) hi = *reinterpret_cast<const v4i*>(row + k_hi);
  return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::NT) fp8_gemm_skinny_kernel(const Args p) {
  constexpr int MF = Cfg::MF, WAVES = Cfg::WAVES, U = Cfg::UNROLL;
  __shared__ v4f red[WAVES][MF][64];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;

  const int nt = blockIdx.x % p.tiles_n;
  const int split = blockIdx.x / p.tiles_n;
  const int n0 = nt * Cfg::BN;
  const int kb0 = split * p.kb_per_split;
  const int kb1 = min(p.kblocks, kb0 + p.kb_per_split);

  const uint8_t* w_row = p.b + static_cast<int64_t>(min(n0 + l16, p.N - 1)) * p.K;
  const float* bs_row = p.b_s + static_cast<int64_t>(n0 / kScaleBlock) * p.kblocks;
  const uint8_t* x_row[MF];
  const float* as_row[MF];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi) {
    const int m = min(mi * 16 + l16, p.M - 1);
    x_row[mi] = p.a + static_cast<int64_t>(m) * p.K;
    as_row[mi] = p.a_s + static_cast<int64_t>(m) * p.as_sm;
  }

  v4f acc[MF];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi) acc[mi] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int kb = kb0 + wave; kb < kb1; kb += WAVES * U) {
    v8i wf[U];
    v8i xf[U][MF];
    float s[U][MF];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kbu = kb + u * WAVES;
      const bool valid = kbu < kb1;
      wf[u] = skinny_load_frag(w_row, kbu, q, p.K, valid);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kbu = kb + u * WAVES;
      const bool valid = kbu < kb1;
      const float sb = valid ? bs_row[kbu] : 0.f;
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        xf[u][mi] = skinny_load_frag(x_row[mi], kbu, q, p.K, valid);
        s[u][mi] = valid ? as_row[mi][static_cast<int64_t>(kbu) * p.as_sk] * sb : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const v4f part = mfma_16x16x128_e4m3(wf[u], xf[u][mi], v4f{0.f, 0.f, 0.f, 0.f});
        acc[mi] += part * s[u][mi];
      }
    }
  }

#pragma unroll
  for (int mi = 0; mi < MF; ++mi) red[wave][mi][lane] = acc[mi];
  __syncthreads();
  if (wave != 0) return;

#pragma unroll
  for (int mi = 0; mi < MF; ++mi) {
    v4f sum = red[0][mi][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][mi][lane];
    acc[mi] = sum;
  }

  if (p.splitk > 1) {
    float* wst = p.ws + static_cast<int64_t>(nt) * p.splitk * (MF * 256);
    float* mine = wst + static_cast<int64_t>(split) * (MF * 256);
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) *reinterpret_cast<v4f*>(mine + (mi * 64 + lane) * 4) = acc[mi];
    __threadfence();
    int last = 0;
    if (lane == 0) last = (atomicAdd(&p.ctr[nt], 1u) == static_cast<unsigned>(p.splitk - 1));
    last = __shfl(last, 0);
    if (!last) return;
    __threadfence();
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) acc[mi] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.splitk; ++s) {
      const float* src = wst + static_cast<int64_t>(s) * (MF * 256);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) acc[mi] += *reinterpret_cast<const v4f*>(src + (mi * 64 + lane) * 4);
    }
    if (lane == 0) p.ctr[nt] = 0u;
  }

  const int64_t esz = p.out_f32 ? 4 : 2;
  const int n = n0 + q * 4;
#pragma unroll
  for (int mi = 0; mi < MF; ++mi) {
    const int m = mi * 16 + l16;
    if (m >= p.M) continue;
    char* c_row = static_cast<char*>(p.c) + static_cast<int64_t>(m) * p.N * esz;
    if (p.out_f32)
      store_row4<true>(c_row, n, acc[mi], p.N - n, p.vec_store);
    else
      store_row4<false>(c_row, n, acc[mi], p.N - n, p.vec_store);
  }
}

}  // namespace dlb
