// LDS-tiled FP8 block-scaled GEMM for gfx950: one workgroup computes BM x BN outputs per tile and walks
// K in 128-byte steps (= one scale block), staging A and B tiles through a double-buffered LDS ring.
//
// Operand roles are swapped relative to the textbook picture: the MFMA "A" operand is fed with 16 rows of
// the WEIGHT tile and the "B" operand with 16 rows of the ACTIVATION tile, so a lane's four accumulator
// components are four consecutive n of one m.  That makes the per-row activation scale a single value per
// lane (m = lane & 15) and lets every lane store 4 contiguous outputs.
//
// Follows the data flow of fp8_gemm_kernel (dlblas/kernels/fp8_gemm.py:38-65); the grouped modes follow the
// buffer conventions of dlblas/kernels/fused_moe_v3.py:262-308 and dlblas/layers/moe/ep_moe.py:199-261.
#pragma once

#include "fp8_gemm_common.h"

namespace dlb {

template <int BM_, int BN_, int WGM_, int WGN_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static constexpr int NT = WGM * WGN * 64;        // threads per workgroup
  static constexpr int WM = BM / WGM;              // rows of the wave tile (m)
  static constexpr int WN = BN / WGN;              // columns of the wave tile (n)
  static constexpr int MF = WM / 16;               // 16-row MFMA fragments along m
  static constexpr int NF = WN / 16;               // 16-row MFMA fragments along n
  static constexpr int A_LD = BM * 8 / NT;         // 16-byte chunks each thread moves per A tile
  static constexpr int B_LD = BN * 8 / NT;
  static constexpr int STAGE_BYTES = (BM + BN) * kScaleBlock;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wave tile must be made of 16x16 fragments");
  static_assert(WN <= 128 && 128 % WN == 0, "a wave's n span must stay inside one 128-wide scale block");
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "tile loads must divide evenly over the threads");
};

// Global -> registers: NLD 16-byte chunks per thread of a [ROWS][128 B] tile whose rows start at `row0`;
// rows past `row_last` re-read row_last (their results are never stored), bytes at or past K read as zero.
template <int NLD, int NT>
__device__ __forceinline__ void tile_load_global(v4i (&r)[NLD], const uint8_t* base, int64_t ld, int row0,
                                                 int row_last, int kbyte0, int K, int tid) {
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int ch = tid + i * NT;
    const int row = ch >> 3, c = ch & 7;
    const int gr = min(row0 + row, row_last);
    const int kk = kbyte0 + c * 16;
    v4i v = {0, 0, 0, 0};
    if (kk < K) v = *reinterpret_cast<const v4i*>(base + static_cast<int64_t>(gr) * ld + kk);
    r[i] = v;
  }
}

template <int NLD, int NT>
__device__ __forceinline__ void tile_store_lds(uint8_t* tile, const v4i (&r)[NLD], int tid) {
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int ch = tid + i * NT;
    *reinterpret_cast<v4i*>(tile + lds_off(ch >> 3, ch & 7)) = r[i];
  }
}

// Bijective remap of a linear workgroup id so that the workgroups the hardware places on one XCD
// (ids congruent modulo 8) own one contiguous range of tile ids and therefore share that XCD's L2.
__device__ __forceinline__ int xcd_remap(int vb, int total) {
  constexpr int kXcds = 8;
  const int q = total / kXcds, r = total % kXcds;
  const int x = vb % kXcds, idx = vb / kXcds;
  return x * q + min(x, r) + idx;
}

template <class Cfg, int MODE>
__global__ void __launch_bounds__(Cfg::NT) fp8_gemm_tiled_kernel(const Args p) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, NT = Cfg::NT, MF = Cfg::MF, NF = Cfg::NF;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int wm0 = (wave / Cfg::WGN) * Cfg::WM;
  const int wn0 = (wave % Cfg::WGN) * Cfg::WN;

  const int tiles = p.tiles_m * p.tiles_n;
  const int total = tiles * p.splitk;  // unused in masked mode

  // masked mode: running position of the device-side walk over masked_m
  int walk_g = 0;
  int walk_base = 0;

  for (int vb = blockIdx.x;; vb += gridDim.x) {
    int g = 0, mt, nt, split = 0, t = 0, m_end;
    if (MODE == kMasked) {
      int mtiles = 0;
      while (walk_g < p.G) {
        const int valid = min(max(p.gidx[walk_g], 0), p.M);
        mtiles = (valid + BM - 1) / BM;
        const int cnt = mtiles * p.tiles_n;
        if (vb < walk_base + cnt) break;
        walk_base += cnt;
        ++walk_g;
      }
      if (walk_g >= p.G) break;
      g = walk_g;
      const int local = vb - walk_base;
      mt = local % mtiles;
      nt = local / mtiles;
      m_end = min(max(p.gidx[g], 0), p.M);
    } else {
      if (vb >= total) break;
      const int id = xcd_remap(vb, total);
      split = id / tiles;
      t = id - split * tiles;
      const int width = p.group_m * p.tiles_n;
      const int grp = t / width;
      const int first_m = grp * p.group_m;
      const int gsz = min(p.tiles_m - first_m, p.group_m);
      const int in_grp = t - grp * width;
      mt = first_m + in_grp % gsz;
      nt = in_grp / gsz;
      m_end = p.M;
      if (MODE == kContiguous) {
        g = p.gidx[mt * BM];  // BM divides 128, so a tile never straddles two experts' row blocks
        if (g < 0 || g >= p.G) continue;
      }
    }
    const int m0 = mt * BM;
    const int n0 = nt * BN;

    const uint8_t* a_base = p.a;
    const float* as_base = p.a_s;
    char* c_base = static_cast<char*>(p.c);
    const int64_t esz = p.out_f32 ? 4 : 2;
    if (MODE == kMasked) {
      a_base += static_cast<int64_t>(g) * p.a_gs;
      as_base += static_cast<int64_t>(g) * p.as_gs;
      c_base += static_cast<int64_t>(g) * p.c_gs * esz;
    }
    const uint8_t* b_base = p.b + static_cast<int64_t>(g) * p.b_gs;
    const float* bs_row =
        p.b_s + static_cast<int64_t>(g) * p.bs_gs + static_cast<int64_t>(min((n0 + wn0) / kScaleBlock, p.nblocks - 1)) * p.kblocks;

    const int kb0 = split * p.kb_per_split;
    const int kb1 = min(p.kblocks, kb0 + p.kb_per_split);

    // per-lane activation-scale row pointers: fragment mi of this wave covers rows wm0 + 16 mi + (lane & 15)
    const float* as_ptr[MF];
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) {
      const int m = min(m0 + wm0 + mi * 16 + l16, m_end - 1);
      as_ptr[mi] = as_base + static_cast<int64_t>(m) * p.as_sm;
    }

    v4f acc[MF][NF];
#pragma unroll
    for (int mi = 0; mi < MF; ++mi)
#pragma unroll
      for (int ni = 0; ni < NF; ++ni) acc[mi][ni] = v4f{0.f, 0.f, 0.f, 0.f};

    v4i ra[Cfg::A_LD], rb[Cfg::B_LD];
    float sa[MF];
    float sb = 0.f;

    __syncthreads();  // previous tile of this workgroup has finished reading the LDS ring
    if (kb0 < kb1) {
      tile_load_global<Cfg::A_LD, NT>(ra, a_base, p.K, m0, m_end - 1, kb0 * kScaleBlock, p.K, tid);
      tile_load_global<Cfg::B_LD, NT>(rb, b_base, p.K, n0, p.N - 1, kb0 * kScaleBlock, p.K, tid);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) sa[mi] = as_ptr[mi][static_cast<int64_t>(kb0) * p.as_sk];
      sb = bs_row[kb0];
      tile_store_lds<Cfg::A_LD, NT>(smem, ra, tid);
      tile_store_lds<Cfg::B_LD, NT>(smem + BM * kScaleBlock, rb, tid);
    }
    __syncthreads();

    int cur = 0;
    for (int kb = kb0; kb < kb1; ++kb) {
      const bool more = kb + 1 < kb1;
      float sa_n[MF];
      float sb_n = 0.f;
      if (more) {
        tile_load_global<Cfg::A_LD, NT>(ra, a_base, p.K, m0, m_end - 1, (kb + 1) * kScaleBlock, p.K, tid);
        tile_load_global<Cfg::B_LD, NT>(rb, b_base, p.K, n0, p.N - 1, (kb + 1) * kScaleBlock, p.K, tid);
#pragma unroll
        for (int mi = 0; mi < MF; ++mi) sa_n[mi] = as_ptr[mi][static_cast<int64_t>(kb + 1) * p.as_sk];
        sb_n = bs_row[kb + 1];
      }

      const uint8_t* sA = smem + cur * Cfg::STAGE_BYTES;
      const uint8_t* sB = sA + BM * kScaleBlock;
      v8i wf[NF];
#pragma unroll
      for (int ni = 0; ni < NF; ++ni) wf[ni] = lds_read_frag(sB, wn0 + ni * 16 + l16, q);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const v8i xf = lds_read_frag(sA, wm0 + mi * 16 + l16, q);
        const float s = sa[mi] * sb;
#pragma unroll
        for (int ni = 0; ni < NF; ++ni) {
          const v4f part = mfma_16x16x128_e4m3(wf[ni], xf, v4f{0.f, 0.f, 0.f, 0.f});
          acc[mi][ni] += part * s;
        }
      }

      if (more) {
        uint8_t* nA = smem + (cur ^ 1) * Cfg::STAGE_BYTES;
        tile_store_lds<Cfg::A_LD, NT>(nA, ra, tid);
        tile_store_lds<Cfg::B_LD, NT>(nA + BM * kScaleBlock, rb, tid);
#pragma unroll
        for (int mi = 0; mi < MF; ++mi) sa[mi] = sa_n[mi];
        sb = sb_n;
      }
      __syncthreads();
      cur ^= 1;
    }

    if (MODE == kDense && p.splitk > 1) {
      // Split-K, first pass: this workgroup's K slice goes to the workspace as a plain fp32 [M][N] matrix of its
      // own; fp8_splitk_reduce_kernel, launched behind this kernel on the same stream, adds the slices in index
      // order (deterministic) and casts.  No fence, no counter: stream order makes the partial sums visible.
      float* mine = p.ws + static_cast<int64_t>(split) * p.M * p.N;
      const bool vec_ok = (p.N % 4) == 0;
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const int m = m0 + wm0 + mi * 16 + l16;
        if (m >= m_end) continue;
        float* w_row = mine + static_cast<int64_t>(m) * p.N;
#pragma unroll
        for (int ni = 0; ni < NF; ++ni) {
          const int n = n0 + wn0 + ni * 16 + q * 4;
          store_row4<true>(w_row, n, acc[mi][ni], p.N - n, vec_ok);
        }
      }
      continue;
    }

    // epilogue: lane holds c[m0 + wm0 + 16 mi + (lane & 15)][n0 + wn0 + 16 ni + 4 (lane >> 4) + 0..3]
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) {
      const int m = m0 + wm0 + mi * 16 + l16;
      if (m >= m_end) continue;
      char* c_row = c_base + static_cast<int64_t>(m) * p.N * esz;
#pragma unroll
      for (int ni = 0; ni < NF; ++ni) {
        const int n = n0 + wn0 + ni * 16 + q * 4;
        if (p.out_f32)
          store_row4<true>(c_row, n, acc[mi][ni], p.N - n, p.vec_store);
        else
          store_row4<false>(c_row, n, acc[mi][ni], p.N - n, p.vec_store);
      }
    }
  }
}

// Split-K, second pass: c[i] = sum over s (in index order) of ws[s][i], i over the M x N outputs, four per thread.
__global__ void __launch_bounds__(256) fp8_splitk_reduce_kernel(const float* ws, void* c, int64_t total, int splits,
                                                                int out_f32, int vec_ok) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  const int left = static_cast<int>(total - i < 4 ? total - i : 4);
  v4f sum = {0.f, 0.f, 0.f, 0.f};
  if (vec_ok) {  // total % 4 == 0 and 16-byte aligned slices
    for (int s = 0; s < splits; ++s)
      sum += __builtin_nontemporal_load(reinterpret_cast<const v4f*>(ws + static_cast<int64_t>(s) * total + i));
  } else {
    for (int s = 0; s < splits; ++s) {
      const float* src = ws + static_cast<int64_t>(s) * total + i;
      sum.x += src[0];
      if (left > 1) sum.y += src[1];
      if (left > 2) sum.z += src[2];
      if (left > 3) sum.w += src[3];
    }
  }
  if (out_f32)
    store_row4<true>(c, i, sum, left, vec_ok != 0);
  else
    store_row4<false>(c, i, sum, left, vec_ok != 0);
}

}  // namespace dlb
