// Weight-streaming FP8 block-scaled GEMM for decode-sized M (M <= 16 * MF) on gfx950.
//
// The problem is bound by reading B once from HBM, so the kernel is organised around keeping as many 16-byte
// weight loads in flight as possible and never staging through LDS: a workgroup owns 16 * NFS rows of B, its
// waves take interleaved 128-byte K blocks, every lane loads its own MFMA operand bytes straight from global
// memory, and the per-wave partial sums meet in LDS at the end (fixed order, so results do not depend on
// scheduling).  K is never split across workgroups: a device-scope fence per workgroup costs far more on this
// part (it empties the XCD's L2 under every other workgroup) than the idle CUs of a small grid do.
//
// Arithmetic is that of fp8_gemm_kernel (dlblas/kernels/fp8_gemm.py:49-60): one scale FMA per K block.
#pragma once

#include "fp8_gemm_common.h"

namespace dlb {

template <int MF_, int WAVES_, int UNROLL_, int NFS_>
struct SkinnyCfg {
  static constexpr int MF = MF_;          // 16-row activation fragments (M <= 16 * MF)
  static constexpr int WAVES = WAVES_;    // waves per workgroup, each taking every WAVES-th K block
  static constexpr int UNROLL = UNROLL_;  // K blocks whose loads are issued before the first MFMA
  static constexpr int NFS = NFS_;        // 16-row weight fragments per workgroup
  static constexpr int NT = WAVES * 64;
  static constexpr int BN = 16 * NFS;
  static constexpr int RED_BYTES = WAVES * MF * NFS * 64 * 16;
  static constexpr int STAGING_BYTES = WAVES * UNROLL * (NFS + MF) * 2048;
  // the reduction buffer reuses the staging areas once every wave is through with its K blocks
  static constexpr int DMA_LDS_BYTES = STAGING_BYTES > RED_BYTES ? STAGING_BYTES : RED_BYTES;
};

// 32 operand bytes of one lane for K block `kb`: bytes [16 q, 16 q + 16) and [64 + 16 q, 64 + 16 q + 16) of the
// block.  Any assignment of K bytes to lanes is valid as long as both MFMA operands use the same one; this
// one makes each of the two load instructions of a wave cover 64 contiguous bytes per row.
// KTAIL: K is not a multiple of 128, bytes at or past K read as zero (predicated loads).  Without it the loads
// are unconditional, which keeps the whole load phase one straight-line block.
template <bool KTAIL, bool STREAM>
__device__ __forceinline__ v8i skinny_load_frag(const uint8_t* row, int kb, int q, int K) {
  const int k_lo = kb * kScaleBlock + q * 16;
  const int k_hi = k_lo + 64;
  v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
  const v4i* p_lo = reinterpret_cast<const v4i*>(row + k_lo);
  const v4i* p_hi = reinterpret_cast<const v4i*>(row + k_hi);
  if (!KTAIL || k_lo < K) lo = STREAM ? __builtin_nontemporal_load(p_lo) : *p_lo;
  if (!KTAIL || k_hi < K) hi = STREAM ? __builtin_nontemporal_load(p_hi) : *p_hi;
  return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

template <class Cfg, bool KTAIL>
__global__ void __launch_bounds__(Cfg::NT) fp8_gemm_skinny_kernel(const Args p) {
  constexpr int MF = Cfg::MF, WAVES = Cfg::WAVES, U = Cfg::UNROLL, NFS = Cfg::NFS;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  v4f(*red)[MF * NFS][64] = reinterpret_cast<v4f(*)[MF * NFS][64]>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;

  const int n0 = blockIdx.x * Cfg::BN;
  const int nk = p.kblocks;

  const uint8_t* w_row[NFS];
  const float* bs_row[NFS];
#pragma unroll
  for (int ni = 0; ni < NFS; ++ni) {
    w_row[ni] = p.b + static_cast<int64_t>(min(n0 + ni * 16 + l16, p.N - 1)) * p.K;
    bs_row[ni] = p.b_s + static_cast<int64_t>(min((n0 + ni * 16) / kScaleBlock, p.nblocks - 1)) * nk;
  }
  const uint8_t* x_row[MF];
  const float* as_row[MF];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi) {
    const int m = min(mi * 16 + l16, p.M - 1);
    x_row[mi] = p.a + static_cast<int64_t>(m) * p.K;
    as_row[mi] = p.a_s + static_cast<int64_t>(m) * p.as_sm;
  }

  v4f acc[MF][NFS];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi)
#pragma unroll
    for (int ni = 0; ni < NFS; ++ni) acc[mi][ni] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int kb = wave; kb < nk; kb += WAVES * U) {
    v8i wf[U][NFS];
    v8i xf[U][MF];
    float sa[U][MF];
    float sb[U][NFS];
    // Weights first: they are the HBM stream; everything else hits L2.  A K block past the end re-reads the
    // last one and enters with scale 0.
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kbu = min(kb + u * WAVES, nk - 1);
#pragma unroll
      for (int ni = 0; ni < NFS; ++ni) wf[u][ni] = skinny_load_frag<KTAIL, true>(w_row[ni], kbu, q, p.K);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool valid = kb + u * WAVES < nk;
      const int kbu = min(kb + u * WAVES, nk - 1);
#pragma unroll
      for (int ni = 0; ni < NFS; ++ni) {
        const float v = bs_row[ni][kbu];
        sb[u][ni] = valid ? v : 0.f;
      }
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        xf[u][mi] = skinny_load_frag<KTAIL, false>(x_row[mi], kbu, q, p.K);
        sa[u][mi] = as_row[mi][static_cast<int64_t>(kbu) * p.as_sk];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NFS; ++ni) {
          const v4f part = mfma_16x16x128_e4m3(wf[u][ni], xf[u][mi], v4f{0.f, 0.f, 0.f, 0.f});
          acc[mi][ni] += part * (sa[u][mi] * sb[u][ni]);
        }
      }
    }
  }

#pragma unroll
  for (int mi = 0; mi < MF; ++mi)
#pragma unroll
    for (int ni = 0; ni < NFS; ++ni) red[wave][mi * NFS + ni][lane] = acc[mi][ni];
  __syncthreads();

  // fragment j of the output is summed (in wave order) and stored by wave j % WAVES
  const int64_t esz = p.out_f32 ? 4 : 2;
  for (int j = wave; j < MF * NFS; j += WAVES) {
    const int mi = j / NFS, ni = j % NFS;
    v4f sum = red[0][j][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][j][lane];
    const int m = mi * 16 + l16;
    const int n = n0 + ni * 16 + q * 4;
    if (m >= p.M) continue;
    char* c_row = static_cast<char*>(p.c) + static_cast<int64_t>(m) * p.N * esz;
    if (p.out_f32)
      store_row4<true>(c_row, n, sum, p.N - n, p.vec_store);
    else
      store_row4<false>(c_row, n, sum, p.N - n, p.vec_store);
  }
}


// ---------------------------------------------------------------------------------------------------------------
// Same computation with full-cache-line global accesses: every wave moves the 16 x 128-byte blocks of its K blocks
// (weights AND activations) into a wave-private LDS area with the DMA path, 8 rows x 128 bytes per instruction, and
// reads its MFMA operands back with ds_read_b128.  The register-load kernel above touches every line with two
// half-line requests of 16 rows each; measured on MI355X that costs 1.3 us of a 7 us launch for the weights and
// 2 us for the activations.  No barrier is involved: a wave only reads what it moved itself.  K % 128 == 0 only
// (the DMA cannot zero-fill a ragged last block).
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ int skinny_swizzle(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// cache policy of the weight DMA: every weight byte is read by exactly one workgroup, so the loads carry the
// non-temporal bit (1 - 3 % on the decode shapes; the activation rows, which every workgroup reads, do not)
constexpr int kWeightsOnce = 2;

template <class Cfg>
__global__ void __launch_bounds__(Cfg::NT) fp8_gemm_skinny_dma_kernel(const Args p) {
  constexpr int MF = Cfg::MF, WAVES = Cfg::WAVES, U = Cfg::UNROLL, NFS = Cfg::NFS;
  constexpr int FRAGS = NFS + MF;                 // 2 KB blocks per K block: weights first, then activations
  constexpr int WAVE_BYTES = U * FRAGS * 2048;    // staging area of one wave
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  v4f(*red)[MF * NFS][64] = reinterpret_cast<v4f(*)[MF * NFS][64]>(smem);  // over the staging areas, behind a barrier

  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* global_ptr_t;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;
  const int q = lane >> 4;
  // the workgroup owns columns [n0, n0 + cols): p.sk_bn of them (a multiple of 4, at most 16 NFS, chosen on the
  // host so that the workgroups cover the CUs evenly), fewer at the end of N; fragment rows past them re-read the
  // last owned row and their results are dropped
  const int n0 = blockIdx.x * p.sk_bn;
  const int cols = min(p.sk_bn, p.N - n0);
  const int nk = p.kblocks;
  uint8_t* stage = smem + wave * WAVE_BYTES;
  // Workgroup b starts its walk over K at block b (mod nk): at any moment the workgroups of the chip then ask for
  // different K blocks of the activation rows instead of all for the same few cache lines (9 % at M <= 32,
  // 7168 x 2048; with 64 and more rows the spread-out walk costs L2 hits instead and is left out).  The order of a
  // wave's partial sums changes with b, the result stays a fixed function of the inputs.
  const int rot = MF <= 2 ? static_cast<int>(blockIdx.x % static_cast<unsigned>(nk)) : 0;

  // DMA source offsets: instruction j (0 / 1) of a block fills rows 8 j .. 8 j + 7; lane i fills physical chunk
  // (i & 7) of row 8 j + (i >> 3), which holds logical chunk (i & 7) ^ swizzle(row)
  uint32_t w_off[NFS][2], x_off[MF][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = 8 * j + (lane >> 3);
    const uint32_t chunk = static_cast<uint32_t>(((lane & 7) ^ skinny_swizzle(row)) * 16);
#pragma unroll
    for (int ni = 0; ni < NFS; ++ni)
      w_off[ni][j] = static_cast<uint32_t>(min(ni * 16 + row, cols - 1)) * static_cast<uint32_t>(p.K) + chunk;
#pragma unroll
    for (int mi = 0; mi < MF; ++mi)
      x_off[mi][j] = static_cast<uint32_t>(min(mi * 16 + row, p.M - 1)) * static_cast<uint32_t>(p.K) + chunk;
  }
  const uint8_t* w_base = p.b + static_cast<int64_t>(n0) * p.K;
  // operand read offsets: lane (row = lane & 15, q) reads logical chunks 2 q and 2 q + 1 of its row
  const int sw = skinny_swizzle(l16);
  const int rd0 = l16 * 128 + (((2 * q) ^ sw) << 4);
  const int rd1 = l16 * 128 + (((2 * q + 1) ^ sw) << 4);

  // weight scales per lane: n0 is any multiple of 4, so a fragment can straddle two 128-column scale blocks, the four
  // columns of a lane (n0 + 16 ni + 4 q ..) cannot
  const float* bs_row[NFS];
#pragma unroll
  for (int ni = 0; ni < NFS; ++ni)
    bs_row[ni] = p.b_s + static_cast<int64_t>(min((n0 + ni * 16 + q * 4) / kScaleBlock, p.nblocks - 1)) * nk;
  const float* as_row[MF];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi) as_row[mi] = p.a_s + static_cast<int64_t>(min(mi * 16 + l16, p.M - 1)) * p.as_sm;

  v4f acc[MF][NFS];
#pragma unroll
  for (int mi = 0; mi < MF; ++mi)
#pragma unroll
    for (int ni = 0; ni < NFS; ++ni) acc[mi][ni] = v4f{0.f, 0.f, 0.f, 0.f};

  // One block in flight per wave (U == 1): the activation scales of FOUR consecutive blocks of the wave are fetched by
  // one load per fragment - lane group q takes the block q rounds ahead - and handed to all lanes with a lane
  // permute when their block comes up.  The four addresses of a row usually share a cache line (row-major a_s), so a
  // wave asks for a quarter of the scale lines it would ask for block by block.
  float sa_ahead[MF];
  int it = 0;
  for (int kb = wave; kb < nk; kb += WAVES * U, ++it) {
    float sa[U][MF], sb[U][NFS];
    // weights first: they are the HBM stream.  A K block past the end re-reads the last one with scale 0.
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int kbu = min(kb + u * WAVES, nk - 1) + rot;
      kbu = kbu >= nk ? kbu - nk : kbu;
      const uint8_t* wk = w_base + static_cast<int64_t>(kbu) * kScaleBlock;
#pragma unroll
      for (int ni = 0; ni < NFS; ++ni)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(wk + w_off[ni][j]),
                                           (lds_ptr_t)(stage + (u * FRAGS + ni) * 2048 + j * 1024), 16, 0, kWeightsOnce);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool valid = kb + u * WAVES < nk;
      int kbu = min(kb + u * WAVES, nk - 1) + rot;
      kbu = kbu >= nk ? kbu - nk : kbu;
      const uint8_t* xk = p.a + static_cast<int64_t>(kbu) * kScaleBlock;
#pragma unroll
      for (int mi = 0; mi < MF; ++mi)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(xk + x_off[mi][j]),
                                           (lds_ptr_t)(stage + (u * FRAGS + NFS + mi) * 2048 + j * 1024), 16, 0, 0);
#pragma unroll
      for (int ni = 0; ni < NFS; ++ni) {
        const float v = bs_row[ni][kbu];
        sb[u][ni] = valid ? v : 0.f;
      }
      if constexpr (U > 1) {
#pragma unroll
        for (int mi = 0; mi < MF; ++mi) sa[u][mi] = as_row[mi][static_cast<int64_t>(kbu) * p.as_sk];
      }
    }
    if constexpr (U == 1) {
      if ((it & 3) == 0) {
        int kq = min(kb + q * WAVES, nk - 1) + rot;
        kq = kq >= nk ? kq - nk : kq;
#pragma unroll
        for (int mi = 0; mi < MF; ++mi) sa_ahead[mi] = as_row[mi][static_cast<int64_t>(kq) * p.as_sk];
      }
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) sa[0][mi] = __shfl(sa_ahead[mi], ((it & 3) << 4) | l16);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): this wave's DMA groups have landed in its LDS area
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v8i wf[NFS], xf[MF];
#pragma unroll
      for (int f = 0; f < FRAGS; ++f) {
        const uint8_t* blk = stage + (u * FRAGS + f) * 2048;
        const v4i lo = *reinterpret_cast<const v4i*>(blk + rd0);
        const v4i hi = *reinterpret_cast<const v4i*>(blk + rd1);
        const v8i v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        if (f < NFS)
          wf[f] = v;
        else
          xf[f - NFS] = v;
      }
#pragma unroll
      for (int mi = 0; mi < MF; ++mi)
#pragma unroll
        for (int ni = 0; ni < NFS; ++ni) {
          const v4f part = mfma_16x16x128_e4m3(wf[ni], xf[mi], v4f{0.f, 0.f, 0.f, 0.f});
          acc[mi][ni] += part * (sa[u][mi] * sb[u][ni]);
        }
    }
    // the next round of DMA overwrites the staging area: its reads above have returned (their values were used)
  }

  __syncthreads();  // every wave has read its last staged block: the staging areas become the reduction buffer
#pragma unroll
  for (int mi = 0; mi < MF; ++mi)
#pragma unroll
    for (int ni = 0; ni < NFS; ++ni) red[wave][mi * NFS + ni][lane] = acc[mi][ni];
  __syncthreads();

  const int64_t esz = p.out_f32 ? 4 : 2;
  for (int j = wave; j < MF * NFS; j += WAVES) {
    const int mi = j / NFS, ni = j % NFS;
    v4f sum = red[0][j][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][j][lane];
    const int m = mi * 16 + l16;
    const int n = n0 + ni * 16 + q * 4;
    if (m >= p.M || n >= n0 + cols) continue;
    char* c_row = static_cast<char*>(p.c) + static_cast<int64_t>(m) * p.N * esz;
    if (p.out_f32)
      store_row4<true>(c_row, n, sum, n0 + cols - n, p.vec_store);
    else
      store_row4<false>(c_row, n, sum, n0 + cols - n, p.vec_store);
  }
}

}  // namespace dlb
