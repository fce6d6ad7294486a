// Compute-bound FP8 block-scaled GEMM for gfx950: 32x32x64 e4m3 MFMA, tiles streamed HBM -> LDS by the DMA
// path of the memory pipeline (global_load_lds_dwordx4, no VGPR staging), multi-stage LDS ring, one barrier
// per 128-wide K step, block scales applied with one FMA per accumulator element and K step.
//
// Workgroup = WGM x WGN waves, one wave per SIMD; a wave owns MF x NF fragments of 32 x 32 outputs.
// MFMA operand roles: "A" = 32 rows of the weight tile (n), "B" = 32 rows of the activation tile (m), so a lane's
// 16 accumulator components of a fragment are 4 groups of 4 consecutive n for ONE m (= lane & 31): the activation
// scale is one value per lane and fragment row block, and every lane stores 4 contiguous outputs at a time.
//
// Arithmetic: fp8_gemm_kernel of the reference (dlblas/kernels/fp8_gemm.py:49-60).  Requires K % 128 == 0.
#pragma once

#include <type_traits>

#include "fp8_gemm_common.h"
#include "fp8_gemm_tiled.h"  // xcd_remap

namespace dlb {

// D = A_op * B_op^T, A_op / B_op [32 x 64] e4m3: lane l supplies row (l & 31), 32 K-bytes selected by (l >> 5).
// Lane l receives D[8 * (t / 4) + 4 * (l >> 5) + (t % 4)][l & 31] in component t.
__device__ __forceinline__ v16f mfma_32x32x64_e4m3(v8i a_op, v8i b_op, v16f c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_op, b_op, c, 0, 0, 0, 0, 0, 0);
}

// XOR pattern of the 16-byte chunk index inside a 128-byte LDS row: distinct within any 8 consecutive rows, and
// rows r and r + 8 that share a pattern differ in row parity, i.e. in the 128-byte half of a 256-byte bank line.
__device__ __forceinline__ int chunk_swizzle(int row) { return (row & 7) ^ ((row >> 3) & 1); }

__device__ __forceinline__ int lds_off32(int row, int chunk) {
  return row * kScaleBlock + ((chunk ^ chunk_swizzle(row)) << 4);
}

// A lane reads four 16-byte chunks of "its" row (lane & 31) of every 32-row fragment: logical chunks 2 h, 2 h + 1
// (K half 0) and 4 + 2 h, 5 + 2 h (K half 1), h = lane >> 5.  Fragments start at multiples of 32 rows, which leaves
// the swizzle untouched, so these four byte offsets are the same for every fragment of every tile.
struct LaneChunks {
  int off[4];
};

__device__ __forceinline__ LaneChunks make_lane_chunks(int l32, int h) {
  LaneChunks lc;
#pragma unroll
  for (int i = 0; i < 4; ++i) lc.off[i] = lds_off32(l32, (i >> 1) * 4 + 2 * h + (i & 1));
  return lc;
}

// 8 VGPRs = the 32 operand bytes of one lane for the fragment whose first row starts `frag_bytes` into the LDS
// ring (wave-uniform) and K half `kk` of the 128-byte step.
__device__ __forceinline__ v8i lds_read_frag32(const uint8_t* ring, int frag_bytes, const LaneChunks& lc, int kk) {
  const v4i lo = *reinterpret_cast<const v4i*>(ring + frag_bytes + lc.off[2 * kk]);
  const v4i hi = *reinterpret_cast<const v4i*>(ring + frag_bytes + lc.off[2 * kk + 1]);
  return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

// Cache policy operand of the DMA instruction: kDmaStream sets the non-temporal bit.  It is for bytes that few
// workgroups ask for: a chip-wide stream of 256-row panels from HBM runs at 7.1 TB/s with it and 6.1 TB/s without
// (the lines are not kept in the L2 ahead of others), while operands that an XCD's workgroups share through the L2
// lose by it (dense 4096 x 7168 x 18432: 3 % slower with it on the weights, 15 % on both operands).
constexpr int kDmaKeep = 0, kDmaStream = 2;

// One wave-wide DMA: lane i moves 16 bytes from (base + voff) to lds_dst + 16 i.
template <int POLICY = kDmaKeep>
__device__ __forceinline__ void dma_16(const uint8_t* base, uint32_t voff, uint8_t* lds_dst) {
  __builtin_amdgcn_global_load_lds((global_ptr_t)(base + voff), (lds_ptr_t)lds_dst, 16, 0, POLICY);
}
// lane i moves 4 bytes from (base + voff) to lds_dst + 4 i.
__device__ __forceinline__ void dma_4(const uint8_t* base, uint32_t voff, uint8_t* lds_dst) {
  __builtin_amdgcn_global_load_lds((global_ptr_t)(base + voff), (lds_ptr_t)lds_dst, 4, 0, 0);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt with only vmcnt constrained: vmcnt = simm16[3:0] | simm16[15:14] << 4, expcnt [6:4], lgkmcnt [11:8]
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (((N >> 4) & 0x3) << 14) | (0x7 << 4) | (0xF << 8));
}

// Workgroup barrier that orders LDS traffic only: every wave's LDS reads have returned (lgkmcnt) before it
// arrives.  Unlike __syncthreads() it does not drain the vector-memory counter, so DMA groups that were issued
// for later stages stay in flight across it; the caller waits for the group it needs with wait_vmcnt first.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Four floats to / from memory that another workgroup of the same launch reads / wrote: device-scope accesses
// (write-through, and read past the caches that are not coherent between the XCDs), 8 bytes each, relaxed.
__device__ __forceinline__ void coherent_store16(float* dst, v4f v) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  uint64_t* d = reinterpret_cast<uint64_t*>(dst);
  __hip_atomic_store(d, __builtin_bit_cast(uint64_t, v2f{v.x, v.y}), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(d + 1, __builtin_bit_cast(uint64_t, v2f{v.z, v.w}), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ v4f coherent_load16(const float* src) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  const uint64_t* s = reinterpret_cast<const uint64_t*>(src);
  const v2f lo = __builtin_bit_cast(v2f, __hip_atomic_load(s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  const v2f hi = __builtin_bit_cast(v2f, __hip_atomic_load(s + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  return v4f{lo.x, lo.y, hi.x, hi.y};
}

// PARTS_: 2 = the scale FMAs of a fragment run under the MFMAs of the NEXT fragment of the same wave (two partial
// accumulators); 1 = they follow their own MFMAs and overlap with the other wave of the SIMD instead (16 fewer VGPRs).
// PREFETCH_: true (one wave per SIMD, 512 registers) = every fragment of the NEXT K step is read into a second
// register set while the current step computes, so no MFMA of a step waits for LDS.
// SCTAB_: true = the activation scales of a tile's rows for ALL K blocks of the workgroup's K range (at most
// SCTAB_KB) are fetched once per tile into a table behind the ring, lanes along K: a row-major a_s then costs one
// cache-line request per row and tile instead of one per row and K step, and needs no re-layout pass in front.
template <int WGM_, int WGN_, int MF_, int NF_, int STAGES_, int PARTS_ = 2, bool PREFETCH_ = false, bool SCTAB_ = false, int SCTAB_KB_ = 32>
struct PipeCfg {
  static constexpr int WGM = WGM_, WGN = WGN_, MF = MF_, NF = NF_, STAGES = STAGES_, PARTS = PARTS_;
  static constexpr bool PREFETCH = PREFETCH_;
  static constexpr bool SCTAB = SCTAB_;
  static constexpr bool UNIFORM_W = (128 % (NF_ * 32)) == 0;
  static constexpr int WAVES = WGM * WGN;
  static constexpr int NT = WAVES * 64;
  static constexpr int BM = WGM * MF * 32;
  static constexpr int BN = WGN * NF * 32;
  static constexpr int A_INST = BM / 8 / WAVES;  // 16-byte DMA instructions per wave and stage for the A tile
  static constexpr int B_INST = BN / 8 / WAVES;
  static constexpr int S_INST = SCTAB ? 0 : (BM + NT - 1) / NT;  // 4-byte DMA instructions per wave for the a_s slice
  static constexpr int A_BYTES = BM * kScaleBlock;
  static constexpr int B_BYTES = BN * kScaleBlock;
  static constexpr int S_BYTES = S_INST * NT * 4;  // activation scales of the tile rows for one K block
  static constexpr int W_BYTES = NT * 4;           // weight scale of each wave's n block, one copy per lane
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + S_BYTES + W_BYTES;
  static constexpr int SCTAB_KB = SCTAB_KB_;       // K blocks per workgroup the table holds
  static constexpr int SCTAB_OFF = STAGES * STAGE_BYTES;
  static constexpr int SCTAB_BYTES = SCTAB ? BM * (SCTAB_KB + 1) * 4 : 0;  // rows of an odd pitch (bank spread), at most SCTAB_KB + 1 floats
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES + SCTAB_BYTES;
  static constexpr int LOADS_PER_STAGE = A_INST + B_INST + S_INST + 1;  // vmcnt units per wave and stage
  static_assert(BM % (8 * WAVES) == 0 && BN % (8 * WAVES) == 0, "tile rows must divide over the DMA instructions");
  static_assert(NF <= 4, "weight scales are fetched for at most four fragments per wave");
  static_assert(LOADS_PER_STAGE * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
};

// Re-lays activation scales from [groups][rows][kblocks] (any strides) to [groups][kblocks][rows_pad], rows
// contiguous, so that the GEMM's per-K-step fetch of one scale per tile row is a handful of full cache lines
// instead of one line per row.  32 x 32 tiles through LDS keep both sides coalesced.  (The reference does the same
// re-layout before its grouped GEMMs, dlblas/kernels/quant_dequant.py:42-83.)
// rows_map (or NULL): row r of the re-laid copy is row rows_map[r] of src.  (bx, by, g): the block's 32 x 32 tile and group.
__device__ __forceinline__ void scale_transpose_block(const float* src, float* dst, int rows, int kblocks, int rows_pad,
                                                      int64_t s_g, int64_t s_m, int64_t s_k, const int32_t* rows_map, int bx,
                                                      int by, int g) {
  __shared__ float tile[32][33];
  const int r0 = bx * 32, k0 = by * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const float* in = src + static_cast<int64_t>(g) * s_g;
  float* out = dst + static_cast<int64_t>(g) * kblocks * rows_pad;
#pragma unroll
  for (int i = 0; i < 32; i += 8) {
    const int r = r0 + ty + i, k = k0 + tx;
    const bool live = r < rows && k < kblocks;
    const int64_t sr = (live && rows_map != nullptr) ? max(rows_map[r], 0) : r;
    tile[ty + i][tx] = live ? in[sr * s_m + static_cast<int64_t>(k) * s_k] : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 32; i += 8) {
    const int k = k0 + ty + i, r = r0 + tx;
    if (k < kblocks && r < rows_pad) out[static_cast<int64_t>(k) * rows_pad + r] = tile[tx][ty + i];
  }
}

__global__ void __launch_bounds__(256) fp8_scale_transpose_kernel(const float* src, float* dst, int rows, int kblocks,
                                                                  int rows_pad, int64_t s_g, int64_t s_m, int64_t s_k,
                                                                  const int32_t* rows_map) {
  scale_transpose_block(src, dst, rows, kblocks, rows_pad, s_g, s_m, s_k, rows_map, blockIdx.x, blockIdx.y, blockIdx.z);
}

constexpr int kTileListHeader = 3;  // tile counts in front of the three tile lists of an expert-contiguous launch

// Work of one workgroup: tiles vb_first, vb_first + gridDim.x, ... of a region that is tiles_m x tiles_n tiles of
// BM x BN and starts at column n_base of the output.
template <class Cfg, int MODE>
__device__ __forceinline__ void pipelined_body(const Args& p, uint8_t* smem, int vb_first, int tiles_m, int tiles_n,
                                               int n_base) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, MF = Cfg::MF, NF = Cfg::NF, WAVES = Cfg::WAVES, STAGES = Cfg::STAGES;
  // One weight scale per wave and K step when the wave's n span cannot straddle a 128-column scale block,
  // otherwise one per 32-column fragment.
  constexpr bool kUniformW = Cfg::UNIFORM_W;
  constexpr int NS = kUniformW ? 1 : NF;
  constexpr bool kList = MODE == kContigList || MODE == kContigListAct;
  // Fused activation: a tile's 256 weight rows are 128 gate rows and the 128 up rows of the same output columns, so
  // that the epilogue has silu(gate) * up of 128 columns - one quantisation group - for every row of the tile.
  constexpr bool kAct = MODE == kContigListAct || MODE == kMaskedAct;
  constexpr bool kMaskedLike = MODE == kMasked || MODE == kMaskedAct;
  // Grouped modes: an expert's weight tile is read by the one to three row tiles of that expert, not by a column of
  // the grid: streamed (2 - 7 % faster from 128 to 768 rows per expert at 32 x 4096 x 7168).
  constexpr int kWeightPolicy = MODE == kDense ? kDmaKeep : kDmaStream;
  static_assert(!kAct || (BN == 256 && kUniformW), "the fused activation pairs 128 gate columns with 128 up columns");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;
  const int wm0 = (wave / Cfg::WGN) * (MF * 32);
  const int wn0 = (wave % Cfg::WGN) * (NF * 32);
  const LaneChunks lc = make_lane_chunks(l32, h);

  const int tiles = tiles_m * tiles_n;
  int walk_g = 0;
  int walk_base = 0;

  for (int vb = vb_first;; vb += gridDim.x) {
    int g = 0, mt = 0, nt, m_end, m_first = -1, split = 0, tile_lin = 0;
    if (kMaskedLike) {
      // The tile count is only known on the device, so the grid is persistent; the hardware deals consecutive
      // workgroups to the 8 XCDs in turn.  Of every 32 consecutive tiles each XCD takes 4 consecutive ones: the row
      // tiles of an expert, which are adjacent in the order and read the same weight tile, meet in one L2, and the
      // last, partial round still spreads over all XCDs (the grid is a multiple of 32).
      const int grid = static_cast<int>(gridDim.x);
      const int w = vb % grid;
      const int tile_id = vb - w + (w / 32) * 32 + (w % 8) * 4 + (w / 8) % 4;
      int mtiles = 0;
      while (walk_g < p.G) {
        const int valid = min(max(p.gidx[walk_g], 0), p.M);
        mtiles = (valid + BM - 1) / BM;
        const int cnt = mtiles * tiles_n;
        if (tile_id < walk_base + cnt) break;
        walk_base += cnt;
        ++walk_g;
      }
      if (walk_g >= p.G) break;
      g = walk_g;
      const int local = tile_id - walk_base;
      mt = local % mtiles;
      nt = local / mtiles;
      m_end = min(max(p.gidx[g], 0), p.M);
    } else if (kList) {
      // tiles of this height come from the list the pre-pass built: entry = first 128-row block of the tile.  The
      // column tiles of one row block are adjacent in the order, so they share the activation tile in L2.
      static_assert(BM == 256 || BM == 192 || BM == 128, "tile heights of the three lists");
      constexpr int kWhich = BM == 256 ? 0 : (BM == 192 ? 1 : 2);
      const int cnt = p.tlist[kWhich];
      const int total = cnt * tiles_n;
      if (vb >= total) break;
      const int t = xcd_remap(vb, total);
      int li;
      if (BM == 192) {
        // the two tiles of a pair side by side for every column tile: neighbours in the order run on one XCD at the same time
        const int pair = t / (2 * tiles_n), r = t - pair * 2 * tiles_n;
        nt = r >> 1;
        li = 2 * pair + (r & 1);
      } else {
        li = t / tiles_n;
        nt = t - li * tiles_n;
      }
      m_first = p.tlist[kTileListHeader + kWhich * p.tlist_cap + li] * 64;
      g = p.gidx[m_first];
      m_end = min(p.M, m_first + BM);
    } else {
      // dense split-K: the K range is cut into p.splitk slices of p.kb_per_split blocks, every (tile, slice) pair is a
      // unit of work, slices of one tile far apart in the order
      const int units = MODE == kDense ? tiles * p.splitk : tiles;
      if (vb >= units) break;
      const int id = xcd_remap(vb, units);
      split = MODE == kDense ? id / tiles : 0;
      const int t = id - split * tiles;
      tile_lin = t;
      const int width = p.group_m * tiles_n;
      const int grp = t / width;
      const int first_m = grp * p.group_m;
      const int gsz = min(tiles_m - first_m, p.group_m);
      const int in_grp = t - grp * width;
      mt = first_m + in_grp % gsz;
      nt = in_grp / gsz;
      m_end = p.M;
      if (MODE == kContiguous) {
        g = p.gidx[mt * BM];
        if (g < 0 || g >= p.G) continue;
      }
    }
    g = __builtin_amdgcn_readfirstlane(g);
    const int m0 = __builtin_amdgcn_readfirstlane(kList ? m_first : mt * BM);
    // fused activation: n0 is the first OUTPUT column of the tile; weight row of tile column c: see w_row below
    const int n0 = __builtin_amdgcn_readfirstlane(kAct ? nt * (BN / 2) : n_base + nt * BN);
    auto w_row = [&](int c) { return c < BN / 2 ? n0 + c : p.act_cols + n0 + c - BN / 2; };

    const int64_t esz = p.out_f32 ? 4 : 2;
    const bool sliced = MODE == kDense && p.splitk > 1;
    const int kb_first = sliced ? split * p.kb_per_split : 0;  // the host leaves no slice empty
    const int nk = sliced ? min(p.kblocks, kb_first + p.kb_per_split) - kb_first : p.kblocks;  // K blocks of this unit
    // activation rows named by a table (the fused gate/up kernel reading the tokens where they lie, instead of a copy
    // sorted by expert): per-lane offsets then count from the first row of the matrix
    const bool a_indirect = MODE == kContigListAct && p.a_rows != nullptr;
    const uint8_t* a_tile = p.a + static_cast<int64_t>(a_indirect ? 0 : m0) * p.K + static_cast<int64_t>(kb_first) * kScaleBlock;
    const float* as_tile = p.a_s + static_cast<int64_t>(m0) * p.as_sm + static_cast<int64_t>(kb_first) * p.as_sk;
    char* c_base = static_cast<char*>(p.c);
    if (kMaskedLike) {
      a_tile += static_cast<int64_t>(g) * p.a_gs;
      as_tile += static_cast<int64_t>(g) * p.as_gs;
      c_base += static_cast<int64_t>(g) * p.c_gs * esz;
    }
    const uint8_t* b_tile = p.b + static_cast<int64_t>(g) * p.b_gs + static_cast<int64_t>(kAct ? 0 : n0) * p.K +
                            static_cast<int64_t>(kb_first) * kScaleBlock;
    // weight scales: lane i of the wave fetches the scale of the wave's fragment (i & 3) (fragment 0 beyond NF)
    const float* bs_g = p.b_s + static_cast<int64_t>(g) * p.bs_gs + kb_first;
    const int bs_frag = (lane & 3) < NF ? (lane & 3) : 0;
    const uint32_t bs_off =
        static_cast<uint32_t>(min((kAct ? w_row(wn0 + 32 * bs_frag) : n0 + wn0 + 32 * bs_frag) / kScaleBlock, p.nblocks - 1)) *
        static_cast<uint32_t>(p.kblocks) * 4u;

    // DMA addressing.  Instruction j of this wave fills LDS rows 8 (j WAVES + wave) .. + 7; lane i fills physical
    // chunk (i & 7) of row (i >> 3), which holds logical chunk (i & 7) ^ swizzle(row).  WAVES is even, so the
    // swizzle does not depend on j and one per-lane chunk offset serves every instruction; the row part is
    // recomputed per instruction (two VALU ops) instead of being kept in registers.  Rows past the valid range
    // re-read the last valid row.
    static_assert(WAVES % 2 == 0, "chunk swizzle must not depend on the DMA instruction index");
    const int a_last = m_end - 1 - m0;
    const int b_last = p.N - 1 - n0;
    const int dma_row = 8 * wave + (lane >> 3);
    const uint32_t dma_chunk = static_cast<uint32_t>(((lane & 7) ^ chunk_swizzle(dma_row)) * 16);
    const uint32_t uK = static_cast<uint32_t>(p.K);

    // Per-lane source offsets of every DMA instruction of a stage, computed once per tile: the K loop then issues
    // its DMA group without any vector ALU work (32-bit multiplies are quarter rate and, issued right behind the
    // barrier by every wave at once, kept the matrix pipe waiting).
    uint32_t a_off[Cfg::A_INST], b_off[Cfg::B_INST], s_off[Cfg::S_INST > 0 ? Cfg::S_INST : 1];
#pragma unroll
    for (int j = 0; j < Cfg::A_INST; ++j) {
      const int r = min(dma_row + 8 * j * WAVES, a_last);
      a_off[j] = static_cast<uint32_t>(a_indirect ? max(p.a_rows[m0 + r], 0) : r) * uK + dma_chunk;
    }
#pragma unroll
    for (int j = 0; j < Cfg::B_INST; ++j)
      b_off[j] = static_cast<uint32_t>(kAct ? w_row(dma_row + 8 * j * WAVES) : min(dma_row + 8 * j * WAVES, b_last)) * uK + dma_chunk;
#pragma unroll
    for (int j = 0; j < Cfg::S_INST; ++j)
      s_off[j] = static_cast<uint32_t>(min((j * WAVES + wave) * 64 + lane, a_last)) * static_cast<uint32_t>(p.as_sm) * 4u;

    auto issue_stage = [&](int kb, int stage) {
      uint8_t* sbase = smem + stage * Cfg::STAGE_BYTES;
      const uint8_t* ag = a_tile + static_cast<int64_t>(kb) * kScaleBlock;
      const uint8_t* bg = b_tile + static_cast<int64_t>(kb) * kScaleBlock;
      const uint8_t* sg = reinterpret_cast<const uint8_t*>(as_tile + static_cast<int64_t>(kb) * p.as_sk);
      // the empty asm keeps each offset a 32-bit register here, so that the load uses the scalar-base + 32-bit
      // vector-offset form instead of a 64-bit address built outside the loop (two registers per instruction)
#pragma unroll
      for (int j = 0; j < Cfg::A_INST; ++j) {
        uint32_t o = a_off[j];
        asm volatile("" : "+v"(o));
        dma_16(ag, o, sbase + (j * WAVES + wave) * 1024);
      }
#pragma unroll
      for (int j = 0; j < Cfg::B_INST; ++j) {
        uint32_t o = b_off[j];
        asm volatile("" : "+v"(o));
        dma_16<kWeightPolicy>(bg, o, sbase + Cfg::A_BYTES + (j * WAVES + wave) * 1024);
      }
#pragma unroll
      for (int j = 0; j < Cfg::S_INST; ++j) {
        uint32_t o = s_off[j];
        asm volatile("" : "+v"(o));
        dma_4(sg, o, sbase + Cfg::A_BYTES + Cfg::B_BYTES + (j * WAVES + wave) * 256);
      }
      // weight scales of the wave's fragments at this K block, one per lane slot
      dma_4(reinterpret_cast<const uint8_t*>(bs_g + kb), bs_off,
            sbase + Cfg::A_BYTES + Cfg::B_BYTES + Cfg::S_BYTES + wave * 256);
    };
    // The same group, one instruction at a time (i = 0 .. LOADS_PER_STAGE - 1, compile-time): the in-place K loop
    // spreads a stage's DMA over several tile slots instead of issuing it in one burst behind the barrier, where
    // the eight waves' 80 instructions queue up in front of the texture path and keep the waves from their MFMAs.
    auto issue_one = [&](auto idx, int kb, int stage) __attribute__((always_inline)) {
      constexpr int i = decltype(idx)::value;
      uint8_t* sbase = smem + stage * Cfg::STAGE_BYTES;
      if constexpr (i < Cfg::A_INST) {
#ifdef DLB_ABLATE_A
        return;
#endif
        uint32_t o = a_off[i];
        asm volatile("" : "+v"(o));
        dma_16(a_tile + static_cast<int64_t>(kb) * kScaleBlock, o, sbase + (i * WAVES + wave) * 1024);
      } else if constexpr (i < Cfg::A_INST + Cfg::B_INST) {
        constexpr int j = i - Cfg::A_INST;
        uint32_t o = b_off[j];
        asm volatile("" : "+v"(o));
        dma_16<kWeightPolicy>(b_tile + static_cast<int64_t>(kb) * kScaleBlock, o, sbase + Cfg::A_BYTES + (j * WAVES + wave) * 1024);
      } else if constexpr (i < Cfg::A_INST + Cfg::B_INST + Cfg::S_INST) {
        constexpr int j = i - Cfg::A_INST - Cfg::B_INST;
        uint32_t o = s_off[j];
        asm volatile("" : "+v"(o));
        dma_4(reinterpret_cast<const uint8_t*>(as_tile + static_cast<int64_t>(kb) * p.as_sk), o,
              sbase + Cfg::A_BYTES + Cfg::B_BYTES + (j * WAVES + wave) * 256);
      } else {
        dma_4(reinterpret_cast<const uint8_t*>(bs_g + kb), bs_off,
              sbase + Cfg::A_BYTES + Cfg::B_BYTES + Cfg::S_BYTES + wave * 256);
      }
    };

    v16f acc[MF][NF];
#pragma unroll
    for (int mi = 0; mi < MF; ++mi)
#pragma unroll
      for (int ni = 0; ni < NF; ++ni)
#pragma unroll
        for (int t = 0; t < 16; ++t) acc[mi][ni][t] = 0.f;

    // ---- K loop ---------------------------------------------------------------------------------------------
    // One operand's fragments are held in registers for the whole K step ("held": the one with fewer fragments),
    // the other's are streamed past them one fragment at a time.  Tiles are visited streamed-major.  Registers
    // are reloaded in place as soon as the last MFMA that reads them has been issued, and the single barrier of a
    // K step sits before the tiles of the LAST streamed fragment: by then every LDS read of the current stage
    // has returned, so the stage can be handed to the DMA, and the first fragments of the next stage are fetched
    // while those last tiles run on the matrix pipe.  The step body is branch-free (the last steps are peeled
    // through template flags) so that the scheduling fences inside it hold.
    constexpr bool kHoldX = MF <= NF;          // hold activations (x), stream weights (w); else the reverse
    constexpr int H = kHoldX ? MF : NF;        // held fragments
    constexpr int S = kHoldX ? NF : MF;        // streamed fragments
    constexpr int T = H * S;
    constexpr int kFragBytes = 32 * kScaleBlock;
    const int held0 = (kHoldX ? wm0 : Cfg::BM + wn0) * kScaleBlock;      // byte offset of held fragment 0 in a stage
    const int strm0 = (kHoldX ? Cfg::BM + wn0 : wm0) * kScaleBlock;
    constexpr int kScaleOff = Cfg::A_BYTES + Cfg::B_BYTES;
    constexpr int kWScaleOff = kScaleOff + Cfg::S_BYTES;

    __syncthreads();  // the previous tile's readers and DMA groups are done with the ring
    if constexpr (Cfg::SCTAB) {
      // scale table [BM][p.sct_pitch]: entry (r, j) = a_s of tile row r at the workgroup's j-th K block.  One DMA
      // instruction moves 64 consecutive entries, i.e. whole runs of a row's scales; issued ahead of the first stages,
      // so the wait for stage 0 covers them.  The pitch is odd: the 32 rows a wave reads at one K block then lie in 32
      // different banks (with a power-of-two pitch of 32 floats they shared two banks, and every such read held the
      // LDS for 16 turns while the other waves' fragment reads waited: 256 x 7168 x 4096 27.2 -> 24 us).
      const int pitch = p.sct_pitch;
      const float inv_pitch = 1.0f / static_cast<float>(pitch);
      const int n_inst = (BM * pitch + 63) >> 6;
      for (int i = wave; i < n_inst; i += WAVES) {
        const int e = i * 64 + lane;
        const int row = static_cast<int>((static_cast<float>(e) + 0.5f) * inv_pitch);  // e / pitch, exact for e < 2^20
        const uint32_t r = static_cast<uint32_t>(min(row, a_last));
        const uint32_t j = static_cast<uint32_t>(min(e - row * pitch, nk - 1));
        dma_4(reinterpret_cast<const uint8_t*>(as_tile),
              (r * static_cast<uint32_t>(p.as_sm) + j * static_cast<uint32_t>(p.as_sk)) * 4u, smem + Cfg::SCTAB_OFF + i * 256);
      }
    }
    // kExactK: only K blocks that exist are fetched - a tile shorter than the ring, and the last STAGES steps of every
    // tile, issue nothing (wave-uniform branches), so no load is in flight when the tile ends and the next tile starts
    // without waiting for loads nobody reads.  The kernels whose wave tile fills the register file (64 x 128) cannot
    // afford those branches' scalar registers inside the K loop (wave tiles above 64 x 64): they keep every step the same code, fetch the last
    // block again past the end of K into a stage nobody reads, and drain at the end of the tile.
    constexpr bool kExactK = MF * NF <= 4;
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
      if (!kExactK || s < nk) issue_stage(min(s, nk - 1), s);
    if (!kExactK || nk >= STAGES)
      wait_vmcnt<(STAGES - 1) * Cfg::LOADS_PER_STAGE>();  // all but the first stage's group may still be on their way
    else
      wait_vmcnt<0>();
    lds_barrier();

    // first table entry of this lane's rows (scale-table kernels)
    int tab_row[MF];
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) tab_row[mi] = Cfg::SCTAB ? (wm0 + mi * 32 + l32) * p.sct_pitch : 0;

    if constexpr (Cfg::PREFETCH) {
      static_assert(kUniformW, "the register-double-buffered path assumes one weight scale per wave");
      // ---- full register double buffering (one wave per SIMD) ------------------------------------------------
      v8i xr[2][MF][2];
      v8i wr[2][NF][2];
      float scb[2][MF];
      float sc_last = 0.f;
      v16f part[2];
#pragma unroll
      for (int u = 0; u < 16; ++u) part[0][u] = part[1][u] = 0.f;
      const int x0 = wm0 * kScaleBlock;
      const int w0 = (Cfg::BM + wn0) * kScaleBlock;
      auto load_scales = [&](int base, int kbl, float (&dst)[MF]) {
        const float sb = *reinterpret_cast<const float*>(smem + base + kWScaleOff + wave * 256);
        if constexpr (Cfg::SCTAB) {
          const float* tab = reinterpret_cast<const float*>(smem + Cfg::SCTAB_OFF);
#pragma unroll
          for (int mi = 0; mi < MF; ++mi) dst[mi] = tab[tab_row[mi] + kbl] * sb;
        } else {
          const float* sS = reinterpret_cast<const float*>(smem + base + kScaleOff);
#pragma unroll
          for (int mi = 0; mi < MF; ++mi) dst[mi] = sS[wm0 + mi * 32 + l32] * sb;
        }
      };
      // half-fragment q of a stage: q < 2 MF -> activation fragment q / 2, K half q % 2; else weight fragment
      constexpr int kHalves = 2 * (MF + NF);
      constexpr int kPerTile = (kHalves + (MF * NF) - 2) / (MF * NF - 1);  // spread over the first T - 1 tiles
      load_scales(0, 0, scb[0]);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        xr[0][mi][0] = lds_read_frag32(smem, x0 + mi * kFragBytes, lc, 0);
        xr[0][mi][1] = lds_read_frag32(smem, x0 + mi * kFragBytes, lc, 1);
      }
#pragma unroll
      for (int ni = 0; ni < NF; ++ni) {
        wr[0][ni][0] = lds_read_frag32(smem, w0 + ni * kFragBytes, lc, 0);
        wr[0][ni][1] = lds_read_frag32(smem, w0 + ni * kFragBytes, lc, 1);
      }

      // Every step is the same code: a step always prefetches "the next stage" into registers (garbage after the
      // last one, never used); whether it hands its stage to the DMA and how many groups it leaves in flight at its
      // barrier are wave-uniform branches on the step's distance from the end of K.
      auto k_step = [&](auto buf_tag, int kb, int stage) __attribute__((always_inline)) {
        constexpr int B = decltype(buf_tag)::value;
        const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
        const int nxt_base = next_stage * Cfg::STAGE_BYTES;
        // every wave holds this stage's fragments in registers and has its share of the next stage in LDS
        // the group of step kb + 1 has landed: behind it at most STAGES - 2 younger groups are out, fewer at the tile's end
        if (kExactK && kb + STAGES > nk)
          wait_vmcnt<0>();
        else
          wait_vmcnt<(STAGES - 2) * Cfg::LOADS_PER_STAGE>();
        lds_barrier();
        if (!kExactK || kb + STAGES < nk) issue_stage(min(kb + STAGES, nk - 1), stage);
#pragma unroll
        for (int t = 0; t < T; ++t) {
          const int mi = t / NF, ni = t % NF;
          __builtin_amdgcn_sched_barrier(0);
          v16f z;
#pragma unroll
          for (int u = 0; u < 16; ++u) z[u] = 0.f;
          z = mfma_32x32x64_e4m3(wr[B][ni][0], xr[B][mi][0], z);
          part[t & 1] = mfma_32x32x64_e4m3(wr[B][ni][1], xr[B][mi][1], z);
          __builtin_amdgcn_sched_barrier(0);
          if (t == 0) load_scales(nxt_base, min(kb + 1, nk - 1), scb[B ^ 1]);
#pragma unroll
          for (int q = t * kPerTile; q < (t + 1) * kPerTile && q < kHalves; ++q) {
            if (q < 2 * MF)
              xr[B ^ 1][q / 2][q % 2] = lds_read_frag32(smem, nxt_base + x0 + (q / 2) * kFragBytes, lc, q % 2);
            else
              wr[B ^ 1][(q - 2 * MF) / 2][q % 2] =
                  lds_read_frag32(smem, nxt_base + w0 + ((q - 2 * MF) / 2) * kFragBytes, lc, q % 2);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (t == 0)
            acc[MF - 1][NF - 1] += part[(T - 1) & 1] * sc_last;  // last tile of the previous K step
          else
            acc[(t - 1) / NF][(t - 1) % NF] += part[(t - 1) & 1] * scb[B][(t - 1) / NF];
        }
        sc_last = scb[B][MF - 1];
      };
      typedef std::integral_constant<int, 0> B0;
      typedef std::integral_constant<int, 1> B1;
      int stage = 0;
      int kb = 0;
      for (; kb + 1 < nk; kb += 2) {
        k_step(B0{}, kb, stage);
        stage = stage + 1 == STAGES ? 0 : stage + 1;
        k_step(B1{}, kb + 1, stage);
        stage = stage + 1 == STAGES ? 0 : stage + 1;
      }
      if (kb < nk) k_step(B0{}, kb, stage);
      acc[MF - 1][NF - 1] += part[(T - 1) & 1] * sc_last;
      if (!kExactK) wait_vmcnt<0>();  // the trailing re-read groups must not land in the next tile's ring
    } else {
    v8i hf[H][2];
    v8i sf[2];
    float sc[MF][NS];
    float sc_last = 0.f;
    v16f part[2];
#pragma unroll
    for (int u = 0; u < 16; ++u) part[0][u] = part[1][u] = 0.f;

    auto load_scales = [&](int base, int kbl, float (&dst)[MF][NS]) {
      float sb[NS];
#pragma unroll
      for (int j = 0; j < NS; ++j) sb[j] = *reinterpret_cast<const float*>(smem + base + kWScaleOff + wave * 256 + j * 4);
      const float* sS = reinterpret_cast<const float*>(smem + base + kScaleOff);
      const float* tab = reinterpret_cast<const float*>(smem + Cfg::SCTAB_OFF);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const float sa = Cfg::SCTAB ? tab[tab_row[mi] + kbl] : sS[wm0 + mi * 32 + l32];
#pragma unroll
        for (int j = 0; j < NS; ++j) dst[mi][j] = sa * sb[j];
      }
    };
    load_scales(0, 0, sc);
#pragma unroll
    for (int hi = 0; hi < H; ++hi) {
      hf[hi][0] = lds_read_frag32(smem, held0 + hi * kFragBytes, lc, 0);
      hf[hi][1] = lds_read_frag32(smem, held0 + hi * kFragBytes, lc, 1);
    }
    sf[0] = lds_read_frag32(smem, strm0, lc, 0);
    sf[1] = lds_read_frag32(smem, strm0, lc, 1);

    // One K step; every step is the same code (see the note in the register-double-buffered path above).
    auto k_step = [&](int kb, int stage) __attribute__((always_inline)) {
      const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
      const int cur_base = stage * Cfg::STAGE_BYTES;
      const int nxt_base = next_stage * Cfg::STAGE_BYTES;
      float sc_next[MF][NS];
      // DMA slots: the group that refills this step's stage starts at the barrier slot kP and is spread over kSlots
      // tile slots, wrapping into the next step (whose slots t < kP therefore finish the PREVIOUS step's group)
      constexpr int kP = (S - 1) * H;
      constexpr int kSlots = T >= 8 ? 5 : (T >= 4 ? 3 : 1);  // measured: 3 to 5 of 8 slots are equally good, 6 and 7 leave the loads too little time
      constexpr int L = Cfg::LOADS_PER_STAGE;
      const int prev_stage = stage == 0 ? STAGES - 1 : stage - 1;
      const int kb_new = kExactK ? kb + STAGES : min(kb + STAGES, nk - 1), kb_prev = kExactK ? kb + STAGES - 1 : min(kb + STAGES - 1, nk - 1);
      const bool do_new = !kExactK || kb_new < nk, do_prev = !kExactK || kb_prev < nk;  // kExactK: K blocks past the end are not fetched
      auto issue_slot = [&](auto qtag, int kbx, int stg) __attribute__((always_inline)) {
        constexpr int q = decltype(qtag)::value;
        constexpr int i0 = q * L / kSlots, i1 = (q + 1) * L / kSlots;
        if constexpr (i0 + 0 < i1) issue_one(std::integral_constant<int, i0 + 0>{}, kbx, stg);
        if constexpr (i0 + 1 < i1) issue_one(std::integral_constant<int, i0 + 1>{}, kbx, stg);
        if constexpr (i0 + 2 < i1) issue_one(std::integral_constant<int, i0 + 2>{}, kbx, stg);
        if constexpr (i0 + 3 < i1) issue_one(std::integral_constant<int, i0 + 3>{}, kbx, stg);
        static_assert(i1 - i0 <= 4, "at most four DMA instructions per slot");
      };
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const int si = t / H, hi = t % H;
        if (si == S - 1 && hi == 0) {
          // every LDS read of this stage has been issued and the barrier waits for their return: hand it over
          // (DLB_ABLATE_*: measurement builds with one part of the K step compiled out - their results are wrong on
          // purpose; what a launch gains by it is what that part costs.  Never defined in the library build.)
#ifndef DLB_ABLATE_VMCNT
          // the group of step kb + 1 has landed: behind it at most STAGES - 2 younger groups are out, fewer at the tile's end
          if (kExactK && kb + STAGES > nk)
            wait_vmcnt<0>();
          else
            wait_vmcnt<(STAGES - 2) * Cfg::LOADS_PER_STAGE>();
#endif
#ifndef DLB_ABLATE_BARRIER
          lds_barrier();
#else
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#endif
        }
#ifndef DLB_ABLATE_DMA
        if (t >= kP) {
          if (t - kP < kSlots && do_new) {
            if (t - kP == 0) issue_slot(std::integral_constant<int, 0>{}, kb_new, stage);
            if (t - kP == 1) issue_slot(std::integral_constant<int, 1>{}, kb_new, stage);
            if (t - kP == 2) issue_slot(std::integral_constant<int, 2>{}, kb_new, stage);
            if (t - kP == 3) issue_slot(std::integral_constant<int, 3>{}, kb_new, stage);
            if (t - kP == 4) issue_slot(std::integral_constant<int, 4>{}, kb_new, stage);
          }
        } else if (t + T - kP < kSlots && do_prev) {
          if (t + T - kP == 1) issue_slot(std::integral_constant<int, 1>{}, kb_prev, prev_stage);
          if (t + T - kP == 2) issue_slot(std::integral_constant<int, 2>{}, kb_prev, prev_stage);
          if (t + T - kP == 3) issue_slot(std::integral_constant<int, 3>{}, kb_prev, prev_stage);
          if (t + T - kP == 4) issue_slot(std::integral_constant<int, 4>{}, kb_prev, prev_stage);
        }
#endif
        // The scheduling fences pin the order MFMA pair -> reloads -> scale FMAs; without them the compiler
        // hoists the reloads above the MFMAs into fresh registers and the kernel spills.
        __builtin_amdgcn_sched_barrier(0);
        v16f z;
#pragma unroll
        for (int u = 0; u < 16; ++u) z[u] = 0.f;
        constexpr int kSlot = Cfg::PARTS == 2 ? 1 : 0;
#ifdef DLB_ABLATE_MFMADEP
        if (kHoldX) {  // the two MFMAs of a tile independent of each other (the first one's product is dropped)
          v16f z2;
#pragma unroll
          for (int u = 0; u < 16; ++u) z2[u] = 0.f;
          z = mfma_32x32x64_e4m3(sf[0], hf[hi][0], z);
          part[t & kSlot] = mfma_32x32x64_e4m3(sf[1], hf[hi][1], z2);
          asm volatile("" ::"v"(z));
        } else
#endif
        if (kHoldX) {
          z = mfma_32x32x64_e4m3(sf[0], hf[hi][0], z);
          part[t & kSlot] = mfma_32x32x64_e4m3(sf[1], hf[hi][1], z);
        } else {
          z = mfma_32x32x64_e4m3(hf[hi][0], sf[0], z);
          part[t & kSlot] = mfma_32x32x64_e4m3(hf[hi][1], sf[1], z);
        }
        __builtin_amdgcn_sched_barrier(0);
        // in-place reloads: the MFMAs above were the last readers of these registers
#ifndef DLB_ABLATE_LDSREAD
        if (hi == H - 1 && si + 1 < S) {
          sf[0] = lds_read_frag32(smem, cur_base + strm0 + (si + 1) * kFragBytes, lc, 0);
          sf[1] = lds_read_frag32(smem, cur_base + strm0 + (si + 1) * kFragBytes, lc, 1);
        }
        if (si == S - 1) {
#ifndef DLB_ABLATE_A
          hf[hi][0] = lds_read_frag32(smem, nxt_base + held0 + hi * kFragBytes, lc, 0);
          hf[hi][1] = lds_read_frag32(smem, nxt_base + held0 + hi * kFragBytes, lc, 1);
#else
          asm volatile("" : "+v"(hf[hi][0]), "+v"(hf[hi][1]));
#endif
          if (hi == 0) load_scales(nxt_base, min(kb + 1, nk - 1), sc_next);
          if (hi == H - 1) {
            sf[0] = lds_read_frag32(smem, nxt_base + strm0, lc, 0);
            sf[1] = lds_read_frag32(smem, nxt_base + strm0, lc, 1);
          }
        }
#else
        if (si == S - 1 && hi == 0) load_scales(nxt_base, min(kb + 1, nk - 1), sc_next);
        asm volatile("" : "+v"(sf[0]), "+v"(sf[1]), "+v"(hf[hi][0]), "+v"(hf[hi][1]));  // the operands change for all the compiler knows
#endif
        __builtin_amdgcn_sched_barrier(0);
#ifdef DLB_ABLATE_SCALE
        {  // one of the 16 scale FMAs of a tile, so that its MFMAs stay
          const int mi = kHoldX ? hi : si, ni = kHoldX ? si : hi;
          acc[mi][ni][0] += part[t & kSlot][0] * sc[mi][kUniformW ? 0 : ni];
        }
#else
        if (Cfg::PARTS == 1) {
          // scale-and-accumulate this tile; the other wave of the SIMD owns the matrix pipe meanwhile
          const int mi = kHoldX ? hi : si, ni = kHoldX ? si : hi;
          acc[mi][ni] += part[0] * sc[mi][kUniformW ? 0 : ni];
        } else if (t == 0) {
          // scale-and-accumulate the previous tile while this tile's MFMAs run
          acc[MF - 1][NF - 1] += part[(T - 1) & 1] * sc_last;  // last tile of the previous K step (zero at kb = 0)
        } else {
          const int pt = t - 1;
          const int pmi = kHoldX ? pt % H : pt / H, pni = kHoldX ? pt / H : pt % H;
          acc[pmi][pni] += part[pt & 1] * sc[pmi][kUniformW ? 0 : pni];
        }
#endif
      }
      sc_last = sc[MF - 1][NS - 1];
#pragma unroll
      for (int m2 = 0; m2 < MF; ++m2)
#pragma unroll
        for (int j = 0; j < NS; ++j) sc[m2][j] = sc_next[m2][j];
    };
    int stage = 0;
    for (int kb = 0; kb < nk; ++kb) {
      k_step(kb, stage);
      stage = stage + 1 == STAGES ? 0 : stage + 1;
    }
    if (Cfg::PARTS == 2) acc[MF - 1][NF - 1] += part[(T - 1) & 1] * sc_last;
    if (!kExactK) wait_vmcnt<0>();  // the trailing re-read groups must not land in the next tile's ring
    }

    // epilogue: lane holds c[m0 + wm0 + 32 mi + (lane & 31)][n0 + wn0 + 32 ni + 8 u + 4 (lane >> 5) + 0..3], u = 0..3
    if constexpr (kAct) {
      // The tile goes to LDS as the bf16 matrix the unfused GEMM would have written ([BM][gate 128 | up 128], 8-byte
      // chunks XOR-ed with an even function of the row so that the 32 rows of a store instruction spread over the
      // banks and 16-byte reads stay whole), then 16 lanes per row compute silu(gate) * up rounded to bf16 and quantise
      // the 128 values exactly as silu_and_mul + per_token_group_quant_fp8 do (moe_activation.h, fp8_quant.h).
      constexpr int kRowB = BN * 2;
      static_assert(BM * kRowB <= Cfg::LDS_BYTES, "the staged tile fits in the ring");
      __syncthreads();  // every wave is done reading the ring
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const int row = wm0 + mi * 32 + l32;
        const int x = (row & 31) << 1;
#pragma unroll
        for (int ni = 0; ni < NF; ++ni)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const v4f v = {acc[mi][ni][4 * u], acc[mi][ni][4 * u + 1], acc[mi][ni][4 * u + 2], acc[mi][ni][4 * u + 3]};
            const int chunk = (wn0 + ni * 32 + u * 8 + h * 4) >> 2;
            *reinterpret_cast<v4bf*>(smem + row * kRowB + ((chunk ^ x) << 3)) = __builtin_convertvector(v, v4bf);
          }
      }
      __syncthreads();
      const int sub = tid & 15;
      uint8_t* q_out = static_cast<uint8_t*>(p.c);
      float* s_out = p.act_s;
      if (kMaskedLike) {
        q_out += static_cast<int64_t>(g) * p.M * p.act_q_stride;
        s_out += static_cast<int64_t>(g) * p.act_s_gs;
      }
#pragma unroll 2
      for (int r0 = 0; r0 < BM; r0 += Cfg::NT / 16) {
        const int row = r0 + (tid >> 4);
        const int x = (row & 31) << 1;
        const v4i graw = *reinterpret_cast<const v4i*>(smem + row * kRowB + (((2 * sub) ^ x) << 3));
        const v4i uraw = *reinterpret_cast<const v4i*>(smem + row * kRowB + (((BN / 4 / 2 + 2 * sub) ^ x) << 3));
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t gw = static_cast<uint32_t>(graw[i]), uw = static_cast<uint32_t>(uraw[i]);
          const float g0 = __builtin_bit_cast(float, gw << 16), g1 = __builtin_bit_cast(float, gw & 0xffff0000u);
          const float u0 = __builtin_bit_cast(float, uw << 16), u1 = __builtin_bit_cast(float, uw & 0xffff0000u);
          if (kMaskedLike) {  // the masked activation rounds silu(gate) before the product (moe.py:256-257)
            v[2 * i] = static_cast<float>(static_cast<__bf16>(u0 * static_cast<float>(static_cast<__bf16>(act_silu_f32(g0)))));
            v[2 * i + 1] = static_cast<float>(static_cast<__bf16>(u1 * static_cast<float>(static_cast<__bf16>(act_silu_f32(g1)))));
          } else {
            v[2 * i] = static_cast<float>(static_cast<__bf16>(act_silu_f32(g0) * u0));
            v[2 * i + 1] = static_cast<float>(static_cast<__bf16>(act_silu_f32(g1) * u1));
          }
        }
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 16));
        const float scale = fmaxf(amax, p.act_eps) / 448.0f;
        const float inv_scale = 1.0f / scale;
        int packed[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          float c4[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) c4[j] = fminf(fmaxf(act_div_by_scale(v[4 * i + j], scale, inv_scale), -448.0f), 448.0f);
          int wd = __builtin_amdgcn_cvt_pk_fp8_f32(c4[0], c4[1], 0, false);
          wd = __builtin_amdgcn_cvt_pk_fp8_f32(c4[2], c4[3], wd, true);
          packed[i] = wd;
        }
        const int m = m0 + row;
        if (row < BM && m < m_end) {
          *reinterpret_cast<v2i*>(q_out + static_cast<int64_t>(m) * p.act_q_stride + n0 + sub * 8) = v2i{packed[0], packed[1]};
          if (sub == 0) s_out[static_cast<int64_t>(m) * p.act_s_sm + static_cast<int64_t>(n0 / kScaleBlock) * p.act_s_sk] = scale;
        }
      }
      continue;
    }
    if (sliced && p.fused_reduce) {
      // Split-K in one launch.  The workgroups of a tile (one per K slice) park their fp32 sums in the workspace,
      // count themselves in on the tile's arrival counter, wait - for a bounded time - until all slices are in, and
      // then each adds up its share of the tile: the slices in index order (the same order, and so the same bits, as
      // fp8_splitk_reduce_kernel), cast, store.  Nobody depends on that wait for correctness: a workgroup that gives
      // up sets its bit in the tile's word of abandoned shares and looks at the counter once more (all in after all:
      // it adds its share anyway); the workgroup whose arrival completed the tile reads that word after its own share
      // and adds the shares named there.  A share that both of them add is stored twice with the same bits.  The last
      // workgroup to leave the tile zeroes its three counters: the workspace head is all zero when the launch ends.
      // Partial sums are written in accumulator order: unit ((wave MF + mi) NF + ni) 4 + u holds, for lane l, the four
      // floats c[32 mi + (l & 31)][32 ni + 8 u + 4 (l >> 5) + 0..3] of that wave's tile.
      constexpr int kTileFloats = BM * BN;
      constexpr int kUnits = kTileFloats / 4;
      const int S = p.splitk;
      float* tbase = p.ws + static_cast<int64_t>(tile_lin) * S * kTileFloats;
      float* mine = tbase + static_cast<int64_t>(split) * kTileFloats;
#pragma unroll
      for (int mi = 0; mi < MF; ++mi)
#pragma unroll
        for (int ni = 0; ni < NF; ++ni)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const v4f v = {acc[mi][ni][4 * u], acc[mi][ni][4 * u + 1], acc[mi][ni][4 * u + 2], acc[mi][ni][4 * u + 3]};
            coherent_store16(mine + ((((wave * MF + mi) * NF + ni) * 4 + u) * 64 + lane) * 4, v);
          }
      // The stores above are write-through, device-scope stores: once the memory counter has drained they are where
      // every XCD reads them.  (A release fence here would also write back the whole L2 of this XCD, once per
      // workgroup: measured at 4 - 11 us per launch.)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // ... those of every wave; the ring is idle from here on
      uint32_t* ctr = p.ctr + static_cast<int64_t>(tile_lin) * 4;
      volatile uint32_t* flag = reinterpret_cast<volatile uint32_t*>(smem);
      const uint32_t uS = static_cast<uint32_t>(S);
      if (tid == 0) {
        // the arrival and the first look at the counter travel together: one round trip instead of two
        const uint32_t ticket = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t seen = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = ticket + 1u == uS;
        bool all_in = last || seen >= uS;
#pragma unroll 1
        for (int spin = 0; !all_in && spin < p.spin_limit; ++spin) {
          __builtin_amdgcn_s_sleep(2);
          all_in = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= uS;
        }
        if (!all_in) {
          __hip_atomic_fetch_or(ctr + 1, 1u << split, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_AGENT);
          all_in = __hip_atomic_load(ctr, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_AGENT) >= uS;
        }
        flag[0] = all_in ? 1u << split : 0u;
        flag[1] = last ? 1u : 0u;
      }
      __syncthreads();
      const bool last = flag[1] != 0;
      const int64_t esz_c = p.out_f32 ? 4 : 2;
      auto add_unit = [&](int u, const v4f& sum) {
        const int ul = u & 63, uu = (u >> 6) & 3, f = u >> 8;  // f = (wave MF + mi) NF + ni
        const int fni = f % NF, fmi = (f / NF) % MF, fw = f / (NF * MF);
        const int m = m0 + (fw / Cfg::WGN) * (MF * 32) + fmi * 32 + (ul & 31);
        const int n = n0 + (fw % Cfg::WGN) * (NF * 32) + fni * 32 + uu * 8 + (ul >> 5) * 4;
        if (m >= m_end) return;
        char* c_row = c_base + static_cast<int64_t>(m) * p.N * esz_c;
        if (p.out_f32)
          store_row4<true>(c_row, n, sum, p.N - n, p.vec_store);
        else
          store_row4<false>(c_row, n, sum, p.N - n, p.vec_store);
      };
      for (int round = 0; round < (last ? 2 : 1); ++round) {
        if (round == 1) {
          // the arrival that completed the tile, done with its own share: the shares their owners gave up on
          __syncthreads();
          if (tid == 0) flag[0] = __hip_atomic_load(ctr + 1, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_AGENT);
          __syncthreads();
        }
        const uint32_t todo = flag[0];
        for (int j = 0; j < S; ++j) {
          if (!((todo >> j) & 1u)) continue;
          const int u0 = static_cast<int>(static_cast<int64_t>(j) * kUnits / S);
          const int u1 = static_cast<int>(static_cast<int64_t>(j + 1) * kUnits / S);
          // two units per thread and pass, the loads of up to eight slices of both in flight before the first sum
          for (int ua = u0 + tid; ua < u1; ua += 2 * Cfg::NT) {
            const int ub = ua + Cfg::NT;
            const bool has_b = ub < u1;
            v4f sum_a = {0.f, 0.f, 0.f, 0.f}, sum_b = {0.f, 0.f, 0.f, 0.f};
            for (int sb = 0; sb < S; sb += 8) {
              v4f pa[8], pb[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                pa[i] = pb[i] = v4f{0.f, 0.f, 0.f, 0.f};
                if (sb + i < S) {
                  pa[i] = coherent_load16(tbase + static_cast<int64_t>(sb + i) * kTileFloats + ua * 4);
                  if (has_b) pb[i] = coherent_load16(tbase + static_cast<int64_t>(sb + i) * kTileFloats + ub * 4);
                }
              }
#pragma unroll
              for (int i = 0; i < 8; ++i)
                if (sb + i < S) sum_a += pa[i], sum_b += pb[i];
            }
            add_unit(ua, sum_a);
            if (has_b) add_unit(ub, sum_b);
          }
        }
      }
      __syncthreads();  // flag[] is read; the next tile may use the ring
      if (tid == 0) {
        const uint32_t left = __hip_atomic_fetch_add(ctr + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left + 1u == uS) {
          __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(ctr + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(ctr + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      continue;
    }
    if (sliced) {
      // first pass of split-K: the slice's sums go to the workspace as an fp32 [M][N] matrix of their own;
      // fp8_splitk_reduce_kernel, launched behind this kernel on the same stream, adds the slices in index order
      float* mine = p.ws + static_cast<int64_t>(split) * p.M * p.N;
      const bool vec_ok = (p.N % 4) == 0;
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const int m = m0 + wm0 + mi * 32 + l32;
        if (m >= m_end) continue;
        float* w_row = mine + static_cast<int64_t>(m) * p.N;
#pragma unroll
        for (int ni = 0; ni < NF; ++ni)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int n = n0 + wn0 + ni * 32 + u * 8 + h * 4;
            const v4f v = {acc[mi][ni][4 * u], acc[mi][ni][4 * u + 1], acc[mi][ni][4 * u + 2], acc[mi][ni][4 * u + 3]};
            store_row4<true>(w_row, n, v, p.N - n, vec_ok);
          }
      }
      continue;
    }
    if (p.c_vec16) {
      // bf16 through LDS: stored straight from the accumulator layout every instruction would touch 32 rows with
      // 16 bytes each, partial sectors that the L2 has to merge.  Each wave parks its 64-row tile in its own slice of
      // the (now idle) ring, rows rotated by their index to spread the banks, and reads it back row-wise: a store
      // instruction then writes whole rows, 16 bytes per lane.
      constexpr int kRowBytes = NF * 32 * 2;
      constexpr int kCpr = kRowBytes / 16;   // 16-byte chunks per row
      constexpr int kRpi = 64 / kCpr;        // rows per store instruction
      static_assert(MF * 32 * kRowBytes * WAVES <= Cfg::LDS_BYTES, "the staging slices fit in the ring");
      __syncthreads();  // every wave is done reading the ring
      uint8_t* st = smem + wave * (MF * 32 * kRowBytes);
#pragma unroll
      for (int mi = 0; mi < MF; ++mi) {
        const int row = mi * 32 + l32;
#pragma unroll
        for (int ni = 0; ni < NF; ++ni)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const v4f v = {acc[mi][ni][4 * u], acc[mi][ni][4 * u + 1], acc[mi][ni][4 * u + 2], acc[mi][ni][4 * u + 3]};
            const int chunk = (ni * 4 + u + row) % kCpr;
            *reinterpret_cast<v4bf*>(st + row * kRowBytes + chunk * 16 + h * 8) = __builtin_convertvector(v, v4bf);
          }
      }
      // a wave reads only what it wrote: no barrier, the LDS counter orders the two
      const int r_in = lane / kCpr, ch = lane % kCpr;
      __bf16* c_tile = reinterpret_cast<__bf16*>(c_base) + static_cast<int64_t>(m0 + wm0) * p.N + n0 + wn0;
#pragma unroll 4
      for (int r0 = 0; r0 < MF * 32; r0 += kRpi) {
        const int row = r0 + r_in;
        if (lane >= kRpi * kCpr || row >= MF * 32) continue;
        const v4i v = *reinterpret_cast<const v4i*>(st + row * kRowBytes + ((ch + row) % kCpr) * 16);
        if (m0 + wm0 + row < m_end && n0 + wn0 + ch * 8 < p.N)
          *reinterpret_cast<v4i*>(c_tile + static_cast<int64_t>(row) * p.N + ch * 8) = v;
      }
      continue;
    }
#pragma unroll
    for (int mi = 0; mi < MF; ++mi) {
      const int m = m0 + wm0 + mi * 32 + l32;
      if (m >= m_end) continue;
      char* c_row = c_base + static_cast<int64_t>(m) * p.N * esz;
#pragma unroll
      for (int ni = 0; ni < NF; ++ni) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int n = n0 + wn0 + ni * 32 + u * 8 + h * 4;
          const v4f v = {acc[mi][ni][4 * u], acc[mi][ni][4 * u + 1], acc[mi][ni][4 * u + 2], acc[mi][ni][4 * u + 3]};
          if (p.out_f32)
            store_row4<true>(c_row, n, v, p.N - n, p.vec_store);
          else
            store_row4<false>(c_row, n, v, p.N - n, p.vec_store);
        }
      }
    }
  }
}

template <class Cfg, int MODE>
__global__ void __launch_bounds__(Cfg::NT) fp8_gemm_pipelined_kernel(const Args p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  pipelined_body<Cfg, MODE>(p, smem, blockIdx.x, p.tiles_m, p.tiles_n, 0);
}

// Dense GEMM whose columns are cut at p.n_split into a region of CfgA tiles and a region of narrower CfgB tiles,
// one workgroup per tile, region A first.  The host picks the cut so that the last round of workgroups fills the
// chip: e.g. 448 tiles of 256 x 256 on 256 CUs leave a quarter of the chip idle in the second round, while 256
// tiles of 256 x 256 followed by 256 tiles of 256 x 192 cover the same output and keep every CU busy.
// Expert-contiguous rows: a one-block pre-pass turns m_indices into three tile lists.  A run of R adjacent 128-row
// blocks of one expert becomes R / 2 tiles of 256 rows when R is even, one tile of 128 rows when R = 1, and
// (R - 3) / 2 tiles of 256 rows followed by two tiles of 192 rows when R is odd: most weight tiles are then fetched
// once per expert instead of once per 128 rows, and the two 192-row tiles of an odd run, which are adjacent in their
// list, run side by side on one XCD at the same pace, so that the second finds the weight tile in the L2 (a 256-row
// and a 128-row tile drift apart and stream it twice).  Blocks whose first index is negative (or not an expert)
// appear in no list.  list layout: [0] = n256, [1] = n192, [2] = n128, then the three lists of `cap` entries each;
// an entry is the tile's first row in units of 64 rows.
constexpr int kTileListMaxBlocks = 4096;  // 512 K rows; more rows fall back to uniform 128-row tiles

__device__ __forceinline__ void contiguous_tile_list_block(const int32_t* m_indices, int M, int G, int32_t* tlist, int cap) {
  __shared__ int eb[kTileListMaxBlocks];   // expert of every 128-row block, -1 = skip
  __shared__ int rs[kTileListMaxBlocks];   // first block of the run of equal experts the block belongs to
  __shared__ int re[kTileListMaxBlocks];   // last block of that run
  __shared__ int chunk_last[256], chunk_first[256];
  __shared__ int n256, n192, n128;
  const int tid = threadIdx.x;
  const int nblk = (M + 127) / 128;
  if (tid == 0) n256 = n192 = n128 = 0;
  for (int b = tid; b < nblk; b += 256) {
    const int e = m_indices[static_cast<int64_t>(b) * 128];
    eb[b] = (e >= 0 && e < G) ? e : -1;
  }
  __syncthreads();
  const int chunk = (nblk + 255) / 256;
  const int b0 = min(nblk, tid * chunk), b1 = min(nblk, b0 + chunk);
  int last = -1;
  for (int b = b0; b < b1; ++b) {
    if (b == 0 || eb[b] != eb[b - 1]) last = b;
    rs[b] = last;
  }
  chunk_last[tid] = last;
  int first = nblk;  // the same from the right: nearest run end at or after the block
  for (int b = b1 - 1; b >= b0; --b) {
    if (b == nblk - 1 || eb[b] != eb[b + 1]) first = b;
    re[b] = first;
  }
  chunk_first[tid] = first;
  __syncthreads();
  // what the chunks before (after) this one carry in: running maximum of chunk_last from the left, running minimum of
  // chunk_first from the right, as two scans over the 256 chunk values in eight steps
  for (int off = 1; off < 256; off <<= 1) {
    const int from_left = tid >= off ? chunk_last[tid - off] : -1;
    const int from_right = tid + off < 256 ? chunk_first[tid + off] : nblk;
    __syncthreads();
    chunk_last[tid] = max(chunk_last[tid], from_left);
    chunk_first[tid] = min(chunk_first[tid], from_right);
    __syncthreads();
  }
  const int carry = tid > 0 ? chunk_last[tid - 1] : -1;
  for (int b = b0; b < b1 && rs[b] < 0; ++b) rs[b] = carry;
  const int carry_r = tid < 255 ? chunk_first[tid + 1] : nblk;
  for (int b = b1 - 1; b >= b0 && re[b] >= nblk; --b) re[b] = carry_r;
  __syncthreads();
  int32_t* l256 = tlist + kTileListHeader;
  int32_t* l192 = l256 + cap;
  int32_t* l128 = l192 + cap;
  for (int b = tid; b < nblk; b += 256) {
    if (eb[b] < 0) continue;
    const int pos = b - rs[b], len = re[b] - rs[b] + 1;
    const bool odd_tail = (len & 1) && len >= 3 && pos >= len - 3;  // the last three blocks of an odd run: two 192-row tiles
    if (odd_tail) {
      if (pos == len - 3) {
        const int at = atomicAdd(&n192, 2);
        l192[at] = 2 * b;
        l192[at + 1] = 2 * b + 3;
      }
    } else if (len == 1) {
      l128[atomicAdd(&n128, 1)] = 2 * b;
    } else if (!(pos & 1)) {
      l256[atomicAdd(&n256, 1)] = 2 * b;  // even position: first half of a 256-row tile
    }
  }
  __syncthreads();
  if (tid == 0) tlist[0] = n256, tlist[1] = n192, tlist[2] = n128;
}

__global__ void __launch_bounds__(256) contiguous_tile_list_kernel(const int32_t* m_indices, int M, int G, int32_t* tlist,
                                                                   int cap) {
  contiguous_tile_list_block(m_indices, M, G, tlist, cap);
}

// Both pre-passes of an expert-contiguous launch in one: the blocks of the scale re-layout, and one more column of
// blocks (x == tiles_x) whose first builds the tile list.  One launch less in front of the GEMM (about 5 us).
__global__ void __launch_bounds__(256) contiguous_prepass_kernel(const int32_t* m_indices, int M, int G, int32_t* tlist, int cap,
                                                                 const float* src, float* dst, int kblocks, int rows_pad,
                                                                 int64_t s_m, int64_t s_k, const int32_t* rows_map, int tiles_x) {
  if (static_cast<int>(blockIdx.x) == tiles_x) {
    if (blockIdx.y == 0) contiguous_tile_list_block(m_indices, M, G, tlist, cap);
    return;
  }
  scale_transpose_block(src, dst, M, kblocks, rows_pad, 0, s_m, s_k, rows_map, blockIdx.x, blockIdx.y, 0);
}

// First workgroup-order index of a list's tiles for this workgroup when the lists before it hold `before` tiles: the
// round robin continues where they ended.
__device__ __forceinline__ int continue_round_robin(int before) {
  const int grid = static_cast<int>(gridDim.x);
  return (static_cast<int>(blockIdx.x) + grid - before % grid) % grid;
}

template <class CfgA, class CfgC, class CfgB>
__global__ void __launch_bounds__(CfgA::NT) fp8_gemm_contig_list_kernel(const Args p) {
  static_assert(CfgA::NT == CfgB::NT && CfgA::NT == CfgC::NT && CfgA::BN == CfgB::BN && CfgA::BN == CfgC::BN,
                "the tile heights use the same workgroup shape and width");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // persistent workgroups: the 192-row pairs first - every workgroup starts at the same moment, so the two tiles of a
  // pair run in step from their first K block (2 - 4 % over starting them behind the 256-row tiles) - then the 256-row
  // tiles, then the 128-row ones
  const int total_a = p.tlist[0] * p.tiles_n, total_c = p.tlist[1] * p.tiles_n;
  pipelined_body<CfgC, kContigList>(p, smem, blockIdx.x, 0, p.tiles_n, 0);
  pipelined_body<CfgA, kContigList>(p, smem, continue_round_robin(total_c), 0, p.tiles_n, 0);
  pipelined_body<CfgB, kContigList>(p, smem, continue_round_robin(total_a + total_c), 0, p.tiles_n, 0);
}

// The gate/up projection of an expert MLP with the activation and the quantiser of its output fused into the epilogue
// (dlblas/kernels/fused_moe_v3.py:307-334 as one kernel): weights [G][2 I][K] with the gate rows first, output
// e4m3 [M][I] + scales [M][I / 128].  Same tile lists and schedule as fp8_gemm_contig_list_kernel; tiles_n = I / 128.
template <class CfgA, class CfgC, class CfgB>
__global__ void __launch_bounds__(CfgA::NT) fp8_gemm_contig_list_act_kernel(const Args p) {
  static_assert(CfgA::NT == CfgB::NT && CfgA::NT == CfgC::NT && CfgA::BN == CfgB::BN && CfgA::BN == CfgC::BN,
                "the tile heights use the same workgroup shape and width");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int total_a = p.tlist[0] * p.tiles_n, total_c = p.tlist[1] * p.tiles_n;
  pipelined_body<CfgC, kContigListAct>(p, smem, blockIdx.x, 0, p.tiles_n, 0);
  pipelined_body<CfgA, kContigListAct>(p, smem, continue_round_robin(total_c), 0, p.tiles_n, 0);
  pipelined_body<CfgB, kContigListAct>(p, smem, continue_round_robin(total_a + total_c), 0, p.tiles_n, 0);
}

template <class CfgA, class CfgB>
__global__ void __launch_bounds__(CfgA::NT) fp8_gemm_pipelined_mixed_kernel(const Args p) {
  static_assert(CfgA::NT == CfgB::NT && CfgA::BM == CfgB::BM, "both regions use the same workgroup shape and tile height");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int bid = blockIdx.x;
  if (bid < p.tiles_a)
    pipelined_body<CfgA, kDense>(p, smem, bid, p.tiles_m, p.tiles_n_a, 0);
  else
    pipelined_body<CfgB, kDense>(p, smem, bid - p.tiles_a, p.tiles_m, p.tiles_n_b, p.n_split);
}

}  // namespace dlb
