// Shared device-side definitions of the gfx950 FP8 block-scaled GEMM kernels.
//
// Arithmetic contract (dlblas/kernels/fp8_gemm.py:38-65 of the reference):
//   acc[m, n] += dot_128(A[m, kb], B[n, kb]) * a_s[m, kb] * b_s[n / 128, kb]      for every K block kb
// Products of two e4m3 values are exact in fp32 and the MFMA accumulates in fp32; the per-block scale
// is applied with one fp32 FMA per accumulator element and K block.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dlb {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));

constexpr int kScaleBlock = 128;  // K (and N) extent covered by one scale; also bytes per LDS tile row

// kContigList: contiguous, tiles from a device-built list.  kContigListAct: the same for the gate/up projection of an
// expert MLP with silu(gate) * up and the 1 x 128 quantiser applied in the epilogue (see fp8_gemm_contig_list_act_kernel).
// kMaskedAct: that epilogue on the masked layout, with the masked activation's two roundings (dlblas/kernels/moe.py:256-257).
enum Mode : int { kDense = 0, kContiguous = 1, kMasked = 2, kContigList = 3, kContigListAct = 4, kMaskedAct = 5 };

// Everything a kernel needs; passed by value as the single kernel argument.
struct Args {
  const uint8_t* a;
  const uint8_t* b;
  const float* a_s;
  const float* b_s;
  void* c;
  const int32_t* gidx;  // m_indices (contiguous) / masked_m (masked) / nullptr (dense)
  float* ws;            // scratch: split-K partial matrices [splitk][M][N]
  uint32_t* ctr;        // head of the workspace: per-tile arrival / claim / exit counters of the one-launch split-K (all zero between launches)
  int64_t a_gs;         // per-expert strides in elements (masked mode)
  int64_t as_gs;
  int64_t c_gs;
  int64_t b_gs;         // per-expert strides of the weights (both grouped modes)
  int64_t bs_gs;
  int64_t as_sm;        // a_s strides in floats
  int64_t as_sk;
  int M;                // dense: M; contiguous: M_sum; masked: M_max
  int N;
  int K;
  int G;
  int kblocks;          // ceil(K / 128)
  int nblocks;          // ceil(N / 128)
  int tiles_m;
  int tiles_n;
  int sk_bn;            // decode kernels with DMA staging: output columns per workgroup (multiple of 4, <= 16 NFS)
  int splitk;
  int kb_per_split;
  int fused_reduce;     // split-K in one launch: the workgroups of a tile add its K slices themselves (see splitk_fused_epilogue)
  int spin_limit;       //   polls (about half a microsecond apart) a workgroup waits for the other slices of its tile before it leaves its share to the last one
  int sct_pitch;        // kernels with a scale table in LDS: floats per table row (odd, >= K blocks per workgroup)
  int group_m;          // m-tiles per L2 swizzle group
  int out_f32;
  int vec_store;        // rows of c are aligned for 4-element vector stores
  int c_vec16;          // bf16 c whose rows are 16-byte aligned (N % 8 == 0): the LDS-transposed epilogue applies
  int n_split;          // mixed-width launch: first column of the narrow-tile region
  int tiles_a;          //   tiles in the wide region (tiles_m x tiles_n_a)
  int tiles_n_a;
  int tiles_n_b;
  const int32_t* tlist;  // kContigList: [0] = 256-row tiles, [1] = 128-row tiles, then the two lists of 128-row block indices
  int tlist_cap;         //   entries per list
  // kContigListAct / kMaskedAct: c is the e4m3 output [G][M][act_cols] with row stride act_q_stride (bytes);
  // N = 2 act_cols weight rows
  const int32_t* a_rows; //   kContigListAct, or NULL: row r of the GEMM is row a_rows[r] of a (its scales arrive re-laid by r)
  float* act_s;          //   scales of the output, element (g, m, j) at [g * act_s_gs + m * act_s_sm + j * act_s_sk]
  int64_t act_s_gs, act_s_sm, act_s_sk;
  int64_t act_q_stride;
  int act_cols;
  float act_eps;
};

// Arithmetic shared by the activation kernels, the quantisers and the GEMM epilogue that fuses both, so that the
// fused and the separate paths give the same bits.
//   act_silu_f32       gate / (1 + exp(-gate)) with the hardware exponential and reciprocal
//   act_div_by_scale   v / s from r = 1 / s (correctly rounded, once per group): q0 = v r, then one correction with
//                      the exact remainder, q = fma(fma(-q0, s, v), r, q0)
__device__ __forceinline__ float act_silu_f32(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }
__device__ __forceinline__ float act_div_by_scale(float v, float s, float r) {
  const float q0 = v * r;
  return fmaf(fmaf(-q0, s, v), r, q0);
}

// D = A_op * B_op^T with A_op [16 x 128] and B_op [16 x 128] e4m3; lane l supplies row (l & 15) of each
// operand, 32 consecutive K bytes starting at 32 * (l >> 4).  Lane l receives D[4 * (l >> 4) + r][l & 15]
// in component r.  Scale operands 0 select the unscaled instruction (v_mfma_f32_16x16x128_f8f6f4).
__device__ __forceinline__ v4f mfma_16x16x128_e4m3(v8i a_op, v8i b_op, v4f c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a_op, b_op, c, 0, 0, 0, 0, 0, 0);
}

// Byte offset of 16-byte chunk `chunk` (0..7) of row `row` inside a [rows][128 B] LDS tile.  The chunk index
// is XOR-swizzled with bits 1..3 of the row so that the 16 lanes of one ds_read_b128 phase (16 rows, same
// logical chunk) touch 16 distinct 16-byte bank groups.
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * kScaleBlock + (((chunk ^ (row >> 1)) & 7) << 4);
}

__device__ __forceinline__ v8i lds_read_frag(const uint8_t* tile, int row, int q) {
  const v4i lo = *reinterpret_cast<const v4i*>(tile + lds_off(row, 2 * q));
  const v4i hi = *reinterpret_cast<const v4i*>(tile + lds_off(row, 2 * q + 1));
  return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

// OCP e4m3fn -> fp32 (bias 7, subnormals m * 2^-9, 0x7f / 0xff = NaN, no infinities).
__device__ __forceinline__ float e4m3_to_f32(uint8_t v) {
  const uint32_t sign = static_cast<uint32_t>(v & 0x80u) << 24;
  const uint32_t e = (v >> 3) & 0xfu;
  const uint32_t m = v & 0x7u;
  if (e == 0) {
    const float mag = static_cast<float>(m) * 0x1p-9f;
    return __uint_as_float(__float_as_uint(mag) | sign);
  }
  if (e == 15 && m == 7) return __uint_as_float(0x7fc00000u | sign);
  return __uint_as_float(sign | ((e + 120u) << 23) | (m << 20));
}

// Store up to four consecutive output elements c[0..3] of one row; `n_left` = elements left in the row.
template <bool F32>
__device__ __forceinline__ void store_row4(void* c_row, int64_t col, v4f v, int n_left, bool vec_ok) {
  if (n_left <= 0) return;
  if (F32) {
    float* dst = static_cast<float*>(c_row) + col;
    if (vec_ok && n_left >= 4) {
      *reinterpret_cast<v4f*>(dst) = v;
    } else {
      dst[0] = v.x;
      if (n_left > 1) dst[1] = v.y;
      if (n_left > 2) dst[2] = v.z;
      if (n_left > 3) dst[3] = v.w;
    }
  } else {
    __bf16* dst = static_cast<__bf16*>(c_row) + col;
    const v4bf h = __builtin_convertvector(v, v4bf);  // round-to-nearest-even
    if (vec_ok && n_left >= 4) {
      *reinterpret_cast<v4bf*>(dst) = h;
    } else {
      dst[0] = h.x;
      if (n_left > 1) dst[1] = h.y;
      if (n_left > 2) dst[2] = h.z;
      if (n_left > 3) dst[3] = h.w;
    }
  }
}

}  // namespace dlb
