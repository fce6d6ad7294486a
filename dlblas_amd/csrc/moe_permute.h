// Token permutation around the expert-contiguous grouped GEMMs, for gfx950.  Restates
//   ep_scatter   dlblas/kernels/fused_moe_v3.py:18-158   rows of recv_x (fp8) and their scales are copied next to
//                                                        the other rows of the same expert; m_indices, output_index
//   ep_gather    dlblas/kernels/fused_moe_v3.py:161-233  weighted sum of a token's expert outputs, fp32 accumulate
// The reference hands out destination rows with one global atomic per (token, slot), in whatever order the atomics
// resolve.  Here the order is fixed - token-major, slot-minor, the order of the reference's single-program variant
// (dlblas/kernels/ascend/fused_moe_v3.py:137) - and no global atomic is used: a stable counting sort in three
// launches (per-block histograms, scan, rank + copy; the scan launch is dropped while the histogram matrix is small
// enough for every copy block to sum the rows of the blocks before it itself).  The copies are HBM-bound: every source row is read once and
// written once per valid slot, 16 bytes per lane.
#pragma once

#include "fp8_gemm_common.h"
#include "fp8_quant.h"

namespace dlb {

constexpr int kPermuteThreads = 256;  // entries (token, slot) per block of the scatter kernels
constexpr int kMaxTopk = 64;

__device__ __forceinline__ int64_t load_index(const void* base, int is64, int64_t off) {
  return is64 ? static_cast<const int64_t*>(base)[off] : static_cast<int64_t>(static_cast<const int32_t*>(base)[off]);
}
__device__ __forceinline__ void store_index(void* base, int is64, int64_t off, int64_t v) {
  if (is64)
    static_cast<int64_t*>(base)[off] = v;
  else
    static_cast<int32_t*>(base)[off] = static_cast<int32_t>(v);
}

struct ScatterArgs {
  const uint8_t* x;       // [T][H] e4m3fn
  const float* xs;        // [T][H / 128]
  const void* topk;       // [T][topk] expert ids, < 0 or >= E: no expert
  const int32_t* counts;  // [E] rows reserved per expert (padded)
  void* start_loc;        // [E] out: first free row of every expert after the call
  uint8_t* out;           // [rows][H]
  float* out_s;           // [rows][H / 128]
  int32_t* m_indices;     // [m_len]
  void* out_index;        // [T][topk]
  int32_t* block_hist;    // workspace [nblocks][E]: histogram, then first destination row of (block, expert)
  int64_t* start_excl;    // workspace [E + 1]: exclusive prefix sum of counts
  int64_t x_row_stride, xs_sm, xs_sk, topk_s0, topk_s1, out_row_stride, os_sm, os_sk, oi_s0, oi_s1;
  int64_t T, m_len;
  int H, E, topk_n, tokens_per_block, nblocks;
  int topk_is64, start_is64, oi_is64;
  int fused_scan;  // the copy kernel derives the block's first rows from the raw histograms itself (no scan launch)
  int32_t* src_row;  // [m_len] or NULL: source token of every destination row (0 for rows nobody is copied to)
  int index_only;    // fill the tables only: no row of x or xs is moved
};

// Expert id of entry `i` (token-major) of block `b`, or -1.
__device__ __forceinline__ int scatter_entry_id(const ScatterArgs& p, int b, int i) {
  const int64_t t = static_cast<int64_t>(b) * p.tokens_per_block + i / p.topk_n;
  const int j = i % p.topk_n;
  if (i >= p.tokens_per_block * p.topk_n || t >= p.T) return -1;
  const int64_t id = load_index(p.topk, p.topk_is64, t * p.topk_s0 + j * p.topk_s1);
  return (id < 0 || id >= p.E) ? -1 : static_cast<int>(id);
}

// Pass 1: block_hist[b][e] = entries of block b routed to expert e.
__global__ void __launch_bounds__(kPermuteThreads) ep_scatter_count_kernel(const ScatterArgs p) {
  extern __shared__ int hist[];
  for (int e = threadIdx.x; e < p.E; e += kPermuteThreads) hist[e] = 0;
  __syncthreads();
  const int id = scatter_entry_id(p, blockIdx.x, threadIdx.x);
  if (id >= 0) atomicAdd(&hist[id], 1);
  __syncthreads();
  for (int e = threadIdx.x; e < p.E; e += kPermuteThreads) p.block_hist[static_cast<int64_t>(blockIdx.x) * p.E + e] = hist[e];
  // rows that no slot is copied to (the padding of every expert's span) name token 0: any valid row will do for them,
  // and this launch is ordered before the one that writes the real entries
  if (p.src_row != nullptr)
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * kPermuteThreads + threadIdx.x; r < p.m_len;
         r += static_cast<int64_t>(gridDim.x) * kPermuteThreads)
      p.src_row[r] = 0;
}

// Pass 2 (one block of 1024): start_excl = exclusive prefix sum of counts; block_hist[b][e] becomes the first row
// block b writes for expert e; start_loc[e] = start_excl[e] + entries routed to e.  The histogram matrix is staged
// through LDS in slabs of whole blocks (coalesced both ways).  Inside a slab a column (expert) is shared by
// P = 1024 / E threads, each summing, then rewriting, its own run of rows.
constexpr int kScanThreads = 1024;
constexpr int kScanTileInts = 24576;  // 96 KB of LDS for the slab
constexpr int kScanMaxExperts = 2048;

__global__ void __launch_bounds__(kScanThreads) ep_scatter_scan_kernel(const ScatterArgs p) {
  extern __shared__ int tile[];  // [slab rows][E]
  __shared__ int64_t part[kScanThreads];
  __shared__ int64_t run[kScanMaxExperts];  // first free row of every expert, advanced slab by slab
  __shared__ int psum[kScanThreads];
  const int tid = threadIdx.x;
  const int per = (p.E + kScanThreads - 1) / kScanThreads;
  const int e0 = min(tid * per, p.E), e1 = min(e0 + per, p.E);
  int64_t sum = 0;
  for (int e = e0; e < e1; ++e) sum += max(p.counts[e], 0);
  part[tid] = sum;
  __syncthreads();
  for (int off = 1; off < kScanThreads; off <<= 1) {  // inclusive Hillis-Steele scan of the chunk sums
    const int64_t add = tid >= off ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += add;
    __syncthreads();
  }
  int64_t first = part[tid] - sum;
  for (int e = e0; e < e1; ++e) {
    p.start_excl[e] = first;
    run[e] = first;
    first += max(p.counts[e], 0);
  }
  if (tid == kScanThreads - 1) p.start_excl[p.E] = part[tid];
  __syncthreads();

  const int slab = max(1, min(p.nblocks, kScanTileInts / p.E));
  const int cols = min(p.E, kScanThreads);           // columns handled at a time
  const int P = kScanThreads / cols;                 // threads per column
  const int my_part = tid / cols, my_col = tid % cols;
  for (int b0 = 0; b0 < p.nblocks; b0 += slab) {
    const int nb = min(slab, p.nblocks - b0);
    int32_t* src = p.block_hist + static_cast<int64_t>(b0) * p.E;
    for (int i = tid; i < nb * p.E; i += kScanThreads) tile[i] = src[i];
    __syncthreads();
    const int R = (nb + P - 1) / P;
    const int r_lo = min(nb, my_part * R), r_hi = min(nb, r_lo + R);
    for (int c0 = 0; c0 < p.E; c0 += cols) {
      const int e = c0 + my_col;
      const bool on = my_part < P && e < p.E;
      int s_rows = 0;
      if (on)
        for (int r = r_lo; r < r_hi; ++r) s_rows += tile[r * p.E + e];
      psum[tid] = s_rows;
      __syncthreads();
      int64_t off = 0;
      if (on) {
        off = run[e];
        for (int q = 0; q < my_part; ++q) off += psum[q * cols + my_col];
        for (int r = r_lo; r < r_hi; ++r) {
          const int h = tile[r * p.E + e];
          tile[r * p.E + e] = static_cast<int>(off);
          off += h;
        }
      }
      __syncthreads();
      if (on && my_part == P - 1) run[e] = off;  // the last part ends at the expert's first free row after this slab
    }
    __syncthreads();
    for (int i = tid; i < nb * p.E; i += kScanThreads) src[i] = tile[i];
    __syncthreads();
  }
  for (int e = tid; e < p.E; e += kScanThreads) store_index(p.start_loc, p.start_is64, e, run[e]);
}

// Pass 3 (blocks of 1024 threads over the same 256 entries as pass 1): rank of every entry among the earlier entries
// of its block with the same expert, destination row = block_hist[b][e] + rank; then the 16 waves copy the block's
// tokens to their destination rows.  Every block also fills its slice of m_indices.
constexpr int kCopyThreads = 1024;

constexpr int kFusedScanMaxInts = 32768;  // histogram entries up to which a copy block scans for itself

__global__ void __launch_bounds__(kCopyThreads) ep_scatter_copy_kernel(const ScatterArgs p) {
  __shared__ int ids[kPermuteThreads];
  __shared__ int64_t dest[kPermuteThreads];
  __shared__ int64_t excl_l[kScanMaxExperts + 1];  // fused scan: exclusive prefix sum of counts
  __shared__ int64_t base_l[kScanMaxExperts];      //             first row this block writes for every expert
  __shared__ int psum[kCopyThreads];
  const int tid = threadIdx.x;
  const int nthreads = static_cast<int>(blockDim.x);  // kCopyThreads when rows are copied, kPermuteThreads for the tables only
  const int b = blockIdx.x;
  int id = -1;
  if (tid < kPermuteThreads) {
    id = scatter_entry_id(p, b, tid);
    ids[tid] = id;
  }
  if (p.fused_scan) {
    // what the scan launch would have left in start_excl and block_hist[b][.], computed by every block for itself:
    // the first wave scans counts 64 at a time, then all threads add up the histogram rows of the blocks before b
    if (tid < 64) {
      int64_t carry = 0;
      for (int e0 = 0; e0 < p.E; e0 += 64) {
        const int e = e0 + tid;
        const int64_t c = e < p.E ? max(p.counts[e], 0) : 0;
        int64_t incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int64_t up = __shfl_up(incl, off);
          if (tid >= off) incl += up;
        }
        if (e < p.E) excl_l[e] = carry + incl - c;
        carry += __shfl(incl, 63);
      }
      if (tid == 0) excl_l[p.E] = carry;
    }
    const int cols = min(p.E, nthreads);
    const int P = nthreads / cols;
    const int my_part = tid / cols, my_col = tid % cols;
    for (int c0 = 0; c0 < p.E; c0 += cols) {
      const int e = c0 + my_col;
      int s_rows = 0;
      if (my_part < P && e < p.E)
        for (int r = my_part; r < b; r += P) s_rows += p.block_hist[static_cast<int64_t>(r) * p.E + e];
      psum[tid] = s_rows;
      __syncthreads();  // also orders excl_l
      if (my_part == 0 && e < p.E) {
        int64_t first = excl_l[e];
        for (int q = 0; q < P; ++q) first += psum[q * cols + my_col];
        base_l[e] = first;
        if (b == static_cast<int>(gridDim.x) - 1)  // the last block knows every expert's first free row after the call
          store_index(p.start_loc, p.start_is64, e, first + p.block_hist[static_cast<int64_t>(b) * p.E + e]);
      }
      __syncthreads();
    }
  }
  __syncthreads();
  if (tid < kPermuteThreads) {
    int64_t d = -1;
    if (id >= 0) {
      int rank = 0;
      for (int j = 0; j < tid; ++j) rank += (ids[j] == id);
      d = (p.fused_scan ? base_l[id] : static_cast<int64_t>(p.block_hist[static_cast<int64_t>(b) * p.E + id])) + rank;
      const int64_t t = static_cast<int64_t>(b) * p.tokens_per_block + tid / p.topk_n;
      store_index(p.out_index, p.oi_is64, t * p.oi_s0 + (tid % p.topk_n) * p.oi_s1, d);
      if (p.src_row != nullptr && d < p.m_len) p.src_row[d] = static_cast<int32_t>(t);
    }
    dest[tid] = d;
  }
  __syncthreads();

  // m_indices: rows [0, start_excl[E]) in slices over the blocks; expert of a row by binary search
  {
    const int64_t* excl = p.fused_scan ? excl_l : p.start_excl;
    const int64_t total = min(excl[p.E], p.m_len);
    const int64_t per = (total + gridDim.x - 1) / gridDim.x;
    const int64_t r1 = min(total, (b + 1) * per);
    for (int64_t r = b * per + tid; r < r1; r += nthreads) {
      int lo = 0, hi = p.E;  // largest e with start_excl[e] <= r
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (excl[mid] <= r)
          lo = mid;
        else
          hi = mid;
      }
      p.m_indices[r] = lo;
    }
  }

  if (p.index_only) return;
  // copies: one wave per token; a lane loads up to 8 chunks of 16 bytes (8 KB per wave and trip) before it stores
  // them to the row of every routed slot
  const int lane = tid & 63, wave = tid >> 6;
  const int groups = p.H / 128;
  for (int lt = wave; lt < p.tokens_per_block; lt += nthreads / 64) {
    const int64_t t = static_cast<int64_t>(b) * p.tokens_per_block + lt;
    if (t >= p.T) break;
    const uint8_t* src = p.x + t * p.x_row_stride;
    const int64_t* drow = dest + lt * p.topk_n;
    for (int c0 = 0; c0 < p.H; c0 += 8 * 64 * 16) {
      v4i v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int c = c0 + (u * 64 + lane) * 16;
        if (c < p.H) v[u] = *reinterpret_cast<const v4i*>(src + c);
      }
      for (int j = 0; j < p.topk_n; ++j) {
        const int64_t dj = drow[j];
        if (dj < 0) continue;
        uint8_t* dst = p.out + dj * p.out_row_stride;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int c = c0 + (u * 64 + lane) * 16;
          if (c < p.H) *reinterpret_cast<v4i*>(dst + c) = v[u];
        }
      }
    }
    for (int k = lane; k < groups; k += 64) {
      const float sv = p.xs[t * p.xs_sm + k * p.xs_sk];
      for (int j = 0; j < p.topk_n; ++j) {
        const int64_t dj = drow[j];
        if (dj >= 0) p.out_s[dj * p.os_sm + k * p.os_sk] = sv;
      }
    }
  }
}

struct GatherArgs {
  const void* in;       // [rows][H]
  const void* topk;     // [T][topk]
  const float* weight;  // [T][topk]
  const void* index;    // [T][topk] source row of every slot
  void* out;            // [T][H]
  int64_t in_row_stride, topk_s0, topk_s1, w_s0, w_s1, idx_s0, idx_s1, out_row_stride;
  int64_t T;
  int H, topk_n;
  int topk_is64, idx_is64;
};

template <int OUT>
__device__ __forceinline__ void gather_store8(void* out, int64_t elem, const float (&v)[8]) {
  if (OUT == kInF32) {
    v4f* p = reinterpret_cast<v4f*>(static_cast<float*>(out) + elem);
    p[0] = v4f{v[0], v[1], v[2], v[3]};
    p[1] = v4f{v[4], v[5], v[6], v[7]};
  } else {
    v4i raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t lo, hi;
      if (OUT == kInBf16) {
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

// grid = (tokens, column parts).  A wave owns a token and a contiguous part of its columns.  Lane j holds slot j of
// the token's routing table; the slot loop is wave-uniform (slots without an expert are skipped by a scalar branch)
// and every routed slot contributes 8 chunks of 8 elements per lane and trip, all loaded before the fp32 FMAs, which
// run in slot order.  H % 8 == 0; rows 16-byte aligned.
template <int IN, int OUT>
__global__ void __launch_bounds__(64) ep_gather_kernel(const GatherArgs p) {
  constexpr int U = 8;
  const int lane = threadIdx.x;
  const int64_t t = blockIdx.x;
  int64_t my_row = -1;
  float my_w = 0.f;
  if (lane < p.topk_n) {
    const int64_t id = load_index(p.topk, p.topk_is64, t * p.topk_s0 + lane * p.topk_s1);
    if (id >= 0) {
      my_row = load_index(p.index, p.idx_is64, t * p.idx_s0 + lane * p.idx_s1);
      my_w = p.weight[t * p.w_s0 + lane * p.w_s1];
    }
  }
  const int chunks = p.H / 8;
  const int per_part = (chunks + gridDim.y - 1) / gridDim.y;
  const int c0 = blockIdx.y * per_part, c1 = min(chunks, c0 + per_part);
  for (int cb = c0; cb < c1; cb += U * 64) {
    float acc[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[u][i] = 0.f;
    for (int j = 0; j < p.topk_n; ++j) {
      const int64_t row = __shfl(my_row, j);  // every lane is active here: the loops above are wave-uniform
      const float w = __shfl(my_w, j);
      if (row < 0) continue;
      const int64_t base = row * p.in_row_stride;
      Raw8 raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = cb + u * 64 + lane;
        if (c < c1) raw[u] = quant_load_raw<IN>(p.in, base + static_cast<int64_t>(c) * 8);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (cb + u * 64 + lane >= c1) continue;
        float v[8];
        quant_unpack8<IN>(raw[u], v);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[u][i] = fmaf(v[i], w, acc[u][i]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = cb + u * 64 + lane;
      if (c < c1) gather_store8<OUT>(p.out, t * p.out_row_stride + static_cast<int64_t>(c) * 8, acc[u]);
    }
  }
}

}  // namespace dlb
