// C ABI of the gfx950 FP8 block-scaled GEMM library: argument validation, kernel selection, launches.
// The declarations and the contract of every entry point are in include/dlblas_fp8_gemm.h.
#include "../../include/dlblas_fp8_gemm.h"
#include "../../include/dlblas_fp8_moe.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "fp8_gemm_common.h"
#include "host_common.h"
#include "fp8_gemm_pipelined.h"
#include "fp8_gemm_skinny.h"
#include "fp8_gemm_tiled.h"
#include "fp8_quant.h"

// Scratch for dlb_fp8_gemm_noalloc: device memory that is part of the loaded code object, so a caller that cannot
// allocate (HIP graph capture, a serving loop that forbids hipMalloc) needs no workspace of its own.  Every GPU the
// library runs on holds its own copy at its own address until the process ends.  The name is only a host-side
// handle: host code uses the per-device address hipGetSymbolAddress returns (static_scratch_ptr below), never the
// name itself.
static __device__ __align__(256) unsigned char scratch[DLB_STATIC_SCRATCH_BYTES];

namespace dlb {

// ---------------------------------------------------------------------------------------------------------
// Exact path for shapes the MFMA kernels do not take (K not a multiple of 16): one thread per output
// element, e4m3 decoded in software, fp32 FMA chain per 128 block, scales applied as in
// dlblas/kernels/fp8_gemm.py:55.
// ---------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) fp8_gemm_exact_kernel(const Args p) {
  const int n = blockIdx.x * 64 + (threadIdx.x & 63);
  if (n >= p.N) return;
  const uint8_t* b_row = p.b + static_cast<int64_t>(n) * p.K;
  const float* bs_row = p.b_s + static_cast<int64_t>(n / kScaleBlock) * p.kblocks;
  for (int64_t m = blockIdx.y * 4 + (threadIdx.x >> 6); m < p.M; m += static_cast<int64_t>(gridDim.y) * 4) {
    const uint8_t* a_row = p.a + m * p.K;
    const float* as_row = p.a_s + m * p.as_sm;
    float acc = 0.f;
    for (int kb = 0; kb < p.kblocks; ++kb) {
      const int k1 = min(p.K, (kb + 1) * kScaleBlock);
      float dot = 0.f;
      for (int k = kb * kScaleBlock; k < k1; ++k) dot = fmaf(e4m3_to_f32(a_row[k]), e4m3_to_f32(b_row[k]), dot);
      acc += dot * as_row[static_cast<int64_t>(kb) * p.as_sk] * bs_row[kb];
    }
    if (p.out_f32)
      static_cast<float*>(p.c)[m * p.N + n] = acc;
    else
      static_cast<__bf16*>(p.c)[m * p.N + n] = static_cast<__bf16>(acc);
  }
}

// ---------------------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------------------
thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_err[0] = '\0'; }

int device_cu_count(int* dev_out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  *dev_out = dev;
  if (dev < 0 || dev >= kMaxDevices) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}

namespace {

thread_local int g_forced_variant = -1;
enum Knob : int {
  kKnobSplitK = 0,
  kKnobSkinnyWaves,
  kKnobSkinnyUnroll,
  kKnobSkinnyNFrags,
  kKnobGroupM,
  kKnobSkinnyDma,  // 0 / 1: DMA-staged decode kernel where possible, 2: register-load decode kernel
  kKnobEpilogue,   // 0 / 1: bf16 output of the pipelined kernels goes through LDS where it can, 2: straight from registers
  kKnobSkinnyBn,   // columns per workgroup of the DMA-staged decode kernels (0 = heuristic)
  kKnobSplitKMode, // 1: K slices of the ring kernels are added inside the launch where that applies; 0 / 2: by a second launch (faster on MI355X)
  kKnobSpinLimit,  // one-launch split-K: value - 1 polls for the other slices of a tile (0 = default; 1 = none: the last arrival adds every share)
  kKnobScaleTable, // 0 / 1: row-major activation scales of the small ring kernels go through the per-tile table, 2: never
  kKnobLdsOversize,  // test hook: 1 = ask for more LDS than the GPU has, so that the launch is refused before anything is enqueued
  kKnobMaskedGrid,   // workgroups per CU of the masked layout's persistent grid (0 = default)
  kKnobTileList,     // expert-contiguous rows: 1 = device-built tile lists whenever possible, 2 = never (0 = by batch size)
  kKnobCount
};
thread_local int g_knob[kKnobCount] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
// set while run() asks every kernel of the call for its launch attributes, before the first pre-pass is enqueued
thread_local bool g_prepare_only = false;
constexpr int kDefaultSpinLimit = 400;  // x about 0.5 us: far beyond the spread of the slices of one round of workgroups

enum Variant : int {
  kVarExact = 0,
  kVarTile128x128,
  kVarTile64x128,
  kVarTile128x64,
  kVarSkinny16,
  kVarSkinny32,
  kVarSkinny64,
  kVarSkinny128,
  kVarPipe256x256,
  kVarPipe128x256w8,
  kVarPipe256mix,
  kVarPipe128x128,
  kVarPipe128x64,
  kVarCount
};

const char* const kVariantNames[kVarCount] = {
    "exact", "tile128x128", "tile64x128", "tile128x64", "skinny16", "skinny32", "skinny64", "skinny128", "pipe256x256", "pipe128x256w8", "pipe256mix", "pipe128x128", "pipe128x64",
};

typedef TileCfg<128, 128, 2, 2> Tile128x128;
typedef TileCfg<64, 128, 2, 2> Tile64x128;
typedef TileCfg<128, 64, 2, 2> Tile128x64;
typedef PipeCfg<4, 2, 2, 4, 2, 2> Pipe256x256;  // 8 waves, wave tile 64 x 128
typedef PipeCfg<4, 2, 2, 3, 2, 2> Pipe256x192;  // narrow tiles of the mixed-width launch
typedef PipeCfg<2, 4, 3, 2, 2, 2> Pipe192x256;  // the two tiles of an expert's run of three 128-row blocks

// bytes of the three tile lists of an expert-contiguous launch over nblk 128-row blocks
constexpr size_t tile_list_bytes(int64_t nblk) {
  return (static_cast<size_t>(kTileListHeader + 3 * nblk) * sizeof(int32_t) + 255) / 256 * 256;
}
typedef PipeCfg<2, 4, 2, 2, 3> Pipe128x256w8;  // 8 waves, wave tile 64 x 64
constexpr int kListLds = Pipe256x256::LDS_BYTES > Pipe128x256w8::LDS_BYTES
                             ? (Pipe256x256::LDS_BYTES > Pipe192x256::LDS_BYTES ? Pipe256x256::LDS_BYTES : Pipe192x256::LDS_BYTES)
                             : (Pipe128x256w8::LDS_BYTES > Pipe192x256::LDS_BYTES ? Pipe128x256w8::LDS_BYTES : Pipe192x256::LDS_BYTES);
// small tiles for problems with few of the large ones (M of a few hundred, or a narrow N): 4 waves, deep rings
#ifdef DLB_EXP_P128
typedef PipeCfg<2, 2, 2, 2, DLB_EXP_P128, 2, false> Pipe128x128;  // experiment: 4 waves, in-place K loop, DLB_EXP_P128 stages
#else
typedef PipeCfg<2, 2, 2, 2, 4, 2, true> Pipe128x128;  // wave tile 64 x 64, 4 stages of 34 KB
#endif
typedef PipeCfg<2, 2, 2, 1, 5, 2, true> Pipe128x64;   // wave tile 64 x 32, 5 stages of 26 KB
// the same with the activation scales of a tile in a table behind the ring (row-major a_s; as many K blocks per
// workgroup as the LDS left by the ring holds: 54 and 64)
typedef PipeCfg<2, 2, 2, 2, 4, 2, true, true, 54> Pipe128x128T;
typedef PipeCfg<2, 2, 2, 1, 5, 2, true, true, 64> Pipe128x64T;
typedef PipeCfg<2, 4, 2, 2, 3, 2, false, true, 16> Pipe128x256w8T;  // the masked layout's tiles (K of at most 16 blocks: 8 KB next to the 150 KB ring)
static_assert(Pipe128x256w8T::LDS_BYTES <= 160 * 1024 && Pipe128x128T::LDS_BYTES <= 160 * 1024 && Pipe128x64T::LDS_BYTES <= 160 * 1024, "ring + table fit the LDS");
constexpr int kFusedMaxTiles = DLB_WS_COUNTER_BYTES / 16;  // four counter words per tile in the workspace head

// Raise a kernel's dynamic LDS limit once per (kernel, device).
template <class Kernel>
hipError_t ensure_lds(Kernel kernel, int bytes, int dev, std::atomic<unsigned long long>* done_mask) {
  if (g_knob[kKnobLdsOversize] == 1) {
    const hipError_t e =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes + (1 << 20));
    if (e != hipSuccess) (void)hipGetLastError();  // the refusal is reported through the return code, not left for the caller's next HIP call
    return e;
  }
  if (bytes <= 48 * 1024) return hipSuccess;
  const unsigned long long bit = 1ull << (dev & 63);
  if (done_mask->load(std::memory_order_acquire) & bit) return hipSuccess;
  const hipError_t e =
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess)
    done_mask->fetch_or(bit, std::memory_order_release);
  else
    (void)hipGetLastError();
  return e;
}

template <class Cfg, int MODE>
hipError_t launch_tiled(const Args& args, int grid, int dev, hipStream_t stream) {
  static std::atomic<unsigned long long> lds_done{0};
  auto kernel = fp8_gemm_tiled_kernel<Cfg, MODE>;
  hipError_t e = ensure_lds(kernel, Cfg::LDS_BYTES, dev, &lds_done);
  if (e != hipSuccess || g_prepare_only) return e;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
  return hipGetLastError();
}

template <class Cfg>
hipError_t launch_tiled_mode(int mode, const Args& args, int grid, int dev, hipStream_t stream) {
  switch (mode) {
    case kDense:
      return launch_tiled<Cfg, kDense>(args, grid, dev, stream);
    case kContiguous:
      return launch_tiled<Cfg, kContiguous>(args, grid, dev, stream);
    default:
      return launch_tiled<Cfg, kMasked>(args, grid, dev, stream);
  }
}

template <class Cfg, int MODE>
hipError_t launch_pipelined(const Args& args, int grid, int dev, hipStream_t stream) {
  static std::atomic<unsigned long long> lds_done{0};
  auto kernel = fp8_gemm_pipelined_kernel<Cfg, MODE>;
  hipError_t e = ensure_lds(kernel, Cfg::LDS_BYTES, dev, &lds_done);
  if (e != hipSuccess || g_prepare_only) return e;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
  return hipGetLastError();
}

template <class Cfg>
hipError_t launch_pipelined_mode(int mode, const Args& args, int grid, int dev, hipStream_t stream) {
  switch (mode) {
    case kDense:
      return launch_pipelined<Cfg, kDense>(args, grid, dev, stream);
    case kContiguous:
      return launch_pipelined<Cfg, kContiguous>(args, grid, dev, stream);
    default:
      return launch_pipelined<Cfg, kMasked>(args, grid, dev, stream);
  }
}

template <class Cfg>
hipError_t launch_skinny_cfg(bool dma, const Args& args, int dev, hipStream_t stream) {
  static std::atomic<unsigned long long> lds_done{0}, lds_done_tail{0}, lds_done_dma{0};
  const bool ktail = args.K % kScaleBlock != 0;
  // full-line DMA staging where it fits in LDS and K has no ragged block; else the register-load kernel
  if (dma && !ktail && Cfg::DMA_LDS_BYTES <= 160 * 1024 && g_knob[kKnobSkinnyDma] != 2) {
    auto kernel = fp8_gemm_skinny_dma_kernel<Cfg>;
    hipError_t e = ensure_lds(kernel, Cfg::DMA_LDS_BYTES, dev, &lds_done_dma);
    if (e != hipSuccess || g_prepare_only) return e;
    const unsigned grid = static_cast<unsigned>(ceil_div(args.N, args.sk_bn));  // its own column split, see pick_skinny_bn
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(Cfg::NT), Cfg::DMA_LDS_BYTES, stream, args);
    return hipGetLastError();
  }
  auto kernel = ktail ? fp8_gemm_skinny_kernel<Cfg, true> : fp8_gemm_skinny_kernel<Cfg, false>;
  hipError_t e = ensure_lds(kernel, Cfg::RED_BYTES, dev, ktail ? &lds_done_tail : &lds_done);
  if (e != hipSuccess || g_prepare_only) return e;
  hipLaunchKernelGGL(kernel, dim3(args.tiles_n), dim3(Cfg::NT), Cfg::RED_BYTES, stream, args);
  return hipGetLastError();
}

// Skinny kernel instances: MF in {1, 2}, (waves, unroll) in a small set, n fragments in {1, 2}.
template <int MF, int NFS>
hipError_t launch_skinny_wu(int waves, int unroll, bool dma, const Args& args, int dev, hipStream_t stream) {
  if (waves >= 16) {
    if (unroll >= 4) return launch_skinny_cfg<SkinnyCfg<MF, 16, 4, NFS>>(dma, args, dev, stream);
    if (unroll >= 2) return launch_skinny_cfg<SkinnyCfg<MF, 16, 2, NFS>>(dma, args, dev, stream);
    return launch_skinny_cfg<SkinnyCfg<MF, 16, 1, NFS>>(dma, args, dev, stream);
  }
  if (waves >= 8) {
    if (unroll >= 4) return launch_skinny_cfg<SkinnyCfg<MF, 8, 4, NFS>>(dma, args, dev, stream);
    if (unroll >= 2) return launch_skinny_cfg<SkinnyCfg<MF, 8, 2, NFS>>(dma, args, dev, stream);
    return launch_skinny_cfg<SkinnyCfg<MF, 8, 1, NFS>>(dma, args, dev, stream);
  }
  if (unroll >= 4) return launch_skinny_cfg<SkinnyCfg<MF, 4, 4, NFS>>(dma, args, dev, stream);
  return launch_skinny_cfg<SkinnyCfg<MF, 4, 2, NFS>>(dma, args, dev, stream);
}

// Large activation blocks (M up to 64 / 128) keep to one K block in flight per wave: their fragments fill the registers.
template <int MF, int NFS>
hipError_t launch_skinny_big(int waves, bool dma, const Args& args, int dev, hipStream_t stream) {
  if (waves >= 16) return launch_skinny_cfg<SkinnyCfg<MF, 16, 1, NFS>>(dma, args, dev, stream);
  if (waves >= 8) return launch_skinny_cfg<SkinnyCfg<MF, 8, 1, NFS>>(dma, args, dev, stream);
  return launch_skinny_cfg<SkinnyCfg<MF, 4, 1, NFS>>(dma, args, dev, stream);
}

hipError_t launch_skinny(int mf, int nfs, int waves, int unroll, bool dma, const Args& args, int dev, hipStream_t stream) {
  switch (mf) {
    case 1:
      return nfs == 2 ? launch_skinny_wu<1, 2>(waves, unroll, dma, args, dev, stream)
                      : launch_skinny_wu<1, 1>(waves, unroll, dma, args, dev, stream);
    case 2:
      return nfs == 2 ? launch_skinny_wu<2, 2>(waves, unroll, dma, args, dev, stream)
                      : launch_skinny_wu<2, 1>(waves, unroll, dma, args, dev, stream);
    case 4:
      return nfs == 2 ? launch_skinny_big<4, 2>(waves, dma, args, dev, stream) : launch_skinny_big<4, 1>(waves, dma, args, dev, stream);
    default:
      return nfs == 2 ? launch_skinny_big<8, 2>(waves, dma, args, dev, stream) : launch_skinny_big<8, 1>(waves, dma, args, dev, stream);
  }
}


// Makespan (in units of one 256 x 256 tile) of `ta` tiles of cost 1 followed by `tb` tiles of cost `cb` < 1, handed
// out in order, each to the worker that becomes free first.  After the unit tiles `ra = ta % workers` workers are busy
// until qa + 1 and the others until qa = ta / workers; every later tile starts at one of the times qa + j cb (on one
// of the workers - ra early ones) or qa + 1 + j cb (on one of the ra late ones), smallest first, so the last start is
// found by merging two arithmetic sequences: a few steps per round of workgroups instead of one heap operation per tile.
double mixed_makespan(int64_t ta, int64_t tb, double cb, int workers) {
  const int64_t qa = ta / workers, ra = ta % workers;
  const int64_t n_early = workers - ra, n_late = ra;
  double end = ta > 0 ? static_cast<double>(qa + (ra > 0 ? 1 : 0)) : 0.0;
  int64_t left = tb, i = 0, j = 0;
  while (left > 0) {
    const double t_early = static_cast<double>(qa) + static_cast<double>(i) * cb;
    const double t_late = static_cast<double>(qa + 1) + static_cast<double>(j) * cb;
    const bool take_early = n_late == 0 || t_early <= t_late;
    const int64_t n = take_early ? n_early : n_late;
    const double start = take_early ? t_early : t_late;
    (take_early ? i : j) += 1;
    left -= n < left ? n : left;
    if (start + cb > end) end = start + cb;
  }
  return end;
}

// Columns [0, n_split) in 256-wide tiles, the rest in 192-wide tiles; returns n_split (== N: no narrow region).
// Cost: (N / 256 + 1) candidate cuts x a few steps per round, a few microseconds at most, no state.
// *makespan (optional): the launch's length in units of one 256-wide tile.
int64_t pick_mixed_split(int64_t M, int64_t N, int cus, double* makespan = nullptr) {
  const int64_t tm = ceil_div(M, 256);
  const double narrow_cost = 0.78;  // 192 / 256 of the work plus the fixed per-tile part
  int64_t best_split = N;
  if (tm * ceil_div(N, 256) > 16 * static_cast<int64_t>(cus)) {  // many rounds: the tail no longer matters
    if (makespan) *makespan = static_cast<double>(ceil_div(tm * ceil_div(N, 256), cus));
    return N;
  }
  const double uniform = mixed_makespan(tm * ceil_div(N, 256), 0, narrow_cost, cus);
  double best = uniform;
  for (int64_t ca = N / 256; ca >= 0; --ca) {
    const int64_t split = ca * 256;
    if (split >= N) continue;
    const double t = mixed_makespan(tm * ca, tm * ceil_div(N - split, 192), narrow_cost, cus);
    if (t < best - 1e-6 && t < 0.96 * uniform) best = t, best_split = split;  // a uniform launch of many rounds runs resident, worth 4 %
  }
  if (makespan) *makespan = best;
  return best_split;
}

// Prefill-sized dense problems: 256-row tiles (256 and 192 columns wide, mixed so that the rounds come out even) or
// 128 x 256 tiles?  Both run from the L2 at the pace of the matrix pipe there - 1.62 us per K step of a 256 x 256 tile,
// 1.0 us for 128 x 256 - and a tile costs a fixed 11.5 / 5.5 us on top (its first loads, its output; 4.3 us in a launch
// of four rounds or more, which runs as resident workgroups; measured on MI355X, 192 ... 4096 rows, K = 512 ... 18432).
// The larger tile wins unless its rows are mostly padding (384 rows are two 256-row tiles but three of 128), its tiles
// leave much of a round empty (2048 x 4096: 128 tiles of 256 x 256 on 256 CUs, but 256 tiles of 128 x 256), or K is so
// short that the fixed part decides: 384 x 18432 x 7168 82 -> 67 us, 2048 x 4096 x 7168 79 -> 67 us,
// 4096 x 32768 x 512 166 -> 155 us.
bool prefers_128_row_tiles(int64_t M, int64_t N, int kblocks, int cus) {
  double span = 0.0;
  pick_mixed_split(M, N, cus, &span);
  const double wide_us = span * (11.5 + 1.62 * kblocks);
  const int64_t rounds = ceil_div(ceil_div(M, 128) * ceil_div(N, 256), cus);
  const double half_us = static_cast<double>(rounds) * ((rounds >= 4 ? 4.3 : 5.5) + 1.0 * kblocks);
  return half_us < 0.95 * wide_us;
}

struct Plan {
  int variant;
  int bm, bn;
  int splitk;
  int sk_waves, sk_unroll, sk_nfrags;  // skinny kernel shape
  int sk_bn;                           // columns per workgroup of its DMA-staged form
  bool sk_dma;                         // decode kernels may use the DMA-staged form
};

void tile_dims(int variant, int* bm, int* bn) {
  switch (variant) {
    case kVarTile64x128:
      *bm = 64, *bn = 128;
      break;
    case kVarTile128x64:
      *bm = 128, *bn = 64;
      break;
    case kVarSkinny16:
      *bm = 16, *bn = 16;
      break;
    case kVarSkinny32:
      *bm = 32, *bn = 16;
      break;
    case kVarSkinny64:
      *bm = 64, *bn = 16;
      break;
    case kVarSkinny128:
      *bm = 128, *bn = 16;
      break;
    case kVarPipe128x256w8:
      *bm = 128, *bn = 256;
      break;
    case kVarPipe256x256:
    case kVarPipe256mix:
      *bm = 256, *bn = 256;
      break;
    case kVarPipe128x64:
      *bm = 128, *bn = 64;
      break;
    default:
      *bm = 128, *bn = 128;
  }
}

bool is_skinny(int v) { return v >= kVarSkinny16 && v <= kVarSkinny128; }
int skinny_rows(int v) { return 16 << (v - kVarSkinny16); }
bool is_pipelined(int v) { return v >= kVarPipe256x256 && v <= kVarPipe128x64; }

// Split count no larger than `want` whose slices hold at least two K blocks and whose fp32 partial matrices fit.
int clamp_splitk(int want, int64_t M, int64_t N, int kblocks, size_t avail) {
  int s = want > 32 ? 32 : want;
  if (s > kblocks / 2) s = kblocks / 2;
  const size_t per_split = static_cast<size_t>(M) * N * sizeof(float);
  if (per_split > 0 && static_cast<size_t>(s) * per_split > avail) s = static_cast<int>(avail / per_split);
  return s < 1 ? 1 : s;
}

// Output columns per workgroup of the DMA-staged decode kernels.  A CU streams weights at a rate of its own (about
// 1 / 256 of what the chip reaches), so the launch takes as long as its busiest CU: the split that gives every CU
// the same number of weight rows wins, e.g. 28 columns for N = 7168 on 256 CUs (256 workgroups) instead of 32 (224),
// or 12 for N = 2112 (176 workgroups) instead of 16 (132).  Every workgroup also reads all activation rows (from the
// L2, cheaper per row); several rounds of workgroups cost in proportion.  Multiples of 4 keep a lane's four output
// columns inside one workgroup and one 128-column scale block.
int pick_skinny_bn(int64_t N, int act_rows, int cus) {
  int best = 16;
  double best_cost = 0.0;
  for (int bn = 4; bn <= 32; bn += 4) {
    const int64_t wgs = ceil_div(N, bn);
    const double cost = static_cast<double>(ceil_div(wgs, cus)) * (bn + 0.4 * act_rows);
    if (bn == 4 || cost < best_cost - 1e-9) best = bn, best_cost = cost;
  }
  return best;
}

// Dense problems between decode and prefill (a few hundred rows, or more rows against a narrow weight matrix): too
// few 256 x 256 tiles to fill the chip, and weight rows that come from HBM because only one or two row tiles use
// them.  There a K step of a DMA-ring kernel lasts about (latency of HBM under load) / (stages in flight), whatever
// the tile size, so the estimate below is: launches + rounds of workgroups x (fixed part of a tile + K steps x time
// per step) + the second pass when K is split.  Constants measured on MI355X (microseconds; bytes per microsecond).
struct MidChoice {
  int variant, splitk;
  double us;
};

constexpr int64_t kRelayoutMinRows = 128;  // dense / grouped launches with more rows re-lay row-major activation scales first

MidChoice pick_mid_plan(int64_t M, int64_t N, int kblocks, int cus, size_t ws_avail) {
  struct Cand { int variant, bm, bn; double step_us; };
  static const Cand cands[] = {{kVarPipe128x256w8, 128, 256, 0.85}, {kVarPipe128x128, 128, 128, 0.65}, {kVarPipe128x64, 128, 64, 0.50}};
  const double launch = 2.6, relayout = M > kRelayoutMinRows ? 2.3 : 0.5, tile_fixed = 2.5, second_pass = 2.5, ws_rate = 3.5e6;
  // scales fetched in place (no re-layout pass): one more line request per row and K step
  const double scattered = M > kRelayoutMinRows ? 1.0 : 1.0 + 0.25 * static_cast<double>(M) / 128.0;
  MidChoice best{kVarPipe128x256w8, 1, 1e30};
  const double out_bytes = static_cast<double>(M) * N * sizeof(float);
  // fewer rows than the 128 of a tile: the clamped rows repeat lines that are already on their way
  const double short_rows = M >= 128 ? 1.0 : 0.6 + 0.4 * static_cast<double>(M) / 128.0;
  for (const Cand& c : cands) {
    for (int want : {1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16}) {
      if (want > 1 && (kblocks / want < 4 || out_bytes * want > static_cast<double>(ws_avail))) continue;
      // more than 8 slices only while a slice keeps 8 K blocks (48 x 1024 x 16384: 17.9 -> 14.9 us with 16 slices;
      // 64 x 576 x 7168: 11.0 -> 12.1 us with 14)
      if (want > 8 && kblocks / want < 8) continue;
      const int per = static_cast<int>(ceil_div(kblocks, want));
      const int sk = static_cast<int>(ceil_div(kblocks, per));
      const int64_t units = ceil_div(M, c.bm) * ceil_div(N, c.bn) * sk;
      // the small tiles fetch a tile's scales once, into a table in LDS, when the slice is short enough: no re-layout
      // launch and no scattered scale lines per K step
      const bool table = (c.variant == kVarPipe128x64 && per <= Pipe128x64T::SCTAB_KB) || (c.variant == kVarPipe128x128 && per <= Pipe128x128T::SCTAB_KB);
      double us = launch + (table ? 0.0 : relayout) +
                  static_cast<double>(ceil_div(units, cus)) * (tile_fixed + per * c.step_us * short_rows * (table ? 1.0 : scattered));
      if (sk > 1) us += second_pass + (2.0 * sk + 0.5) * out_bytes / ws_rate;  // partial sums written, read back, result written
      if (us < best.us) best = MidChoice{c.variant, sk, us};
    }
  }
  return best;
}

// dma_ok: the DMA kernels address their sources with 32-bit byte offsets from the tile's first row (up to 256 rows x K
// bytes, 512 scale rows x stride); false sends such problems to the kernels with 64-bit addressing.
// G, hint_rows (grouped layouts): experts, and the masked layout's typical rows per expert (<= 0: unknown).
// fixed_grouped: the caller needs the 128 x 256 kernel (the fused activation epilogues exist for it only).
Plan make_plan(int mode, int64_t M, int64_t N, int64_t K, int cus, size_t ws_bytes, bool dma_ok, int G = 1,
               int64_t hint_rows = -1, bool fixed_grouped = false) {
  Plan pl{kVarTile128x128, 128, 128, 1, 4, 4, 1, 16, dma_ok};
  const int kblocks = static_cast<int>(ceil_div(K, kScaleBlock));
  const size_t ws_avail = ws_bytes > DLB_WS_COUNTER_BYTES ? ws_bytes - DLB_WS_COUNTER_BYTES : 0;
  int mid_splitk = 0;  // K slices chosen together with a DMA-ring variant
  int v = g_forced_variant;
  if (v < 0) {
    const bool whole_blocks = K > 0 && K % kScaleBlock == 0;
    if (K % 16 != 0) {
      v = kVarExact;
    } else if (mode == kDense && M <= 128) {
      // decode: stream the weights once, K split over the waves of a workgroup
      v = M <= 16 ? kVarSkinny16 : (M <= 32 ? kVarSkinny32 : (M <= 64 ? kVarSkinny64 : kVarSkinny128));
      // more than 64 rows against a narrow weight matrix: the few workgroups of the streaming kernel would each
      // re-read the whole activation matrix from L2; K split over workgroups in two passes is twice as fast there
      // (measured at M = 128: 2112 x 7168 44 -> 22 us, 4096 x 7168 45 -> 23 us; 7168 x 2048 stays: 16 vs 19 us)
      if (M > 64 && kblocks >= 32 && ceil_div(N, 128) * 2 <= cus) v = kVarTile128x128;
      if (M > 32 && whole_blocks) {
        // 33 .. 128 rows: the streaming kernel costs what is larger of its workgroups each reading all activation rows
        // from the L2 (about 8.5 TB/s over the chip) and of its waves' K blocks, fetched one after the other: a round
        // of 8 blocks lasts 0.8 x (0.14 us + 24 ns per activation row + 40 ns per weight row of the workgroup) (measured at
        // 33 .. 128 rows, 4 .. 28 weight rows, K = 2048 .. 16384).  A K-split tile kernel wins when the weight matrix
        // is narrow and K long (2112 x 7168: 18.3 -> 14.1 us at 64 rows, 29 -> 17.4 us at 128; at 33 rows the streaming
        // kernel stays ahead, 11.9 against 13.2 us)
        const int rows = M <= 64 ? 64 : 128;
        const int bn = pick_skinny_bn(N, rows, cus);
        const int64_t wgs = ceil_div(N, bn);
        const double m_eff = M <= 64 ? static_cast<double>(M) : 0.5 * (M + 128.0);  // the 128-row kernel computes all 8 row fragments
        const double round_us = 0.14 + 0.0239 * m_eff + 0.04 * bn;
        const double chain_us = 0.8 * round_us * static_cast<double>(ceil_div(kblocks, 8)) * static_cast<double>(ceil_div(wgs, cus));
        const double l2_us = static_cast<double>(wgs) * M * K / 8.5e6;
        const double stream_us = 2.6 + (l2_us > chain_us ? l2_us : chain_us);
        const MidChoice mid = pick_mid_plan(M, N, kblocks, cus, ws_avail);
        if (mid.us < stream_us) v = mid.variant, mid_splitk = mid.splitk;
        else v = M <= 64 ? kVarSkinny64 : kVarSkinny128;
      }
    } else if (whole_blocks && mode == kDense) {
      const int64_t t256 = ceil_div(M, 256) * ceil_div(N, 256);
      if (t256 * 2 >= cus) {
        v = prefers_128_row_tiles(M, N, kblocks, cus) ? kVarPipe128x256w8 : kVarPipe256mix;
      } else {
        const MidChoice mid = pick_mid_plan(M, N, kblocks, cus, ws_avail);
        v = mid.variant, mid_splitk = mid.splitk;
      }
    } else if (whole_blocks) {
      v = kVarPipe128x256w8;  // grouped: 128-row tiles never straddle two experts / waste at most 127 masked rows
      const int64_t tn = ceil_div(N, 256);
      if (fixed_grouped || (mode == kContiguous && g_knob[kKnobTileList] == 1)) {
      } else if (mode == kContiguous) {
        // a small batch: 128 x 128 tiles while 128 x 256 ones would leave half the CUs idle
        // (8 experts x 128 rows x 4096 x 7168: 67 -> 54 us)
        if (ceil_div(M, 128) * tn * 2 <= cus) v = kVarPipe128x128;
      } else if (hint_rows > 0) {
        // masked, with the caller's hint: few rows per expert and few experts - smaller tiles, as above (8 experts,
        // 4096 x 7168, up to 128 rows each: 54 - 75 -> 44 - 55 us); several hundred rows per expert - 256-row tiles,
        // which fetch an expert's weights once per 256 rows (32 experts x ~520 rows x 4096 x 7168: 665 -> 573 us,
        // 7168 x 2048: 363 -> 335 us)
        // (or two 128-row tiles per expert that fill one round at most: 8 experts x ~240 rows: 121 -> 110 us)
        const int64_t em = hint_rows < M ? hint_rows : M;
        const int64_t units = static_cast<int64_t>(G) * ceil_div(em, 128) * tn;
        if (units * 2 <= cus) v = kVarPipe128x128;
        else if (em >= 384 || (em >= 192 && units <= cus)) v = kVarPipe256x256;
      }
    } else {
      v = (M <= 64 && mode != kContiguous) ? kVarTile64x128 : kVarTile128x128;
    }
  }
  if (K % 16 != 0) v = kVarExact;
  if (is_pipelined(v) && (K % kScaleBlock != 0 || K == 0 || !dma_ok)) v = kVarTile128x128;  // DMA path moves whole K blocks
  if ((v == kVarPipe256x256 || v == kVarPipe256mix) && mode == kContiguous) v = kVarPipe128x256w8;
  if (v == kVarPipe256mix && mode != kDense) v = kVarPipe256x256;
  if (is_skinny(v) && (mode != kDense || M > skinny_rows(v))) v = kVarTile128x128;
  if (v == kVarExact && mode != kDense) v = kVarTile128x128;
  pl.variant = v;
  tile_dims(v, &pl.bm, &pl.bn);
  if (mode == kDense && is_pipelined(v) && mid_splitk > 1) pl.splitk = mid_splitk;
  // tuning knob: a K slice count for the dense tile kernels (twice the block count lets clamp_splitk go down to one
  // block per slice)
  const bool knob_splitk = g_knob[kKnobSplitK] > 0 && mode == kDense && v != kVarExact && !is_skinny(v) && v != kVarPipe256mix;
  if (knob_splitk) pl.splitk = clamp_splitk(g_knob[kKnobSplitK], M, N, kblocks * 2, ws_avail);
  if (mode != kDense || v == kVarExact || is_pipelined(v) || (kblocks < 2 && !is_skinny(v))) return pl;

  const int64_t tiles_n = ceil_div(N, pl.bn);
  const size_t avail = ws_bytes > DLB_WS_COUNTER_BYTES ? ws_bytes - DLB_WS_COUNTER_BYTES : 0;
  if (is_skinny(v)) {
    // K is split over the waves of a workgroup only.  Pick the wave count so that every wave has two or so K
    // blocks and the unroll so that a wave issues all of its loads before its first MFMA.
    int waves = kblocks >= 4 ? 8 : 4;  // (4 K blocks: 16 x 32768 x 512 7.4 -> 6.4 us with 8 waves, half of them without a block)
    // A long K against few rows: 16 waves keep twice the weight bytes in flight (1 x 2112 x 7168: 7.3 -> 6.0 us) - as
    // long as the workgroup's share of the weights is small (up to 16 rows of K = 7168: 16 x 4096 x 7168 8.4 -> 8.2 us,
    // 16 x 1536 x 7168 7.6 -> 6.4 us; from 20 rows on 8 waves are ahead: 16 x 7168 x 16384 21.7 -> 20.5 us) and one
    // round of workgroups covers the matrix (16 x 36864 x 7168: 55 -> 47 us with 8 waves).
    // (from 24 K blocks on for up to 8 rows: 1 x 4096 x 4096 6.0 -> 5.25 us, 1 x 3072 x 3072 4.9 -> 4.4 us)
    if (skinny_rows(v) == 16 && kblocks >= (M <= 8 ? 24 : 48) && K % kScaleBlock == 0) {
      const int bn16 = g_knob[kKnobSkinnyBn] > 0 ? g_knob[kKnobSkinnyBn] : pick_skinny_bn(N, 16, cus);
      // (a single row moves the limit up: 1 x 4608 x 7168, 20 rows of K = 7168 per workgroup, 9.4 -> 8.5 us with 16 waves)
      const int64_t share_limit = (M <= 8 ? 160 : 128) * 1024;
      if (static_cast<int64_t>(bn16) * K <= share_limit && ceil_div(N, bn16) <= cus) waves = 16;
    }
    if (g_knob[kKnobSkinnyWaves] > 0) waves = g_knob[kKnobSkinnyWaves] >= 16 ? 16 : (g_knob[kKnobSkinnyWaves] >= 8 ? 8 : 4);
    const int per_wave = static_cast<int>(ceil_div(kblocks, waves));
    // measured on MI355X: one K block in flight per wave is as good as more once eight waves share a row block
    int unroll = waves >= 8 ? 1 : (per_wave >= 3 ? 4 : 2);
    if (g_knob[kKnobSkinnyUnroll] > 0) unroll = g_knob[kKnobSkinnyUnroll];
    // two weight fragments per workgroup halve the activation re-reads, but only while the grid still covers the chip
    int nfrags = ceil_div(N, 32) * 4 >= 3 * cus ? 2 : 1;
    if (g_knob[kKnobSkinnyNFrags] > 0) nfrags = g_knob[kKnobSkinnyNFrags];
    pl.sk_waves = waves, pl.sk_unroll = unroll, pl.sk_nfrags = nfrags >= 2 ? 2 : 1;
    pl.sk_bn = 16 * pl.sk_nfrags;
    if (g_knob[kKnobSkinnyNFrags] <= 0 && K % kScaleBlock == 0) {
      pl.sk_bn = g_knob[kKnobSkinnyBn] > 0 ? g_knob[kKnobSkinnyBn] : pick_skinny_bn(N, skinny_rows(v), cus);
      if (pl.sk_bn % 4 != 0 || pl.sk_bn < 4 || pl.sk_bn > 32) pl.sk_bn = 16 * pl.sk_nfrags;
      pl.sk_nfrags = pl.sk_bn > 16 ? 2 : 1;
    }
    pl.bn = 16 * pl.sk_nfrags;
    // the reduction buffer (waves x fragments x 1 KB) has to fit the 160 KB of LDS whatever the knobs ask for
    const int frags = skinny_rows(v) / 16 * pl.sk_nfrags;
    while (pl.sk_waves > 4 && pl.sk_waves * frags * 1024 > 160 * 1024) pl.sk_waves /= 2;
  } else if (!knob_splitk) {
    // few tiles and a long K: split K over workgroups (partial sums in the workspace, second pass adds them)
    const int64_t tiles = ceil_div(M, pl.bm) * tiles_n;
    if (tiles * 2 > cus) return pl;
    pl.splitk = clamp_splitk(static_cast<int>(cus / tiles), M, N, kblocks, avail);  // one workgroup per CU: a single round
  }
  return pl;
}

// Everything the host decides about one launch, from shapes, strides and the workspace size alone: run() launches
// exactly this and dlb_fp8_gemm_plan reports it.
struct Resolved {
  Plan pl;
  int splitk, kb_per_split;  // K slices summed in a second pass (1 = none), K blocks per slice
  bool tile_list;            // expert-contiguous rows: device-built lists of 256-, 192- and 128-row tiles
  int64_t nblk;              //   128-row blocks it covers
  bool relayout;             // activation scales re-laid rows-contiguous in the workspace first
  int64_t rows_pad;          //   rows per K block of the re-laid copy
  size_t ws_used;            // bytes of the workspace's data region taken by list and scales; partial sums follow
  int64_t n_split;           // mixed-width launch: first column of the 192-wide tiles (N: uniform 256-wide tiles)
  int64_t grid;              // workgroups of the main kernel
  bool resident;             // dense launch of many rounds: one resident workgroup per CU walks the tiles
  bool sctab;                // small ring kernels: row-major activation scales through the per-tile table in LDS
  int sct_pitch;             //   floats per table row (odd)
  bool fused;                // K slices added inside the launch (counters in the workspace head), no second pass
};

// fused_act: the launch is one of the gate/up GEMMs with the activation in its epilogue (their kernels take no scale table)
Resolved resolve(int mode, int64_t rows, int64_t N, int64_t K, int G, int64_t as_sm, int64_t as_sk, bool have_ws,
                 size_t ws_bytes, int cus, bool gather_scales = false, bool fused_act = false, int64_t hint_rows = -1) {
  Resolved r{};
  const int64_t kblocks = ceil_div(K, kScaleBlock);
  const int64_t groups = mode == kMasked ? G : 1;  // a_s is per expert only in the masked layout; contiguous rows are one matrix
  const bool dma_ok = K < (1ll << 24) && as_sm < (1ll << 21);
  const bool usable_ws = have_ws && ws_bytes > DLB_WS_COUNTER_BYTES;
  r.pl = make_plan(mode, rows, N, K, cus, usable_ws ? ws_bytes : 0, dma_ok, G, hint_rows, fused_act || gather_scales);
  const Plan& pl = r.pl;
  const int want = usable_ws ? pl.splitk : 1;
  r.kb_per_split = static_cast<int>(ceil_div(kblocks > 0 ? kblocks : 1, want));
  r.splitk = static_cast<int>(ceil_div(kblocks > 0 ? kblocks : 1, r.kb_per_split));  // no empty slice
  r.n_split = N;
  if (mode == kContiguous && pl.variant == kVarPipe128x256w8 && g_forced_variant < 0 && usable_ws && kblocks > 0) {
    const int64_t nblk = ceil_div(rows, kScaleBlock);
    const size_t bytes = tile_list_bytes(nblk);
    // Taller tiles save weight traffic, not time per tile.  Estimates (microseconds, constants as in
    // prefers_128_row_tiles): uniform 128-row tiles take rounds x (5.5 + 1.2 K blocks: most of their weights come from HBM) or, when that is longer, the time
    // to stream every block's weight matrix (6.4 TB/s: neighbouring tiles of an expert share some of it in the L2);
    // the lists take 5 us for their pre-pass + rounds x (11.5 + 1.62 K blocks) or the weights of their tiles at
    // 4.85 TB/s, with as many tiles as pairs of blocks, but at least one per expert.  8 experts, 1408 rows, 4096 x
    // 7168: 107 us with lists, 69 us without; 2432 rows: 106 us with, 128 us without; 32 experts x 128 rows: 183 / 174.
    // The fused epilogues exist for the list kernel only.
    bool worth_it = fused_act || gather_scales || g_knob[kKnobTileList] == 1;
    if (!worth_it && g_knob[kKnobTileList] != 2 && nblk > G) {
      const int64_t tn = ceil_div(N, 256);
      const double mat_mb = static_cast<double>(N) * static_cast<double>(K) * 1e-6;
      const double plain_us = std::max(static_cast<double>(ceil_div(nblk * tn, cus)) * (5.5 + 1.2 * static_cast<double>(kblocks)),
                                       static_cast<double>(nblk) * mat_mb / 6.4);
      const int64_t tall = std::max(ceil_div(nblk, 2), std::min<int64_t>(nblk, G));
      const double list_us = 5.0 + std::max(static_cast<double>(ceil_div(tall * tn, cus)) * (11.5 + 1.62 * static_cast<double>(kblocks)),
                                            static_cast<double>(tall) * mat_mb / 4.85);
      worth_it = list_us < plain_us;
    }
    if (worth_it && nblk <= kTileListMaxBlocks && DLB_WS_COUNTER_BYTES + bytes <= ws_bytes) r.tile_list = true, r.nblk = nblk, r.ws_used = bytes;
  }
  // Small ring kernels with at most 32 K blocks per workgroup fetch a tile's row-major scales once, into a table in
  // LDS: no re-layout pass, one cache-line request per row and tile.
  const bool small_ring = pl.variant == kVarPipe128x128 || pl.variant == kVarPipe128x64;
  // (the masked layout's 128 x 256 tiles take the table too: a decode-sized K, no re-layout launch in front)
  const bool masked_ring = mode == kMasked && pl.variant == kVarPipe128x256w8 && !gather_scales && !fused_act && g_forced_variant < 0;
  auto table_fits = [&](int kb_per) {
    return ((mode == kDense && small_ring) || masked_ring) && g_knob[kKnobScaleTable] != 2 && as_sm != 1 &&
           kb_per <= (masked_ring ? Pipe128x256w8T::SCTAB_KB
                                  : (pl.variant == kVarPipe128x64 ? Pipe128x64T::SCTAB_KB : Pipe128x128T::SCTAB_KB)) &&
           as_sk < (1ll << 20) && dma_ok;
  };
  r.sctab = table_fits(r.kb_per_split);
  // gather_scales: the re-layout pass also brings the rows into the GEMM's order, so it runs whatever the strides
  if (is_pipelined(pl.variant) && usable_ws && !r.sctab &&
      (gather_scales ? kblocks > 0 : as_sk == 1 && as_sm > 1 && kblocks > 1 && rows > kRelayoutMinRows)) {
    // row-major activation scales: re-lay them rows-contiguous in the workspace first (a few microseconds) so the
    // GEMM fetches 8 cache lines of scales per K step and tile instead of 256.  Up to 128 rows the extra launch costs
    // more than the scattered scale lines (64 x 2112 x 7168: 15.9 -> 14.1 us without it)
    const int64_t rows_pad = (rows + 3) / 4 * 4;
    const int64_t need = groups * kblocks * rows_pad * static_cast<int64_t>(sizeof(float));
    if (static_cast<size_t>(need) + r.ws_used + DLB_WS_COUNTER_BYTES <= ws_bytes && rows_pad * kblocks < (1ll << 31)) {
      r.relayout = true, r.rows_pad = rows_pad;
      r.ws_used += (static_cast<size_t>(need) + 255) / 256 * 256;
    }
  }
  if (r.splitk > 1 && is_pipelined(pl.variant)) {
    // One launch: the workgroups of a tile add its slices themselves.  Needs a single round of workgroups (they wait
    // for each other, for a bounded time), a counter slot per tile and at most 32 slices (one claim bit each).
    const int64_t tiles = ceil_div(rows, pl.bm) * ceil_div(N, pl.bn);
    // Opt-in: on MI355X the device-scope round trips of that hand-over (stores out, counter, loads back) cost about
    // 3 us more than ending the launch and starting a reduction kernel behind it.
    r.fused = mode == kDense && g_knob[kKnobSplitKMode] == 1 && tiles <= kFusedMaxTiles && r.splitk <= 32 && tiles * r.splitk <= cus;
    // the partial sums of the K slices follow whatever else lives in the workspace (whole tiles in the one-launch
    // form, a [rows][N] matrix per slice otherwise); fewer slices if they do not fit
    const size_t avail = ws_bytes - DLB_WS_COUNTER_BYTES - r.ws_used;
    const size_t per_slice = r.fused ? static_cast<size_t>(tiles) * pl.bm * pl.bn * sizeof(float) : static_cast<size_t>(rows) * N * sizeof(float);
    if (per_slice * r.splitk > avail) {
      const int fit = per_slice > 0 && avail / per_slice >= 1 ? static_cast<int>(avail / per_slice) : 1;
      r.kb_per_split = static_cast<int>(ceil_div(kblocks, fit));
      r.splitk = static_cast<int>(ceil_div(kblocks, r.kb_per_split));
    }
    if (r.splitk <= 1) r.fused = false;
  }
  if (r.sctab && !table_fits(r.kb_per_split)) r.sctab = false;  // fewer, longer slices than the table holds: scales in place
  if (r.sctab)
    r.sct_pitch = r.kb_per_split | 1;
  if (pl.variant == kVarPipe256mix) r.n_split = pick_mixed_split(rows, N, cus);
  const int64_t tiles_m = ceil_div(rows, pl.bm), tiles_n = ceil_div(N, pl.bn);
  int64_t grid = tiles_m * tiles_n * r.splitk;
  if (mode == kMasked) {
    // the real tile count is only known on the device: a persistent grid
    const int64_t worst = tiles_m * tiles_n * G;
    // One resident workgroup per CU that walks its tiles: equal tiles need no balancing by the hardware's dispatcher,
    // and every further workgroup a CU has to start costs it about 2 us (32 x 256 x 7168 x 2048: 145 -> 137 us).
    const int64_t per_cu = g_knob[kKnobMaskedGrid] > 0 ? g_knob[kKnobMaskedGrid] : 1;
    grid = worst < static_cast<int64_t>(cus) * per_cu ? worst : static_cast<int64_t>(cus) * per_cu;
    grid = (grid + 31) / 32 * 32;  // the ring kernels deal tiles to the XCDs four at a time
  }
  // Dense launches of many rounds of equal tiles run one resident workgroup per CU that walks its tiles itself (the
  // ring kernels loop over tiles anyway): saves the hardware's per-workgroup start, 4 % at six rounds.
  r.resident = mode == kDense && grid >= 4ll * cus;
  r.grid = grid;
  return r;
}

struct Problem {
  int mode;
  const void *a, *b;
  const float *a_s, *b_s;
  void* c;
  const int32_t* gidx;
  int64_t rows;  // dense: M, contiguous: M_sum, masked: M_max
  int64_t N, K;
  int G;
  int64_t as_sg, as_sm, as_sk;
  int out_dtype;
  void* ws;
  size_t ws_bytes;
  hipStream_t stream;
  // fused gate/up epilogue (dlb_fp8_gemm_grouped_{contiguous,masked}_silu_quant): c is then the e4m3 output
  // [rows][N / 2] ([G][rows][N / 2] masked)
  float* act_s = nullptr;
  int64_t act_s_sg = 0, act_s_sm = 0, act_s_sk = 0;
  // ... reading its activation rows through a table (dlb_fp8_gemm_grouped_contiguous_gather_silu_quant): row r of the
  // GEMM is row a_rows[r] of a [a_src_rows][K]; a_s has a_src_rows rows too
  const int32_t* a_rows = nullptr;
  int64_t a_src_rows = 0;
  float act_eps = 0.f;
  bool act = false;
  int64_t hint_rows = -1;  // masked layout: the caller's expected_m
};


// Argument checks that need no device.  Returns DLB_OK with *empty set when there is nothing to compute.
int check_problem(const Problem& pr, bool* empty) {
  g_err[0] = '\0';
  *empty = false;
  if (pr.out_dtype != DLB_OUT_BF16 && pr.out_dtype != DLB_OUT_F32)
    return fail(DLB_ERR_BAD_DTYPE, "out_dtype %d is neither DLB_OUT_BF16 nor DLB_OUT_F32", pr.out_dtype);
  if (pr.rows < 0 || pr.N < 0 || pr.K < 0)
    return fail(DLB_ERR_BAD_SHAPE, "negative dimension (rows=%lld N=%lld K=%lld)", (long long)pr.rows,
                (long long)pr.N, (long long)pr.K);
  const int64_t lim = (1ll << 31) - 1024;
  if (pr.rows > lim || pr.N > lim || pr.K > lim)
    return fail(DLB_ERR_BAD_SHAPE, "dimension beyond 2^31 (rows=%lld N=%lld K=%lld)", (long long)pr.rows,
                (long long)pr.N, (long long)pr.K);
  if (pr.mode != kDense && pr.G < 0) return fail(DLB_ERR_BAD_SHAPE, "negative group count %d", pr.G);
  const int64_t groups = pr.mode == kDense ? 1 : pr.G;
  if (pr.rows == 0 || pr.N == 0 || groups == 0) {
    *empty = true;
    return DLB_OK;
  }
  if (!pr.c) return fail(DLB_ERR_NULL_POINTER, "c is NULL");
  if (pr.mode != kDense && !pr.gidx)
    return fail(DLB_ERR_NULL_POINTER, "%s is NULL", pr.mode == kContiguous ? "m_indices" : "masked_m");
  if (pr.K > 0 && (!pr.a || !pr.b || !pr.a_s || !pr.b_s))
    return fail(DLB_ERR_NULL_POINTER, "a, b, a_s or b_s is NULL");
  if (pr.mode != kDense && pr.K % 16 != 0)
    return fail(DLB_ERR_BAD_SHAPE, "grouped GEMM needs K %% 16 == 0 (K=%lld)", (long long)pr.K);
  const int64_t kblocks = ceil_div(pr.K, kScaleBlock);
  if (pr.K > 0) {
    if (pr.as_sm < 0 || pr.as_sk < 0 || pr.as_sg < 0)
      return fail(DLB_ERR_BAD_STRIDE, "negative a_s stride");
    if (pr.rows > 1 && pr.as_sm == 0) return fail(DLB_ERR_BAD_STRIDE, "a_s row stride is 0 for %lld rows", (long long)pr.rows);
    if (kblocks > 1 && pr.as_sk == 0) return fail(DLB_ERR_BAD_STRIDE, "a_s K-block stride is 0 for %lld blocks", (long long)kblocks);
    if (pr.mode == kMasked && pr.G > 1 && pr.as_sg == 0) return fail(DLB_ERR_BAD_STRIDE, "a_s group stride is 0");
  }
  const bool mfma_path = pr.K % 16 == 0;
  if (mfma_path && pr.K > 0 && (misaligned(pr.a, 16) || misaligned(pr.b, 16)))
    return fail(DLB_ERR_ALIGNMENT, "a and b must be 16-byte aligned");
  if (misaligned(pr.c, 2) || misaligned(pr.a_s, 4) || misaligned(pr.b_s, 4))
    return fail(DLB_ERR_ALIGNMENT, "c / a_s / b_s are not aligned to their element size");
  return DLB_OK;
}

int run(const Problem& pr) {
  bool empty = false;
  const int bad = check_problem(pr, &empty);
  if (bad != DLB_OK || empty) return bad;
  const int64_t groups = pr.mode == kDense ? 1 : pr.G;
  const int64_t kblocks = ceil_div(pr.K, kScaleBlock);

  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");

  if (pr.ws && misaligned(pr.ws, 16)) return fail(DLB_ERR_ALIGNMENT, "workspace must be 16-byte aligned");
  const Resolved rs = resolve(pr.mode, pr.rows, pr.N, pr.K, pr.G, pr.as_sm, pr.as_sk, pr.ws != nullptr, pr.ws_bytes, cus,
                              pr.a_rows != nullptr, pr.act, pr.hint_rows);
  const Plan& pl = rs.pl;
  // everything that can refuse the launch is checked before the first pre-pass kernel is enqueued
  if (rs.grid > (1ll << 30)) return fail(DLB_ERR_BAD_SHAPE, "too many tiles (%lld)", (long long)rs.grid);
  if (pl.variant == kVarExact && pr.mode != kDense) return fail(DLB_ERR_BAD_SHAPE, "exact path is dense only");
  if (pr.act) {
    // the fused epilogue exists for the tile-list kernel (contiguous) and the 128 x 256 ring kernel (masked) only:
    // whole 128-blocks of K and of the output, a workspace for the list, no forced variant; anything else is the
    // caller's cue to run the GEMM and the activation apart
    const bool kernel_ok = pr.mode == kContiguous ? rs.tile_list : pr.mode == kMasked && pl.variant == kVarPipe128x256w8;
    if (!kernel_ok || pr.K % kScaleBlock != 0 || pr.N % (2 * kScaleBlock) != 0 || pr.N * pr.K >= (1ll << 32))
      return fail(DLB_ERR_BAD_SHAPE,
                  "fused activation needs K %% 128 == 0, N %% 256 == 0, N K < 2^32%s (N=%lld K=%lld)",
                  pr.mode == kContiguous ? " and a workspace for the tile list" : "", (long long)pr.N, (long long)pr.K);
    if (!pr.act_s || misaligned(pr.act_s, 4) || misaligned(pr.c, 8))
      return fail(DLB_ERR_ALIGNMENT, "out_s is NULL or misaligned, or out_q is not 8-byte aligned");
    if (pr.act_s_sm < 0 || pr.act_s_sk < 0 || pr.act_s_sg < 0) return fail(DLB_ERR_BAD_STRIDE, "negative out_s stride");
    if (pr.a_rows) {
      // 32-bit DMA offsets count from the first row of the source matrix; its scales are gathered by the re-layout pass
      if (pr.mode != kContiguous || !rs.relayout || pr.a_src_rows <= 0 || pr.a_src_rows * pr.K >= (1ll << 32))
        return fail(DLB_ERR_BAD_SHAPE, "gathered activation rows need a workspace for their scales and rows * K < 2^32 (rows=%lld K=%lld)",
                    (long long)pr.a_src_rows, (long long)pr.K);
      if (misaligned(pr.a_rows, 4)) return fail(DLB_ERR_ALIGNMENT, "a_row_index is misaligned");
    }
  }
  if (pl.variant == kVarExact && ceil_div(pr.N, 64) > (1ll << 31) - 1) return fail(DLB_ERR_BAD_SHAPE, "N too large for the exact path");

  Args ar;
  memset(&ar, 0, sizeof(ar));
  ar.a = static_cast<const uint8_t*>(pr.a);
  ar.b = static_cast<const uint8_t*>(pr.b);
  ar.a_s = pr.a_s;
  ar.b_s = pr.b_s;
  ar.c = pr.c;
  ar.gidx = pr.gidx;
  ar.M = static_cast<int>(pr.rows);
  ar.N = static_cast<int>(pr.N);
  ar.K = static_cast<int>(pr.K);
  ar.G = pr.mode == kDense ? 1 : pr.G;
  ar.kblocks = static_cast<int>(kblocks);
  ar.nblocks = static_cast<int>(ceil_div(pr.N, kScaleBlock));
  ar.as_sm = pr.as_sm;
  ar.as_sk = pr.as_sk;
  ar.as_gs = pr.as_sg;
  ar.a_gs = pr.rows * pr.K;
  ar.c_gs = pr.rows * pr.N;
  ar.b_gs = pr.N * pr.K;
  ar.bs_gs = static_cast<int64_t>(ar.nblocks) * kblocks;
  ar.tiles_m = static_cast<int>(ceil_div(pr.rows, pl.bm));
  ar.tiles_n = static_cast<int>(ceil_div(pr.N, pl.bn));
  ar.sk_bn = pl.sk_bn;
  ar.splitk = rs.splitk;
  ar.kb_per_split = rs.kb_per_split;
  ar.group_m = g_knob[kKnobGroupM] > 0 ? g_knob[kKnobGroupM] : 8;
  ar.out_f32 = pr.out_dtype == DLB_OUT_F32;
  ar.a_rows = pr.a_rows;
  ar.act_s = pr.act_s;
  ar.act_s_gs = pr.act_s_sg;
  ar.act_s_sm = pr.act_s_sm;
  ar.act_s_sk = pr.act_s_sk;
  ar.act_eps = pr.act_eps;
  ar.act_cols = static_cast<int>(pr.N / 2);
  ar.act_q_stride = pr.N / 2;
  ar.vec_store = (pr.N % 4 == 0) && !misaligned(pr.c, 4 * (ar.out_f32 ? 4 : 2));
  ar.c_vec16 = !ar.out_f32 && pr.N % 8 == 0 && !misaligned(pr.c, 16) && g_knob[kKnobEpilogue] != 2;
  if (pr.ws && pr.ws_bytes >= DLB_WS_COUNTER_BYTES) {
    ar.ctr = static_cast<uint32_t*>(pr.ws);
    ar.ws = reinterpret_cast<float*>(static_cast<char*>(pr.ws) + DLB_WS_COUNTER_BYTES);
  }

  hipError_t e = hipSuccess;
  ar.fused_reduce = rs.fused ? 1 : 0;
  ar.spin_limit = g_knob[kKnobSpinLimit] > 0 ? g_knob[kKnobSpinLimit] - 1 : kDefaultSpinLimit;
  ar.sct_pitch = rs.sct_pitch;
  const bool tile_list = rs.tile_list;
  const size_t esz = ar.out_f32 ? 4 : 2;

  // The main kernel of the call.  With g_prepare_only set it only raises the kernel's dynamic-LDS limit (the one
  // step of a launch that can still fail), so that run() can do that before it enqueues the first pre-pass.
  auto main_kernel = [&]() -> hipError_t {
    switch (pl.variant) {
      case kVarExact: {
        if (g_prepare_only) return hipSuccess;
        // rows in a grid-stride loop: the second grid dimension is limited to 65535
        const int64_t row_groups = ceil_div(pr.rows, 4);
        const dim3 grid(static_cast<unsigned>(ceil_div(pr.N, 64)), static_cast<unsigned>(row_groups < 65535 ? row_groups : 65535));
        hipLaunchKernelGGL(fp8_gemm_exact_kernel, grid, dim3(256), 0, pr.stream, ar);
        return hipGetLastError();
      }
      case kVarSkinny16:
        return launch_skinny(1, pl.sk_nfrags, pl.sk_waves, pl.sk_unroll, pl.sk_dma, ar, dev, pr.stream);
      case kVarSkinny32:
        return launch_skinny(2, pl.sk_nfrags, pl.sk_waves, pl.sk_unroll, pl.sk_dma, ar, dev, pr.stream);
      case kVarSkinny64:
        return launch_skinny(4, pl.sk_nfrags, pl.sk_waves, pl.sk_unroll, pl.sk_dma, ar, dev, pr.stream);
      case kVarSkinny128:
        return launch_skinny(8, pl.sk_nfrags, pl.sk_waves, pl.sk_unroll, pl.sk_dma, ar, dev, pr.stream);
      default:
        break;
    }
    const int g = static_cast<int>(rs.grid);
    const int g_dense = rs.resident ? cus : g;
    if (pl.variant == kVarPipe256mix) {
      const int64_t split = rs.n_split;
      if (split >= pr.N) return launch_pipelined_mode<Pipe256x256>(pr.mode, ar, g_dense, dev, pr.stream);
      static std::atomic<unsigned long long> lds_done{0};
      auto kernel = fp8_gemm_pipelined_mixed_kernel<Pipe256x256, Pipe256x192>;
      ar.n_split = static_cast<int>(split);
      ar.tiles_n_a = static_cast<int>(split / 256);
      ar.tiles_n_b = static_cast<int>(ceil_div(pr.N - split, 192));
      ar.tiles_a = ar.tiles_m * ar.tiles_n_a;
      const hipError_t le = ensure_lds(kernel, Pipe256x256::LDS_BYTES, dev, &lds_done);
      if (le != hipSuccess || g_prepare_only) return le;
      hipLaunchKernelGGL(kernel, dim3(ar.tiles_a + ar.tiles_m * ar.tiles_n_b), dim3(Pipe256x256::NT), Pipe256x256::LDS_BYTES,
                         pr.stream, ar);
      return hipGetLastError();
    }
    if (pl.variant == kVarPipe256x256) return launch_pipelined_mode<Pipe256x256>(pr.mode, ar, g_dense, dev, pr.stream);
    if (pl.variant == kVarPipe128x256w8 && tile_list && pr.act) {
      static std::atomic<unsigned long long> lds_done{0};
      auto kernel = fp8_gemm_contig_list_act_kernel<Pipe256x256, Pipe192x256, Pipe128x256w8>;
      const hipError_t le = ensure_lds(kernel, kListLds, dev, &lds_done);
      if (le != hipSuccess || g_prepare_only) return le;
      ar.tiles_n = static_cast<int>(pr.N / 256);  // 128 output columns = 128 gate + 128 up weight rows per tile
      hipLaunchKernelGGL(kernel, dim3(cus), dim3(Pipe256x256::NT), kListLds, pr.stream, ar);
      return hipGetLastError();
    }
    if (pl.variant == kVarPipe128x256w8 && tile_list) {
      static std::atomic<unsigned long long> lds_done{0};
      auto kernel = fp8_gemm_contig_list_kernel<Pipe256x256, Pipe192x256, Pipe128x256w8>;
      const hipError_t le = ensure_lds(kernel, kListLds, dev, &lds_done);
      if (le != hipSuccess || g_prepare_only) return le;
      ar.tiles_n = static_cast<int>(ceil_div(pr.N, 256));
      hipLaunchKernelGGL(kernel, dim3(cus), dim3(Pipe256x256::NT), kListLds, pr.stream, ar);  // one resident workgroup per CU
      return hipGetLastError();
    }
    if (pl.variant == kVarPipe128x256w8 && pr.act)
      return launch_pipelined<Pipe128x256w8, kMaskedAct>(ar, g, dev, pr.stream);  // N / 256 column tiles, as the plain GEMM
    if (pl.variant == kVarPipe128x256w8 && pr.mode == kMasked && rs.sctab) return launch_pipelined<Pipe128x256w8T, kMasked>(ar, g, dev, pr.stream);
    if (pl.variant == kVarPipe128x256w8) return launch_pipelined_mode<Pipe128x256w8>(pr.mode, ar, g_dense, dev, pr.stream);
    if (pl.variant == kVarPipe128x128)
      return rs.sctab ? launch_pipelined<Pipe128x128T, kDense>(ar, g, dev, pr.stream)
                      : launch_pipelined_mode<Pipe128x128>(pr.mode, ar, g, dev, pr.stream);
    if (pl.variant == kVarPipe128x64)
      return rs.sctab ? launch_pipelined<Pipe128x64T, kDense>(ar, g, dev, pr.stream)
                      : launch_pipelined_mode<Pipe128x64>(pr.mode, ar, g, dev, pr.stream);
    if (pl.variant == kVarTile64x128) return launch_tiled_mode<Tile64x128>(pr.mode, ar, g, dev, pr.stream);
    if (pl.variant == kVarTile128x64) return launch_tiled_mode<Tile128x64>(pr.mode, ar, g, dev, pr.stream);
    return launch_tiled_mode<Tile128x128>(pr.mode, ar, g, dev, pr.stream);
  };
  g_prepare_only = true;
  e = main_kernel();
  g_prepare_only = false;
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "the kernel's LDS size was refused, nothing enqueued: %s", hipGetErrorString(e));

  // workspace data region: [tile list][re-laid scales][partial sums of the K slices]
  size_t ws_used = 0;
  const bool one_prepass = tile_list && rs.relayout && pr.mode == kContiguous;
  if (one_prepass) {
    // tile list and scale re-layout in one launch
    int32_t* tl = reinterpret_cast<int32_t*>(ar.ws);
    ws_used = tile_list_bytes(rs.nblk);
    float* relaid = reinterpret_cast<float*>(reinterpret_cast<char*>(ar.ws) + ws_used);
    const int tiles_x = static_cast<int>(ceil_div(rs.rows_pad, 32));
    const dim3 pgrid(static_cast<unsigned>(tiles_x + 1), static_cast<unsigned>(ceil_div(kblocks, 32)), 1);
    hipLaunchKernelGGL(contiguous_prepass_kernel, pgrid, dim3(256), 0, pr.stream, pr.gidx, static_cast<int>(pr.rows), pr.G, tl,
                       static_cast<int>(rs.nblk), pr.a_s, relaid, static_cast<int>(kblocks), static_cast<int>(rs.rows_pad), pr.as_sm,
                       pr.as_sk, pr.a_rows, tiles_x);
    e = hipGetLastError();
    if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "pre-pass launch failed: %s", hipGetErrorString(e));
    ar.tlist = tl;
    ar.tlist_cap = static_cast<int>(rs.nblk);
    ar.a_s = relaid;
    ar.as_sm = 1;
    ar.as_sk = rs.rows_pad;
    ar.as_gs = kblocks * rs.rows_pad;
  }
  if (tile_list && !one_prepass) {
    // expert-contiguous rows: device-built lists of 256-, 192- and 128-row tiles (see contiguous_tile_list_block)
    int32_t* tl = reinterpret_cast<int32_t*>(ar.ws);
    hipLaunchKernelGGL(contiguous_tile_list_kernel, dim3(1), dim3(256), 0, pr.stream, pr.gidx, static_cast<int>(pr.rows), pr.G, tl,
                       static_cast<int>(rs.nblk));
    e = hipGetLastError();
    if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "tile list launch failed: %s", hipGetErrorString(e));
    ar.tlist = tl;
    ar.tlist_cap = static_cast<int>(rs.nblk);
    ws_used = tile_list_bytes(rs.nblk);
  }
  if (rs.relayout && !one_prepass) {
    float* relaid = reinterpret_cast<float*>(reinterpret_cast<char*>(ar.ws) + ws_used);
    const dim3 tgrid(static_cast<unsigned>(ceil_div(rs.rows_pad, 32)), static_cast<unsigned>(ceil_div(kblocks, 32)),
                     static_cast<unsigned>(pr.mode == kMasked ? groups : 1));
    hipLaunchKernelGGL(fp8_scale_transpose_kernel, tgrid, dim3(256), 0, pr.stream, pr.a_s, relaid, static_cast<int>(pr.rows),
                       static_cast<int>(kblocks), static_cast<int>(rs.rows_pad), pr.mode == kMasked ? pr.as_sg : 0, pr.as_sm,
                       pr.as_sk, pr.a_rows);
    e = hipGetLastError();
    if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "scale re-layout launch failed: %s", hipGetErrorString(e));
    ar.a_s = relaid;
    ar.as_sm = 1;
    ar.as_sk = rs.rows_pad;
    ar.as_gs = kblocks * rs.rows_pad;
  }
  if (ar.splitk > 1 && is_pipelined(pl.variant)) ar.ws = reinterpret_cast<float*>(reinterpret_cast<char*>(ar.ws) + rs.ws_used);
  e = main_kernel();
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  if (ar.splitk > 1 && !rs.fused && pr.mode == kDense && pl.variant != kVarExact && !is_skinny(pl.variant)) {
    const int64_t total = pr.rows * pr.N;
    const int vec_ok = total % 4 == 0 && !misaligned(pr.c, 4 * esz);
    hipLaunchKernelGGL(fp8_splitk_reduce_kernel, dim3(static_cast<unsigned>(ceil_div(ceil_div(total, 4), 256))), dim3(256), 0,
                       pr.stream, ar.ws, pr.c, total, ar.splitk, ar.out_f32, vec_ok);
    e = hipGetLastError();
    if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "split-K reduction launch failed: %s", hipGetErrorString(e));
  }
  return DLB_OK;
}

// The slice of `scratch` that calls on `stream` work in.  The array's device address is looked up once per device
// (with that device current) and kept; a stream is bound to the first free slice of its device at its first call and
// keeps it until the process ends, so calls on different streams never share scratch memory.  More streams than slices:
// DLB_ERR_WORKSPACE.
int static_scratch_slice(hipStream_t stream, void** out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void*> ptr_of[kMaxDevices];
  static std::atomic<uintptr_t> owner[kMaxDevices][DLB_STATIC_SCRATCH_SLICES];  // 0 = free, else the stream handle + 1
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  if (dev < 0 || dev >= kMaxDevices) return fail(DLB_ERR_LAUNCH, "device ordinal %d beyond the %d this library tracks", dev, kMaxDevices);
  void* ptr = ptr_of[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail(DLB_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    ptr_of[dev].store(ptr, std::memory_order_release);
  }
  const uintptr_t key = reinterpret_cast<uintptr_t>(stream) + 1;
  for (int i = 0; i < DLB_STATIC_SCRATCH_SLICES; ++i) {
    uintptr_t cur = owner[dev][i].load(std::memory_order_acquire);
    if (cur == 0 && owner[dev][i].compare_exchange_strong(cur, key, std::memory_order_acq_rel)) cur = key;
    if (cur == key) {
      *out = static_cast<char*>(ptr) + static_cast<size_t>(i) * DLB_STATIC_SCRATCH_SLICE_BYTES;
      return DLB_OK;
    }
  }
  return fail(DLB_ERR_WORKSPACE,
              "the %d slices of the static scratch of device %d are bound to other streams; use dlb_fp8_gemm with a workspace "
              "for this stream", DLB_STATIC_SCRATCH_SLICES, dev);
}

template <int IN>
void launch_quant_group(const QuantArgs& qa, int lanes, unsigned blocks, hipStream_t st) {
  const dim3 grid(blocks), block(256);
  switch (lanes) {
    case 1: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 1>), grid, block, 0, st, qa); break;
    case 2: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 2>), grid, block, 0, st, qa); break;
    case 4: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 4>), grid, block, 0, st, qa); break;
    case 8: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 8>), grid, block, 0, st, qa); break;
    case 16: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 16>), grid, block, 0, st, qa); break;
    case 32: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 32>), grid, block, 0, st, qa); break;
    case 64: hipLaunchKernelGGL((fp8_quant_group_kernel<IN, 64>), grid, block, 0, st, qa); break;
    default: hipLaunchKernelGGL(fp8_quant_group_generic_kernel<IN>, grid, block, 0, st, qa);
  }
}

}  // namespace
}  // namespace dlb

// ---------------------------------------------------------------------------------------------------------
// extern "C" surface
// ---------------------------------------------------------------------------------------------------------
extern "C" {

int dlb_abi_version(void) { return DLB_ABI_VERSION; }

const char* dlb_last_error(void) { return dlb::g_err; }

size_t dlb_fp8_gemm_workspace_bytes(int64_t rows, int64_t N, int64_t K) {
  (void)K;
  if (rows <= 0 || N <= 0) return DLB_WS_COUNTER_BYTES;
  // Split-K only runs while the un-split grid cannot fill the chip, so (tiles x splits) stays within a few
  // hundred fp32 tiles of at most 128 x 128: 32 MiB covers every plan; the planner lowers the split count to
  // fit whatever it is given.
  const size_t cap = static_cast<size_t>(32) << 20;
  const int64_t padded = dlb::ceil_div(rows, 128) * dlb::ceil_div(N, 128);
  const size_t want = padded > 1024 ? cap : static_cast<size_t>(padded) * 128 * 128 * sizeof(float) * 16;
  return DLB_WS_COUNTER_BYTES + (want < cap ? want : cap);
}

int dlb_fp8_gemm(const void* a, const void* b, const float* a_s, const float* b_s, void* c, int64_t M, int64_t N,
                 int64_t K, int64_t as_stride_m, int64_t as_stride_k, int out_dtype, void* workspace,
                 size_t workspace_bytes, void* stream) {
  dlb::Problem pr{dlb::kDense, a, b, a_s, b_s, c, nullptr, M, N, K, 1, 0, as_stride_m, as_stride_k, out_dtype,
                  workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  return dlb::run(pr);
}

int dlb_fp8_gemm_noalloc(const void* a, const void* b, const float* a_s, const float* b_s, void* c, int64_t M, int64_t N,
                         int64_t K, int64_t as_stride_m, int64_t as_stride_k, int out_dtype, void* stream) {
  dlb::Problem pr{dlb::kDense, a, b, a_s, b_s, c, nullptr, M, N, K, 1, 0, as_stride_m, as_stride_k, out_dtype,
                  nullptr, 0, static_cast<hipStream_t>(stream)};
  bool empty = false;
  const int bad = dlb::check_problem(pr, &empty);
  if (bad != DLB_OK || empty) return bad;
  // What the plan of this problem would keep in a workspace of any size besides the partial sums of K slices (those
  // adapt to the space there is): the activation scales re-laid rows-contiguous.  That has to fit a slice.
  int dev = 0;
  const int cus = dlb::device_cu_count(&dev);
  if (cus < 0) return dlb::fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  const dlb::Resolved want = dlb::resolve(dlb::kDense, M, N, K, 1, as_stride_m, as_stride_k, true, static_cast<size_t>(1) << 40, cus);
  const size_t room = DLB_STATIC_SCRATCH_SLICE_BYTES - DLB_WS_COUNTER_BYTES;
  if (want.ws_used > room)
    return dlb::fail(DLB_ERR_WORKSPACE,
                     "M=%lld x ceil(K/128)=%lld needs %lld bytes of re-laid scales, a slice of the static scratch holds %lld; use "
                     "dlb_fp8_gemm with a workspace", (long long)M, (long long)dlb::ceil_div(K, dlb::kScaleBlock), (long long)want.ws_used,
                     (long long)room);
  void* ws = nullptr;
  const int rc = dlb::static_scratch_slice(pr.stream, &ws);
  if (rc != DLB_OK) return rc;
  pr.ws = ws;
  pr.ws_bytes = DLB_STATIC_SCRATCH_SLICE_BYTES;
  return dlb::run(pr);
}

int dlb_fp8_gemm_grouped_contiguous(const void* a, const void* b, const float* a_s, const float* b_s, void* c,
                                    const int32_t* m_indices, int64_t M_sum, int64_t N, int64_t K, int32_t G,
                                    int64_t as_stride_m, int64_t as_stride_k, int out_dtype, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  dlb::Problem pr{dlb::kContiguous, a, b, a_s, b_s, c, m_indices, M_sum, N, K, G, 0, as_stride_m, as_stride_k,
                  out_dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  return dlb::run(pr);
}

int dlb_fp8_gemm_grouped_contiguous_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s, void* out_q,
                                               float* out_s, const int32_t* m_indices, int64_t M_sum, int64_t N, int64_t K,
                                               int32_t G, int64_t as_stride_m, int64_t as_stride_k, int64_t os_stride_m,
                                               int64_t os_stride_k, float eps, void* workspace, size_t workspace_bytes,
                                               void* stream) {
  dlb::Problem pr{dlb::kContiguous, a, b, a_s, b_s, out_q, m_indices, M_sum, N, K, G, 0, as_stride_m, as_stride_k,
                  DLB_OUT_BF16, workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  pr.act = true;
  pr.act_s = out_s;
  pr.act_s_sm = os_stride_m;
  pr.act_s_sk = os_stride_k;
  pr.act_eps = eps;
  if (M_sum > 0 && N > 0 && G > 0 && !out_s) return dlb::fail(DLB_ERR_NULL_POINTER, "out_s is NULL");
  return dlb::run(pr);
}

int dlb_fp8_gemm_grouped_contiguous_gather_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s,
                                                      void* out_q, float* out_s, const int32_t* m_indices,
                                                      const int32_t* a_row_index, int64_t a_rows, int64_t M_sum, int64_t N,
                                                      int64_t K, int32_t G, int64_t as_stride_m, int64_t as_stride_k,
                                                      int64_t os_stride_m, int64_t os_stride_k, float eps, void* workspace,
                                                      size_t workspace_bytes, void* stream) {
  dlb::Problem pr{dlb::kContiguous, a, b, a_s, b_s, out_q, m_indices, M_sum, N, K, G, 0, as_stride_m, as_stride_k,
                  DLB_OUT_BF16, workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  pr.act = true;
  pr.act_s = out_s;
  pr.act_s_sm = os_stride_m;
  pr.act_s_sk = os_stride_k;
  pr.act_eps = eps;
  pr.a_rows = a_row_index;
  pr.a_src_rows = a_rows;
  if (M_sum > 0 && N > 0 && G > 0 && !out_s) return dlb::fail(DLB_ERR_NULL_POINTER, "out_s is NULL");
  if (M_sum > 0 && N > 0 && G > 0 && !a_row_index) return dlb::fail(DLB_ERR_NULL_POINTER, "a_row_index is NULL");
  return dlb::run(pr);
}

int dlb_fp8_gemm_grouped_masked_silu_quant(const void* a, const void* b, const float* a_s, const float* b_s, void* out_q,
                                           float* out_s, const int32_t* masked_m, int32_t expected_m, int64_t M_max,
                                           int64_t N, int64_t K, int32_t G, int64_t as_stride_g, int64_t as_stride_m,
                                           int64_t as_stride_k, int64_t os_stride_g, int64_t os_stride_m, int64_t os_stride_k,
                                           float eps, void* workspace, size_t workspace_bytes, void* stream) {
  (void)expected_m;
  dlb::Problem pr{dlb::kMasked, a, b, a_s, b_s, out_q, masked_m, M_max, N, K, G, as_stride_g, as_stride_m, as_stride_k,
                  DLB_OUT_BF16, workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  pr.act = true;
  pr.act_s = out_s;
  pr.act_s_sg = os_stride_g;
  pr.act_s_sm = os_stride_m;
  pr.act_s_sk = os_stride_k;
  pr.act_eps = eps;
  if (M_max > 0 && N > 0 && G > 0 && !out_s) return dlb::fail(DLB_ERR_NULL_POINTER, "out_s is NULL");
  return dlb::run(pr);
}

int dlb_fp8_gemm_grouped_masked(const void* a, const void* b, const float* a_s, const float* b_s, void* c,
                                const int32_t* masked_m, int32_t expected_m, int64_t M_max, int64_t N, int64_t K,
                                int32_t G, int64_t as_stride_g, int64_t as_stride_m, int64_t as_stride_k,
                                int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  dlb::Problem pr{dlb::kMasked, a, b, a_s, b_s, c, masked_m, M_max, N, K, G, as_stride_g, as_stride_m, as_stride_k,
                  out_dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
  pr.hint_rows = expected_m;
  return dlb::run(pr);
}

int dlb_fp8_quant_group(const void* x, int x_dtype, void* q, float* s, int64_t rows, int64_t K, int64_t group_size,
                        int64_t x_row_stride, int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream) {
  using namespace dlb;
  g_err[0] = '\0';
  if (x_dtype < kInBf16 || x_dtype > kInF32) return fail(DLB_ERR_BAD_DTYPE, "x_dtype %d is not DLB_IN_BF16 / F16 / F32", x_dtype);
  if (rows < 0 || K < 0) return fail(DLB_ERR_BAD_SHAPE, "negative dimension (rows=%lld K=%lld)", (long long)rows, (long long)K);
  if (group_size <= 0) return fail(DLB_ERR_BAD_SHAPE, "group size %lld is not positive", (long long)group_size);
  if (K % group_size != 0)
    return fail(DLB_ERR_BAD_SHAPE, "K=%lld is not a multiple of the group size %lld", (long long)K, (long long)group_size);
  if (rows == 0 || K == 0) return DLB_OK;
  if (!x || !q || !s) return fail(DLB_ERR_NULL_POINTER, "x, q or s is NULL");
  const int64_t esz = x_dtype == kInF32 ? 4 : 2;
  if (x_row_stride < K) return fail(DLB_ERR_BAD_STRIDE, "x row stride %lld < K", (long long)x_row_stride);
  if (s_stride_m < 0 || s_stride_k < 0) return fail(DLB_ERR_BAD_STRIDE, "negative scale stride");
  if (misaligned(x, esz) || misaligned(s, 4)) return fail(DLB_ERR_ALIGNMENT, "x or s is not aligned to its element size");
  // the vector kernel: whole 16-byte loads and 8-byte stores per lane
  const bool vector_ok = group_size % 8 == 0 && group_size <= 512 && !misaligned(x, 16) && (x_row_stride * esz) % 16 == 0 && !misaligned(q, 8);
  if (group_size == kScaleBlock && !vector_ok) return fail(DLB_ERR_ALIGNMENT, "x rows must be 16-byte aligned, q 8-byte aligned");
  int lanes = 0;  // 0 = generic kernel
  if (vector_ok)
    for (lanes = 1; lanes * 8 < group_size; lanes *= 2) {
    }
  int dev = 0;
  const int cus = device_cu_count(&dev);
  if (cus < 0) return fail(DLB_ERR_LAUNCH, "hipGetDevice failed");
  QuantArgs qa{x, static_cast<uint8_t*>(q), s, rows, K / group_size, group_size, x_row_stride, s_stride_m, s_stride_k, eps};
  const int64_t groups = rows * (K / group_size);
  const int64_t per_block = lanes > 0 ? 4 * (64 / lanes) : 4;  // 4 waves x groups per wave and step
  int64_t blocks = ceil_div(groups, per_block);
  const int64_t cap = static_cast<int64_t>(cus) * 16;
  if (blocks > cap) blocks = cap;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (x_dtype == kInBf16)
    launch_quant_group<kInBf16>(qa, lanes, static_cast<unsigned>(blocks), st);
  else if (x_dtype == kInF16)
    launch_quant_group<kInF16>(qa, lanes, static_cast<unsigned>(blocks), st);
  else
    launch_quant_group<kInF32>(qa, lanes, static_cast<unsigned>(blocks), st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return DLB_OK;
}

int dlb_fp8_quant_1x128(const void* x, int x_dtype, void* q, float* s, int64_t rows, int64_t K, int64_t x_row_stride,
                        int64_t s_stride_m, int64_t s_stride_k, float eps, void* stream) {
  return dlb_fp8_quant_group(x, x_dtype, q, s, rows, K, dlb::kScaleBlock, x_row_stride, s_stride_m, s_stride_k, eps, stream);
}

int dlb_fp8_quant_128x128(const void* w, int w_dtype, void* q, float* s, int64_t G, int64_t N, int64_t K,
                          int64_t w_row_stride, float eps, void* stream) {
  using namespace dlb;
  g_err[0] = '\0';
  if (w_dtype < kInBf16 || w_dtype > kInF32) return fail(DLB_ERR_BAD_DTYPE, "w_dtype %d is not DLB_IN_BF16 / F16 / F32", w_dtype);
  if (G < 0 || N < 0 || K < 0)
    return fail(DLB_ERR_BAD_SHAPE, "negative dimension (G=%lld N=%lld K=%lld)", (long long)G, (long long)N, (long long)K);
  if (K % 8 != 0) return fail(DLB_ERR_BAD_SHAPE, "K=%lld is not a multiple of 8", (long long)K);
  if (G == 0 || N == 0 || K == 0) return DLB_OK;
  if (!w || !q || !s) return fail(DLB_ERR_NULL_POINTER, "w, q or s is NULL");
  const int64_t esz = w_dtype == kInF32 ? 4 : 2;
  if (w_row_stride < K) return fail(DLB_ERR_BAD_STRIDE, "w row stride %lld < K", (long long)w_row_stride);
  if (misaligned(w, 16) || (w_row_stride * esz) % 16 != 0 || misaligned(q, 8) || misaligned(s, 4))
    return fail(DLB_ERR_ALIGNMENT, "w rows must be 16-byte aligned, q 8-byte aligned");
  const int64_t nbn = ceil_div(N, kScaleBlock), nbk = ceil_div(K, kScaleBlock);
  const int64_t blocks = G * nbn * nbk;
  if (blocks >= (1ll << 31) || nbn >= (1ll << 30) || nbk >= (1ll << 30)) return fail(DLB_ERR_BAD_SHAPE, "too many blocks");
  BlockQuantArgs a{w, static_cast<uint8_t*>(q), s, N, K, w_row_stride, static_cast<int>(nbn), static_cast<int>(nbk), eps};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  if (w_dtype == kInBf16)
    hipLaunchKernelGGL(fp8_quant_128x128_kernel<kInBf16>, grid, block, 0, st, a);
  else if (w_dtype == kInF16)
    hipLaunchKernelGGL(fp8_quant_128x128_kernel<kInF16>, grid, block, 0, st, a);
  else
    hipLaunchKernelGGL(fp8_quant_128x128_kernel<kInF32>, grid, block, 0, st, a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return DLB_OK;
}

int dlb_fp8_gemm_plan(int mode, int64_t rows, int64_t N, int64_t K, size_t workspace_bytes, int compute_units, int* variant,
                      int* k_slices, int* decode_columns, int64_t* narrow_from) {
  dlb::clear_error();
  if (mode < dlb::kDense || mode > dlb::kMasked) return dlb::fail(DLB_ERR_BAD_SHAPE, "mode %d is not 0 (dense), 1 (contiguous) or 2 (masked)", mode);
  if (rows < 0 || N < 0 || K < 0) return dlb::fail(DLB_ERR_BAD_SHAPE, "negative dimension (rows=%lld, N=%lld, K=%lld)", (long long)rows, (long long)N, (long long)K);
  const int64_t lim = (1ll << 31) - 1024;
  if (rows > lim || N > lim || K > lim) return dlb::fail(DLB_ERR_BAD_SHAPE, "dimension beyond 2^31");
  if (compute_units <= 0) return dlb::fail(DLB_ERR_BAD_SHAPE, "compute_units must be positive");
  // row-major activation scales, as the dense Python entry point hands them over
  const dlb::Resolved rs = dlb::resolve(mode, rows, N, K, mode == dlb::kDense ? 1 : 32, dlb::ceil_div(K, dlb::kScaleBlock), 1,
                                        workspace_bytes > 0, workspace_bytes, compute_units);
  if (variant) *variant = rs.pl.variant;
  if (k_slices) *k_slices = rs.splitk;
  if (decode_columns) *decode_columns = dlb::is_skinny(rs.pl.variant) ? rs.pl.sk_bn : 0;
  if (narrow_from) *narrow_from = rs.n_split;
  return DLB_OK;
}

int dlb_fp8_gemm_plan_grouped(int mode, int64_t rows, int64_t N, int64_t K, int32_t G, int32_t expected_m, size_t workspace_bytes,
                              int compute_units, int* variant, int* tile_lists) {
  dlb::clear_error();
  if (mode != dlb::kContiguous && mode != dlb::kMasked) return dlb::fail(DLB_ERR_BAD_SHAPE, "mode %d is not 1 (contiguous) or 2 (masked)", mode);
  if (rows < 0 || N < 0 || K < 0 || G < 0) return dlb::fail(DLB_ERR_BAD_SHAPE, "negative dimension (rows=%lld, N=%lld, K=%lld, G=%d)", (long long)rows, (long long)N, (long long)K, G);
  const int64_t lim = (1ll << 31) - 1024;
  if (rows > lim || N > lim || K > lim) return dlb::fail(DLB_ERR_BAD_SHAPE, "dimension beyond 2^31");
  if (compute_units <= 0) return dlb::fail(DLB_ERR_BAD_SHAPE, "compute_units must be positive");
  const dlb::Resolved rs = dlb::resolve(mode, rows, N, K, G, dlb::ceil_div(K, dlb::kScaleBlock), 1, workspace_bytes > 0, workspace_bytes,
                                        compute_units, false, false, mode == dlb::kMasked ? expected_m : -1);
  if (variant) *variant = rs.pl.variant;
  if (tile_lists) *tile_lists = rs.tile_list ? 1 : 0;
  return DLB_OK;
}

int dlb_fp8_gemm_force_variant(int variant) {
  if (variant >= dlb::kVarCount) return dlb::fail(DLB_ERR_BAD_SHAPE, "unknown kernel variant %d", variant);
  dlb::g_forced_variant = variant < 0 ? -1 : variant;
  return DLB_OK;
}

int dlb_fp8_gemm_tune(int knob, int value) {
  if (knob < 0 || knob >= dlb::kKnobCount) return dlb::fail(DLB_ERR_BAD_SHAPE, "unknown tuning knob %d", knob);
  if (value < 0 || value > 1024) return dlb::fail(DLB_ERR_BAD_SHAPE, "tuning value %d outside [0, 1024]", value);
  dlb::g_knob[knob] = value;
  return DLB_OK;
}

const char* dlb_fp8_gemm_variant_name(int variant) {
  if (variant < 0 || variant >= dlb::kVarCount) return nullptr;
  return dlb::kVariantNames[variant];
}

// declared in include/dlblas_fp8_moe.h; lives here next to the kernel it shares with the GEMM's own pre-pass
int dlb_scale_relayout(const float* src, float* dst, int64_t rows, int64_t kblocks, int64_t rows_pad,
                       int64_t src_stride_m, int64_t src_stride_k, void* stream) {
  using namespace dlb;
  clear_error();
  if (rows < 0 || kblocks < 0 || rows_pad < rows)
    return fail(DLB_ERR_BAD_SHAPE, "bad dimensions (rows=%lld kblocks=%lld rows_pad=%lld)", (long long)rows, (long long)kblocks,
                (long long)rows_pad);
  if (rows_pad == 0 || kblocks == 0) return DLB_OK;
  if (!dst || (rows > 0 && !src)) return fail(DLB_ERR_NULL_POINTER, "src or dst is NULL");
  if (rows_pad >= (1ll << 31) || kblocks >= (1ll << 31) || ceil_div(kblocks, 32) > 65535)
    return fail(DLB_ERR_BAD_SHAPE, "dimensions beyond the supported range");
  const dim3 grid(static_cast<unsigned>(ceil_div(rows_pad, 32)), static_cast<unsigned>(ceil_div(kblocks, 32)), 1);
  hipLaunchKernelGGL(fp8_scale_transpose_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), src, dst,
                     static_cast<int>(rows), static_cast<int>(kblocks), static_cast<int>(rows_pad), static_cast<int64_t>(0),
                     src_stride_m, src_stride_k, static_cast<const int32_t*>(nullptr));
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DLB_ERR_LAUNCH, "scale_relayout launch failed: %s", hipGetErrorString(e));
  return DLB_OK;
}

}  // extern "C"
