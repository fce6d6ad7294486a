#!/usr/bin/env python3
"""Benchmark of the FP8 block-scaled GEMM hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path (one GEMM launch through the C ABI) over one batch of synthetic, already
quantised inputs that are resident in HBM before the timed region starts.  The default workload is the
compute-bound prefill GEMM M=4096, N=7168, K=18432 the metric is quoted on; the decode (HBM-bound) shape
M=16, N=7168, K=2048 is measured after the timed region and reported in the same JSON line under "decode".
Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA peak, TFLOP/s
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E peak, GB/s

WORKLOADS = {
    # name: (kind, M, N, K)
    'prefill_4096x7168x18432': ('dense', 4096, 7168, 18432),
    'prefill_4096x24576x1536': ('dense', 4096, 24576, 1536),
    'decode_16x7168x2048': ('dense', 16, 7168, 2048),
    'decode_16x2112x7168': ('dense', 16, 2112, 7168),
    'cpu_case_64x512x1024': ('dense', 64, 512, 1024),
}


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def algorithmic_bytes(M, N, K):
    """Each operand once, bf16 output once: M K + N K + 4 M ceil(K/128) + 4 ceil(N/128) ceil(K/128) + 2 M N."""
    kb, nb = -(-K // 128), -(-N // 128)
    return M * K + N * K + 4 * M * kb + 4 * nb * kb + 2 * M * N


def quantise_act(x):
    """1x128 groups: s = max(amax, 1e-10) / 448, q = clamp(x / s) -> e4m3fn (torch ops on the device)."""
    import torch
    M, K = x.shape
    g = x.float().reshape(M, K // 128, 128)
    s = g.abs().amax(-1, keepdim=True).clamp_min(1e-10) / 448.0
    q = (g / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).reshape(M, K)
    return q.contiguous(), s.reshape(M, K // 128).contiguous()


def quantise_weight(w):
    """128x128 blocks (ragged last N block allowed): s = block amax / 448."""
    import torch
    N, K = w.shape
    nb = -(-N // 128)
    pad = torch.zeros(nb * 128, K, dtype=torch.float32, device=w.device)
    pad[:N] = w.float()
    blk = pad.reshape(nb, 128, K // 128, 128)
    s = blk.abs().amax(dim=(1, 3), keepdim=True).clamp_min(1e-10) / 448.0
    q = (blk / s).clamp(-448.0, 448.0).reshape(nb * 128, K)[:N].to(torch.float8_e4m3fn)
    return q.contiguous(), s.reshape(nb, K // 128).contiguous()


def make_inputs(M, N, K, dev, seed=20, weight_copies=1):
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    a = torch.randn(M, K, device=dev, generator=g).to(torch.bfloat16)
    a_q, a_s = quantise_act(a)
    del a
    ws = []
    for _ in range(weight_copies):
        w = (torch.randn(N, K, device=dev, generator=g) * 0.02).to(torch.bfloat16)
        ws.append(quantise_weight(w))
        del w
    return a_q, a_s, ws


class DenseLauncher:
    """Pre-marshalled ctypes call of dlb_fp8_gemm on torch's current stream (no per-call tensor handling)."""

    def __init__(self, a_q, a_s, weights, out):
        import torch

        from dlblas_amd import _lib
        self.lib = _lib.load()
        self.keep = (a_q, a_s, weights, out)
        stream = torch.cuda.current_stream().cuda_stream
        ws = _lib.workspace(a_q.device, stream)
        M, K = a_q.shape
        self.calls = []
        for (b_q, b_s) in weights:
            N = b_q.shape[0]
            self.calls.append((ctypes.c_void_p(a_q.data_ptr()), ctypes.c_void_p(b_q.data_ptr()),
                               ctypes.c_void_p(a_s.data_ptr()), ctypes.c_void_p(b_s.data_ptr()),
                               ctypes.c_void_p(out.data_ptr()), M, N, K, a_s.stride(0), a_s.stride(1), _lib.OUT_BF16,
                               ctypes.c_void_p(ws.data_ptr()), ws.numel(), ctypes.c_void_p(stream)))
        self.i = 0

    def __call__(self):
        rc = self.lib.dlb_fp8_gemm(*self.calls[self.i])
        self.i = (self.i + 1) % len(self.calls)
        if rc != 0:
            from dlblas_amd import _lib
            _lib.check(rc)


def time_steps(launch, steps, warmup):
    """Wall clock over exactly `steps` launches between two synchronisations, plus the HIP-event time of the same
    launches on the launch stream (average kernel duration when launches are back to back)."""
    import torch
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        launch()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, start.elapsed_time(stop) / steps


def cpu_baseline(kind, M, N, K, a_q, a_s, b_q, b_s, budget_s=15.0):
    """The reference CPU path (dequantise to fp32, torch.matmul) timed on this host on a bounded row sample."""
    import torch

    from oracle import fp8_block_gemm as orc
    a_q, a_s, b_q, b_s = a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu()
    probe_rows = min(M, 32)
    t0 = time.perf_counter()
    orc.dequant_ref(a_q[:probe_rows], a_s[:probe_rows], b_q, b_s, torch.bfloat16)
    probe = time.perf_counter() - t0
    # the weight dequantisation is a fixed cost; scale rows so that the whole sample takes about budget_s
    t0 = time.perf_counter()
    orc.dequant_ref(a_q[:1], a_s[:1], b_q, b_s, torch.bfloat16)
    fixed = time.perf_counter() - t0
    per_row = max((probe - fixed) / max(probe_rows - 1, 1), 1e-9)
    rows = int(max(probe_rows, min(M, (budget_s - fixed) / per_row)))
    t0 = time.perf_counter()
    orc.dequant_ref(a_q[:rows], a_s[:rows], b_q, b_s, torch.bfloat16)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * N * K
    return {
        'value': flops / dt / 1e12,
        'unit': 'TFLOP/s',
        'cores': torch.get_num_threads(),
        'kind': 'port',
        'sample': f'first {rows} of {M} rows x N={N} x K={K} (dequantise both operands to fp32 + torch.matmul), '
                  f'{dt:.1f} s',
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='prefill_4096x7168x18432', choices=sorted(WORKLOADS))
    ap.add_argument('--variant', default=None, help='force a kernel variant (tuning)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-decode', action='store_true')
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import torch

    import dlblas_amd  # noqa: F401
    from dlblas_amd import _lib
    _lib.load()
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    if args.variant:
        _lib.force_variant(args.variant)

    kind, M, N, K = WORKLOADS[args.workload]
    log(f'workload {args.workload}: generating inputs')
    memory_bound = M <= 128
    copies = 24 if memory_bound else 1  # rotate weights so decode reads come from HBM, not the 256 MB cache
    a_q, a_s, weights = make_inputs(M, N, K, dev, weight_copies=copies)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    launch = DenseLauncher(a_q, a_s, weights, out)
    log('timing')
    ms_per_step, ev_ms = time_steps(launch, args.steps, args.warmup)
    flops = 2.0 * M * N * K
    nbytes = algorithmic_bytes(M, N, K)
    if memory_bound:
        value, unit = nbytes / (ms_per_step * 1e-3) / 1e9, 'GB/s'
        roofline = {'bound': 'hbm', 'achieved': nbytes / (ev_ms * 1e-3) / 1e9, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s'}
    else:
        value, unit = flops / (ms_per_step * 1e-3) / 1e12, 'TFLOP/s'
        roofline = {'bound': 'mfma', 'achieved': flops / (ev_ms * 1e-3) / 1e12, 'peak': PEAK_FP8_TFLOPS,
                    'unit': 'TFLOP/s'}
    roofline['frac'] = roofline['achieved'] / roofline['peak']
    roofline['traffic'] = None
    roofline['kernel_ms'] = ev_ms

    result = {
        'metric': 'FP8 block-scaled GEMM TFLOP/s (% FP8 MFMA peak); decode-M HBM GB/s',
        'value': value,
        'unit': unit,
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': ms_per_step,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'fp8_e4m3 x fp8_e4m3 -> f32 accumulate -> bf16',
        'data': 'synthetic',
        'config': {'workload': args.workload, 'M': M, 'N': N, 'K': K, 'a_scale': '1x128 f32', 'b_scale': '128x128 f32',
                   'out': 'bf16', 'seed': 20},
        'roofline': roofline,
    }

    if not args.no_decode and not memory_bound:
        dM, dN, dK = 16, 7168, 2048
        log(f'decode M={dM} N={dN} K={dK}')
        da_q, da_s, dws = make_inputs(dM, dN, dK, dev, weight_copies=24)
        dout = torch.empty(dM, dN, dtype=torch.bfloat16, device=dev)
        dl = DenseLauncher(da_q, da_s, dws, dout)
        d_wall, d_ev = time_steps(dl, 480, 48)
        db = algorithmic_bytes(dM, dN, dK)
        result['decode'] = {
            'workload': f'decode_{dM}x{dN}x{dK}', 'us_per_launch': d_ev * 1e3, 'GBps': db / (d_ev * 1e-3) / 1e9,
            'frac_of_hbm_peak': db / (d_ev * 1e-3) / 1e9 / PEAK_HBM_GBS, 'bytes': db,
            'note': '24 distinct weight copies in rotation (353 MB) so reads miss the 256 MB cache'
        }

    if not args.no_cpu_baseline:
        log('cpu baseline')
        b_q, b_s = weights[0]
        result['cpu_baseline'] = cpu_baseline(kind, M, N, K, a_q, a_s, b_q, b_s)
    print(json.dumps(result), flush=True)


if __name__ == '__main__':
    main()
