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
    'decode_64x2112x7168': ('dense', 64, 2112, 7168),
    'decode_128x2112x7168': ('dense', 128, 2112, 7168),
    'cpu_case_64x512x1024': ('dense', 64, 512, 1024),
}
# measured after the timed region and reported under "other_workloads" (name: M, N, K)
DECODE_SWEEP = [(m, n, k) for (n, k) in ((7168, 2048), (2112, 7168)) for m in (1, 16, 64, 128)]
# the dense MLP's projections of the same model at 16 rows: weight matrices large enough that the launch is not
# most of the time (132 and 264 MB)
DECODE_SWEEP += [(16, 7168, 18432), (16, 36864, 7168)]
GROUPED_CONTIGUOUS = dict(G=32, tokens=8192, N=4096, K=7168)
GROUPED_MASKED = dict(G=32, M_max=256, N=7168, K=2048)


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


def _timed(launch, steps):
    """Wall clock and HIP-event time (events on the launch stream) of exactly `steps` back-to-back launches."""
    import torch
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


SETTLE_MAX_LAUNCHES = 120


def settle(launch, block=10, tol=0.01):
    """Untimed launches of the step until the power controller has settled: a GPU that goes from idle to this load
    boosts, overshoots into a throttle and recovers over the first few tens of milliseconds (per-launch series in
    profiles/).  Blocks of `block` launches are timed until two consecutive blocks agree within `tol`, at most
    SETTLE_MAX_LAUNCHES launches.  Returns the number of launches made."""
    import torch
    done, prev = 0, None
    while done < SETTLE_MAX_LAUNCHES:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(block):
            launch()
        stop.record()
        torch.cuda.synchronize()
        done += block
        cur = start.elapsed_time(stop)
        if prev is not None and abs(cur - prev) <= tol * prev:
            break
        prev = cur
    return done


def time_steps(launch, steps, warmup):
    """The measurement of the headline workload.

    1. From an idle GPU: `warmup` untimed + `steps` timed launches.  Reported as "from_idle": on this part it is the
       power controller's start-up transient, not the kernel's rate.
    2. settle(): untimed launches until the per-launch time stops moving.
    3. `warmup` untimed launches, then EXACTLY `steps` timed launches between two synchronisations: wall clock
       (ms_per_step, value) and HIP events on the launch stream (roofline)."""
    import torch
    time.sleep(0.2)
    for _ in range(warmup):
        launch()
    idle_wall, idle_ev = _timed(launch, steps)
    settled = settle(launch)
    for _ in range(warmup):
        launch()
    wall, ev = _timed(launch, steps)
    return wall, ev, {'ms_per_step': idle_wall, 'kernel_ms': idle_ev, 'settle_launches': settled,
                      'launches_before_the_timed_region': warmup + steps + settled + warmup}


def cpu_baseline(kind, M, N, K, a_q, a_s, b_q, b_s, budget_s=12.0):
    """The reference CPU path (dequantise both operands to fp32, torch.matmul, cast to bf16) timed on this host:
    whole passes over a row sample of the workload, repeated until about `budget_s` seconds of CPU work are done."""
    import torch

    from oracle import fp8_block_gemm as orc
    a_q, a_s, b_q, b_s = a_q.cpu(), a_s.cpu(), b_q.cpu(), b_s.cpu()
    rows = min(M, 1024)
    t0 = time.perf_counter()
    orc.dequant_ref(a_q[:rows], a_s[:rows], b_q, b_s, torch.bfloat16)
    first = time.perf_counter() - t0
    if first < budget_s / 8 and rows < M:
        rows = M
    times = []
    spent = 0.0
    while spent < budget_s and len(times) < 50:
        t0 = time.perf_counter()
        orc.dequant_ref(a_q[:rows], a_s[:rows], b_q, b_s, torch.bfloat16)
        times.append(time.perf_counter() - t0)
        spent += times[-1]
    times.sort()
    dt = times[len(times) // 2]
    flops = 2.0 * rows * N * K
    return {
        'value': flops / dt / 1e12,
        'unit': 'TFLOP/s',
        'cores': torch.get_num_threads(),
        'kind': 'port',
        'sample': f'first {rows} of {M} rows x N={N} x K={K}: dequantise both operands to fp32 + torch.matmul + bf16 '
                  f'cast, median of {len(times)} passes ({spent:.1f} s of CPU work, {dt:.2f} s per pass)',
    }


def time_call(fn, iters, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def decode_sweep(dev):
    """HBM-bound shapes: distinct weight copies in rotation (24 of the small matrices, > 256 MB in all) so that reads
    come from HBM."""
    import torch
    rows = []
    for (M, N, K) in DECODE_SWEEP:
        copies = max(2, min(24, -(-400_000_000 // (N * K))))
        a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=copies)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        small = N * K < 50_000_000
        # 1500 untimed launches of a small matrix (~10 ms): clocks at their loaded level
        ms = time_call(DenseLauncher(a_q, a_s, ws, out), 480 if small else 120, 1500 if small else 300)
        nbytes = algorithmic_bytes(M, N, K)
        rows.append({'workload': f'decode_{M}x{N}x{K}', 'us_per_launch': ms * 1e3, 'GBps': nbytes / ms / 1e6,
                     'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'TFLOPs': 2.0 * M * N * K / ms / 1e9,
                     'bytes': nbytes})
        del a_q, a_s, ws, out
    return rows


FLOOR_LIB = os.path.join(ROOT, 'bench_kernels', 'libfloor_kernels.so')


def decode_floor(dev, N=7168, K=2048, copies=24):
    """What one launch of the decode shape costs on this GPU without any arithmetic (bench_kernels/floor_kernels.hip):
    an empty kernel of the decode kernel's grid, and a kernel that only reads the N x K weight bytes with 16-byte loads,
    both launched back to back on one stream over the same rotation of `copies` weight buffers as the decode sweep."""
    import torch
    if not os.path.exists(FLOOR_LIB):
        return None
    lib = ctypes.CDLL(FLOOR_LIB)
    lib.floor_empty.argtypes = [ctypes.c_int, ctypes.c_void_p]
    lib.floor_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.floor_read_store.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64,
                                     ctypes.c_void_p]
    bufs = [torch.randint(0, 255, (N * K, ), dtype=torch.uint8, device=dev) for _ in range(copies)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    state = {'i': 0}

    def reader(wgs, depth):
        def read():
            b = bufs[state['i']]
            state['i'] = (state['i'] + 1) % copies
            lib.floor_read(ctypes.c_void_p(b.data_ptr()), N * K, wgs, depth, stream)
        return read

    empty_ms = time_call(lambda: lib.floor_empty(cus, stream), 480, 1500)
    # the best of a few shapes of the read-only kernel: workgroups per CU x 16-byte loads in flight per thread
    tried = {}
    for per_cu in (1, 2, 4):
        for depth in (2, 4, 8):
            tried[f'{per_cu} wg/cu x {depth} loads'] = time_call(reader(cus * per_cu, depth), 240, 240) * 1e3
    best = min(tried, key=tried.get)
    read_us = time_call(reader(cus * int(best.split()[0]), int(best.split()[3])), 480, 1500) * 1e3
    # the same reads + one exchange between a workgroup's waves + the store of a 16-row bf16 result (fastest shape again)
    out16 = torch.empty(16 * N, dtype=torch.bfloat16, device=dev)

    def storer(wgs, depth):
        def run():
            b = bufs[state['i']]
            state['i'] = (state['i'] + 1) % copies
            lib.floor_read_store(ctypes.c_void_p(b.data_ptr()), N * K, wgs, depth, ctypes.c_void_p(out16.data_ptr()), out16.numel() * 2, stream)
        return run

    tried_store = {}
    for per_cu in (1, 2, 4):
        for depth in (2, 4, 8):
            tried_store[f'{per_cu} wg/cu x {depth} loads'] = time_call(storer(cus * per_cu, depth), 240, 240) * 1e3
    best_store = min(tried_store, key=tried_store.get)
    read_store_us = time_call(storer(cus * int(best_store.split()[0]), int(best_store.split()[3])), 480, 1500) * 1e3
    del bufs
    return {'empty_launch_us': empty_ms * 1e3, 'read_only_us': read_us, 'read_only_GBps': N * K / read_us / 1e3,
            'read_exchange_store_us': read_store_us, 'read_exchange_store_shape': best_store,
            'gemm_16_rows_us': decode_stream_loop(dev, 16, N, K, copies),
            'read_only_shape': best, 'bytes_read': N * K, 'gemm_16_rows_graph_replay_us': decode_graph_replay(dev, 16, N, K, copies),
            'note': 'bench-only kernels (bench_kernels/floor_kernels.hip), same rotation of weight buffers and same launch '
                    'loop as the decode rows; read_only = fastest of 9 shapes of a kernel that only loads the weight bytes; '
                    'read_exchange_store = the same reads, one LDS exchange between the waves of a workgroup and the store of a 16-row bf16 result; '
                    'graph_replay = the GEMM itself, 48 launches captured in a HIP graph and replayed'}


def decode_graph_replay(dev, M, N, K, copies):
    """Per-launch time of the decode GEMM when 48 launches over the rotating weight buffers are captured in a HIP graph
    and the graph is replayed: what is left of a launch when the host's part of it is taken away."""
    import torch
    a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=copies)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    per_graph = 2 * copies
    with torch.cuda.stream(side):
        launch = DenseLauncher(a_q, a_s, ws, out)  # its calls carry the side stream
        for _ in range(per_graph):
            launch()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(per_graph):
                launch()
        for _ in range(30):
            graph.replay()
        side.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(side)
        for _ in range(10):
            graph.replay()
        stop.record(side)
        side.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    return start.elapsed_time(stop) / (10 * per_graph) * 1e3


def decode_stream_loop(dev, M, N, K, copies):
    """Per-launch time of the decode GEMM in the loop the floors are measured in (launches back to back on one stream)."""
    import torch
    a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=copies)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    return time_call(DenseLauncher(a_q, a_s, ws, out), 480, 1500) * 1e3


def ceilings(dev):
    """What the GPU gives the prefill kernel's instruction mix and the grouped kernels' weight stream with everything
    else taken away (bench_kernels/floor_kernels.hip), measured like the workloads: launches back to back on one stream,
    timed after ~100 ms of the same load so that clocks are at their loaded level."""
    import torch
    if not os.path.exists(FLOOR_LIB):
        return None
    lib = ctypes.CDLL(FLOOR_LIB)
    lib.floor_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.floor_panel_stream.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                                       ctypes.c_int, ctypes.c_void_p]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    g = torch.Generator().manual_seed(20)
    codes = torch.randint(0, 256, (12288, ), generator=g, dtype=torch.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x30                       # no NaN codes
    operands = {'constant 1.0': torch.full((12288, ), 0x38, dtype=torch.uint8).to(dev), 'random e4m3 codes': codes.to(dev)}
    sink = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    iters = 400                                                 # ~1 ms per launch
    flop = cus * 8.0 * iters * 16 * 131072
    res = {'mfma_loop_TFLOPs': {}, 'panel_stream_GBps': {}}
    for name, buf in operands.items():
        for reads in (0, 3):
            def run(buf=buf, reads=reads):
                lib.floor_mfma(ctypes.c_void_p(buf.data_ptr()), ctypes.c_void_p(sink.data_ptr()), cus, iters, reads, stream)
            ms = time_call(run, 40, 100)
            res['mfma_loop_TFLOPs'][f'{name}, {reads} ds_read_b128 per MFMA pair'] = flop / ms / 1e9
    # 256-row panels of a [65536, 7168]-byte matrix (470 MB: past the 256 MB cache), the rows of one expert's weight tile
    panels, row_bytes = 256, 7168
    mat = torch.randint(0, 255, (panels * 256 * row_bytes, ), dtype=torch.uint8, device=dev)
    hot = torch.randint(0, 255, (16 * 256 * row_bytes, ), dtype=torch.uint8, device=dev)
    for hint in (0, 1):
        tag = ', non-temporal loads' if hint else ''
        for depth in (1, 2, 4):
            def run(depth=depth, hint=hint):
                lib.floor_panel_stream(ctypes.c_void_p(mat.data_ptr()), panels, row_bytes, cus, depth, None, 0, hint, stream)
            ms = time_call(run, 20, 20)
            res['panel_stream_GBps'][f'{depth} K steps (x 32 KB) in flight per workgroup{tag}'] = panels * 256 * row_bytes / ms / 1e6
        for depth in (1, 4):
            def run(depth=depth, hint=hint):
                lib.floor_panel_stream(ctypes.c_void_p(mat.data_ptr()), panels, row_bytes, 8, depth, None, 0, hint, stream)
            ms = time_call(run, 5, 3)
            res['panel_stream_GBps'][f'8 workgroups only (one per XCD), {depth} K steps in flight{tag}: per workgroup'] = \
                panels * 256 * row_bytes / ms / 1e6 / 8
        for depth in (1, 2):
            def run(depth=depth, hint=hint):
                lib.floor_panel_stream(ctypes.c_void_p(mat.data_ptr()), panels, row_bytes, cus, depth, ctypes.c_void_p(hot.data_ptr()), 16, hint,
                                       stream)
            ms = time_call(run, 20, 20)
            res['panel_stream_GBps'][f'{depth} K steps in flight, plus a shared (L2-resident) 256-row panel per step{tag}: HBM panel bytes only'] = \
                panels * 256 * row_bytes / ms / 1e6
    # what the path from the L2 into a CU delivers when every request hits: all workgroups pull the same 512 rows, 64 KB per
    # K step (the bytes a 256 x 256 tile needs per step), through the LDS DMA and through 16-byte register loads
    lib.floor_l2_stream.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    res['l2_stream'] = {}
    strip = torch.randint(0, 255, (512 * 18432, ), dtype=torch.uint8, device=dev)
    steps_per_launch = 2000
    for mode, name in ((0, 'LDS DMA'), (1, 'register loads')):
        for depth in (1, 2):
            def run(mode=mode, depth=depth):
                lib.floor_l2_stream(ctypes.c_void_p(strip.data_ptr()), 18432, cus, steps_per_launch, mode, depth, stream)
            ms = time_call(run, 10, 10)
            res['l2_stream'][f'{name}, {depth} K steps in flight'] = {'GBps_per_cu': steps_per_launch * 65536 / ms / 1e6,
                                                                       'ns_per_64KB_step': ms * 1e6 / steps_per_launch}
    res['note'] = ('l2_stream: one workgroup per CU, every request an L2 hit after the first touch (the prefill kernel moves 64 KB '
                   'per K step of about 1600 ns). mfma_loop: pairs of v_mfma_f32_32x32x64_f8f6f4 + 16 scale FMAs from registers, 8 waves per CU, no memory '
                   'traffic except the optional LDS reads (the prefill kernel issues 3 per pair); peak 5000 TFLOP/s. '
                   'panel_stream: one workgroup per CU pulls 256 x 7168-byte panels from HBM through the LDS DMA path, '
                   '128 bytes per row and K step, and computes nothing')
    return res


def second_prefill_workload(dev):
    """The other prefill shape of the metric's configuration: 4096 x 24576 x 1536, where the 201 MB of bf16 output are
    most of the bytes."""
    import torch
    M, N, K = 4096, 24576, 1536
    a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=1)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ms = time_call(DenseLauncher(a_q, a_s, ws, out), 60, 150)  # past the power controller's start-up transient
    flops, nbytes = 2.0 * M * N * K, algorithmic_bytes(M, N, K)
    return [{'workload': f'prefill_{M}x{N}x{K}', 'us_per_launch': ms * 1e3, 'TFLOPs': flops / ms / 1e9,
             'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS, 'GBps': nbytes / ms / 1e6,
             'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes}]


def chunked_prefill_workloads(dev):
    """Dense shapes between decode and prefill (a few hundred rows against the same weight matrices): too few large tiles
    for the chip, weights streamed from HBM.  Four weight copies in rotation."""
    import torch
    rows = []
    for (M, N, K) in ((256, 7168, 2048), (512, 4096, 7168), (256, 7168, 16384)):
        a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=4)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        ms = time_call(DenseLauncher(a_q, a_s, ws, out), 100, 10)
        flops, nbytes = 2.0 * M * N * K, algorithmic_bytes(M, N, K)
        rows.append({'workload': f'chunk_{M}x{N}x{K}', 'us_per_launch': ms * 1e3, 'TFLOPs': flops / ms / 1e9,
                     'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS, 'GBps': nbytes / ms / 1e6,
                     'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes})
        del a_q, a_s, ws, out
    return rows


def expert_weights(G, N, K, dev, seed):
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    qs, ss = [], []
    for _ in range(G):
        q, s = quantise_weight((torch.randn(N, K, device=dev, generator=g) * 0.02).to(torch.bfloat16))
        qs.append(q)
        ss.append(s)
    return torch.stack(qs), torch.stack(ss)


def grouped_workloads(dev):
    """One GPU's expert share of the two MoE layouts; FLOPs count real tokens only, bytes count every operand once."""
    import torch

    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous, fp8_gemm_grouped_masked
    rows = []
    # expert-contiguous (prefill): per-expert counts from a seeded multinomial, padded to multiples of 128
    c = GROUPED_CONTIGUOUS
    G, N, K = c['G'], c['N'], c['K']
    g = torch.Generator().manual_seed(20)
    assign = torch.multinomial(torch.full((G, ), 1.0 / G), c['tokens'], replacement=True, generator=g)
    counts = torch.bincount(assign, minlength=G)
    padded = (counts + 127) // 128 * 128
    M_sum = int(padded.sum())
    m_indices = torch.repeat_interleave(torch.arange(G, dtype=torch.int32), padded).to(dev)
    gd = torch.Generator(device=dev).manual_seed(21)
    a_q, a_s = quantise_act(torch.randn(M_sum, K, device=dev, generator=gd).to(torch.bfloat16))
    w_q, w_s = expert_weights(G, N, K, dev, 22)
    out = torch.empty(M_sum, N, dtype=torch.bfloat16, device=dev)
    ms = time_call(lambda: fp8_gemm_grouped_contiguous(a_q, a_s, w_q, w_s, out, m_indices), 40, 80)
    flops = 2.0 * c['tokens'] * N * K
    nbytes = M_sum * K + G * N * K + 4 * M_sum * (K // 128) + 4 * G * (N // 128) * (K // 128) + 2 * M_sum * N + 4 * M_sum
    rows.append({'workload': f'grouped_contiguous_E{G}_T{c["tokens"]}_N{N}_K{K}', 'M_sum_padded': M_sum,
                 'us_per_launch': ms * 1e3, 'TFLOPs': flops / ms / 1e9, 'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS,
                 'GBps': nbytes / ms / 1e6, 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS})
    # the same GEMM as the gate/up projection of the expert MLP (N = 2 x 2048), with silu * up and the 1 x 128 quantiser
    # in its epilogue; bytes: the bf16 output is replaced by the e4m3 activations and their scales
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous_silu_quant
    ms = time_call(lambda: fp8_gemm_grouped_contiguous_silu_quant(a_q, a_s, w_q, w_s, m_indices), 40, 80)
    nbytes_act = nbytes - 2 * M_sum * N + M_sum * (N // 2) + 4 * M_sum * (N // 256)
    rows.append({'workload': f'grouped_contiguous_silu_quant_E{G}_T{c["tokens"]}_I{N // 2}_K{K}', 'M_sum_padded': M_sum,
                 'us_per_launch': ms * 1e3, 'TFLOPs': flops / ms / 1e9, 'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS,
                 'GBps': nbytes_act / ms / 1e6, 'frac_of_hbm_peak': nbytes_act / ms / 1e6 / PEAK_HBM_GBS,
                 'note': 'includes the allocation of its two outputs'})
    del a_q, a_s, w_q, w_s, out
    # masked (decode): valid rows uniform in [0, M_max]
    c = GROUPED_MASKED
    G, M_max, N, K = c['G'], c['M_max'], c['N'], c['K']
    masked_m = torch.randint(0, M_max + 1, (G, ), generator=torch.Generator().manual_seed(20), dtype=torch.int32)
    a_q, a_s = quantise_act(torch.randn(G * M_max, K, device=dev, generator=gd).to(torch.bfloat16))
    a_q, a_s = a_q.reshape(G, M_max, K), a_s.reshape(G, M_max, K // 128)
    w_q, w_s = expert_weights(G, N, K, dev, 24)
    out = torch.empty(G, M_max, N, dtype=torch.bfloat16, device=dev)
    mm = masked_m.to(dev)
    hint = int(masked_m.float().mean())
    ms = time_call(lambda: fp8_gemm_grouped_masked(a_q, a_s, w_q, w_s, out, mm, hint), 60, 150)
    valid = int(masked_m.sum())
    flops = 2.0 * valid * N * K
    nbytes = valid * K + G * N * K + 4 * valid * (K // 128) + 4 * G * (N // 128) * (K // 128) + 2 * valid * N + 4 * G
    rows.append({'workload': f'grouped_masked_E{G}_Mmax{M_max}_N{N}_K{K}', 'valid_rows': valid,
                 'us_per_launch': ms * 1e3, 'TFLOPs': flops / ms / 1e9, 'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS,
                 'GBps': nbytes / ms / 1e6, 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS})
    return rows


def masked_gate_up_workload(dev):
    """The first half of the decode MoE layer (gate/up projection: 2 x 2048 weight rows, K = 7168) on 32 experts x 256 row
    slots with masked_m uniform in [0, 256]: masked GEMM + masked activation + quantiser as one kernel, and as the two
    kernels it replaces."""
    import torch

    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_masked, fp8_gemm_grouped_masked_silu_quant
    from dlblas_amd.kernels.moe import silu_and_mul_masked_post_quant_fwd
    c = GROUPED_MASKED
    G, M_max = c['G'], c['M_max']
    N, K = GROUPED_CONTIGUOUS['N'], GROUPED_CONTIGUOUS['K']
    masked_m = torch.randint(0, M_max + 1, (G, ), generator=torch.Generator().manual_seed(20), dtype=torch.int32)
    mm, hint, valid = masked_m.to(dev), int(masked_m.float().mean()), int(masked_m.sum())
    gd = torch.Generator(device=dev).manual_seed(23)
    a_q, a_s = quantise_act(torch.randn(G * M_max, K, device=dev, generator=gd).to(torch.bfloat16))
    a_q, a_s = a_q.reshape(G, M_max, K), a_s.reshape(G, M_max, K // 128)
    w_q, w_s = expert_weights(G, N, K, dev, 25)
    q = torch.empty(G, M_max, N // 2, dtype=torch.float8_e4m3fn, device=dev)
    q_s = torch.empty(G, M_max, N // 256, dtype=torch.float32, device=dev)
    gate_up = torch.empty(G, M_max, N, dtype=torch.bfloat16, device=dev)

    def two_steps():
        fp8_gemm_grouped_masked(a_q, a_s, w_q, w_s, gate_up, mm, hint)
        silu_and_mul_masked_post_quant_fwd(gate_up, q, q_s, 128, mm)

    ms2 = time_call(two_steps, 60, 150)
    ms = time_call(lambda: fp8_gemm_grouped_masked_silu_quant(a_q, a_s, w_q, w_s, q, q_s, mm, hint), 60, 150)
    flops = 2.0 * valid * N * K
    nbytes = valid * K + G * N * K + 4 * valid * (K // 128) + 4 * G * (N // 128) * (K // 128) + valid * (N // 2) + 4 * valid * (N // 256) + 4 * G
    return [{'workload': f'grouped_masked_silu_quant_E{G}_Mmax{M_max}_I{N // 2}_K{K}', 'valid_rows': valid,
             'us_per_launch': ms * 1e3, 'us_as_two_kernels': ms2 * 1e3, 'TFLOPs': flops / ms / 1e9,
             'frac_of_fp8_peak': flops / ms / 1e9 / PEAK_FP8_TFLOPS, 'GBps': nbytes / ms / 1e6,
             'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS}]


def quantiser_workload(dev):
    """The producer of (a, a_s): 1 x 128 quantisation of a bf16 [4096, 18432] activation; bytes = read + write."""
    import torch

    from dlblas_amd.kernels.fp8 import per_token_group_quant_fp8
    M, K = 4096, 18432
    x = torch.randn(M, K, device=dev, generator=torch.Generator(device=dev).manual_seed(20)).to(torch.bfloat16)
    from dlblas_amd import _lib
    x_q, x_s = per_token_group_quant_fp8(x, 128)
    lib = _lib.load()
    vp = ctypes.c_void_p
    args = (vp(x.data_ptr()), _lib.IN_CODES[x.dtype], vp(x_q.data_ptr()), vp(x_s.data_ptr()), M, K, K, K // 128, 1, 1e-10,
            vp(torch.cuda.current_stream().cuda_stream))
    ms = time_call(lambda: lib.dlb_fp8_quant_1x128(*args), 100, 10)
    nbytes = 2 * M * K + M * K + 4 * M * (K // 128)
    row = {'workload': f'quant_1x128_bf16_{M}x{K}', 'us_per_launch': ms * 1e3, 'GBps': nbytes / ms / 1e6,
           'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes}
    # the producer of (b, b_s): 128 x 128 block quantisation of a bf16 [7168, 18432] weight
    from dlblas_amd.kernels.fp8 import per_block_quant_fp8
    N = 7168
    w = (torch.randn(N, K, device=dev, generator=torch.Generator(device=dev).manual_seed(21)) * 0.02).to(torch.bfloat16)
    w_q, w_s = per_block_quant_fp8(w)
    wargs = (vp(w.data_ptr()), _lib.IN_CODES[w.dtype], vp(w_q.data_ptr()), vp(w_s.data_ptr()), 1, N, K, K, 1e-10,
             vp(torch.cuda.current_stream().cuda_stream))
    ms = time_call(lambda: lib.dlb_fp8_quant_128x128(*wargs), 50, 5)
    nbytes = 2 * N * K + N * K + 4 * (N // 128) * (K // 128)
    return [row, {'workload': f'quant_128x128_bf16_{N}x{K}', 'us_per_launch': ms * 1e3, 'GBps': nbytes / ms / 1e6,
                  'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes}]


def activation_workloads(dev):
    """The step between the two grouped GEMMs: silu(gate) * up + 1 x 128 quantisation.  Contiguous layout at the
    expert-contiguous shape (9728 padded rows, gate_up 4096 wide -> 2048 fp8), masked layout at the decode shape
    (32 experts x 256 rows capacity, gate_up 4096 wide).  bytes = bf16 read + fp8 and scale written (valid rows)."""
    import torch

    from dlblas_amd import _lib
    gd = torch.Generator(device=dev).manual_seed(20)
    rows = []
    M, N = 9728, 2048
    x = torch.randn(M, 2 * N, device=dev, generator=gd).to(torch.bfloat16)
    q2 = torch.empty(M, N, device=dev, dtype=torch.float8_e4m3fn)
    s2 = torch.empty(M, N // 128, device=dev, dtype=torch.float32)
    # pre-marshalled C calls with caller-owned outputs: the kernels take 10-30 us, less than a torch op dispatch
    lib = _lib.load()
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    args = (vp(x.data_ptr()), _lib.IN_CODES[x.dtype], vp(q2.data_ptr()), vp(s2.data_ptr()), M, N, 2 * N, N // 128, 1, 1e-10, stream)
    _lib.check(lib.dlb_silu_mul_quant(*args))
    ms = time_call(lambda: lib.dlb_silu_mul_quant(*args), 100, 10)
    nbytes = 4 * M * N + M * N + 4 * M * (N // 128)
    rows.append({'workload': f'silu_mul_quant_bf16_{M}x{2 * N}', 'us_per_launch': ms * 1e3, 'GBps': nbytes / ms / 1e6,
                 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes})
    G, M_max = GROUPED_MASKED['G'], GROUPED_MASKED['M_max']
    masked_m = torch.randint(0, M_max + 1, (G, ), generator=torch.Generator().manual_seed(20), dtype=torch.int32)
    x3 = torch.randn(G, M_max, 2 * N, device=dev, generator=gd).to(torch.bfloat16)
    q = torch.empty(G, M_max, N, device=dev, dtype=torch.float8_e4m3fn)
    s = torch.empty(G, M_max, N // 128, device=dev, dtype=torch.float32)
    mm = masked_m.to(dev)
    args3 = (vp(x3.data_ptr()), _lib.IN_CODES[x3.dtype], vp(q.data_ptr()), vp(s.data_ptr()), vp(mm.data_ptr()), G, M_max, N,
             s.stride(0), s.stride(1), s.stride(2), stream)
    _lib.check(lib.dlb_silu_mul_quant_masked(*args3))
    ms = time_call(lambda: lib.dlb_silu_mul_quant_masked(*args3), 100, 10)
    valid = int(masked_m.sum())
    nbytes = 4 * valid * N + valid * N + 4 * valid * (N // 128) + 4 * G
    rows.append({'workload': f'silu_mul_quant_masked_bf16_E{G}_Mmax{M_max}_{2 * N}', 'valid_rows': valid,
                 'us_per_launch': ms * 1e3, 'GBps': nbytes / ms / 1e6, 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS,
                 'bytes': nbytes})
    return rows


def permutation_workloads(dev):
    """ep_scatter / ep_gather at the expert-contiguous shape: 8192 tokens x top-8 over 256 experts of which 32 are
    local (about one local slot per token), hidden 7168.  bytes = rows read + rows written (+ scales, tables)."""
    import torch

    from dlblas_amd import _lib
    lib = _lib.load()
    T, H, E, topk = 8192, 7168, 32, 8
    gd = torch.Generator(device=dev).manual_seed(20)
    x = torch.randint(0, 127, (T, H), device=dev, generator=gd, dtype=torch.uint8).view(torch.float8_e4m3fn)
    xs = torch.rand(T, H // 128, device=dev, generator=gd)
    ids = torch.randint(0, 256, (T, topk), device=dev, generator=gd)
    ids[ids >= E] = -1
    wts = torch.rand(T, topk, device=dev, generator=gd)
    routed = torch.bincount(ids[ids >= 0], minlength=E)
    counts = ((routed + 127) // 128 * 128).to(torch.int32)
    rows, n_routed = int(counts.sum()), int(routed.sum())
    out = torch.empty(rows, H, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    out_s = torch.empty(rows, H // 128, device=dev)
    m_indices = torch.empty(rows, dtype=torch.int32, device=dev)
    out_idx = torch.empty_like(ids)
    start = torch.empty(E, dtype=torch.int32, device=dev)
    sargs = _lib.ep_scatter_args(x, xs, ids, counts, start, out, out_s, m_indices, out_idx)
    _lib.check(lib.dlb_ep_scatter(*sargs))
    ms = time_call(lambda: lib.dlb_ep_scatter(*sargs), 50, 5)
    nbytes = (T + n_routed) * (H + 4 * (H // 128)) + 2 * 8 * T * topk + 4 * rows
    res = [{'workload': f'ep_scatter_T{T}_top{topk}_E{E}_H{H}', 'routed_rows': n_routed, 'us_per_launch': ms * 1e3,
            'GBps': nbytes / ms / 1e6, 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes}]
    down = torch.randn(rows, H, device=dev, generator=gd).to(torch.bfloat16)
    gout = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    gargs = _lib.ep_gather_args(down, ids, wts, out_idx, gout)
    _lib.check(lib.dlb_ep_gather(*gargs))
    ms = time_call(lambda: lib.dlb_ep_gather(*gargs), 50, 5)
    nbytes = 2 * H * (n_routed + T) + (8 + 4 + 8) * T * topk
    res.append({'workload': f'ep_gather_T{T}_top{topk}_H{H}_bf16', 'routed_rows': n_routed, 'us_per_launch': ms * 1e3,
                'GBps': nbytes / ms / 1e6, 'frac_of_hbm_peak': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'bytes': nbytes})
    return res


def fused_moe_workload(dev):
    """The whole expert-contiguous MLP of one GPU's 32 local experts (dlblas_amd.kernels.fused_moe_v3.fused_moe_v3):
    ep_scatter -> gate/up GEMM -> silu * up + quantisation -> down GEMM -> ep_gather, every intermediate allocated per call
    as in the reference driver.  8192 tokens x top-8 over 256 experts (about one local slot per token), hidden 7168,
    intermediate 2048.  The row also gives the sum of the five steps measured one by one, so the driver's own cost shows."""
    import torch

    from dlblas_amd.kernels.fused_moe_v3 import fused_moe_v3
    T, H, I, E, topk = 8192, 7168, 2048, 32, 8
    gd = torch.Generator(device=dev).manual_seed(20)
    x_q, x_s = quantise_act(torch.randn(T, H, device=dev, generator=gd).to(torch.bfloat16))
    ids = torch.randint(0, 256, (T, topk), device=dev, generator=gd)
    ids[ids >= E] = -1
    wts = torch.rand(T, topk, device=dev, generator=gd)
    routed = torch.bincount(ids[ids >= 0], minlength=E)
    counts = [int(c) for c in ((routed + 127) // 128 * 128).tolist()]
    w13_q, w13_s = expert_weights(E, 2 * I, H, dev, 31)
    w2_q, w2_s = expert_weights(E, H, I, dev, 32)
    call = lambda: fused_moe_v3((x_q, x_s), ids, wts, (w13_q, w13_s), (w2_q, w2_s), counts)
    call()
    torch.cuda.synchronize()
    ms = time_call(call, 30, 60)
    rows, n_routed = sum(counts), int(routed.sum())
    flops = 2.0 * n_routed * (2 * I * H + H * I)
    out = [{'workload': f'fused_moe_v3_T{T}_top{topk}_E{E}_H{H}_I{I}', 'routed_rows': n_routed, 'rows_padded': rows,
            'us_per_call': ms * 1e3, 'TFLOPs_on_routed_rows': flops / ms / 1e9,
            'note': 'row tables, fused gate/up GEMM on the unsorted tokens, down GEMM, gather with their pre-passes + per-call allocation of every intermediate, timed as one call of the Python driver'}]
    # the decode counterpart: the masked expert MLP (dlblas_amd.kernels.moe.low_latency_experts) on 32 experts x 256
    # row slots with masked_m uniform in [0, 256]: fused gate/up GEMM + activation + quantiser, then the down GEMM
    from dlblas_amd.kernels.moe import low_latency_experts
    M_max = GROUPED_MASKED['M_max']
    masked_m = torch.randint(0, M_max + 1, (E, ), generator=torch.Generator().manual_seed(20), dtype=torch.int32)
    a_q, a_s = quantise_act(torch.randn(E * M_max, H, device=dev, generator=gd).to(torch.bfloat16))
    a_q, a_s = a_q.reshape(E, M_max, H), a_s.reshape(E, M_max, H // 128)
    mm, hint = masked_m.to(dev), int(masked_m.float().mean())
    call = lambda: low_latency_experts((a_q, a_s), w13_q, w13_s, w2_q, w2_s, mm, hint)
    call()
    torch.cuda.synchronize()
    ms = time_call(call, 30, 60)
    valid = int(masked_m.sum())
    out.append({'workload': f'low_latency_experts_E{E}_Mmax{M_max}_H{H}_I{I}', 'valid_rows': valid, 'us_per_call': ms * 1e3,
                'TFLOPs_on_valid_rows': 2.0 * valid * (2 * I * H + H * I) / ms / 1e9,
                'weight_GBps': E * 3 * I * H / ms / 1e6,
                'note': 'fused masked gate/up GEMM + down GEMM + per-call allocation of the intermediates; the weights (1.41 GB) are read once'})
    return out


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel from the rocprofv3 --pmc runs kept under profiles/ (None when
    no counter run for this workload has been recorded).  Not measured in this run: counters need the profiler."""
    path = os.path.join(ROOT, 'profiles', 'hbm_traffic.json')
    try:
        with open(path) as fh:
            return json.load(fh).get(workload, {}).get('bytes_per_launch')
    except (OSError, ValueError):
        return None


def copy_calibration(dev):
    """Three 1 GiB device copies: the kernel of known size that the HBM counters of a profiled run are scaled by."""
    import torch
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


PLANNER_SWEEP_WEIGHTS = [(2112, 7168), (24576, 1536), (32768, 512), (7168, 16384), (4096, 7168), (7168, 2048), (1536, 7168),
                         (7168, 18432), (36864, 7168), (576, 7168), (4608, 7168), (7168, 2304), (18432, 7168)]


def planner_sweep(dev, which):
    """The planner's launch against every alternative forced in turn; prints one line per problem and returns the rows.
    'dense': kernel variants (no K split forced) over 13 weight shapes x 15 row counts; 'mid': the three small ring
    kernels x 1 ... 16 K slices where the planner picks one of them; 'decode': columns per workgroup x waves x blocks in
    flight of the streaming kernels at 1, 16 and 32 rows; 'grouped': ring variants for both grouped layouts, 8 and 32
    experts.  A row's 'regret' is default / best - 1."""
    import torch

    from dlblas_amd import _lib
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous, fp8_gemm_grouped_masked
    rows = []

    def report(name, plan, t_default, best_t, best_what):
        row = {'problem': name, 'plan': plan, 'default_us': t_default, 'best_us': best_t, 'best': best_what,
               'regret': t_default / best_t - 1.0}
        rows.append(row)
        print(f"{name}: default {plan} {t_default:.1f} us; best {best_what} {best_t:.1f} us; regret {100 * row['regret']:.0f} %", flush=True)

    def dense_problem(M, N, K):
        copies = max(2, min(24, int(400e6 // (N * K))))
        a_q, a_s, ws = make_inputs(M, N, K, dev, weight_copies=copies)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        launch = DenseLauncher(a_q, a_s, ws, out)
        reps = int(max(10, min(200, 3e-2 / max(2.0 * M * N * K / 2e15, 5e-6))))
        time_call(launch, reps, reps)
        return launch, reps

    def timed(launch, reps):
        try:
            launch()
            torch.cuda.synchronize()
            return time_call(launch, reps, max(5, reps // 4)) * 1e3
        except Exception:  # the variant does not take this shape
            return None

    try:
        if which == 'dense':
            names = [n for n in _lib.variant_names() if n.startswith('pipe') or n.startswith('skinny')]
            for (N, K) in PLANNER_SWEEP_WEIGHTS:
                for M in (1, 16, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 2048, 4096):
                    if M * N * K > 4096 * 7168 * 18432:
                        continue
                    launch, reps = dense_problem(M, N, K)
                    plan = _lib.plan(0, M, N, K)
                    t0 = timed(launch, reps)
                    best = (t0, 'default')
                    if plan[1] == 1:  # forcing a variant drops the K split the planner chose with it
                        for v in names:
                            _lib.force_variant(v)
                            t = timed(launch, reps)
                            if t is not None and t < best[0]:
                                best = (t, v)
                        _lib.force_variant(None)
                        t0 = min(t0, timed(launch, reps))
                    report(f'{M}x{N}x{K}', plan[:2], t0, min(best[0], t0), best[1])
        elif which == 'mid':
            for (N, K) in PLANNER_SWEEP_WEIGHTS + [(4096, 4096), (1024, 16384), (7168, 4096)]:
                for M in (48, 64, 96, 128, 192, 256, 384, 512, 1024):
                    plan = _lib.plan(0, M, N, K)
                    if plan[0] not in ('pipe128x256w8', 'pipe128x128', 'pipe128x64') or M * N * K > 4096 * 7168 * 4096:
                        continue
                    launch, reps = dense_problem(M, N, K)
                    t0 = timed(launch, reps)
                    best = (t0, 'default')
                    for v in ('pipe128x256w8', 'pipe128x128', 'pipe128x64'):
                        _lib.force_variant(v)
                        for sk in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16):
                            if sk > 1 and (K // 128) // sk < 2:
                                continue
                            _lib.tune('splitk', sk)
                            t = timed(launch, max(10, reps // 2))
                            if t is not None and t < best[0]:
                                best = (t, f'{v} / {sk} slices')
                        _lib.tune('splitk', 0)
                    _lib.force_variant(None)
                    t0 = min(t0, timed(launch, reps))
                    report(f'{M}x{N}x{K}', plan[:2], t0, min(best[0], t0), best[1])
        elif which == 'decode':
            for (N, K) in PLANNER_SWEEP_WEIGHTS + [(4096, 4096), (8192, 1024), (16384, 2048)]:
                for M in (1, 16, 32):
                    launch, reps = dense_problem(M, N, K)
                    plan = _lib.plan(0, M, N, K)
                    t0 = timed(launch, reps)
                    best = (t0, 'default')
                    for bn in (8, 12, 16, 20, 24, 28, 32):
                        for waves in (4, 8, 16):
                            for unroll in (1, 2):
                                _lib.tune('skinny_bn', bn), _lib.tune('skinny_waves', waves), _lib.tune('skinny_unroll', unroll)
                                t = timed(launch, max(10, reps // 2))
                                if t is not None and t < best[0]:
                                    best = (t, f'{bn} columns, {waves} waves, {unroll} in flight')
                    for knob in ('skinny_bn', 'skinny_waves', 'skinny_unroll'):
                        _lib.tune(knob, 0)
                    t0 = min(t0, timed(launch, reps))
                    report(f'{M}x{N}x{K}', plan, t0, min(best[0], t0), best[1])
        elif which == 'grouped':
            gd = torch.Generator(device=dev).manual_seed(21)
            ring = ('pipe128x256w8', 'pipe256x256', 'pipe128x128')
            for (G, N, K) in ((32, 4096, 7168), (32, 7168, 2048), (8, 4096, 7168), (8, 7168, 2048)):
                w_q, w_s = expert_weights(G, N, K, dev, 22)
                for tokens in (G * 16, G * 64, G * 128, G * 256, G * 512):
                    assign = torch.multinomial(torch.full((G, ), 1.0 / G), tokens, replacement=True,
                                               generator=torch.Generator().manual_seed(20))
                    padded = (torch.bincount(assign, minlength=G) + 127) // 128 * 128
                    M_sum = int(padded.sum())
                    m_indices = torch.repeat_interleave(torch.arange(G, dtype=torch.int32), padded).to(dev)
                    a_q, a_s = quantise_act(torch.randn(M_sum, K, device=dev, generator=gd).to(torch.bfloat16))
                    out = torch.empty(M_sum, N, dtype=torch.bfloat16, device=dev)
                    call = lambda: fp8_gemm_grouped_contiguous(a_q, a_s, w_q, w_s, out, m_indices)  # noqa: E731
                    t0 = timed(call, 30)
                    best = (t0, 'default')
                    for v in ring:
                        _lib.force_variant(v)
                        t = timed(call, 30)
                        if t is not None and t < best[0]:
                            best = (t, v + ', uniform tiles')
                    _lib.force_variant(None)
                    for lists in (1, 2):
                        _lib.tune('tile_list', lists)
                        t = timed(call, 30)
                        if t is not None and t < best[0]:
                            best = (t, 'tile lists' if lists == 1 else 'no tile lists')
                    _lib.tune('tile_list', 0)
                    t0 = min(t0, timed(call, 30))
                    report(f'contiguous, {G} experts, {M_sum} rows, {N}x{K}', _lib.plan_grouped(1, M_sum, N, K, G), t0, min(best[0], t0), best[1])
                    del a_q, a_s, out
                for M_max in (64, 128, 256, 512, 1024):
                    for fill in (0.1, 0.5, 1.0):
                        masked_m = torch.randint(0, int(M_max * fill) + 1, (G, ), generator=torch.Generator().manual_seed(20), dtype=torch.int32)
                        a_q, a_s = quantise_act(torch.randn(G * M_max, K, device=dev, generator=gd).to(torch.bfloat16))
                        a_q, a_s = a_q.reshape(G, M_max, K), a_s.reshape(G, M_max, K // 128)
                        out = torch.empty(G, M_max, N, dtype=torch.bfloat16, device=dev)
                        mm, hint = masked_m.to(dev), int(masked_m.float().mean())
                        call = lambda: fp8_gemm_grouped_masked(a_q, a_s, w_q, w_s, out, mm, hint)  # noqa: E731
                        t0 = timed(call, 30)
                        best = (t0, 'default')
                        for v in ring:
                            _lib.force_variant(v)
                            t = timed(call, 30)
                            if t is not None and t < best[0]:
                                best = (t, v)
                        _lib.force_variant(None)
                        t0 = min(t0, timed(call, 30))
                        report(f'masked, {G} experts x {M_max} slots, {int(masked_m.sum())} valid rows, {N}x{K}',
                               _lib.plan_grouped(2, M_max, N, K, G, hint), t0, min(best[0], t0), best[1])
                        del a_q, a_s, out
                del w_q, w_s
        else:
            raise ValueError(which)
    finally:
        _lib.force_variant(None)
        for knob in _lib.KNOBS:
            _lib.tune(knob, 0)
    worst = sorted(rows, key=lambda r: -r['regret'])[:5]
    print(f"{len(rows)} problems; over 5 %: {sum(r['regret'] > 0.05 for r in rows)}, over 10 %: {sum(r['regret'] > 0.10 for r in rows)}; "
          'largest: ' + '; '.join(f"{r['problem']} {100 * r['regret']:.0f} %" for r in worst), flush=True)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='prefill_4096x7168x18432', choices=sorted(WORKLOADS))
    ap.add_argument('--variant', default=None, help='force a kernel variant (tuning)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run three 1 GiB device copies: the known-size kernel that HBM counters are scaled by')
    ap.add_argument('--no-other', action='store_true', help='skip the decode sweep and the grouped workloads')
    ap.add_argument('--moe-only', action='store_true',
                    help='run only the quantisers, the activation step and ep_scatter / ep_gather and print their rows (the '
                    'command their rocprofv3 summaries are made with)')
    ap.add_argument('--series', type=int, default=0,
                    help='print the duration of each of the first N launches of the workload from an idle GPU (the power '
                    "controller's start-up transient) and exit")
    ap.add_argument('--decode-floor', action='store_true',
                    help='run only the launch-cost floors of the decode shape (empty kernel, read-only kernel) and print them')
    ap.add_argument('--ceilings', action='store_true',
                    help='print what bench-only kernels reach on this GPU: the prefill kernel\'s MFMA + FMA mix from registers '
                         '(constant and random operands, with and without LDS reads) and a bare weight-panel stream through the LDS DMA path')
    ap.add_argument('--grouped-only', action='store_true',
                    help='run only the two grouped MoE workloads and print their rows (the command the rocprofv3 summaries of '
                    'the grouped kernels are made with)')
    ap.add_argument('--planner-sweep', choices=['dense', 'mid', 'decode', 'grouped'], default=None,
                    help="time the planner's launch against every alternative forced in turn over a grid of problems and "
                    'print where it is not the fastest (a minute or two)')
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

    if args.decode_floor:
        print(json.dumps({'decode_floor': decode_floor(dev)}), flush=True)
        return

    if args.planner_sweep:
        planner_sweep(dev, args.planner_sweep)
        return

    if args.ceilings:
        print(json.dumps({'ceilings': ceilings(dev)}), flush=True)
        return

    if args.moe_only:
        rows = (quantiser_workload(dev) + activation_workloads(dev) + permutation_workloads(dev) + masked_gate_up_workload(dev) +
                fused_moe_workload(dev))
        if args.copy_calibration:
            copy_calibration(dev)
        print(json.dumps({'moe_workloads': rows}), flush=True)
        return

    if args.grouped_only:
        rows = grouped_workloads(dev)
        if args.copy_calibration:
            copy_calibration(dev)
        print(json.dumps({'grouped_workloads': rows}), flush=True)
        return

    kind, M, N, K = WORKLOADS[args.workload]
    log(f'workload {args.workload}: generating inputs')
    memory_bound = M <= 128
    copies = 24 if memory_bound else 1  # rotate weights so decode reads come from HBM, not the 256 MB cache
    a_q, a_s, weights = make_inputs(M, N, K, dev, weight_copies=copies)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    launch = DenseLauncher(a_q, a_s, weights, out)
    if args.series > 0:
        time.sleep(0.2)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.series + 1)]
        ev[0].record()
        for i in range(args.series):
            launch()
            ev[i + 1].record()
        torch.cuda.synchronize()
        us = [round(ev[i].elapsed_time(ev[i + 1]) * 1e3, 1) for i in range(args.series)]
        print(json.dumps({'workload': args.workload, 'us_per_launch_in_order': us}), flush=True)
        return
    log('timing')
    ms_per_step, ev_ms, from_idle = time_steps(launch, args.steps, args.warmup)
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
    roofline['traffic'] = measured_traffic(args.workload)
    roofline['traffic_source'] = ('profiles/hbm_traffic.json: FETCH_SIZE + WRITE_SIZE of rocprofv3 --pmc runs of this command, '
                                  'scaled by a 1 GiB copy; read from the committed file, not measured in this run')
    roofline['kernel_ms'] = ev_ms
    from_idle['frac_of_peak'] = (nbytes / 1e9 if memory_bound else flops / 1e12) / (from_idle['kernel_ms'] * 1e-3) / roofline['peak']
    from_idle['note'] = ('the same warmup + steps measured first, on an idle GPU: the power controller boosts, throttles and '
                         'recovers during the first tens of milliseconds of this load; value / roofline are measured after '
                         'settle_launches further untimed launches + one more warmup (effective_warmup_launches in all), when '
                         'the per-launch time has stopped moving')

    result = {
        'metric': 'FP8 block-scaled GEMM TFLOP/s (% FP8 MFMA peak); decode-M HBM GB/s',
        'value': value,
        'unit': unit,
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'effective_warmup_launches': from_idle['launches_before_the_timed_region'],
        'from_idle_ms_per_step': from_idle['ms_per_step'],
        'from_idle_frac_of_peak': from_idle['frac_of_peak'],
        'ms_per_step': ms_per_step,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'fp8_e4m3 x fp8_e4m3 -> f32 accumulate -> bf16',
        'data': 'synthetic',
        'config': {'workload': args.workload, 'M': M, 'N': N, 'K': K, 'a_scale': '1x128 f32', 'b_scale': '128x128 f32',
                   'out': 'bf16', 'seed': 20},
        'roofline': roofline,
        'from_idle': from_idle,
    }

    if not args.no_other:
        log('decode sweep')
        others = decode_sweep(dev)
        m16 = next(r for r in others if r['workload'] == 'decode_16x7168x2048')
        result['decode'] = {'workload': m16['workload'], 'us_per_launch': m16['us_per_launch'], 'GBps': m16['GBps'],
                            'frac_of_hbm_peak': m16['frac_of_hbm_peak'], 'bytes': m16['bytes'],
                            'floor_us': decode_floor(dev),
                            'note': '24 distinct weight copies in rotation (353 MB) so reads miss the 256 MB cache'}
        log('grouped workloads')
        others += second_prefill_workload(dev)
        others += chunked_prefill_workloads(dev)
        others += grouped_workloads(dev)
        others += quantiser_workload(dev)
        others += activation_workloads(dev)
        others += permutation_workloads(dev)
        others += masked_gate_up_workload(dev)
        others += fused_moe_workload(dev)
        result['other_workloads'] = others

    if args.copy_calibration:
        copy_calibration(dev)

    if not args.no_cpu_baseline:
        log('cpu baseline')
        b_q, b_s = weights[0]
        result['cpu_baseline'] = cpu_baseline(kind, M, N, K, a_q, a_s, b_q, b_s)
    print(json.dumps(result), flush=True)


if __name__ == '__main__':
    main()
