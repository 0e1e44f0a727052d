#!/usr/bin/env python3
"""Benchmark of the W4A4 linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step is one W4A4 linear at the Llama-7B gate/up shape (M=4096 tokens, K=4096, N=11008) as
`harness.linear_forward` runs it at this size: the fused Hadamard + scale + quantise kernel on the fp16
activations, writing the INT4 codes in the GEMM's operand form (E2M3 tiles), then the INT4 x INT4 GEMM
on the FP6 matrix instructions with the scale epilogue to fp16 -- the same output bits as the
packed-nibble INT8 kernels, which are timed beside it.  Inputs are synthetic and already resident in
HBM; several activation buffers are rotated so that no step finds its input in the Infinity Cache.
`value` is 2*M*N*K / step time (TOPS of the whole linear, as the reference's published layer times
are converted).  The JSON line also carries
  roofline           the GEMM kernel against the INT8 MFMA peak, the metric's denominator (HIP events around
                     back-to-back launches); the FP6 pipe's own peak and the INT8 kernel's figure beside it,
  roofline_quantize  the fused activation kernel at bf16 [8192, 4096] (heavy-tailed input with
                     outlier channels) against the HBM peak,
  decode             the layer at M in {1, 8, 16}: the weight-streaming GEMM alone and with the activation kernel,
  few_hundred_tokens the same at M in {128, 256, 384} (the small-tile GEMM),
  forward            the 12-layer Llama of the reference's end-to-end benchmark, dense vs W4A4 vs no-op linears,
  cpu_baseline       the CPU oracle (PyTorch restatement of the reference's `backend='pytorch'`
                     path) on the reference's CPU-runnable case, timed on this host's cores.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
REPLAYS = 9                  # timed replays of a batch of launches; the median is reported
WARM_REPLAYS = 3             # untimed replays before them: the first ones run while the clocks still ramp
SUSTAIN_MS = 60.0            # launches_ms(..., sustained=True): untimed replays for this long before a second set of timed ones
EAGER_BATCHES = False        # --eager-batches: time plain launches instead of graph replays
LAST = {'min_ms': None, 'sustained_ms': None}      # fastest replay of the most recent launches_ms() call
INT8_MFMA_PEAK_TOPS = 5000.0
FP6_MFMA_PEAK_TOPS = 10100.0

# HBM bytes per launch from rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE in KiB per dispatch),
# scaled by what the same counters read for calibration_stream() below (FETCH_SIZE x 1.9998, WRITE_SIZE x 1.0);
# the runs are summarised under profiles/.
TRAFFIC_SOURCE = ('constant from a separate rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this script, summarised in '
                  'profiles/bench_gemm_e2m3_M4096_K4096_N11008_and_quantize_8192x4096.md; not measured in this run')
TRAFFIC_GEMM_BYTES = 329496400                 # gemm_e2m3_kernel; of these 219.7 MB fetched (operands: 46.4 MB), 109.8 MB written
TRAFFIC_QUANTIZE_BYTES = 84284627
# what quest_e2m3_gemm_plan reported for M=4096 K=4096 N=11008 on 256 compute units when TRAFFIC_GEMM_BYTES was measured: the
# figure depends on the schedule (which workgroup fetches what), so the line says `traffic_stale` when the plan has changed
TRAFFIC_GEMM_PLAN = [256, 8, 0, 2, 256, 256, 6, 64]


def gemm_plan(lib, m, k, n, dev):
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    plan = (ctypes.c_int * 8)()
    if lib.quest_e2m3_gemm_plan(m, k, n, cus, plan) != 0:
        raise RuntimeError('quest_e2m3_gemm_plan failed')
    return list(plan)


def event_pairs(n):
    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


def mean_ms(pairs):
    return sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)


def current_stream():
    """torch's current HIP stream as the C ABI takes it; read at every launch so that a capturing stream is honoured."""
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def launches_ms(launch, n, warmup=5, sustained=False):
    """Average duration of `n` back-to-back launches of one kernel: HIP events on the stream the launches go to,
    around each of REPLAYS replays of a HIP graph that holds the whole batch (a graph keeps the gap between two dispatches to a
    fraction of a microsecond; whatever gap remains counts as kernel time).  `launch(i)` must be a bare C-ABI call
    that reads torch's current stream at call time."""
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    if EAGER_BATCHES:                            # plain launches (counter collection cannot follow graph replays)
        per_launch = []
        for _ in range(REPLAYS):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for i in range(n):
                launch(i)
            b.record()
            torch.cuda.synchronize()
            per_launch.append(a.elapsed_time(b) / n)
        per_launch.sort()
        LAST['min_ms'], LAST['sustained_ms'] = per_launch[0], None
        return per_launch[len(per_launch) // 2]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(n):
                launch(i)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(WARM_REPLAYS):
        graph.replay()
    per_launch = []
    for _ in range(REPLAYS):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        graph.replay()
        b.record()
        torch.cuda.synchronize()
        per_launch.append(a.elapsed_time(b) / n)
    LAST['all_ms'] = list(per_launch)
    LAST['sustained_ms'] = None
    if sustained:
        # the same graph after SUSTAIN_MS of uninterrupted replays: a bandwidth-bound kernel that runs alone for tens of
        # milliseconds gets a lower core clock from the power management, and whatever of it is not hidden under memory
        # traffic (launch, first and last waves) takes longer
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < SUSTAIN_MS:
            graph.replay()
            torch.cuda.synchronize()
        late = []
        for _ in range(REPLAYS):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            late.append(a.elapsed_time(b) / n)
        late.sort()
        LAST['sustained_ms'] = late[len(late) // 2]
    per_launch.sort()
    LAST['min_ms'] = per_launch[0]
    return per_launch[len(per_launch) // 2]      # median replay: the first ones run while the clocks still ramp


def heavy_tailed_activations(m, k, dtype, device, seed):
    """Student-t (3 degrees of freedom) entries, 1 % of the channels scaled by 20."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    z = torch.randn(m, k, generator=g)
    chi = torch.randn(m, k, 3, generator=g).square_().sum(-1)
    x = z / (chi / 3).sqrt_()
    cols = torch.randperm(k, generator=g)[: max(1, k // 100)]
    x[:, cols] *= 20
    return x.to(dtype).to(device)


def bench_linear(quest, _lib, steps, warmup, dev):
    m, k, n = 4096, 4096, 11008
    dtype = torch.float16
    g = torch.Generator(device='cpu').manual_seed(0)
    n_buf = 6
    acts = [torch.randn(m, k, generator=g).to(dtype).to(dev) for _ in range(n_buf)]
    # weights: uniform codes in [-8, 7], per-channel scales U(0.01, 0.1)
    w_codes = torch.randint(-8, 8, (n, k), generator=g, dtype=torch.int8)
    w_packed = ((w_codes[:, 1::2] << 4) | (w_codes[:, ::2] & 0xF)).view(torch.uint8).to(dev)
    w_scale = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype).to(dev)
    w_add = (w_codes.to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2).to(dev)
    w_tiles = quest.int4_to_e2m3_tiles(w_packed)                 # the weights' operand form, made once (as Linear4bit keeps it)
    a_scale = torch.empty(m, 1, dtype=dtype, device=dev)
    a_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    a_row_sum = torch.empty(m, 1, dtype=torch.int32, device=dev)
    a_tiles = torch.empty(quest.e2m3_tiles_bytes(m, k), dtype=torch.uint8, device=dev)
    out = torch.empty(m, n, dtype=dtype, device=dev)

    def step(i, ev=None):
        x = acts[i % n_buf]
        if ev:
            ev[0].record()
        quest.hadamard_quantize_e2m3(x, a_scale, a_tiles)
        if ev:
            ev[1].record()
        quest.fused_matmul_dequantize_e2m3(a_tiles, w_tiles, a_scale, w_scale, k, out)
        if ev:
            ev[2].record()

    def step_int8(i):
        quest.hadamard_quantize_int4(acts[i % n_buf], a_scale, a_packed, a_row_sum)
        quest.fused_matmul_dequantize_int4_int4t_bf16(a_packed, w_packed, a_row_sum, w_add, a_scale, w_scale, out)

    lib = _lib.load()
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    # The K steps as one HIP graph (every entry point is capturable: no allocation, no synchronisation, the stream an
    # argument), which is how a serving loop would issue them: the gap between dependent kernels drops from the
    # several microseconds of an eager launch to a fraction of one.  The chip needs some 30 ms of this load before
    # its clocks settle (the first replays run 15-25 % slower), so the graph is replayed untimed for 60 ms (ten
    # replays at least) on top of the W warm-up steps; then exactly K steps are timed between two synchronisations,
    # five times over, and the median counts (all five are in the line).
    step_times_ms, untimed_replays = [], 0
    if not EAGER_BATCHES:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(steps):
                    step(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        settle_until = time.perf_counter() + SUSTAIN_MS * 1e-3
        while untimed_replays < 10 or time.perf_counter() < settle_until:
            graph.replay()
            torch.cuda.synchronize()
            untimed_replays += 1
        for _ in range(5):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            step_times_ms.append((time.perf_counter() - t0) * 1e3 / steps)
    # the same K steps as plain launches, right after (the chip still warm): W untimed steps, K timed ones
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms_per_step_eager = (time.perf_counter() - t0) * 1e3 / steps
    ms_per_step = sorted(step_times_ms)[len(step_times_ms) // 2] if step_times_ms else ms_per_step_eager
    # the same layer on the packed-nibble path (activation kernel writing nibbles and row sums, INT8 kernel)
    step_int8_ms = launches_ms(step_int8, steps)
    # the split between the two kernels, from a second pass with events between them (the events cost a few
    # microseconds each, which is why the timed pass above has none)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for i in range(steps):
        step(i, evs[i])
    torch.cuda.synchronize()
    quant_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / steps
    gemm_in_step_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / steps

    # the GEMM alone, bare C-ABI launches: on uniform random activation codes (the stated GEMM workload; the
    # matrix cores draw the most power on them) and on the codes the last step left (Gaussian activations)
    u_codes = torch.randint(-8, 8, (m, k), generator=g, dtype=torch.int8)
    u_packed = ((u_codes[:, 1::2] << 4) | (u_codes[:, ::2] & 0xF)).view(torch.uint8).to(dev)
    u_row_sum = u_codes.to(torch.int32).sum(-1, keepdim=True).to(torch.int32).to(dev)
    u_scale = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype).to(dev)

    u_tiles = quest.int4_to_e2m3_tiles(u_packed)

    def gemm_launcher(codes, row_sum, scale):                      # the INT8 kernel on packed nibbles
        args = (_lib.ptr(out), _lib.ptr(codes), _lib.ptr(w_packed), _lib.ptr(row_sum), _lib.ptr(w_add),
                _lib.ptr(scale), _lib.ptr(w_scale), m, k, n, _lib.DTYPE_CODE[dtype])         # sizes in the ABI's order: M, K, N

        def gemm(_):
            if lib.quest_fused_matmul_dequantize_int4_int4t(*args, current_stream()) != 0:
                raise RuntimeError('GEMM launch failed')
        return gemm

    def e2m3_launcher(tiles, scale, w=None):                       # the FP6 kernel on E2M3 tiles
        args = (_lib.ptr(out), _lib.ptr(tiles), _lib.ptr(w_tiles if w is None else w), _lib.ptr(scale), _lib.ptr(w_scale), m, k, n,
                _lib.DTYPE_CODE[dtype])

        def gemm(_):
            if lib.quest_fused_matmul_dequantize_e2m3(*args, current_stream()) != 0:
                raise RuntimeError('GEMM launch failed')
        return gemm

    # the activation kernel of the step alone (fp16 [4096, 4096], inputs rotating): bare launches in a graph, without the
    # events that quant_ms above has around it
    q_tail = (_lib.ptr(a_scale), _lib.ptr(a_packed), _lib.ptr(a_row_sum), None, k, m, 181. / 2048., _lib.DTYPE_CODE[dtype])
    act_ptrs = [_lib.ptr(x) for x in acts]

    def quant_alone(i):
        if lib.quest_hadamard_quantize_int4(act_ptrs[i % n_buf], *q_tail, current_stream()) != 0:
            raise RuntimeError('activation kernel launch failed')

    t_tail = (_lib.ptr(a_scale), _lib.ptr(a_tiles), None, None, None, k, m, 181. / 2048., _lib.DTYPE_CODE[dtype])

    def quant_tiles_alone(i):
        if lib.quest_hadamard_quantize_e2m3(act_ptrs[i % n_buf], *t_tail, current_stream()) != 0:
            raise RuntimeError('activation kernel launch failed')

    quant_alone_ms = launches_ms(quant_alone, 100)
    quant_tiles_alone_ms = launches_ms(quant_tiles_alone, 100)
    step(0)                                                       # a_tiles / a_packed hold the codes of Gaussian activations again
    step_int8(0)
    gemm_quantized_ms = launches_ms(e2m3_launcher(a_tiles, a_scale), max(steps, 100))
    int8_quantized_ms = launches_ms(gemm_launcher(a_packed, a_row_sum, a_scale), max(steps, 100))
    # the same with the weights rotated through 14 copies (315 MB, more than the Infinity Cache holds), as a model
    # with many layers would stream them from HBM
    w_copies = [w_tiles] + [w_tiles.clone() for _ in range(9)]    # 10 x 33.8 MB
    u_args = (_lib.ptr(u_scale), _lib.ptr(w_scale), m, k, n, _lib.DTYPE_CODE[dtype])
    w_ptrs = [_lib.ptr(w) for w in w_copies]

    def gemm_rotating(i):
        if lib.quest_fused_matmul_dequantize_e2m3(_lib.ptr(out), _lib.ptr(u_tiles), w_ptrs[i % 10], *u_args, current_stream()) != 0:
            raise RuntimeError('GEMM launch failed')

    gemm_rotating_ms = launches_ms(gemm_rotating, 100)
    del w_copies
    int8_gemm_ms = launches_ms(gemm_launcher(u_packed, u_row_sum, u_scale), max(steps, 100))
    gemm_ms = launches_ms(e2m3_launcher(u_tiles, u_scale), max(steps, 100))
    gemm_min_ms = LAST['min_ms']
    # a yardstick, not part of the path: the vendor library's INT8 GEMM (torch._int_mm -> hipBLASLt) on the same codes as
    # int8, int32 out -- twice the operand bytes, no nibbles to split, no scale arithmetic
    vendor_int8_ms = None
    try:
        w8 = w_codes.to(dev)
        u8 = u_codes.to(dev)
        vendor_int8_ms = launches_ms(lambda _: torch._int_mm(u8, w8.t()), 50)
        del w8, u8
    except Exception:                       # not every build of the library has it
        vendor_int8_ms = None
    ops = 2.0 * m * n * k
    return {
        'shape': {'M': m, 'K': k, 'N': n},
        'ms_per_step': ms_per_step,
        'ms_per_step_each': step_times_ms,
        'untimed_replays': untimed_replays,
        'ms_per_step_eager': ms_per_step_eager,
        'tops': ops / (ms_per_step * 1e-3) / 1e12,
        'gemm_ms': gemm_ms,
        'gemm_min_ms': gemm_min_ms,
        'gemm_tops': ops / (gemm_ms * 1e-3) / 1e12,
        'gemm_in_step_ms': gemm_in_step_ms,
        'gemm_quantized_acts_ms': gemm_quantized_ms,
        'gemm_rotating_weights_ms': gemm_rotating_ms,
        'vendor_int8_ms': vendor_int8_ms,
        'quant_ms': quant_ms,
        'quant_alone_ms': quant_alone_ms,
        'quant_tiles_alone_ms': quant_tiles_alone_ms,
        'step_int8_ms': step_int8_ms,
        'int8_gemm_ms': int8_gemm_ms,
        'int8_quantized_ms': int8_quantized_ms,
    }


def bench_quantize(_lib, steps, warmup, dev):
    m, k = 8192, 4096
    dtype = torch.bfloat16
    n_buf = 6                                   # 6 x 64 MiB > the 256 MB Infinity Cache
    xs = [heavy_tailed_activations(m, k, dtype, dev, seed=s) for s in range(n_buf)]
    scale = torch.empty(m, 1, dtype=dtype, device=dev)
    packed = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    row_sum = torch.empty(m, 1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    xp = [_lib.ptr(x) for x in xs]
    tail = (_lib.ptr(scale), _lib.ptr(packed), _lib.ptr(row_sum), None, k, m, 181. / 2048., _lib.DTYPE_CODE[dtype])

    def launch(i):
        if lib.quest_hadamard_quantize_int4(xp[i % n_buf], *tail, current_stream()) != 0:
            raise RuntimeError('activation kernel launch failed')

    ms = launches_ms(launch, steps, warmup, sustained=True)
    ms_min, ms_sustained = LAST['min_ms'], LAST['sustained_ms']
    algo_bytes = m * k * 2 + m * k // 2 + m * 2 + m * 4
    gbs = algo_bytes / (ms * 1e-3) / 1e9

    # a yardstick: torch's device copy moving the same number of bytes in one launch (half read, half written), inputs
    # rotating as above
    half = algo_bytes // 2 // 16 * 16
    flat = [x.view(torch.uint8).view(-1) for x in xs]
    sink = torch.empty(half, dtype=torch.uint8, device=dev)
    copy_same_bytes_ms = launches_ms(lambda i: sink.copy_(flat[i % n_buf][:half]), steps, warmup)
    del flat, sink

    # the same kernel on eight times the rows: what it sustains once launch, fill and drain (about 4 us, a fifth of
    # the 8192-row launch) are amortised, next to a device copy of the same size class
    del xs
    m8 = 8 * m
    big = [torch.randn(m8, k, device=dev).to(dtype) for _ in range(2)]
    scale8 = torch.empty(m8, 1, dtype=dtype, device=dev)
    packed8 = torch.empty(m8, k // 2, dtype=torch.uint8, device=dev)
    row_sum8 = torch.empty(m8, 1, dtype=torch.int32, device=dev)
    bp = [_lib.ptr(x) for x in big]
    tail8 = (_lib.ptr(scale8), _lib.ptr(packed8), _lib.ptr(row_sum8), None, k, m8, 181. / 2048., _lib.DTYPE_CODE[dtype])

    def launch8(i):
        if lib.quest_hadamard_quantize_int4(bp[i % 2], *tail8, current_stream()) != 0:
            raise RuntimeError('activation kernel launch failed')

    ms8 = launches_ms(launch8, 20, 3)
    src, dst = big[0].view(torch.uint8).view(-1), big[1].view(torch.uint8).view(-1)
    copy_ms = launches_ms(lambda i: dst.copy_(src), 10, 2)
    sustained = {'rows': m8, 'us_per_launch': ms8 * 1e3, 'GBs': 8 * algo_bytes / (ms8 * 1e-3) / 1e9,
                 'frac': 8 * algo_bytes / (ms8 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 'device_copy_same_size_GBs': 2 * src.numel() / (copy_ms * 1e-3) / 1e9}
    del big
    torch.cuda.empty_cache()
    return {'bound': 'hbm', 'achieved': gbs, 'peak': HBM_PEAK_GBS, 'unit': 'GB/s', 'frac': gbs / HBM_PEAK_GBS,
            'traffic': TRAFFIC_QUANTIZE_BYTES, 'traffic_source': TRAFFIC_SOURCE, 'kernel': 'hadamard_quantize_mfma_kernel', 'us_per_launch': ms * 1e3, 'us_per_launch_min': ms_min * 1e3,
            'us_per_launch_after_60ms_of_replays': None if ms_sustained is None else ms_sustained * 1e3,
            'device_copy_same_bytes_us': copy_same_bytes_ms * 1e3,
            'algorithmic_bytes': algo_bytes, 'workload': 'bf16 [8192,4096] Student-t(3), 1% channels x20',
            'sustained_at_8x_rows': sustained}


def bench_decode(_lib, dev, ms=(1, 8, 16)):
    """The layer at a few token counts M (default: the decode shapes {1, 8, 16}): weights rotate through copies
    totalling more than the Infinity Cache so that they stream from HBM; bare C-ABI launches, the GEMM alone and the
    activation kernel + GEMM pair."""
    out = []
    lib = _lib.load()
    dtype = torch.float16
    code = _lib.DTYPE_CODE[dtype]
    g = torch.Generator(device='cpu').manual_seed(1)
    work = torch.zeros(16384 + (2 << 20), dtype=torch.uint8, device=dev)       # the split-K workspace, counters zeroed once
    for k, n in [(4096, 4096), (4096, 11008), (11008, 4096)]:
        n_w = max(2, int(600e6 // (n * k // 2)))
        ws = [torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.uint8).to(dev) for _ in range(n_w)]
        w_scale = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype).to(dev)
        w_add = torch.randint(-500, 500, (n, 1), generator=g, dtype=torch.int32).to(dev)
        for m in ms:
            x = torch.randn(m, k, generator=g).to(dtype).to(dev)
            a_scale = torch.empty(m, 1, dtype=dtype, device=dev)
            a_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
            a_row_sum = torch.empty(m, 1, dtype=torch.int32, device=dev)
            y = torch.empty(m, n, dtype=dtype, device=dev)
            q_args = (_lib.ptr(x), _lib.ptr(a_scale), _lib.ptr(a_packed), _lib.ptr(a_row_sum), None, k, m, 181. / 2048., code)
            wp = [_lib.ptr(w) for w in ws]
            g_tail = (_lib.ptr(a_row_sum), _lib.ptr(w_add), _lib.ptr(a_scale), _lib.ptr(w_scale), m, k, n, code)
            yp, ap = _lib.ptr(y), _lib.ptr(a_packed)

            def gemm(i):
                if lib.quest_fused_matmul_dequantize_int4_int4t(yp, ap, wp[i % n_w], *g_tail, current_stream()) != 0:
                    raise RuntimeError('GEMM launch failed')

            def gemm_split(i):
                if lib.quest_fused_matmul_dequantize_int4_int4t_ws(yp, ap, wp[i % n_w], *g_tail, _lib.ptr(work), work.numel(), current_stream()) != 0:
                    raise RuntimeError('GEMM launch failed')

            def layer(i):
                if lib.quest_hadamard_quantize_int4(*q_args, current_stream()) != 0:
                    raise RuntimeError('activation kernel launch failed')
                gemm(i)

            layer(0)
            gemm_us = launches_ms(gemm, 200, 20) * 1e3
            layer_us = launches_ms(layer, 200, 20) * 1e3
            split_us = launches_ms(gemm_split, 200, 20) * 1e3 if lib.quest_gemm_workspace_bytes(m, k, n) else None
            wbytes = n * k // 2
            out.append({'M': m, 'K': k, 'N': n, 'gemm_us': round(gemm_us, 2), 'layer_us': round(layer_us, 2),
                        'gemm_split_k_us': None if split_us is None else round(split_us, 2),
                        'weight_GBs': round(wbytes / gemm_us / 1e3, 1),
                        'frac_hbm': round(wbytes / gemm_us / 1e3 / HBM_PEAK_GBS, 4),
                        'TOPS': round(2.0 * m * n * k / gemm_us / 1e6, 1)})
    return out


def bench_forward(dev):
    """The whole-model row: 12-layer d=1024 Llama, ids (32, 512), bf16, every transformer projection W4A4 with the
    Hadamard on.  Times per forward for the dense model, the INT4 model and the no-op model (everything but the
    linears); the linear-only fraction prices (int4 - noop) against the INT8 matrix peak."""
    from quest_amd import llama
    out = {}
    cfg = llama.LlamaConfig()
    batch, seq = 32, cfg.sequence_length
    for mode in ('bf16', 'bf16_fused_producers', 'int4', 'int4_fused_producers', 'noop'):
        torch.manual_seed(0)
        model = llama.Llama(cfg).to(torch.bfloat16).to(dev).eval()
        llama.quantize_model(model, mode.split('_')[0], use_hadamard=True, fuse_gate_up=True,
                             fuse_producers=mode.endswith('producers'))
        r = llama.bench_forward(model, batch, seq)
        out[mode] = {'eager_ms': r['eager_s'] * 1e3, 'graph_ms': r['graph_s'] * 1e3, 'best_ms': r['best_s'] * 1e3,
                     'graph_matches_eager': r['graph_matches_eager']}
        del model
        torch.cuda.empty_cache()
    ops = cfg.linear_ops_per_token() * batch * seq
    lin_ms = out['int4']['best_ms'] - out['noop']['best_ms']
    return {'model': '12 layers, d=1024, 16 heads, SwiGLU 2816, vocab 32000, random init', 'tokens': batch * seq,
            'modes': out, 'int4_tokens_per_s': batch * seq / (out['int4_fused_producers']['best_ms'] * 1e-3),
            'speedup_over_bf16': out['bf16']['best_ms'] / out['int4_fused_producers']['best_ms'],
            'speedup_over_bf16_with_rotary_kernel': out['bf16_fused_producers']['best_ms'] / out['int4_fused_producers']['best_ms'],
            'linear_int_ops': ops, 'linear_ms': lin_ms,
            'linear_frac_of_int8_peak': ops / (lin_ms * 1e-3) / 1e12 / INT8_MFMA_PEAK_TOPS,
            'wiring': 'QKV fused (as the reference); gate and up share one quantisation and one GEMM'}


def bench_small_layer_gpu(quest, dev):
    """The CPU baseline's workload (fp16 [512,1024] x [1024,1024]^T, Hadamard on, absmax-scaled weights) through the
    HIP path, as a replayed HIP graph of 100 layers: the figure to set beside `cpu_baseline`."""
    from quest_amd import harness
    torch.manual_seed(0)
    m, k, n = 512, 1024, 1024
    x = torch.randn(m, k).half().to(dev)
    w = (torch.randn(n, k) * 0.02).half().to(dev)
    wp, ws, wa, _ = harness.preprocess_weight(w, use_hadamard=True, w_scale_mode='absmax')
    scale = torch.empty(m, 1, dtype=x.dtype, device=dev)
    packed = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    row_sum = torch.empty(m, 1, dtype=torch.int32, device=dev)
    out = torch.empty(m, n, dtype=x.dtype, device=dev)

    def layer(_):
        quest.hadamard_quantize_int4(x, scale, packed, row_sum)
        quest.fused_matmul_dequantize_int4_int4t_bf16(packed, wp, row_sum, wa, scale, ws, out)

    ms = launches_ms(layer, 100, 10)
    # the checker: activation codes of this workload against the full CPU oracle pipeline on the same x (the
    # reference's F.linear Hadamard, torch-CPU scale, quantiser), and the layer output against the oracle's
    from oracle import quest_oracle as qo
    _, o_scale, o_packed, _ = qo.hadamard_quantize_int4(x.cpu(), hadamard='matmul')
    differ = (qo.unpack_int4(packed.cpu()) != qo.unpack_int4(o_packed)).float().mean().item()
    owp, ows, owa, _ = qo.preprocess_weight(w.cpu(), use_hadamard=True, w_scale_mode='absmax')
    want = qo.linear_forward(x.cpu(), owp, ows, owa, use_hadamard=True, hadamard='matmul', via='fp32').double()
    rel = ((out.cpu().double() - want).norm() / want.norm()).item()
    return {'ms_per_call': ms, 'activation_codes_differing_from_oracle_pipeline': differ,
            'weights_bit_exact': bool(torch.equal(wp.cpu(), owp) and torch.equal(wa.cpu(), owa)),
            'output_rel_error_vs_oracle': rel, 'value': 2.0 * m * n * k / (ms * 1e-3) / 1e12, 'unit': 'TOPS',
            'what': 'the same layer through the HIP path on the GPU (graph replay, median of nine)'}


def bench_cpu_baseline():
    """The CPU oracle on the reference's CPU-runnable case: fp16 [512,1024] x [1024,1024]^T, Hadamard
    as F.linear, scale, quantise, integer GEMM through fp64 as the reference's own check does, and
    the scale epilogue."""
    from oracle import quest_oracle as qo
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    m, k, n = 512, 1024, 1024
    x = torch.randn(m, k).half()
    w = (torch.randn(n, k) * 0.02).half()
    wp, ws, wa, _ = qo.preprocess_weight(w, use_hadamard=True, w_scale_mode='absmax')      # pre-quantised, per-row absmax scales
    for _ in range(3):
        qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='matmul', via='fp64')
    times = []
    for _ in range(10):
        t0 = time.perf_counter()
        qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='matmul', via='fp64')
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    t32 = []
    for _ in range(10):
        t0 = time.perf_counter()
        qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='matmul', via='fp32')
        t32.append(time.perf_counter() - t0)
    t32.sort()
    ops = 2.0 * m * n * k
    # the bench step's own workload (fp16 [4096,4096] -> quantise -> x [11008,4096]^T, same generators as the GPU step):
    # a warm-up on 256 tokens, then five whole steps, their median counted -- about ten seconds of CPU work
    sm, sk, sn = 4096, 4096, 11008
    g = torch.Generator(device='cpu').manual_seed(0)
    sx = torch.randn(sm, sk, generator=g).half()
    s_codes = torch.randint(-8, 8, (sn, sk), generator=g, dtype=torch.int8)
    s_packed = ((s_codes[:, 1::2] << 4) | (s_codes[:, ::2] & 0xF)).view(torch.uint8)
    s_scale = (torch.rand(sn, 1, generator=g) * 0.09 + 0.01).half()
    s_add = (s_codes.to(torch.int32).sum(-1, keepdim=True) + sk // 2).to(torch.int32)
    del s_codes
    qo.linear_forward(sx[:256], s_packed, s_scale, s_add, use_hadamard=True, hadamard='matmul', via='fp64')
    t_step = []
    for _ in range(5):
        t0 = time.perf_counter()
        qo.linear_forward(sx, s_packed, s_scale, s_add, use_hadamard=True, hadamard='matmul', via='fp64')
        t_step.append(time.perf_counter() - t0)
    step_workload = {'what': f'one bench step on the CPU: W4A4 linear fp16 M={sm} K={sk} N={sn}, median of five calls',
                     's_per_step': sorted(t_step)[2], 'value': 2.0 * sm * sn * sk / sorted(t_step)[2] / 1e12, 'unit': 'TOPS'}
    del sx, s_packed
    return {'value': ops / med / 1e12, 'unit': 'TOPS', 'cores': torch.get_num_threads(), 'kind': 'port',
            'step_workload': step_workload,
            'sample': f'W4A4 linear fp16 M={m} K={k} N={n}, seed 0, median of 10 calls after 3 warm-ups '
                      f'({med * 1e3:.1f} ms per call; integer GEMM via fp64 matmul as the reference checks it)',
            'ms_per_call': med * 1e3,
            'faster_variant': {'what': 'same path with the integer GEMM as an exact fp32 matmul',
                               'value': ops / t32[len(t32) // 2] / 1e12, 'ms_per_call': t32[len(t32) // 2] * 1e3}}


def calibration_stream(dev):
    """A plain elementwise kernel of known traffic (reads 256 MiB, writes 256 MiB), launched three times so that
    a counter run of this script holds the reference the FETCH_SIZE / WRITE_SIZE readings are scaled by."""
    a = torch.zeros(64 * 1024 * 1024, dtype=torch.int32, device=dev)
    b = torch.empty_like(a)
    for _ in range(3):
        torch.add(a, 1, out=b)
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=100)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-forward', action='store_true', help='skip the whole-model row')
    ap.add_argument('--only', choices=('quantize', 'decode'),
                    help='run one leg only and print its result (for short rocprofv3 runs): the activation kernel or the decode shapes')
    ap.add_argument('--layer-sweep', action='store_true',
                    help='also run the layer benchmark of quest_amd.bench_layer (quick set of token counts) and add it to the line')
    ap.add_argument('--eager-batches', action='store_true',
                    help='time batches of plain launches instead of HIP-graph replays (for rocprofv3 --pmc runs)')
    args = ap.parse_args()
    global EAGER_BATCHES
    EAGER_BATCHES = args.eager_batches
    if args.gpus != 1:
        sys.exit('bench.py: this build runs on one GPU; --gpus above 1 is not supported '
                 '(the path shards by tokens with no exchange, but no multi-GPU run is part of it)')
    if not torch.cuda.is_available():
        sys.exit('bench.py: no GPU visible')
    import quest_amd as quest
    from quest_amd import _lib
    _lib.load()
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)

    if args.only == 'quantize':
        print(json.dumps({'roofline_quantize': bench_quantize(_lib, max(args.steps, 100), args.warmup, dev)}))
        return
    if args.only == 'decode':
        print(json.dumps({'decode': bench_decode(_lib, dev)}))
        return
    # the bandwidth-bound kernel first: after a few hundred GEMM launches the power controller holds the core clock
    # down for a while, which this kernel (a third of its time is arithmetic) would inherit
    rq = bench_quantize(_lib, max(args.steps, 100), args.warmup, dev)
    lin = bench_linear(quest, _lib, args.steps, args.warmup, dev)
    dec = bench_decode(_lib, dev)
    few_hundred = bench_decode(_lib, dev, ms=(128, 256, 384))
    fwd = None if args.no_forward else bench_forward(dev)
    e2e = None
    if not args.no_forward:
        # the reference's end-to-end benchmark (gemm-quest/benchmarks/bench_e2e.py) at its largest batch: the 1600M model,
        # 8 x 512 tokens; every batch size: python -m quest_amd.bench_e2e
        from quest_amd import bench_e2e
        e2e = bench_e2e.get_timing('1600m', (8,))[0]
    layer_sweep = None
    if args.layer_sweep:
        from quest_amd import bench_layer
        layer_sweep = bench_layer.as_records(bench_layer.get_timing(batch_sizes=[32, 512, 4096, 16384]))
    calibration_stream(dev)
    cpu = None if args.no_cpu_baseline else bench_cpu_baseline()
    if cpu is not None:
        cpu['gpu_same_workload'] = bench_small_layer_gpu(quest, dev)

    ops_gemm = 2.0 * 4096 * 4096 * 11008
    plan = gemm_plan(_lib.load(), 4096, 4096, 11008, dev)
    int8_tops = ops_gemm / (lin['int8_gemm_ms'] * 1e-3) / 1e12
    roofline = {'bound': 'mfma', 'achieved': lin['gemm_tops'], 'peak': INT8_MFMA_PEAK_TOPS, 'unit': 'TOP/s',
                'frac': lin['gemm_tops'] / INT8_MFMA_PEAK_TOPS,
                'peak_is': 'INT8 MFMA dense, the peak the metric is stated against; the kernel runs the same INT4 x INT4 products '
                           'on the FP6 (E2M3) matrix instructions, whose own dense peak is 10.1 PFLOP/s: frac_of_fp6_peak',
                'frac_of_fp6_peak': lin['gemm_tops'] / FP6_MFMA_PEAK_TOPS,
                'traffic': TRAFFIC_GEMM_BYTES, 'traffic_source': TRAFFIC_SOURCE, 'traffic_plan': TRAFFIC_GEMM_PLAN, 'plan': plan,
                'traffic_stale': plan != TRAFFIC_GEMM_PLAN,
                'kernel': 'gemm_e2m3_kernel', 'us_per_launch': lin['gemm_ms'] * 1e3,
                'us_per_launch_min': lin['gemm_min_ms'] * 1e3,
                'us_per_launch_weights_from_hbm': lin['gemm_rotating_weights_ms'] * 1e3,
                'int8_kernel_same_codes': {'kernel': 'gemm_w4a4_big_kernel', 'us_per_launch': lin['int8_gemm_ms'] * 1e3,
                                           'achieved': int8_tops, 'frac': int8_tops / INT8_MFMA_PEAK_TOPS},
                'vendor_int8_gemm_same_shape_us': None if lin['vendor_int8_ms'] is None else lin['vendor_int8_ms'] * 1e3,
                'algorithmic_ops': ops_gemm,
                'workload': 'uniform random INT4 codes on both sides (as E2M3 tiles), M=4096 K=4096 N=11008, fp16 out'}
    line = {
        'metric': 'INT4-GEMM TOPS + quantize GB/s at Llama-7B layer shapes, % MI355X roofline',
        'value': lin['tops'], 'unit': 'TOPS', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'untimed_steps': args.warmup + lin['untimed_replays'] * args.steps,
        'ms_per_step': lin['ms_per_step'], 'ms_per_step_eager_launches': lin['ms_per_step_eager'],
        'step_issue': f"one HIP graph of K steps, timed as K steps between two synchronisations after the W warm-up steps and "
                      f"{lin['untimed_replays']} untimed replays (60 ms: the clocks settle); median of five such timings, all in "
                      "ms_per_step_each; the eager figure beside it",
        'ms_per_step_each': lin['ms_per_step_each'], 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'fp6 (E2M3 products of INT4 codes, fp32 accumulation: exact)', 'data': 'synthetic',
        'config': {'workload': 'W4A4 linear, Llama-7B gate/up: fp16 activations [4096,4096] -> fused '
                               'Hadamard-quantize (INT4 codes as E2M3 tiles) -> INT4 x INT4 GEMM [4096,4096]x[11008,4096]^T on the FP6 '
                               'matrix instructions -> fp16 [4096,11008]',
                   'M': 4096, 'K': 4096, 'N': 11008},
        'gemm_tops': lin['gemm_tops'], 'gemm_us_in_step': lin['gemm_in_step_ms'] * 1e3,
        'gemm_tops_on_quantized_activations': 2.0 * 4096 * 4096 * 11008 / (lin['gemm_quantized_acts_ms'] * 1e-3) / 1e12,
        'packed_nibble_path': {'what': 'the same layer through the activation kernel writing nibbles and the INT8 kernels (same output bits)',
                               'us_per_step': lin['step_int8_ms'] * 1e3,
                               'gemm_us_on_quantized_activations': lin['int8_quantized_ms'] * 1e3},
        'quantize_us_in_step': lin['quant_ms'] * 1e3,
        'quantize_GBs': rq['achieved'],
        'quantize_tiles_in_step_shape': {'workload': 'fp16 [4096,4096] -> E2M3 tiles + scales (the step\'s own activation kernel), graph of 100 bare launches',
                                         'us_per_launch': lin['quant_tiles_alone_ms'] * 1e3,
                                         'GBs': (4096 * 4096 * 2.75 + 4096 * 2) / (lin['quant_tiles_alone_ms'] * 1e-3) / 1e9,
                                         'frac_hbm': (4096 * 4096 * 2.75 + 4096 * 2) / (lin['quant_tiles_alone_ms'] * 1e-3) / 1e9 / HBM_PEAK_GBS},
        'quantize_in_step_shape': {'workload': 'fp16 [4096,4096] -> packed nibbles, scales, row sums (the packed path\'s activation kernel), graph of 100 bare launches',
                                   'us_per_launch': lin['quant_alone_ms'] * 1e3,
                                   'GBs': (4096 * 4096 * 2.5 + 4096 * 6) / (lin['quant_alone_ms'] * 1e-3) / 1e9,
                                   'frac_hbm': (4096 * 4096 * 2.5 + 4096 * 6) / (lin['quant_alone_ms'] * 1e-3) / 1e9 / HBM_PEAK_GBS},
        'roofline': roofline, 'roofline_quantize': rq, 'decode': dec, 'few_hundred_tokens': few_hundred, 'forward': fwd, 'e2e_1600m_batch8': e2e,
        'cpu_baseline': cpu,
    }
    if layer_sweep is not None:
        line['layer_sweep'] = layer_sweep
    print(json.dumps(line))


if __name__ == '__main__':
    main()
