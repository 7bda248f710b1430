#!/usr/bin/env python3
"""Benchmark of the quantisation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--all-configs]

A step is one call of the hot-path entry point (through the C ABI, on preallocated device
buffers) over one batch of synthetic, seeded input that already sits in HBM.  The default
workload is the headline one: fused SwiGLU + per-token 1x128 FP8 E4M3 quantisation of a bf16
[8192, 4096] activation.  Steps rotate over several independent buffer sets whose total size
exceeds the 256 MB last-level cache, so every call streams from HBM.

One JSON line goes to stdout.  `value` is algorithmic bytes (input read + codes written + scales
written) per wall-clock second over the timed region; `roofline.achieved` is the same byte count
over the kernel's mean duration taken with HIP events on the launch stream.  `cpu_baseline` times
the CPU oracle (test infrastructure, a restatement of the reference's torch implementation) on the
host cores for the same workload and doubles as the in-run parity check.  `configs` holds the same
figures, in short, for the other four benchmark configurations, and `same_traffic_reference` the time
of a stock PyTorch elementwise kernel that moves the same bytes (no arithmetic to speak of) on the same
buffers, next to the time per launch of this entry point on a four-row input (what a launch costs on
this stack whatever its size).  `launch_structure` says how a launch of this size is spent (gap between launches, start
of the waves, first data, streaming rate, spread between the XCDs), from time stamps the traffic-only kernel takes per
wave; `--timeline` prints only that.

`roofline.traffic` is measured too: before it touches the GPU the script runs itself twice per configuration under
rocprofv3 (FETCH_SIZE, then WRITE_SIZE, each scaled by a copy of known size in the same run; `--no-measure-traffic`
skips this and reports the figures of earlier such runs).

Before the `--warmup` launches the GPU is kept busy with the same launches for `--preheat-ms`
milliseconds (untimed): its clocks need about 15 ms of load to settle, and a handful of 15 us
launches does not provide that.
"""
import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LLC_BYTES = 256 << 20

# HBM bytes per launch from rocprofv3 counter runs of this script (FETCH_SIZE and WRITE_SIZE, each
# scaled by what the same counter reads for the 256 MiB copy of --copy-calibration); the summaries
# are kept under profiles/.  None where no counter run was made.
MEASURED_TRAFFIC_BYTES = {1: 89.04e6, 2: 44.14e6, 3: 84.61e6, 4: 371.83e6, 5: 297.30e6}

WORKLOADS = {
    1: 'per_token_cast e4m3 1x128, bf16 [4096,7168]',
    2: 'per_block_cast e4m3 128x128, bf16 [7168,2048]',
    3: 'swiglu_forward_and_per_token_cast e4m3 1x128, bf16 [8192,4096]',
    4: 'swiglu_forward_and_per_token_cast e4m3 1x128 MoE-expanded (4096 tokens, top-8 of 256, pad 128), bf16 [R,4096]',
    5: 'per_token_cast e2m1 1x32 packed UE8M0, bf16 [16384,7168]',
}


def algorithmic_bytes(cfg: int, data: dict) -> int:
    """Bytes the operator of configuration `cfg` has to move for the input `data` (make_baseline_input): the input
    read once, codes and scales written once.  Configuration 4 reads only the rows that are not padding, plus the
    4-byte mask entry of every row, and writes zero codes and scales for the padding rows."""
    x = data['x']
    M = x.shape[0]
    if cfg in (1, 5):
        K = x.shape[1]
        group, code_bytes, sf_bytes = (128, M * K, 4) if cfg == 1 else (32, M * K // 2, 1)
        return x.numel() * 2 + code_bytes + M * (K // group) * sf_bytes
    if cfg == 2:
        K = x.shape[1]
        return x.numel() * 2 + M * K + (M // 128) * (K // 128) * 4
    H = x.shape[1] // 2
    live = M if cfg == 3 else int((data['pos_to_expert'] >= 0).sum())
    return live * 4 * H + (0 if cfg == 3 else 4 * M) + M * H + M * (H // 128) * 4


class Workload:
    """Device buffers and the C-ABI launch closure of one benchmark configuration."""

    def __init__(self, cfg: int, nsets_min: int = 3):
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        from tilekernels_amd.quant.common import alloc_scaling_factors, get_cast_output_config, sf_leading_dim
        self.cfg = cfg
        self.tk = tk
        self.lib = _ffi.load()
        data = tk.testing.make_baseline_input(cfg)
        self.host = data
        x = data['x']
        M = x.shape[0]
        dev = torch.device('cuda:0')
        if cfg in (1, 5):
            K = x.shape[1]
            fmt, group = ('e4m3', 128) if cfg == 1 else ('e2m1', 32)
            kw = {} if cfg == 1 else dict(use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
            oc = get_cast_output_config(fmt, (1, group), **kw)
            out_shape = (M, K if cfg == 1 else K // 2)
        elif cfg == 2:
            K = x.shape[1]
            oc = get_cast_output_config('e4m3', (128, 128))
            out_shape = (M, K)
        else:
            H = x.shape[1] // 2
            oc = get_cast_output_config('e4m3', (1, 128))
            out_shape = (M, H)
        self.bytes = algorithmic_bytes(cfg, data)
        self.oc = oc
        set_bytes = x.numel() * 2 + out_shape[0] * out_shape[1]
        self.nsets = max(nsets_min, -(-int(1.6 * LLC_BYTES) // set_bytes))
        self.x = [x.to(dev) for _ in range(self.nsets)]
        self.out = [torch.empty(out_shape, dtype=oc.torch_dtype, device=dev) for _ in range(self.nsets)]
        self.sf = [alloc_scaling_factors((M, x.shape[1] if cfg in (1, 2, 5) else x.shape[1] // 2), oc, dev) for _ in range(self.nsets)]
        self.aux = {k: v.to(dev) for k, v in data.items() if k != 'x'}
        stream = torch.cuda.current_stream(dev).cuda_stream
        self.main_stream = stream
        lib = self.lib
        calls = []
        for i in range(self.nsets):
            xp, op, sp, ld = self.x[i].data_ptr(), self.out[i].data_ptr(), self.sf[i].data_ptr(), sf_leading_dim(self.sf[i])
            if cfg in (1, 5):
                args = (xp, 0, M, x.shape[1], x.shape[1], op, sp, ld, oc.fmt_code, oc.sf_block[1], oc.layout_code,
                        int(oc.round_sf), 0, stream)
                calls.append((lib.tk_per_token_cast, args))
            elif cfg == 2:
                args = (xp, 0, M, x.shape[1], op, sp, ld, oc.fmt_code, 128, 128, oc.layout_code, 0, 0, stream)
                calls.append((lib.tk_per_block_cast, args))
            else:
                pe = self.aux['pos_to_expert'].data_ptr() if cfg == 4 else 0
                args = (xp, 0, M, x.shape[1] // 2, op, sp, ld, 128, oc.layout_code, 0, -1.0, 0, 0, 0, pe, 0, 0.0, 0, 0, stream)
                calls.append((lib.tk_swiglu_per_token_cast, args))
        self.calls = calls

    def launch(self, i: int, stream: int = None) -> None:
        fn, args = self.calls[i % self.nsets]
        if stream is not None:
            args = args[:-1] + (stream,)      # the stream is the last argument of every entry point
        rc = fn(*args)
        if rc != 0:
            raise RuntimeError(f'launch failed with status {rc}')

    def small_launch(self, stream: int) -> None:
        """The same entry point on the first four rows (128 for the per-block cast) of buffer set 0."""
        fn, args = self.calls[0]
        rows = 128 if self.cfg == 2 else 4
        rc = fn(*(args[:2] + (rows,) + args[3:-1] + (stream,)))      # the row count is the third argument, the stream the last
        if rc != 0:
            raise RuntimeError(f'launch failed with status {rc}')

    def result(self, i: int = 0):
        """(codes, scales) of buffer set i as the public API would return them."""
        from tilekernels_amd.quant.common import cast_epilogue
        x = self.host['x']
        hidden = x.shape[1] if self.cfg in (1, 2, 5) else x.shape[1] // 2
        return self.out[i], cast_epilogue(self.sf[i], x.shape[0], hidden, self.oc)


def preheat(w: 'Workload', ms: float) -> float:
    """Untimed launches for at least `ms` milliseconds of GPU time; returns the milliseconds spent."""
    if ms <= 0:
        return 0.0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    per_batch = max(16, int(2000.0 / (w.bytes / 6e6)))     # about 2 ms of launches per batch at 6 TB/s
    spent, i = 0.0, 0
    e0.record()
    while spent < ms:
        for _ in range(per_batch):
            w.launch(i)
            i += 1
        e1.record()
        e1.synchronize()
        spent = e0.elapsed_time(e1)
    return spent


def time_gpu_graph(w: 'Workload', steps: int, warmup: int, chunk: int = 100):
    """The same launches enqueued by the GPU instead of the host: `chunk` launches on the rotating buffers are captured into
    one HIP graph and the graph is replayed until `steps` launches have run.  Under a profiler the host needs longer per
    launch than the kernel takes, the GPU idles between launches and the profiler's durations are those of a GPU whose
    clocks have dropped; replays keep the launches back to back.  Returns what time_gpu returns (the per-launch figure is
    the whole region over its launches; the first replay runs untimed)."""
    chunk = max(w.nsets, min(chunk, steps) // w.nsets * w.nsets)      # whole turns of the buffer sets
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for i in range(max(warmup, w.nsets)):
            w.launch(i, side.cuda_stream)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(chunk):
                w.launch(i, side.cuda_stream)
        replays = max(1, -(-steps // chunk))
        graph.replay()
        side.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        e1.record()
        while not e1.query():
            pass
        wall = (time.perf_counter() - t0) * steps / (replays * chunk)
        us = e0.elapsed_time(e1) * 1e3 / (replays * chunk)
    torch.cuda.synchronize()
    n = min(steps, 200)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i in range(n):
        ev[i][0].record()
        w.launch(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    return wall, us, us, [a.elapsed_time(b) * 1e3 for a, b in ev]


class RawEvents:
    """HIP events made by the runtime itself (the copy of it that torch has loaded) with hipEventDisableSystemFence: such an
    event is a time stamp in the stream and nothing else.  An ordinary event (torch's) also makes the kernels before it
    visible to the host, and the kernel behind it starts about 2 us later for that: a tenth of a microsecond per launch
    in a region of 20 launches with one event behind the first, nothing to speak of in a region of thousands."""
    NO_SYSTEM_FENCE = 0x20000000

    def __init__(self):
        import ctypes
        self.ct = ctypes
        hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), 'lib', 'libamdhip64.so'))
        hip.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
        hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        hip.hipEventQuery.argtypes = [ctypes.c_void_p]
        hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip = hip

    def make(self):
        e = self.ct.c_void_p()
        if self.hip.hipEventCreateWithFlags(self.ct.byref(e), self.NO_SYSTEM_FENCE) != 0:
            raise RuntimeError('hipEventCreateWithFlags failed')
        return e

    def record(self, e, stream: int) -> None:
        if self.hip.hipEventRecord(e, self.ct.c_void_p(stream)) != 0:
            raise RuntimeError('hipEventRecord failed')

    def done(self, e) -> bool:
        return self.hip.hipEventQuery(e) == 0

    def elapsed_us(self, a, b) -> float:
        ms = self.ct.c_float()
        if self.hip.hipEventElapsedTime(self.ct.byref(ms), a, b) != 0:
            raise RuntimeError('hipEventElapsedTime failed')
        return ms.value * 1e3

    def destroy(self, *events) -> None:
        for e in events:
            self.hip.hipEventDestroy(e)


def time_gpu(w: 'Workload', steps: int, warmup: int, fenceless: bool = False):
    """Returns (wall seconds for `steps` launches, HIP-event microseconds per launch, the same with the first launch
    left in, list of single-launch durations from per-launch event pairs).  `fenceless`: the three events of the
    timed region are RawEvents instead of torch's.

    The timed region starts on an idle GPU (it follows a synchronisation), and the first launch needs a few
    microseconds to get there that are no part of any kernel's duration (a kernel trace does not show them either).
    The per-launch figure is therefore the period of the launches behind the first: an event goes into the stream
    right behind the first launch, and the time from there to the end of the region is divided by steps - 1.  The wall
    clock covers all `steps` launches."""
    for i in range(warmup):
        w.launch(i)
    torch.cuda.synchronize()
    todo = [w.calls[i % w.nsets] for i in range(steps)]
    if fenceless:
        raw = RawEvents()
        e0, ef, e1 = raw.make(), raw.make(), raw.make()
        record, done = (lambda e: raw.record(e, w.main_stream)), raw.done
        elapsed_us = raw.elapsed_us
    else:
        e0, ef, e1 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        record, done = (lambda e: e.record()), (lambda e: e.query())      # torch's current stream is the stream the launches go to
        elapsed_us = lambda a, b: a.elapsed_time(b) * 1e3
    record(e0)
    t0 = time.perf_counter()
    for n, (fn, call_args) in enumerate(todo):
        if fn(*call_args) != 0:
            raise RuntimeError('launch failed')
        if n == 0:
            record(ef)
    record(e1)
    while not done(e1):     # the end of the region is seen by polling: a blocking wait wakes up tens of microseconds late
        pass
    wall = time.perf_counter() - t0
    torch.cuda.synchronize()
    region_all_us = elapsed_us(e0, e1) / steps
    region_us = elapsed_us(ef, e1) / (steps - 1) if steps >= 4 else region_all_us
    if fenceless:
        raw.destroy(e0, ef, e1)
    # single launches: one event pair around each (adds the cost of the two event records)
    n = min(steps, 200)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i in range(n):
        ev[i][0].record()
        w.launch(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    per = [a.elapsed_time(b) * 1e3 for a, b in ev]
    return wall, region_us, region_all_us, per


def _event_time_us(fn, n: int) -> float:
    for i in range(min(n, 200)):
        fn(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(n):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def same_traffic_reference(w: 'Workload', steps: int):
    """Kernels that move the same bytes as the configuration's operator and do no arithmetic to speak of, timed
    on the same rotating buffers with HIP events:
      * the library's own traffic-only kernel (tk_stream_floor: the operator's loads and stores, nothing else);
      * a stock PyTorch elementwise kernel of the same byte shape (comparison of the input with zero, or of its two
        halves, into a bool tensor of the output's shape);
      * this entry point on four rows, replayed from a HIP graph of 100 launches: what one launch costs between
        dependent launches in a stream, whatever its size.
    They overwrite the output buffers; the caller runs the operator again before looking at results.
    Configuration 5 (half-byte codes) gets the flat traffic-only kernel alone; None for configuration 4 (masked rows)."""
    if w.cfg == 5:
        # half-byte codes: the flat traffic-only kernel with 16-byte loads and 4-byte stores (8 codes per lane), two pieces per
        # wave like the operator; the 3.7 MB of scale bytes are not moved
        n = max(steps, 400)
        in_bytes = w.x[0].numel() * 2

        def floor5(i):
            k = i % w.nsets
            rc = w.lib.tk_stream_floor_flat(w.x[k].data_ptr(), in_bytes, 16, w.out[k].data_ptr(), 4, 2, w.main_stream)
            if rc != 0:
                raise RuntimeError(f'tk_stream_floor_flat failed with status {rc}')
        us = _event_time_us(floor5, n)
        moved = in_bytes + in_bytes // 4
        return {'traffic_only_kernel': {'what': 'tk_stream_floor_flat: the input in 16-byte loads, the codes in 4-byte stores, no scales, no arithmetic',
                                        'us_per_call': round(us, 3), 'pct_of_hbm_peak': round(moved / us / 1e3 / HBM_PEAK_GBS * 100, 2)}}
    if w.cfg not in (1, 2, 3):
        return None
    n = max(steps, 400)
    outs = [o.view(torch.bool) for o in w.out]
    rows, cols = w.x[0].shape[0], w.x[0].shape[1] // (2 if w.cfg == 3 else 1)
    stream = w.main_stream

    def stock(i):
        x = w.x[i % w.nsets]
        if w.cfg == 3:
            torch.gt(x[:, :cols], x[:, cols:], out=outs[i % w.nsets])
        else:
            torch.gt(x, 0, out=outs[i % w.nsets])

    def floor(i):
        k = i % w.nsets
        rc = w.lib.tk_stream_floor(w.x[k].data_ptr(), rows, cols, 1 if w.cfg == 3 else 0, w.out[k].data_ptr(),
                                   0 if w.cfg == 2 else w.sf[k].data_ptr(), stream)
        if rc != 0:
            raise RuntimeError(f'tk_stream_floor failed with status {rc}')

    res = {}
    us = _event_time_us(floor, n)
    res['traffic_only_kernel'] = {'what': 'tk_stream_floor: the loads and stores of this operator, no arithmetic',
                                  'us_per_call': round(us, 3), 'pct_of_hbm_peak': round(w.bytes / us / 1e3 / HBM_PEAK_GBS * 100, 2)}
    if w.cfg == 3:
        # the same traffic in the launch shape the operator uses at this size: the last 15 % of the rows by one-piece waves,
        # the 55 % before them by two-piece waves (tk_swiglu_per_token_cast, launches of about one to three occupancy rounds)
        r1, r2 = rows * 15 // 100 // 4 * 4, rows * 55 // 100 // 4 * 4

        def floor_tailed(i):
            k = i % w.nsets
            rc = w.lib.tk_stream_floor_tailed(w.x[k].data_ptr(), rows, cols, 1, w.out[k].data_ptr(), w.sf[k].data_ptr(), r2, r1, stream)
            if rc != 0:
                raise RuntimeError(f'tk_stream_floor_tailed failed with status {rc}')
        us = _event_time_us(floor_tailed, n)
        res['traffic_only_kernel_smaller_waves_at_the_end'] = {
            'what': f'tk_stream_floor_tailed: the same loads and stores, the last {r1} rows by one-piece and the {r2} before them by two-piece waves',
            'us_per_call': round(us, 3), 'pct_of_hbm_peak': round(w.bytes / us / 1e3 / HBM_PEAK_GBS * 100, 2)}
    us = _event_time_us(stock, n)
    moved = w.bytes - (0 if w.cfg == 2 else w.sf[0].numel() * w.sf[0].element_size())      # the stock kernel writes no scales
    res['stock_torch_kernel'] = {'what': 'torch.gt into a bool tensor of the output shape (same bytes per element, no scales)',
                                 'us_per_call': round(us, 3), 'pct_of_hbm_peak': round(moved / us / 1e3 / HBM_PEAK_GBS * 100, 2)}
    # launch cost: 100 launches on four rows in one graph, so that the host's enqueue rate does not limit it
    small = w.small_launch
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        small(side.cuda_stream)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(100):
                small(side.cuda_stream)
    torch.cuda.synchronize()
    us = _event_time_us(lambda i: graph.replay(), 20) / 100
    res['launch_cost_us'] = round(us, 3)
    res['launch_cost_what'] = 'this entry point on four rows (128 for the per-block cast), per launch, 100 launches per HIP graph replay'
    return res


def launch_timeline(cfg: int, launches: int = 14, preheat_ms: float = 40.0) -> dict:
    """How a launch of the configuration's size is spent, from per-wave time stamps of the traffic-only kernel
    (tk_stream_floor_timeline: the operator's loads and stores, every wave reporting its start, the arrival of its last
    load, the issue and the acknowledgement of its stores on the 100 MHz real-time counter, and where it ran).
    `launches` calls go out back to back on the rotating buffers; the first two are left out of the summary.
    All times in microseconds; figures are means over the launches unless they say otherwise."""
    import numpy as np
    if cfg not in (1, 3):
        raise SystemExit('--timeline knows the row-wise traffic of configurations 1 and 3')
    w = Workload(cfg)
    preheat(w, preheat_ms)
    rows, cols = w.x[0].shape[0], w.x[0].shape[1] // (2 if cfg == 3 else 1)
    words = int(w.lib.tk_stream_floor_stamp_words(rows, cols))
    stamps = torch.zeros((launches, words), dtype=torch.int64, device=w.x[0].device)
    torch.cuda.synchronize()
    for i in range(launches):
        k = i % w.nsets
        rc = w.lib.tk_stream_floor_timeline(w.x[k].data_ptr(), rows, cols, 1 if cfg == 3 else 0, w.out[k].data_ptr(), w.sf[k].data_ptr(),
                                            stamps[i].data_ptr(), w.main_stream)
        if rc != 0:
            raise RuntimeError(f'tk_stream_floor_timeline failed with status {rc}')
    torch.cuda.synchronize()
    t = stamps.cpu().numpy().reshape(launches, -1, 6)
    tick = 0.01                                     # 100 MHz
    bytes_per_wave = w.bytes / t.shape[1]
    spans, gaps, ramp50, ramp99, first_data, med_data, xcd_start, xcd_end, mid_rate, tail10 = [], [], [], [], [], [], [], [], [], []
    for i in range(2, launches):
        a = t[i]
        start = a[:, 0].min()
        rel = (a[:, :4] - start) * tick
        end = rel[:, 3].max()
        spans.append(end)
        if i + 1 < launches:
            gaps.append((t[i + 1][:, 0].min() - a[:, 3].max()) * tick)
        ramp50.append(float(np.percentile(rel[:, 0], 50)))
        ramp99.append(float(np.percentile(rel[:, 0], 99)))
        wait = rel[:, 1] - rel[:, 0]
        first_data.append(float(wait.min()))
        med_data.append(float(np.median(wait)))
        xcc = a[:, 5] & 0xF
        xcd_start.append([float(rel[xcc == x, 0].mean()) for x in range(8)])
        xcd_end.append([float(rel[xcc == x, 3].max()) for x in range(8)])
        mid = (rel[:, 1] >= 0.3 * end) & (rel[:, 1] < 0.7 * end)
        mid_rate.append(float(mid.sum() * bytes_per_wave / (0.4 * end) / 1e3))       # GB/s of the operator's bytes
        tail10.append(float(end - np.percentile(rel[:, 1], 90)))
    mean = lambda v: round(float(np.mean(v)), 3)
    xs, xe = np.array(xcd_start), np.array(xcd_end)
    return {
        'timeline': f'tk_stream_floor_timeline on the buffers of config {cfg}, {launches - 2} back-to-back launches',
        'waves_per_launch': int(t.shape[1]),
        'first_wave_to_last_acknowledgement_us': {'mean': mean(spans), 'min': round(min(spans), 3), 'max': round(max(spans), 3)},
        'last_acknowledgement_to_first_wave_of_next_launch_us': {'mean': mean(gaps), 'min': round(min(gaps), 3), 'max': round(max(gaps), 3)},
        'half_of_the_waves_started_after_us': mean(ramp50), 'all_but_1_percent_started_after_us': mean(ramp99),
        'wave_start_to_its_last_load_us': {'shortest': mean(first_data), 'median': mean(med_data)},
        'mean_wave_start_per_xcd_us': [round(float(v), 3) for v in xs.mean(axis=0)],
        'last_acknowledgement_per_xcd_us': {'mean': [round(float(v), 3) for v in xe.mean(axis=0)],
                                             'spread_within_a_launch_mean': mean(xe.max(axis=1) - xe.min(axis=1)),
                                             'spread_within_a_launch_max': round(float((xe.max(axis=1) - xe.min(axis=1)).max()), 3)},
        'operator_bytes_per_second_in_the_middle_40_percent_GBps': mean(mid_rate),
        'last_tenth_of_the_loads_arrives_within_us_of_the_end': mean(tail10),
    }


VARIANTS = {'base': 0, 'pkfloor': 1, 'widest': 2, 'prio': 3, 'piecesf': 4, 'late': 5, 'ahead': 6, 'rounds': 7, 'tail': 8}


def variant_ab(specs, steps: int, rounds: int = 4, preheat_ms: float = 40.0) -> dict:
    """Times alternative structures of the headline kernel (tk_swiglu_cast_variant: measurement aids of the library, not
    reachable from the Python API) against the product entry point on configuration 3's buffers: `rounds` rounds, each
    timing the product and every variant in turn over `steps` launches with HIP events.  Every variant's codes and scales
    are first compared with the product's, bit for bit.  `specs`: names from VARIANTS, each optionally followed by
    ':<parameter>'."""
    w = Workload(3)
    preheat(w, preheat_ms)
    x = w.host['x']
    R, H = x.shape[0], x.shape[1] // 2
    stream = w.main_stream
    legs = [('product', lambda i: w.launch(i))]
    for spec in specs:
        name, _, par = spec.partition(':')
        if name not in VARIANTS:
            raise SystemExit(f'unknown variant {name!r}; known: {", ".join(VARIANTS)}')
        code, param = VARIANTS[name], int(par) if par else 0

        def call(i, code=code, param=param):
            k = i % w.nsets
            rc = w.lib.tk_swiglu_cast_variant(w.x[k].data_ptr(), R, H, w.out[k].data_ptr(), w.sf[k].data_ptr(), code, param, stream)
            if rc != 0:
                raise RuntimeError(f'tk_swiglu_cast_variant failed with status {rc}')
        legs.append((spec, call))
    w.launch(0)
    torch.cuda.synchronize()
    ref_codes, ref_sf = w.out[0].view(torch.uint8).clone(), w.sf[0].clone()
    parity = {}
    for spec, call in legs[1:]:
        w.out[0].view(torch.uint8).fill_(0xAB)
        w.sf[0].fill_(-1.0)
        call(0)
        torch.cuda.synchronize()
        parity[spec] = bool(torch.equal(w.out[0].view(torch.uint8), ref_codes) and torch.equal(w.sf[0], ref_sf))
    times = {spec: [] for spec, _ in legs}
    for _ in range(rounds):
        for spec, call in legs:
            times[spec].append(round(_event_time_us(call, steps), 3))
    return {'workload': WORKLOADS[3], 'steps': steps, 'rounds': rounds,
            'us_per_launch': {k: {'median': round(statistics.median(v), 3), 'runs': v} for k, v in times.items()},
            'identical_to_product': parity}


def time_two_streams(w: Workload, steps: int):
    """Same calls, alternating over two streams: consecutive calls are independent batches, so the
    ramp-up of one overlaps the drain of the other.  Returns microseconds per call."""
    side = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for i in range(200):
        w.launch(i, side[i & 1].cuda_stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        w.launch(i, side[i & 1].cuda_stream)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e6


def copy_calibration(n_copies: int = 20, mib: int = 256):
    """Plain device copies of a known size, so that a hardware-counter run of this script also
    holds a kernel whose HBM bytes are known (reads `mib` MiB, writes `mib` MiB per copy)."""
    src = torch.arange((mib << 20) // 4, dtype=torch.int32, device='cuda:0')
    dst = torch.empty_like(src)
    for _ in range(n_copies):
        torch.add(src, 1, out=dst)      # an ordinary elementwise kernel: one read and one write per element
    torch.cuda.synchronize()
    return {'copy_calibration': {'copies': n_copies, 'bytes_read_each': mib << 20, 'bytes_written_each': mib << 20}}


def under_a_profiler() -> bool:
    """Whether a ROCm profiler is loaded into this process.  Its tool library initialises the GPU before the program
    starts, and a process in that state must not start other programs: the counter leg is skipped then.  (PyTorch
    itself maps librocprofiler-register and libroctracer64; a profiler brings its tool library and its variables.)"""
    env = os.environ
    if env.get('HSA_TOOLS_LIB') or env.get('ROCP_TOOL_LIBRARIES') or any(k.startswith('ROCPROF') for k in env):
        return True
    if any(name in env.get('LD_PRELOAD', '') for name in ('rocprofiler-sdk', 'rocprofiler64', 'roctracer', 'rocprof-')):
        return True
    try:
        with open('/proc/self/maps') as f:
            return any('rocprofiler-sdk' in line or 'rocprofiler64' in line or 'tracer_tool' in line for line in f)
    except OSError:
        return True


def measure_traffic(cfg: int, timeout_s: float = 60.0) -> dict:
    """HBM bytes per launch of configuration `cfg`, from two hardware-counter runs of this script under rocprofv3
    (FETCH_SIZE, then WRITE_SIZE: KiB per dispatch, one counter per run), each scaled by what the same counter reads
    for the 256 MiB copies of --copy-calibration in the same run.  The profiler runs as a child process, so this
    has to be called before the calling process touches the GPU."""
    import collections
    import csv
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    exe = shutil.which('rocprofv3')
    if exe is None:
        raise RuntimeError('rocprofv3 is not on PATH')
    tmp = tempfile.mkdtemp(prefix='tk_traffic_', dir='/tmp')
    cal_bytes = 256 << 20
    result = {}
    try:
        for counter in ('FETCH_SIZE', 'WRITE_SIZE'):
            out_dir = os.path.join(tmp, counter)
            cmd = [exe, '--pmc', counter, '--output-format', 'csv', '-d', out_dir, '-o', 'c', '--', sys.executable,
                   os.path.abspath(__file__), '--only', '--no-cpu', '--single-stream-only', '--config', str(cfg), '--steps', '100',
                   '--warmup', '20', '--preheat-ms', '0', '--copy-calibration', '--no-measure-traffic']
            child = subprocess.Popen(cmd, cwd='/tmp', env=dict(os.environ, TMPDIR='/tmp'), stdout=subprocess.DEVNULL,
                                     stderr=subprocess.DEVNULL, start_new_session=True)
            try:
                rc = child.wait(timeout_s)
            except subprocess.TimeoutExpired:
                os.killpg(child.pid, signal.SIGKILL)
                child.wait()
                raise RuntimeError(f'the {counter} run did not finish within {timeout_s:.0f} s')
            if rc != 0:
                raise RuntimeError(f'the {counter} run exited with {rc}')
            files = glob.glob(os.path.join(out_dir, '**', '*counter_collection.csv'), recursive=True)
            if not files:
                raise RuntimeError(f'the {counter} run left no counter file')
            per_kernel = collections.defaultdict(list)
            with open(files[0], newline='') as f:
                for row in csv.DictReader(f):
                    if row['Counter_Name'] == counter:
                        per_kernel[row['Kernel_Name']].append(float(row['Counter_Value']))
            cal = [v for k, v in per_kernel.items() if 'CUDAFunctorOnSelf_add<int>' in k]
            ours = [v for k, v in per_kernel.items() if 'tk::' in k and 'stream_floor' not in k]
            if len(cal) != 1 or not ours:
                raise RuntimeError(f'the {counter} run holds {len(cal)} calibration kernels and {len(ours)} kernels of the library')
            mine = max(ours, key=len)                           # the timed kernel is the one with the most dispatches
            scale = (cal_bytes / 1024.0) / (sum(cal[0]) / len(cal[0]))
            result[counter] = {'kib_per_dispatch': round(sum(mine) / len(mine), 1), 'dispatches': len(mine), 'scale': round(scale, 5),
                               'bytes': sum(mine) / len(mine) * scale * 1024.0}
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return {'bytes': round(result['FETCH_SIZE']['bytes'] + result['WRITE_SIZE']['bytes']),
            'read_bytes': round(result['FETCH_SIZE']['bytes']), 'written_bytes': round(result['WRITE_SIZE']['bytes']),
            'fetch_scale': result['FETCH_SIZE']['scale'], 'write_scale': result['WRITE_SIZE']['scale'],
            'dispatches': result['FETCH_SIZE']['dispatches']}


def cpu_baseline(w: Workload, budget_s: float = 12.0, min_runs: int = 3):
    """Times the CPU oracle on the full workload (repeated until the budget is used) and checks the
    GPU result of buffer set 0 against it."""
    from oracle import torch_ref
    from tests._util import dense_bytes, fp8_code_report
    # threads: the CPUs this process may run on (the affinity mask and OMP_NUM_THREADS, which the GPU boxes set to
    # their per-GPU share of the host); host_cores: what the machine has
    host_cores = os.cpu_count() or 1
    share = len(os.sched_getaffinity(0)) if hasattr(os, 'sched_getaffinity') else host_cores
    threads = max(1, min(share, int(os.environ.get('OMP_NUM_THREADS', share) or share)))
    torch.set_num_threads(threads)
    d = w.host
    x = d['x']

    def run():
        if w.cfg == 1:
            return torch_ref.cast(x, 'e4m3', (1, 128))
        if w.cfg == 2:
            return torch_ref.cast(x, 'e4m3', (128, 128))
        if w.cfg == 3:
            return torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
        if w.cfg == 4:
            return torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=d['pos_to_expert'])
        return torch_ref.cast(x, 'e2m1', (1, 32), round_sf=True, use_tma_aligned_col_major_sf=True, use_packed_ue8m0=True)

    ref = run()   # warm-up, and the parity reference
    times = []
    t_start = time.perf_counter()
    while len(times) < min_runs or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)

    w.launch(0)        # other legs of the benchmark may have written to the output buffers since
    codes, sf = w.result(0)
    torch.cuda.synchronize()
    frac, one_step = fp8_code_report(dense_bytes(codes.cpu()), dense_bytes(ref[0])) if w.cfg != 5 else \
        (float((dense_bytes(codes.cpu()) != dense_bytes(ref[0])).float().mean()), True)
    a = torch.empty(sf.shape, dtype=sf.dtype).copy_(sf.cpu())
    b = torch.empty(sf.shape, dtype=sf.dtype).copy_(ref[1])
    if a.dtype == torch.float32:
        sf_rel = float(((a - b).abs() / b.abs().clamp(min=1e-30)).max())
    else:
        sf_rel = float((a != b).float().mean())
    parity = {'codes_differing_frac': frac, 'code_diffs_one_step': one_step, 'scale_max_rel_err': sf_rel}
    base = {'value': round(w.bytes / med / 1e9, 3), 'unit': 'GB/s', 'cores': threads, 'host_cores': host_cores, 'kind': 'port',
            'ms_per_call': round(med * 1e3, 3),
            'sample': f'full workload, {len(times)} timed calls of the torch CPU oracle after 1 warm-up (median)'}
    return base, parity


def bench_config(cfg: int, steps: int, warmup: int, with_cpu: bool, with_two_streams: bool = True, preheat_ms: float = 40.0,
                 cpu_budget_s: float = 12.0, with_reference: bool = True, traffic: dict = None, graph: bool = False,
                 fenceless: bool = False):
    w = Workload(cfg)
    heated = preheat(w, preheat_ms)
    wall, kern_us, kern_all_us, per = time_gpu_graph(w, steps, warmup) if graph else time_gpu(w, steps, warmup, fenceless)
    ms_per_step = wall / steps * 1e3
    value = w.bytes / (wall / steps) / 1e9
    achieved = w.bytes / (kern_us * 1e-6) / 1e9
    line = {
        'metric': 'HBM GB/s (% of MI355X peak) + \u00b5s/call, fused SwiGLU+FP8 quant [8192,4096]' if cfg == 3 else f'HBM GB/s, config {cfg}',
        'value': round(value, 1), 'unit': 'GB/s', 'n_gpus': 1, 'steps': steps, 'warmup': warmup,
        'ms_per_step': round(ms_per_step, 6), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': WORKLOADS[cfg], 'algorithmic_bytes': w.bytes, 'buffer_sets': w.nsets,
                   'boundary': 'C ABI (ctypes), preallocated outputs'},
        'preheat_ms': round(heated, 1),
        'us_per_call': round(ms_per_step * 1e3, 3), 'pct_of_hbm_peak': round(100 * value / HBM_PEAK_GBS, 2),
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBS, 4),
                     'traffic': float(traffic['bytes']) if traffic and 'bytes' in traffic else MEASURED_TRAFFIC_BYTES[cfg],
                     'traffic_source': ('rocprofv3 FETCH_SIZE and WRITE_SIZE runs started by this run' if traffic and 'bytes' in traffic
                                        else 'earlier rocprofv3 counter runs of this script (profiles/)'),
                     'kernel_us': round(kern_us, 3),
                     'timing': ('HIP events around replays of a HIP graph of launches on the rotating buffers (about 100 per replay), per launch' if graph else
                                f'HIP events{" without a system fence" if fenceless else ""}: from behind the first of the {steps} timed launches to the end of the region / {steps - 1} '
                                '(the region starts on an idle GPU; what the first launch takes to get there is no kernel time)'
                                if steps >= 4 else f'HIP events around the {steps} timed launches / {steps}'),
                     'kernel_us_first_launch_included': round(kern_all_us, 3),
                     'single_launch_us_median': round(statistics.median(per), 3), 'single_launch_us_min': round(min(per), 3)},
    }
    if with_reference:
        try:        # a side measurement: its failure must not cost the line
            ref = same_traffic_reference(w, steps)
        except Exception as e:      # noqa: BLE001
            ref = {'error': f'{type(e).__name__}: {e}'}
            torch.cuda.synchronize()
        if ref is not None:
            line['same_traffic_reference'] = ref
    # informational: what the same entry point sustains when independent calls overlap
    if with_two_streams:
        us2 = time_two_streams(w, max(steps, 200))
        line['two_streams'] = {'us_per_call': round(us2, 3), 'GBps': round(w.bytes / us2 / 1e3, 1),
                               'pct_of_hbm_peak': round(w.bytes / us2 / 1e3 / HBM_PEAK_GBS * 100, 2),
                               'note': 'calls alternate over two HIP streams; not used for value'}
    if with_cpu:
        line['cpu_baseline'], line['parity'] = cpu_baseline(w, cpu_budget_s, 3 if cpu_budget_s >= 6 else 1)
    return line


def short_form(line: dict, cfg: int) -> dict:
    """One entry of the `configs` array."""
    out = {'cfg': cfg, 'workload': line['config']['workload'], 'us': line['roofline']['kernel_us'],
           'us_wall': line['us_per_call'], 'GBps': line['roofline']['achieved'], 'frac': line['roofline']['frac'],
           'traffic': line['roofline']['traffic']}
    if 'cpu_baseline' in line:
        out['cpu_ms'] = line['cpu_baseline']['ms_per_call']
        out['parity'] = line['parity']
    if 'same_traffic_reference' in line and 'error' not in line['same_traffic_reference']:
        ref = line['same_traffic_reference']
        out['traffic_only_kernel_us'] = ref['traffic_only_kernel']['us_per_call']
        if 'stock_torch_kernel' in ref:
            out['stock_torch_kernel_us'] = ref['stock_torch_kernel']['us_per_call']
            out['launch_cost_us'] = ref['launch_cost_us']
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=5000)
    ap.add_argument('--warmup', type=int, default=2000, help='untimed launches directly before the timed ones')
    ap.add_argument('--preheat-ms', type=float, default=40.0,
                    help='untimed launches for this many milliseconds before the warm-up: the GPU needs ~15 ms of load to '
                         'reach its steady clocks')
    ap.add_argument('--config', type=int, default=3, choices=sorted(WORKLOADS))
    ap.add_argument('--only', action='store_true', help='leave out the `configs` array (the other four configurations)')
    ap.add_argument('--all-configs', action='store_true', help='also print the full line of every other configuration to stderr')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU-oracle baseline / parity leg')
    ap.add_argument('--single-stream-only', action='store_true',
                    help='skip the informational two-stream leg and the same-traffic reference kernel (for kernel traces: '
                         'overlapping launches there would inflate the per-kernel durations)')
    ap.add_argument('--no-measure-traffic', action='store_true',
                    help='skip the hardware-counter leg: by default this script first runs itself twice per configuration under '
                         'rocprofv3 (FETCH_SIZE, then WRITE_SIZE; a few seconds each) and reports the HBM bytes per launch measured '
                         'there as roofline.traffic; without it, or if the profiler fails, the figures of earlier such runs are reported')
    ap.add_argument('--timeline', action='store_true',
                    help='instead of the benchmark, print how a launch of the configuration\'s size is spent (per-wave time stamps '
                         'of the traffic-only kernel over a few back-to-back launches; configurations 1 and 3)')
    ap.add_argument('--no-launch-structure', action='store_true',
                    help='leave out `launch_structure` (what --timeline prints, appended to the full line of configurations 1 and 3)')
    ap.add_argument('--variant', type=str, default=None,
                    help='instead of the benchmark, time alternative structures of the headline kernel against the product: a comma-separated '
                         f'list of {", ".join(VARIANTS)}, each optionally with ":<parameter>" (see csrc/swiglu_cast_variants.hip)')
    ap.add_argument('--graph', action='store_true',
                    help='enqueue the timed launches of --config from a HIP graph (100 launches per replay) instead of from the host: '
                         'for runs under a profiler, where the host is slower than the kernel')
    ap.add_argument('--fenceless-events', action='store_true',
                    help='time the region of --config with HIP events created with hipEventDisableSystemFence (time stamps only) instead '
                         'of torch\'s: the event behind the first launch then does not hold up the second; matters for regions of tens of launches')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run plain device copies of known size (reference kernel for hardware-counter runs)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: this path has no multi-GPU component (rows are independent; '
                 'run one process per GPU on its own row range). Use --gpus 1.')
    if args.timeline:
        if not torch.cuda.is_available():
            sys.exit('bench.py needs a GPU')
        print(json.dumps(launch_timeline(args.config, preheat_ms=args.preheat_ms)), flush=True)
        return
    if args.variant:
        if not torch.cuda.is_available():
            sys.exit('bench.py needs a GPU')
        print(json.dumps(variant_ab(args.variant.split(','), min(args.steps, 4000), preheat_ms=args.preheat_ms)), flush=True)
        return
    traffic = {}
    if not args.no_measure_traffic and not under_a_profiler():        # child processes: started before this process touches the GPU
        for cfg in ([args.config] if args.only else sorted(WORKLOADS)):
            try:
                traffic[cfg] = measure_traffic(cfg)
            except Exception as e:      # noqa: BLE001  (a side measurement: the stored figure is reported instead)
                traffic[cfg] = {'error': f'{type(e).__name__}: {e}'}
                break                   # and the other configurations are not tried
    if not torch.cuda.is_available():
        sys.exit('bench.py needs a GPU')
    two = not args.single_stream_only
    line = bench_config(args.config, args.steps, args.warmup, not args.no_cpu, two, args.preheat_ms, 12.0, two, traffic.get(args.config),
                        args.graph, args.fenceless_events)
    if traffic:
        line['traffic_measurement'] = {str(c): t for c, t in traffic.items()}
    if not args.only:
        # the other configurations with the same steps and warm-up, a short CPU leg each (one timed call of the oracle
        # after its warm-up call, which is also the parity reference)
        others = []
        for cfg in sorted(WORKLOADS):
            if cfg == args.config:
                continue
            try:
                full = bench_config(cfg, args.steps, args.warmup, not args.no_cpu, False, args.preheat_ms, 0.0, two, traffic.get(cfg))
            except Exception as e:      # noqa: BLE001  (the headline line is printed whatever happens to a side leg)
                others.append({'cfg': cfg, 'workload': WORKLOADS[cfg], 'error': f'{type(e).__name__}: {e}'})
                continue
            if args.all_configs:
                print(json.dumps(full), file=sys.stderr, flush=True)
            others.append(short_form(full, cfg))
        line['configs'] = others
    if args.copy_calibration:
        line.update(copy_calibration())
    if not args.only and not args.no_launch_structure and args.config in (1, 3):
        try:        # a side measurement, taken after everything else: its failure must not cost the line
            line['launch_structure'] = launch_timeline(args.config, preheat_ms=args.preheat_ms)
        except Exception as e:      # noqa: BLE001
            line['launch_structure'] = {'error': f'{type(e).__name__}: {e}'}
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()
