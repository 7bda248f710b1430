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
host cores for the same workload and doubles as the in-run parity check.
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
MEASURED_TRAFFIC_BYTES = {1: 89.03e6, 2: 44.13e6, 3: 84.47e6, 4: 371.84e6, 5: 297.31e6}

WORKLOADS = {
    1: 'per_token_cast e4m3 1x128, bf16 [4096,7168]',
    2: 'per_block_cast e4m3 128x128, bf16 [7168,2048]',
    3: 'swiglu_forward_and_per_token_cast e4m3 1x128, bf16 [8192,4096]',
    4: 'swiglu_forward_and_per_token_cast e4m3 1x128 MoE-expanded (4096 tokens, top-8 of 256, pad 128), bf16 [R,4096]',
    5: 'per_token_cast e2m1 1x32 packed UE8M0, bf16 [16384,7168]',
}


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
            self.bytes = x.numel() * 2 + out_shape[0] * out_shape[1] + M * (K // group) * (4 if cfg == 1 else 1)
        elif cfg == 2:
            K = x.shape[1]
            oc = get_cast_output_config('e4m3', (128, 128))
            out_shape = (M, K)
            self.bytes = x.numel() * 2 + M * K + (M // 128) * (K // 128) * 4
        else:
            H = x.shape[1] // 2
            oc = get_cast_output_config('e4m3', (1, 128))
            out_shape = (M, H)
            live = M if cfg == 3 else int((data['pos_to_expert'] >= 0).sum())
            # padding rows are not read; their zero codes and scales are written
            self.bytes = live * 4 * H + (0 if cfg == 3 else 4 * M) + M * H + M * (H // 128) * 4
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

    def result(self, i: int = 0):
        """(codes, scales) of buffer set i as the public API would return them."""
        from tilekernels_amd.quant.common import cast_epilogue
        x = self.host['x']
        hidden = x.shape[1] if self.cfg in (1, 2, 5) else x.shape[1] // 2
        return self.out[i], cast_epilogue(self.sf[i], x.shape[0], hidden, self.oc)


def time_gpu(w: Workload, steps: int, warmup: int):
    """Returns (wall seconds for `steps` launches, HIP-event microseconds per launch over the same
    timed region, list of single-launch durations from per-launch event pairs)."""
    for i in range(warmup):
        w.launch(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()          # torch's current stream is the stream the launches go to
    for i in range(steps):
        w.launch(i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    region_us = e0.elapsed_time(e1) * 1e3 / steps
    # single launches: one event pair around each (adds the cost of the two event records)
    n = min(steps, 200)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i in range(n):
        ev[i][0].record()
        w.launch(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    per = [a.elapsed_time(b) * 1e3 for a, b in ev]
    return wall, region_us, per


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


def cpu_baseline(w: Workload, budget_s: float = 12.0):
    """Times the CPU oracle on the full workload (repeated until the budget is used) and checks the
    GPU result of buffer set 0 against it."""
    from oracle import torch_ref
    from tests._util import dense_bytes, fp8_code_report
    threads = min(16, os.cpu_count() or 1)
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
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)

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
    base = {'value': round(w.bytes / med / 1e9, 3), 'unit': 'GB/s', 'cores': threads, 'kind': 'port',
            'ms_per_call': round(med * 1e3, 3),
            'sample': f'full workload, {len(times)} timed calls of the torch CPU oracle after 1 warm-up (median)'}
    return base, parity


def bench_config(cfg: int, steps: int, warmup: int, with_cpu: bool, with_two_streams: bool = True):
    w = Workload(cfg)
    wall, kern_us, per = time_gpu(w, steps, warmup)
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
        'us_per_call': round(ms_per_step * 1e3, 3), 'pct_of_hbm_peak': round(100 * value / HBM_PEAK_GBS, 2),
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': MEASURED_TRAFFIC_BYTES[cfg],
                     'kernel_us': round(kern_us, 3), 'timing': f'HIP events around the {steps} timed launches / {steps}',
                     'single_launch_us_median': round(statistics.median(per), 3), 'single_launch_us_min': round(min(per), 3)},
    }
    # informational: what the same entry point sustains when independent calls overlap
    if with_two_streams:
        us2 = time_two_streams(w, steps)
        line['two_streams'] = {'us_per_call': round(us2, 3), 'GBps': round(w.bytes / us2 / 1e3, 1),
                               'pct_of_hbm_peak': round(w.bytes / us2 / 1e3 / HBM_PEAK_GBS * 100, 2),
                               'note': 'calls alternate over two HIP streams; not used for value'}
    if with_cpu:
        line['cpu_baseline'], line['parity'] = cpu_baseline(w)
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=5000)
    ap.add_argument('--warmup', type=int, default=2000,
                    help='untimed launches first; the GPU needs ~15 ms of load to reach its steady clocks')
    ap.add_argument('--config', type=int, default=3, choices=sorted(WORKLOADS))
    ap.add_argument('--all-configs', action='store_true', help='also print one line per other configuration to stderr')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU-oracle baseline / parity leg')
    ap.add_argument('--single-stream-only', action='store_true',
                    help='skip the informational two-stream leg (for kernel traces: overlapping launches there would '
                         'inflate the per-kernel durations)')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run plain device copies of known size (reference kernel for hardware-counter runs)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: this path has no multi-GPU component (rows are independent; '
                 'run one process per GPU on its own row range). Use --gpus 1.')
    if not torch.cuda.is_available():
        sys.exit('bench.py needs a GPU')
    if args.all_configs:
        for cfg in sorted(WORKLOADS):
            if cfg != args.config:
                print(json.dumps(bench_config(cfg, args.steps, args.warmup, not args.no_cpu, not args.single_stream_only)),
                      file=sys.stderr, flush=True)
    line = bench_config(args.config, args.steps, args.warmup, not args.no_cpu, not args.single_stream_only)
    if args.copy_calibration:
        line.update(copy_calibration())
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()
