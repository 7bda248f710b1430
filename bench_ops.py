#!/usr/bin/env python3
"""Kernel timings of the operators around the headline path, one JSON line per operator.

    python bench_ops.py [--steps 2000] [--warmup 1000] [--only NAME[,NAME...]]

Companion of bench.py (which measures the headline workload and keeps the driver's contract): the
same method -- C-ABI calls on preallocated device buffers, buffer sets rotated past the 256 MB
last-level cache, HIP events on the launch stream over the timed region -- applied to the
scale-only and given-scale variants of the casts, the weighted MoE form of the headline operator, the
dequantisation, the re-quantisation of quantised input, the MoE layout helpers, the fused SwiGLU
backward and the per-channel cast family.  `bytes` is the algorithmic HBM traffic of one call (inputs read once, outputs written
once); `frac` prices it against 8 TB/s; `cpu_baseline` times the CPU oracle on the same input.
"""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LLC_BYTES = 256 << 20


def nbytes(*tensors) -> int:
    return sum(t.numel() * t.element_size() for t in tensors)


class Op:
    """`build()` returns (callable launching one call on torch's current stream, algorithmic bytes,
    footprint bytes of the buffer set, factory of a callable that runs the CPU oracle on the same input)."""

    def __init__(self, name, workload, build, floor=None):
        # floor: (bytes read, bytes a lane reads per piece, bytes it writes per piece, pieces per wave) of the traffic-only
        # kernel (tk_stream_floor_flat) that moves this operator's code and value bytes in loads and stores of its widths
        self.name, self.workload, self.build, self.floor = name, workload, build, floor


def _sets_needed(footprint: int) -> int:
    # small operators (the mapping) are latency-bound: a handful of sets is enough there
    return min(16, max(3, -(-int(1.6 * LLC_BYTES) // max(footprint, 1))))


def op_cast_back(out_name='bf16'):
    def make():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        M, K = 8192, 4096
        x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
        codes, sf = tk.quant.per_token_cast(x, 'e4m3', num_per_channels=128)
        out = torch.empty((M, K), device='cuda', dtype=torch.bfloat16 if out_name == 'bf16' else torch.float32)
        out_dtype = _ffi.TK_BF16 if out_name == 'bf16' else _ffi.TK_F32
        stream = _ffi.current_stream(x.device)

        def launch():
            rc = lib.tk_cast_back(codes.data_ptr(), 0, M, K, sf.data_ptr(), sf.stride(0), 0, 1, 128, out.data_ptr(), out_dtype, stream)
            assert rc == 0, rc
        def cpu():
            from oracle import torch_ref
            xq = (codes.cpu(), sf.cpu())
            return lambda: torch_ref.cast_back(xq, out_name, (1, 128))
        return launch, nbytes(codes, sf, out), nbytes(codes, sf, out), cpu
    return make


def op_requant():
    import tilekernels_amd as tk
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    M, K = 8192, 4096
    x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
    codes, sf = tk.quant.per_token_cast(x, 'e4m3', num_per_channels=128)
    out = torch.empty((M, K // 2), device='cuda', dtype=torch.int8)
    out_sf = torch.empty((M, K // 32), device='cuda', dtype=torch.float32)
    stream = _ffi.current_stream(x.device)

    def launch():
        # E4M3 1x128 -> E2M1 1x32 (the path per_token_cast takes when handed a (codes, scales) pair)
        rc = lib.tk_per_token_cast_quantized(codes.data_ptr(), 0, M, K, K, sf.data_ptr(), sf.stride(0), 0, 1, 128,
                                             out.data_ptr(), out_sf.data_ptr(), out_sf.stride(0), 1, 32, 0, 0, stream)
        assert rc == 0, rc
    def cpu():
        from oracle import torch_ref
        xq = (codes.cpu(), sf.cpu())
        return lambda: torch_ref.cast(xq, 'e2m1', (1, 32), x_block_size=(1, 128))
    return launch, nbytes(codes, sf, out, out_sf), nbytes(codes, sf, out, out_sf), cpu


def _moe_maps(T=4096, K=8, E=256, alignment=128, seed=0):
    import tilekernels_amd as tk
    g = torch.Generator().manual_seed(seed)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices.contiguous().cuda()
    maps = tk.moe.get_fused_mapping(topk_idx, E, 0, alignment)
    return topk_idx, maps


def op_get_fused_mapping():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, E, alignment = 4096, 8, 256, 128
    topk_idx, maps = _moe_maps(T, K, E, alignment)
    p2e, p2t, ptt, t2p, es, ee, npe = maps[:7]
    R = p2e.numel()
    ws_bytes = lib.tk_fused_mapping_workspace_bytes(T, K, E)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device='cuda')
    stream = _ffi.current_stream(topk_idx.device)

    def launch():
        rc = lib.tk_get_fused_mapping(topk_idx.data_ptr(), T, K, E, alignment, R, p2e.data_ptr(), p2t.data_ptr(),
                                      ptt.data_ptr(), t2p.data_ptr(), es.data_ptr(), ee.data_ptr(), npe.data_ptr(),
                                      ws.data_ptr(), ws_bytes, stream)
        assert rc == 0, rc
    b = nbytes(topk_idx, p2e, p2t, ptt, t2p, es, ee, npe)

    def cpu():
        from oracle import torch_ref
        idx = topk_idx.cpu()
        return lambda: torch_ref.get_fused_mapping(idx, E, alignment)
    return launch, b, b, cpu


def op_expand_to_fused():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, hidden = 4096, 8, 4096
    _, maps = _moe_maps(T, K)
    p2e, t2p = maps[0], maps[3]
    R = p2e.numel()
    x = torch.randn((T, hidden), device='cuda', dtype=torch.bfloat16)
    out = torch.empty((R, hidden), device='cuda', dtype=torch.bfloat16)
    stream = _ffi.current_stream(x.device)

    def launch():
        rc = lib.tk_expand_to_fused(x.data_ptr(), T, hidden * 2, t2p.data_ptr(), K, p2e.data_ptr(), R, out.data_ptr(),
                                    0, 0, 0, 0, 0, stream)
        assert rc == 0, rc
    def cpu():
        from oracle import torch_ref
        xc, tc, pc = x.cpu(), t2p.cpu(), p2e.cpu()
        return lambda: torch_ref.expand_to_fused(xc, tc, pc)
    return launch, nbytes(x, out, t2p, p2e), nbytes(x, out, t2p, p2e), cpu


def op_swiglu_backward(group=128, rows=8192, hidden=2048):
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        R, H, T, K = rows, hidden, (rows + 7) // 8, 8
        x = torch.randn((R, 2 * H), device='cuda', dtype=torch.bfloat16)
        codes, sf = tk.quant.per_token_cast(x, 'e4m3', num_per_channels=group)
        del x
        go = torch.randn((R, H), device='cuda', dtype=torch.bfloat16)
        w = torch.rand((T, K), device='cuda')
        ptt = torch.randperm(T * K, device='cuda').to(torch.int32)
        t2p = torch.empty((T * K,), dtype=torch.int32, device='cuda')
        ptt = ptt[:R].contiguous()
        t2p.fill_(-1)
        t2p[ptt.long()] = torch.arange(R, dtype=torch.int32, device="cuda")
        out = torch.empty((R, H), device='cuda', dtype=torch.bfloat16)
        q = torch.empty((R, 2 * H), device='cuda', dtype=torch.float8_e4m3fn)
        q_sf = torch.empty((R, 2 * H // group), device='cuda', dtype=torch.float32)
        xg = torch.empty((R, 2 * H), device='cuda', dtype=torch.bfloat16)
        wg = torch.empty((T, K), device='cuda')
        stream = _ffi.current_stream(go.device)

        def launch():
            rc = lib.tk_swiglu_backward_per_token_cast(codes.data_ptr(), sf.data_ptr(), R, H, group, go.data_ptr(),
                                                       w.data_ptr(), ptt.data_ptr(), t2p.data_ptr(), T * K, out.data_ptr(),
                                                       q.data_ptr(), q_sf.data_ptr(), xg.data_ptr(), wg.data_ptr(), 1, 0, 0.0,
                                                       stream)
            assert rc == 0, rc
        b = nbytes(codes, sf, go, w, ptt, t2p, out, q, q_sf, xg, wg)

        def cpu():
            from oracle import torch_ref
            xq, goc, wc, pc, tc = (codes.cpu(), sf.cpu()), go.cpu(), w.cpu(), ptt.cpu(), t2p.cpu().view(T, K)
            return lambda: torch_ref.swiglu_backward_and_per_token_cast(xq, goc, wc, pc, tc, group, True, None)
        return launch, b, b, cpu
    return build


def op_per_channel(mode, transpose, num_per_tokens=128, rows=8192, hidden=4096):
    """mode: 'bf16' (plain), 'e4m3' (FP8 input with 1x128 scales), 'swiglu' (bf16 [rows, 2*hidden] in front)."""
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        M, K = rows, hidden
        x_sf = None
        if mode == 'swiglu':
            x = torch.randn((M, 2 * K), device='cuda', dtype=torch.bfloat16)
        else:
            x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
            if mode == 'e4m3':
                x, x_sf = tk.quant.per_token_cast(x, 'e4m3', num_per_channels=128)
        out = torch.empty((K, M) if transpose else (M, K), device='cuda', dtype=torch.float8_e4m3fn)
        out_sf = torch.empty((M // num_per_tokens, K), device='cuda', dtype=torch.float32)
        stream = _ffi.current_stream(out.device)

        def launch():
            rc = lib.tk_per_channel_cast(x.data_ptr(), 0, 0 if x_sf is None else x_sf.data_ptr(), M, K, 0, M, out.data_ptr(),
                                         out_sf.data_ptr(), num_per_tokens, 1, int(transpose), int(mode == 'swiglu'), 0, 0.0,
                                         stream)
            assert rc == 0, rc
        ts = [x, out, out_sf] + ([x_sf] if x_sf is not None else [])

        def cpu():
            from oracle import torch_ref
            xc = x.cpu()
            if mode == 'swiglu':
                return lambda: torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(xc, num_per_tokens, True, not transpose)
            xin = (xc, x_sf.cpu()) if mode == 'e4m3' else xc
            if transpose:
                return lambda: torch_ref.per_channel_cast_and_transpose(xin, num_per_tokens, True)
            return lambda: torch_ref.per_channel_cast_fused(xin, num_per_tokens, 128 if mode == 'e4m3' else None, True, None)
        return launch, nbytes(*ts), nbytes(*ts), cpu
    return build


def op_short_rows(direction):
    """Rows of 576 columns (the shortest row length of the reference's test list): per_token_cast 1x64 and its dequantisation."""
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        M, K, N = 65536, 576, 64
        x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
        codes = torch.empty((M, K), device='cuda', dtype=torch.float8_e4m3fn)
        sf = torch.empty((M, K // N), device='cuda', dtype=torch.float32)
        back = torch.empty((M, K), device='cuda', dtype=torch.bfloat16)
        stream = _ffi.current_stream(x.device)

        def cast():
            rc = lib.tk_per_token_cast(x.data_ptr(), _ffi.TK_BF16, M, K, K, codes.data_ptr(), sf.data_ptr(), K // N, _ffi.TK_E4M3, N,
                                       _ffi.TK_SF_ROW_F32, 0, _ffi.TK_CAST_AND_SF, stream)
            assert rc == 0, rc
        cast()

        def dequant():
            rc = lib.tk_cast_back(codes.data_ptr(), _ffi.TK_E4M3, M, K, sf.data_ptr(), K // N, _ffi.TK_SF_ROW_F32, 1, N, back.data_ptr(),
                                  _ffi.TK_BF16, stream)
            assert rc == 0, rc
        b = nbytes(x, codes, sf)

        def cpu():
            from oracle import torch_ref
            xc = x.cpu()
            if direction == 'cast':
                return lambda: torch_ref.cast(xc, 'e4m3', (1, N))
            q = (codes.cpu(), sf.cpu())
            return lambda: torch_ref.cast_back(q, 'bf16', (1, N))
        return (cast if direction == 'cast' else dequant), b, b, cpu
    return build


def op_cast_variant(kind, mode):
    """The scale-only and given-scale variants of the two casts at their benchmark shapes.
    kind: 'token' (bf16 [4096,7168], 1x128) or 'block' (bf16 [7168,2048], 128x128); mode: 'sf_only' or 'given_sf'."""
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        M, K = (4096, 7168) if kind == 'token' else (7168, 2048)
        x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
        if kind == 'token':
            sf = tk.quant.per_token_cast_with_sf_only(x, 'e4m3', 128)
        else:
            sf = tk.quant.per_block_cast_with_sf_only(x, 'e4m3', (128, 128))
        out = torch.empty((M, K), device='cuda', dtype=torch.float8_e4m3fn)
        stream = _ffi.current_stream(x.device)
        code = _ffi.TK_SF_ONLY if mode == 'sf_only' else _ffi.TK_CAST_GIVEN_SF
        op = 0 if mode == 'sf_only' else out.data_ptr()

        def launch():
            if kind == 'token':
                rc = lib.tk_per_token_cast(x.data_ptr(), _ffi.TK_BF16, M, K, K, op, sf.data_ptr(), sf.stride(0), _ffi.TK_E4M3, 128,
                                           _ffi.TK_SF_ROW_F32, 0, code, stream)
            else:
                rc = lib.tk_per_block_cast(x.data_ptr(), _ffi.TK_BF16, M, K, op, sf.data_ptr(), sf.stride(0), _ffi.TK_E4M3, 128, 128,
                                           _ffi.TK_SF_ROW_F32, 0, code, stream)
            assert rc == 0, rc
        ts = [x, sf] + ([out] if mode == 'given_sf' else [])

        def cpu():
            from oracle import torch_ref
            xc, sc = x.cpu(), sf.cpu()
            blk = (1, 128) if kind == 'token' else (128, 128)
            if mode == 'sf_only':
                return lambda: torch_ref.cast(xc, 'e4m3', blk)[1]      # the oracle has no scale-only mode
            return lambda: torch_ref.cast(xc, 'e4m3', blk, sf=sc)
        return launch, nbytes(*ts), nbytes(x, sf, out), cpu
    return build


def op_expand_to_fused_with_sf():
    import tilekernels_amd as tk
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, hidden = 4096, 8, 4096
    _, maps = _moe_maps(T, K)
    p2e, t2p = maps[0], maps[3]
    R = p2e.numel()
    x, x_sf = tk.quant.per_token_cast(torch.randn((T, hidden), device='cuda', dtype=torch.bfloat16), 'e4m3', 128)
    out = torch.empty((R, hidden), device='cuda', dtype=torch.float8_e4m3fn)
    out_sf = torch.empty((R, hidden // 128), device='cuda', dtype=torch.float32)
    stream = _ffi.current_stream(x.device)

    def launch():
        rc = lib.tk_expand_to_fused(x.data_ptr(), T, hidden, t2p.data_ptr(), K, p2e.data_ptr(), R, out.data_ptr(),
                                    x_sf.data_ptr(), hidden // 128, out_sf.data_ptr(), hidden // 128, 0, stream)
        assert rc == 0, rc
    ts = [x, x_sf, out, out_sf, t2p, p2e]

    def cpu():
        from oracle import torch_ref
        xq, tc, pc = (x.cpu(), x_sf.cpu()), t2p.cpu(), p2e.cpu()
        return lambda: torch_ref.expand_to_fused_with_sf(xq, 128, tc, pc)
    return launch, nbytes(*ts), nbytes(*ts), cpu


def op_swiglu_weighted():
    """The headline operator on the MoE-expanded batch with routing weights (bench.py's config 4 has the mask only)."""
    import tilekernels_amd as tk
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, H = 4096, 8, 2048
    _, maps = _moe_maps(T, K)
    p2e, ptt = maps[0], maps[2]
    R = p2e.numel()
    x = torch.randn((R, 2 * H), device='cuda', dtype=torch.bfloat16)
    w = torch.rand((T, K), device='cuda')
    out = torch.empty((R, H), device='cuda', dtype=torch.float8_e4m3fn)
    sf = torch.empty((R, H // 128), device='cuda', dtype=torch.float32)
    stream = _ffi.current_stream(x.device)

    def launch():
        rc = lib.tk_swiglu_per_token_cast(x.data_ptr(), _ffi.TK_BF16, R, H, out.data_ptr(), sf.data_ptr(), H // 128, 128,
                                          _ffi.TK_SF_ROW_F32, 0, -1.0, ptt.data_ptr(), w.data_ptr(), T * K, p2e.data_ptr(),
                                          0, 0.0, 0, 0, stream)
        assert rc == 0, rc
    live = int((p2e >= 0).sum())
    # padding rows are not read; their codes and scales are written
    algo = live * 2 * H * 2 + nbytes(out, sf, p2e, ptt, w)

    def cpu():
        from oracle import torch_ref
        xc, pc, tc, wc = x.cpu(), p2e.cpu(), ptt.cpu(), w.cpu()
        return lambda: torch_ref.swiglu_forward_and_per_token_cast(xc, 'e4m3', 128, pos_to_token_topk=tc, topk_weights=wc, pos_to_expert=pc)
    return launch, algo, nbytes(x, out, sf), cpu


def op_swiglu_dense(R, H, packed_col_major, count_clamp=False):
    """The headline operator on dense rows of other shapes and scale layouts: packed UE8M0 column-major scales (the layout a
    block-scaled GEMM consumes) at the headline shape, short rows (H = 768), rows of three 512-column pieces (H = 1536), and
    with a clamp at 6 whose hits are counted (clamped_count; N(0,1) data, so next to nothing is clamped)."""
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        from tilekernels_amd.quant.common import alloc_scaling_factors, get_cast_output_config, sf_leading_dim
        lib = _ffi.load()
        x = torch.randn((R, 2 * H), device='cuda', dtype=torch.bfloat16)
        out = torch.empty((R, H), device='cuda', dtype=torch.float8_e4m3fn)
        oc = get_cast_output_config('e4m3', (1, 128), packed_col_major, packed_col_major, packed_col_major)
        sf = alloc_scaling_factors((R, H), oc, x.device)
        stream = _ffi.current_stream(x.device)
        counts = torch.zeros(3, dtype=torch.int64, device='cuda')
        cap = 8 * torch.cuda.get_device_properties(x.device).multi_processor_count      # what the Python wrapper passes

        def launch():
            rc = lib.tk_swiglu_per_token_cast(x.data_ptr(), _ffi.TK_BF16, R, H, out.data_ptr(), sf.data_ptr(), sf_leading_dim(sf), 128,
                                              oc.layout_code, int(packed_col_major), -1.0, 0, 0, 0, 0, int(count_clamp), 6.0 if count_clamp else 0.0,
                                              counts.data_ptr() if count_clamp else 0, cap if count_clamp else 0, stream)
            assert rc == 0, rc
        b = nbytes(x, out) + R * (H // 128) * (1 if packed_col_major else 4)

        def cpu():
            from oracle import torch_ref
            xc = x.cpu()
            cc = torch.zeros(3, dtype=torch.int64) if count_clamp else None
            return lambda: torch_ref.swiglu_forward_and_per_token_cast(xc, 'e4m3', 128, use_tma_aligned_col_major_sf=packed_col_major,
                                                                       round_sf=packed_col_major, use_packed_ue8m0=packed_col_major,
                                                                       swiglu_clamp_value=6.0 if count_clamp else None, clamped_count=cc)
        return launch, b, b, cpu
    return build


def op_e5m6(direction):
    """per_token_cast(fmt='e5m6') of bf16 [8192, 4096] (one scale per row) and its dequantisation."""
    def build():
        import tilekernels_amd as tk
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        M, K = 8192, 4096
        x = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
        codes = torch.empty((M, K * 3 // 2), device='cuda', dtype=torch.uint8)
        sf = torch.empty((M, 1), device='cuda', dtype=torch.float32)
        back = torch.empty((M, K), device='cuda', dtype=torch.bfloat16)
        stream = _ffi.current_stream(x.device)

        def cast():
            rc = lib.tk_per_token_cast(x.data_ptr(), _ffi.TK_BF16, M, K, K, codes.data_ptr(), sf.data_ptr(), 1, _ffi.TK_E5M6, K,
                                       _ffi.TK_SF_ROW_F32, 1, _ffi.TK_CAST_AND_SF, stream)
            assert rc == 0, rc
        def uncast():
            rc = lib.tk_cast_back(codes.data_ptr(), _ffi.TK_E5M6, M, K, sf.data_ptr(), 1, _ffi.TK_SF_ROW_F32, 1, K, back.data_ptr(),
                                  _ffi.TK_BF16, stream)
            assert rc == 0, rc
        cast()
        ts = [x, codes, sf] if direction == 'cast' else [codes, sf, back]

        def cpu():
            from oracle import torch_ref
            if direction == 'cast':
                xc = x.cpu()
                return lambda: torch_ref.cast_to_e5m6(xc, K, round_sf=True)
            xq = (codes.cpu(), sf.cpu())
            return lambda: torch_ref.cast_back_from_e5m6(xq, 'bf16', (1, K))
        return (cast if direction == 'cast' else uncast), nbytes(*ts), nbytes(x, codes, sf, back), cpu
    return build


def op_lossless():
    """FP4 1x32 (packed UE8M0 scales) -> FP8 128x128, a [7168, 2048] weight as in the per-block benchmark shape."""
    import tilekernels_amd as tk
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    M, K = 7168, 2048
    w = torch.randn((M, K), device='cuda', dtype=torch.bfloat16)
    codes, sf = tk.quant.per_token_cast(w, 'e2m1', 32, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    store = sf.T.view(torch.uint8)
    out = torch.empty((M, K), device='cuda', dtype=torch.float8_e4m3fn)
    out_sf = torch.empty((M // 128, K // 128), device='cuda', dtype=torch.float32)
    stream = _ffi.current_stream(w.device)

    def launch():
        rc = lib.tk_per_block_cast_lossless(codes.data_ptr(), M, K, store.data_ptr(), store.stride(0), _ffi.TK_SF_COL_UE8M0, 1, 32,
                                            out.data_ptr(), out_sf.data_ptr(), K // 128, _ffi.TK_SF_ROW_F32, 128, 128, stream)
        assert rc == 0, rc
    algo = codes.numel() + M * (K // 32) + nbytes(out, out_sf)

    def cpu():
        from oracle import torch_ref
        xq = (codes.cpu(), sf.cpu())
        return lambda: torch_ref.per_block_cast_lossless(xq, 'e4m3', (1, 32), (128, 128), round_sf=True)
    return launch, algo, nbytes(codes, out) + store.numel(), cpu


def op_reduce_fused(fp8):
    """The inverse of expand_to_fused at its benchmark shape: bf16 [R, 4096] expanded rows -> [4096, 4096] tokens, top-8."""
    def build():
        from tilekernels_amd import _ffi
        lib = _ffi.load()
        T, K, hidden = 4096, 8, 4096
        _, maps = _moe_maps(T, K)
        p2e, t2p = maps[0], maps[3]
        R = p2e.numel()
        x = torch.randn((R, hidden), device='cuda', dtype=torch.bfloat16)
        w = torch.rand((T, K), device='cuda')
        sf = torch.ones((1,), device='cuda')
        out = torch.empty((T, hidden), device='cuda', dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16)
        stream = _ffi.current_stream(x.device)

        def launch():
            rc = lib.tk_reduce_fused(x.data_ptr(), _ffi.TK_BF16, R, hidden, 0, w.data_ptr(), t2p.data_ptr(), T, K, out.data_ptr(),
                                     _ffi.TK_OUT_E4M3 if fp8 else _ffi.TK_BF16, sf.data_ptr() if fp8 else 0, stream)
            assert rc == 0, rc
        # the T * K live rows are read, padding rows are not
        algo = T * K * hidden * 2 + nbytes(out, w, t2p)

        def cpu():
            from oracle import torch_ref
            xc, wc, tc, sc = x.cpu(), w.cpu(), t2p.cpu(), sf.cpu()
            return lambda: torch_ref.reduce_fused(xc, wc, tc, 'e4m3' if fp8 else '', sc if fp8 else None)
        return launch, algo, nbytes(x, out), cpu
    return build


OPS = [
    Op('reduce_fused', 'reduce_fused bf16 [R,4096] -> bf16 [4096,4096], top-8 of 256 experts, weighted', op_reduce_fused(False)),
    Op('reduce_fused_fp8', 'reduce_fused bf16 [R,4096] -> e4m3 [4096,4096] with output scale, top-8, weighted', op_reduce_fused(True)),
    Op('per_block_cast_lossless', 'per_block_cast_lossless e2m1 1x32 (packed scales) -> e4m3 128x128, [7168,2048]', op_lossless, floor=(7168 * 2048 // 2, 8, 16, 4)),
    Op('per_token_cast_e5m6', "per_token_cast fmt='e5m6' (12-bit, one scale per row) round_sf, bf16 [8192,4096]", op_e5m6('cast')),
    Op('cast_back_e5m6', 'cast_back of e5m6 -> bf16, [8192,4096]', op_e5m6('back')),
    Op('per_token_cast_k576', 'per_token_cast e4m3 1x64, short rows: bf16 [65536,576]', op_short_rows('cast')),
    Op('cast_back_k576', 'cast_back e4m3 1x64 -> bf16, short rows: [65536,576]', op_short_rows('back')),
    Op('per_token_cast_with_sf_only', 'per_token_cast_with_sf_only e4m3 1x128, bf16 [4096,7168]', op_cast_variant('token', 'sf_only'), floor=(4096 * 7168 * 2, 16, 0, 2)),
    Op('per_token_cast_with_precomputed_sf', 'per_token_cast_with_precomputed_sf e4m3 1x128, bf16 [4096,7168]',
       op_cast_variant('token', 'given_sf')),
    Op('per_block_cast_with_sf_only', 'per_block_cast_with_sf_only e4m3 128x128, bf16 [7168,2048]', op_cast_variant('block', 'sf_only'), floor=(7168 * 2048 * 2, 16, 0, 8)),
    Op('per_block_cast_with_precomputed_sf', 'per_block_cast_with_precomputed_sf e4m3 128x128, bf16 [7168,2048]',
       op_cast_variant('block', 'given_sf'), floor=(7168 * 2048 * 2, 16, 8, 8)),
    Op('swiglu_forward_and_per_token_cast_weighted',
       'swiglu_forward_and_per_token_cast e4m3 1x128, MoE-expanded bf16 [R,4096] with mask and routing weights', op_swiglu_weighted),
    Op('swiglu_forward_and_per_token_cast_packed_sf', 'swiglu_forward_and_per_token_cast e4m3 1x128, packed UE8M0 column-major scales, bf16 [8192,4096]',
       op_swiglu_dense(8192, 2048, True)),
    Op('swiglu_forward_and_per_token_cast_clamped_count', 'swiglu_forward_and_per_token_cast e4m3 1x128 with a clamp and clamped_count, bf16 [8192,4096]',
       op_swiglu_dense(8192, 2048, False, True)),
    Op('swiglu_forward_and_per_token_cast_h1536', 'swiglu_forward_and_per_token_cast e4m3 1x128, rows of three pieces: bf16 [10912,3072]',
       op_swiglu_dense(10912, 1536, False)),
    Op('swiglu_forward_and_per_token_cast_h768', 'swiglu_forward_and_per_token_cast e4m3 1x128, short rows: bf16 [32768,1536]',
       op_swiglu_dense(32768, 768, False), floor=(32768 * 1536 * 2, 16, 4, 4)),
    Op('expand_to_fused_with_sf', 'expand_to_fused_with_sf e4m3 [4096,4096] + 1x128 scales -> [R,4096], top-8 of 256 experts, pad 128',
       op_expand_to_fused_with_sf),
    Op('cast_back', 'cast_back e4m3 1x128 -> bf16, [8192,4096]', op_cast_back('bf16')),
    Op('cast_back_fp32', 'cast_back e4m3 1x128 -> fp32, [8192,4096]', op_cast_back('fp32')),
    Op('per_token_cast_quantized', 'per_token_cast of (e4m3 1x128) input -> e2m1 1x32, [8192,4096]', op_requant, floor=(8192 * 4096, 16, 8, 2)),
    Op('get_fused_mapping', 'get_fused_mapping 4096 tokens, top-8 of 256 experts, pad 128', op_get_fused_mapping),
    Op('expand_to_fused', 'expand_to_fused bf16 [4096,4096] -> [R,4096], top-8 of 256 experts, pad 128', op_expand_to_fused),
    Op('swiglu_backward_and_per_token_cast', 'swiglu_backward_and_per_token_cast 1x128 round_sf, x e4m3 [8192,4096]',
       op_swiglu_backward(128)),
    Op('swiglu_backward_and_per_token_cast_g32', 'swiglu_backward_and_per_token_cast 1x32 round_sf, x e4m3 [8192,4096]',
       op_swiglu_backward(32)),
    Op('per_channel_cast', 'per_channel_cast 128x1 round_sf, bf16 [8192,4096]', op_per_channel('bf16', False), floor=(8192 * 4096 * 2, 16, 8, 8)),
    Op('per_channel_cast_fused_fp8_input', 'per_channel_cast_fused 128x1 of (e4m3 1x128) input, [8192,4096]',
       op_per_channel('e4m3', False), floor=(8192 * 4096, 16, 16, 8)),
    Op('per_channel_cast_and_transpose', 'per_channel_cast_and_transpose 128x1 round_sf, bf16 [8192,4096] -> [4096,8192]',
       op_per_channel('bf16', True), floor=(8192 * 4096 * 2, 16, 8, 8)),
    Op('swiglu_forward_and_per_channel_cast_and_transpose',
       'swiglu_forward_and_per_channel_cast_and_transpose 128x1 round_sf, bf16 [8192,4096] -> [2048,8192]',
       op_per_channel('swiglu', True, hidden=2048), floor=(8192 * 4096 * 2, 16, 4, 8)),
    Op('swiglu_forward_and_per_channel_cast', 'same without transpose, bf16 [8192,4096] -> [8192,2048]',
       op_per_channel('swiglu', False, hidden=2048), floor=(8192 * 4096 * 2, 16, 4, 8)),
]


def time_floor(spec, steps: int, warmup: int) -> dict:
    """The traffic-only kernel on flat buffers of the operator's size, rotated past the last-level cache like the
    operator's own: what the same bytes cost on this machine in loads and stores of the same widths, with no arithmetic."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    in_bytes, ipl, opl, pieces = spec
    out_bytes = in_bytes // ipl * opl
    n = _sets_needed(in_bytes + out_bytes)
    ins = [torch.randint(0, 255, (in_bytes,), dtype=torch.uint8, device='cuda') for _ in range(n)]
    outs = [torch.empty((max(out_bytes, 16),), dtype=torch.uint8, device='cuda') for _ in range(n)]
    stream = _ffi.current_stream(ins[0].device)

    def launch(i):
        rc = lib.tk_stream_floor_flat(ins[i % n].data_ptr(), in_bytes, ipl, outs[i % n].data_ptr() if opl else 0, opl, pieces, stream)
        assert rc == 0, rc
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        launch(i)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / steps
    return {'us_per_call': round(us, 2), 'bytes': in_bytes + out_bytes, 'frac': round((in_bytes + out_bytes) / us / 1e3 / HBM_PEAK_GBS, 4),
            'what': f'tk_stream_floor_flat: {in_bytes} bytes read in {ipl}-byte loads, {out_bytes} written in {opl}-byte stores, {pieces} pieces per wave'}


def time_cpu(make) -> dict:
    """The CPU oracle (test infrastructure: a restatement of the reference's torch implementation) on the
    host cores for the same workload: one warm-up call, then two timed calls, the faster one reported."""
    import time
    threads = min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    fn = make()
    fn()
    best = float('inf')
    for _ in range(2):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return {'ms_per_call': round(best * 1e3, 2), 'cores': threads, 'kind': 'port'}


def run(op: Op, steps: int, warmup: int, with_cpu: bool) -> dict:
    sets = []
    launch, algo, footprint, make_cpu = op.build()
    sets.append(launch)
    for _ in range(_sets_needed(footprint) - 1):
        sets.append(op.build()[0])
    n = len(sets)
    for i in range(warmup):
        sets[i % n]()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        sets[i % n]()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / steps
    gbs = algo / us / 1e3
    rec = {'op': op.name, 'workload': op.workload, 'us_per_call': round(us, 2), 'bytes': algo, 'GB/s': round(gbs, 1),
           'frac': round(gbs / HBM_PEAK_GBS, 4), 'buffer_sets': n, 'steps': steps, 'warmup': warmup}
    if op.floor is not None:
        del sets
        torch.cuda.empty_cache()
        rec['traffic_only_kernel'] = time_floor(op.floor, steps, warmup)
        rec['over_traffic_only'] = round(us / rec['traffic_only_kernel']['us_per_call'], 3)
    if with_cpu:
        rec['cpu_baseline'] = time_cpu(make_cpu)
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--steps', type=int, default=2000)
    ap.add_argument('--warmup', type=int, default=1000)
    ap.add_argument('--only', type=str, default=None)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU-oracle timing of each operator')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run plain 256 MiB device copies (reference point for hardware-counter runs)')
    a = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit('bench_ops.py needs a GPU')
    torch.cuda.set_device(0)
    for op in OPS:
        if a.only and op.name not in a.only.split(','):
            continue
        print(json.dumps(run(op, a.steps, a.warmup, not a.no_cpu)), flush=True)
        torch.cuda.empty_cache()
    if a.copy_calibration:
        from bench import copy_calibration
        print(json.dumps(copy_calibration()), flush=True)


if __name__ == '__main__':
    main()
