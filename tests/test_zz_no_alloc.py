"""tk_get_fused_mapping_static (the entry point that allocates nothing: its slice x expert table is a device
array owned by the library) against tk_get_fused_mapping with a caller-provided workspace, bit for bit,
through the C ABI.  Calls follow each other on one GPU with inputs of different sizes, so a later call
finds the table as the earlier one left it."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

NAMES = ['pos_to_expert', 'pos_to_token', 'pos_to_token_topk', 'token_topk_to_pos', 'expert_start', 'expert_end',
         'num_tokens_per_expert']


def _topk_idx(T, K, E, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    return idx.masked_fill(torch.rand(idx.shape, generator=g) < 0.1, -1).contiguous()


def _buffers(T, K, E, R, poison):
    i32 = dict(dtype=torch.int32, device='cuda')
    return [torch.full((R,), poison, **i32), torch.full((R,), poison, **i32), torch.full((R,), poison, **i32),
            torch.full((T * K,), poison, **i32), torch.full((E,), poison, **i32), torch.full((E,), poison, **i32),
            torch.full((E,), poison, **i32)]


def _run_both(lib, T, K, E, alignment, seed):
    idx = _topk_idx(T, K, E, seed).cuda()
    R = (T * K + (alignment - 1) * E) // alignment * alignment
    stream = torch.cuda.current_stream().cuda_stream
    ws_bytes = lib.tk_fused_mapping_workspace_bytes(T, K, E)
    ws = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.int32, device='cuda')
    want = _buffers(T, K, E, R, -7)
    rc = lib.tk_get_fused_mapping(idx.data_ptr(), T, K, E, alignment, R, *[b.data_ptr() for b in want], ws.data_ptr(),
                                  ws.numel() * 4, stream)
    assert rc == 0, lib.tk_strerror(rc)
    got = _buffers(T, K, E, R, -9)
    torch.cuda.synchronize()
    # free device memory as the driver reports it (torch's own counters would only see torch's allocator)
    before, before_torch = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    rc = lib.tk_get_fused_mapping_static(idx.data_ptr(), T, K, E, alignment, R, *[b.data_ptr() for b in got], stream)
    assert rc == 0, lib.tk_strerror(rc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_allocated() == before_torch
    for name, g, w in zip(NAMES, got, want):
        assert torch.equal(g.cpu(), w.cpu()), (name, T, K, E, alignment)
    # the mapping is a bijection between the routed (token, k) pairs and the live positions
    t2p = got[3].cpu()
    live = t2p[t2p >= 0].long()
    assert live.numel() == int((idx >= 0).sum()) and live.unique().numel() == live.numel()
    assert torch.equal(got[2].cpu()[live], torch.nonzero(t2p >= 0).flatten().int())


def test_static_scratch_mapping_matches_workspace_mapping_on_consecutive_calls():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    # large first, then smaller inputs: the table keeps the earlier call's contents.  Lists of 64 Ki pairs or more, and
    # more than 512 experts, take the three launches that go through the table; the others take the single launch
    _run_both(lib, 32768, 8, 256, 128, seed=1)     # 1024 slices x 256 experts = 1 MiB of the 4 MiB table
    _run_both(lib, 20001, 8, 256, 64, seed=2)      # table
    _run_both(lib, 9000, 8, 64, 16, seed=7)        # table: 72000 pairs, fewer experts than the calls before
    _run_both(lib, 4001, 6, 72, 16, seed=3)        # single launch
    _run_both(lib, 7, 1, 1, 16, seed=4)
    _run_both(lib, 16384, 8, 1024, 128, seed=5)    # table: 512 slices x 1024 experts = 2 MiB
    _run_both(lib, 1024, 8, 600, 16, seed=8)       # table (more than 512 experts) although the list is short
    _run_both(lib, 8192, 8, 16, 32, seed=9)        # table: exactly 64 Ki pairs
    _run_both(lib, 513, 9, 32, 16, seed=6)


def test_static_scratch_mapping_rejects_what_does_not_fit():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, E = 262145, 4, 1024      # 4097 slices x 1024 experts x 4 bytes > 4 MiB
    assert lib.tk_fused_mapping_workspace_bytes(T, K, E) > (4 << 20)
    dummy = torch.zeros((8,), dtype=torch.int64, device='cuda')
    p = dummy.data_ptr()
    rc = lib.tk_get_fused_mapping_static(p, T, K, E, 16, 16, p, p, p, p, p, p, p, torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b'large' in lib.tk_strerror(rc).lower()
    # no tokens at all: the start/end tables are still written
    out = _buffers(0, 4, 8, 32, -9)
    rc = lib.tk_get_fused_mapping_static(0, 0, 4, 8, 16, 32, *[b.data_ptr() for b in out], torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.all(out[0].cpu() == -1) and torch.all(out[4].cpu() == 0) and torch.all(out[5].cpu() == 0)
