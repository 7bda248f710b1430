"""The library under HIP graph capture: the C-ABI entry points allocate nothing and record no memset
nodes, so a chain of them can be captured once and replayed.  The chain of an MoE layer's quantisation
front end (mapping with a fixed-size buffer -> expansion -> fused SwiGLU cast -> per-token cast ->
SwiGLU backward) is captured, then replayed several times with new input contents and ordinary eager
work and synchronisations in between; every replay must equal the eager result bit for bit (the same
kernels run on the same data, so this is an equality, not a tolerance)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _chain(tk, topk_idx, x, go, w, E, R, alignment):
    p2e, p2t, ptt, t2p, es, ee, npe, _ = tk.moe.get_fused_mapping(topk_idx, E, R, alignment)
    xe = tk.moe.expand_to_fused(x, t2p, p2e)
    act, act_sf = tk.quant.swiglu_forward_and_per_token_cast(xe, 'e4m3', 128, pos_to_token_topk=ptt, topk_weights=w,
                                                             pos_to_expert=p2e, round_sf=True)
    xq = tk.quant.per_token_cast(xe, 'e4m3', 128, round_sf=True)
    out, (gq, gq_sf), xg, wg = tk.quant.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, 128, round_sf=True,
                                                                           swiglu_clamp_value=10.0)
    pc, pc_sf = tk.quant.per_channel_cast_fused(xe, 'e4m3', 128, round_sf=True)
    return [p2e, ptt, t2p, xe, act, act_sf, xq[0], xq[1], out, gq, gq_sf, xg, wg, pc, pc_sf]


def _new_inputs(seed, T, K, E, H):
    g = torch.Generator().manual_seed(seed)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < 0.15, -1).contiguous()
    x = torch.randn((T, 2 * H), generator=g).to(torch.bfloat16)
    w = torch.rand((T, K), generator=g)
    return topk_idx, x, w


def test_moe_chain_replays_from_a_graph():
    import tilekernels_amd as tk
    T, K, E, H, alignment = 512, 4, 16, 512, 128
    R = (T * K + (alignment - 1) * E) // alignment * alignment      # worst case, fixed: no host sync in the chain
    topk_idx = torch.empty((T, K), dtype=torch.int64, device='cuda')
    x = torch.empty((T, 2 * H), dtype=torch.bfloat16, device='cuda')
    w = torch.empty((T, K), dtype=torch.float32, device='cuda')
    go = torch.randn((R, H), dtype=torch.bfloat16, device='cuda')

    def load(seed):
        a, b, c = _new_inputs(seed, T, K, E, H)
        topk_idx.copy_(a); x.copy_(b); w.copy_(c)

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _chain(tk, topk_idx, x, go, w, E, R, alignment)               # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _chain(tk, topk_idx, x, go, w, E, R, alignment)

    for seed in (1, 2, 3, 4):
        load(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        # ordinary eager work between replays, then the eager chain on the same inputs
        _ = (x.float() * 2).sum().item()
        want = _chain(tk, topk_idx, x, go, w, E, R, alignment)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert a.dtype == b.dtype and a.shape == b.shape
            ab, bb = a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8)
            assert torch.equal(ab, bb), f'seed {seed}: output {i} differs between graph replay and eager run'


@pytest.mark.parametrize('layout', ['row', 'packed'])
def test_swiglu_launch_that_ends_in_smaller_waves_replays_from_a_graph(layout):
    """The launch shape of dense batches of about one to three times the GPU's wave slots (its smaller waves read part of
    their arguments from the argument segment behind their loads) under capture: replays on new contents equal eager runs."""
    import tilekernels_amd as tk
    R, H = 8192, 2048
    kw = dict(round_sf=True, use_tma_aligned_col_major_sf=layout == 'packed', use_packed_ue8m0=layout == 'packed')
    x = torch.empty((R, 2 * H), dtype=torch.bfloat16, device='cuda')
    ptt = torch.arange(R, dtype=torch.int32, device='cuda')
    w = torch.empty((R // 8, 8), dtype=torch.float32, device='cuda')

    def run():
        a = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, **kw)
        b = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_token_topk=ptt, topk_weights=w, swiglu_clamp_value=2.0, **kw)
        return [a[0], a[1], b[0], b[1]]

    def load(seed):
        g = torch.Generator().manual_seed(seed)
        x.copy_(torch.randn((R, 2 * H), generator=g).to(torch.bfloat16))
        w.copy_(torch.rand((R // 8, 8), generator=g) + 0.5)

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for seed in (1, 2, 3):
        load(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        _ = (x.float() * 2).sum().item()
        want = run()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8)), f'seed {seed}: output {i}'
