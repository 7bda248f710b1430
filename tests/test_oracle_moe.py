"""Pins the oracle's MoE layout helpers (mapping and expansion) against naive loops and the
invariants the reference's own tests state (tests/moe/test_get_fused_mapping.py:54-78)."""
import pytest
import torch

from oracle import torch_ref


def naive_mapping(topk_idx, num_experts, alignment):
    T, K = topk_idx.shape
    per = [[] for _ in range(num_experts)]
    for t in range(T):
        for k in range(K):
            e = int(topk_idx[t, k])
            if e >= 0:
                per[e].append(t * K + k)
    p2e, p2t, p2tk = [], [], []
    t2p = [-1] * (T * K)
    starts, ends, padded = [], [], []
    for e in range(num_experts):
        starts.append(len(p2e))
        for i in per[e]:
            t2p[i] = len(p2e)
            p2e.append(e); p2t.append(i // K); p2tk.append(i)
        while len(p2e) % alignment:
            p2e.append(-1); p2t.append(-1); p2tk.append(-1)
        ends.append(len(p2e)); padded.append(ends[-1] - starts[-1])
    return p2e, p2t, p2tk, t2p, starts, ends, padded


@pytest.mark.parametrize('T,K,E,align', [(13, 3, 5, 4), (40, 2, 7, 16), (1, 1, 1, 8), (64, 8, 32, 128), (9, 4, 6, 1)])
def test_mapping_matches_naive_loop_and_invariants(T, K, E, align):
    topk_idx = torch.stack([torch.randperm(E)[:K] if K <= E else torch.randint(0, E, (K,)) for _ in range(T)]).long()
    topk_idx[torch.rand(topk_idx.shape) < 0.15] = -1
    got = torch_ref.get_fused_mapping(topk_idx, E, align)
    want = naive_mapping(topk_idx, E, align)
    for g, w in zip(got, want):
        assert g.dtype == torch.int32 and g.reshape(-1).tolist() == list(w)
    p2e, p2t, p2tk, t2p, starts, ends, padded = got
    # invariants of the reference's test
    live = p2e >= 0
    assert torch.equal(live, p2t >= 0) and torch.equal(live, p2tk >= 0)
    tk = p2tk[live].long()
    assert torch.equal(t2p.reshape(-1)[tk].long(), torch.nonzero(live).flatten())
    assert torch.equal(topk_idx.reshape(-1)[tk], p2e[live].long())
    assert torch.equal(tk // K, p2t[live].long())
    assert int(padded.sum()) == p2e.numel() and torch.all(padded % align == 0)
    for e in range(E):
        seg = p2e[starts[e]:ends[e]]
        assert int((seg == e).sum()) == int((topk_idx == e).sum()) and torch.all((seg == e) | (seg == -1))


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float8_e4m3fn, torch.int8])
def test_expand_matches_naive_loop(dtype):
    T, K, E, H = 11, 3, 4, 64
    topk_idx = torch.stack([torch.randperm(E)[:K] for _ in range(T)]).long()
    topk_idx[2, 1] = -1
    p2e, _, p2tk, t2p, *_ = torch_ref.get_fused_mapping(topk_idx, E, 8)
    x = torch.randn((T, H)).to(dtype) if dtype != torch.int8 else torch.randint(-128, 127, (T, H), dtype=torch.int8)
    out = torch_ref.expand_to_fused(x, t2p, p2e)
    assert out.shape == (p2e.numel(), H) and out.dtype == dtype
    xb, ob = x.view(torch.uint8), out.view(torch.uint8)
    for pos in range(p2e.numel()):
        if p2e[pos] >= 0:
            assert torch.equal(ob[pos], xb[int(p2tk[pos]) // K])
        else:
            assert torch.all(ob[pos] == 0)


@pytest.mark.parametrize('col_major,packed', [(False, False), (True, False), (True, True)])
def test_expand_with_sf_layouts(col_major, packed):
    T, K, E, H = 9, 2, 3, 512
    topk_idx = torch.stack([torch.randperm(E)[:K] for _ in range(T)]).long()
    p2e, _, p2tk, t2p, *_ = torch_ref.get_fused_mapping(topk_idx, E, 16)
    x = torch.randn((T, H)).to(torch.bfloat16)
    codes, sf = torch_ref.cast(x, 'e4m3', (1, 128), round_sf=True, use_tma_aligned_col_major_sf=col_major, use_packed_ue8m0=packed)
    sf = torch.empty(sf.shape, dtype=sf.dtype).copy_(sf)         # the caller hands over contiguous rows
    out, out_sf = torch_ref.expand_to_fused_with_sf((codes, sf), 128, t2p, p2e, col_major)
    R = p2e.numel()
    assert out_sf.shape == (R, sf.shape[1]) and out_sf.dtype == sf.dtype
    assert out_sf.stride() == ((1, (R + 3) // 4 * 4) if col_major else (sf.shape[1], 1))
    for pos in range(R):
        if p2e[pos] >= 0:
            t = int(p2tk[pos]) // K
            assert torch.equal(out_sf[pos], sf[t]) and torch.equal(out.view(torch.uint8)[pos], codes.view(torch.uint8)[t])
        else:
            assert torch.all(out_sf[pos] == 0)
