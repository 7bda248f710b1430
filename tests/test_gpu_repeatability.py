"""Every operator, run 25 times on the same input, must return the same bytes each time: a missing
barrier around an LDS stage, an unordered atomic accumulation or a read of uninitialised memory would
show up here as a run that differs.  Shapes are chosen to exercise partial tiles and every scale layout."""
import pytest
import torch

pytestmark = pytest.mark.gpu

RUNS = 25


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _flat(result):
    """All tensors of a (nested) result, as byte tensors on the GPU."""
    if isinstance(result, torch.Tensor):
        t = result.contiguous() if result.numel() else result
        return [t.view(torch.uint8).flatten().clone()] if t.numel() else []
    out = []
    for r in result:
        if isinstance(r, (torch.Tensor, tuple, list)):
            out += _flat(r)
    return out


def _repeat(fn):
    first = _flat(fn())
    for i in range(1, RUNS):
        again = _flat(fn())
        assert len(again) == len(first)
        for j, (a, b) in enumerate(zip(first, again)):
            assert torch.equal(a, b), f'run {i}: output {j} differs in {(a != b).sum().item()} bytes'


def _x(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator(device='cuda').manual_seed(seed)
    return torch.randn(shape, generator=g, device='cuda', dtype=torch.float32).to(dtype)


@pytest.mark.parametrize('mode', [(False, False, False), (True, True, False), (True, True, True)],
                         ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('fmt,N', [('e4m3', 128), ('e2m1', 32)])
def test_per_token_cast_repeats(fmt, N, mode):
    tk = _tk()
    col, rnd, packed = mode
    x = _x((1003, 3200), 1)
    _repeat(lambda: tk.quant.per_token_cast(x, fmt, N, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed))


def test_per_block_cast_repeats():
    tk = _tk()
    x = _x((1000, 2112), 2)
    _repeat(lambda: tk.quant.per_block_cast(x, 'e4m3', (128, 128)))
    _repeat(lambda: tk.quant.per_block_cast(x, 'e2m1', (32, 32), use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True))


@pytest.mark.parametrize('col', [False, True])
def test_swiglu_forward_repeats(col):
    tk = _tk()
    g = torch.Generator().manual_seed(3)
    pe, ptt, w = tk.testing.generate_moe_layout(301, 16, 8, 16, g, drop_fraction=0.1)
    x = _x((pe.numel(), 2 * 1536), 4)
    pe, ptt, w = pe.cuda(), ptt.cuda(), w.cuda()
    cnt = torch.zeros(3, dtype=torch.int64, device='cuda')

    def run():
        cnt.zero_()
        out = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_token_topk=ptt, topk_weights=w, pos_to_expert=pe,
                                                         use_tma_aligned_col_major_sf=col, round_sf=col,
                                                         swiglu_clamp_value=1.5, clamped_count=cnt)
        return out[0], out[1], cnt
    _repeat(run)


def test_swiglu_backward_repeats():
    tk = _tk()
    T, K, E, H = 257, 4, 8, 1536
    g = torch.Generator().manual_seed(5)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices.contiguous()
    _, _, ptt, t2p, *_ = tk.moe.get_fused_mapping(topk_idx.cuda(), E, 0, 16)
    R = ptt.numel()
    xq = tk.quant.per_token_cast(_x((R, 2 * H), 6), 'e4m3', 128)
    go, w = _x((R, H), 7), torch.rand((T, K), device='cuda')
    # weight_grad is a sum over the row: its order of accumulation must be fixed too
    _repeat(lambda: tk.quant.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, 128, swiglu_clamp_value=2.0))


def test_per_channel_family_repeats():
    tk = _tk()
    x = _x((1024, 1280), 8)
    _repeat(lambda: tk.quant.per_channel_cast(x, 'e4m3', 128))
    _repeat(lambda: tk.quant.per_channel_cast_and_transpose(x, 'e4m3', 32, round_sf=True))
    _repeat(lambda: tk.quant.swiglu_forward_and_per_channel_cast_and_transpose(x, 'e4m3', 128))
    xq = tk.quant.per_token_cast(x, 'e4m3', 128)
    pos = torch.randint(-1, 1024, (512,), dtype=torch.int32, device='cuda')
    _repeat(lambda: tk.quant.per_channel_cast_fused(xq, 'e4m3', 128, num_per_channels=128, pos_to_token=pos))


def test_moe_layout_repeats():
    tk = _tk()
    T, K, E = 2001, 8, 64
    g = torch.Generator().manual_seed(9)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < 0.1, -1).contiguous().cuda()
    _repeat(lambda: tk.moe.get_fused_mapping(topk_idx, E, 0, 64)[:7])
    p2e, _, _, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, E, 0, 64)
    x = _x((T, 2304), 10)
    _repeat(lambda: tk.moe.expand_to_fused(x, t2p, p2e))
    xq = tk.quant.per_token_cast(x, 'e4m3', 128)
    _repeat(lambda: tk.moe.expand_to_fused_with_sf(xq, 128, t2p, p2e, use_tma_aligned_col_major_sf=True))
