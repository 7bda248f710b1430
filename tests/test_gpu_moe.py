"""GPU parity of the MoE layout helpers (mapping, expansion) against the CPU oracle, bit for bit,
and the end-to-end chain mapping -> expansion -> fused SwiGLU cast.  Structure follows the
reference's tests/moe/test_get_fused_mapping.py and tests/moe/test_expand_to_fused.py."""
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same
from tests.test_gpu_swiglu import check_fused

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _topk_idx(T, K, E, drop=0.1, seed=0):
    g = torch.Generator().manual_seed(seed)
    scores = torch.rand((T, E), generator=g)
    idx = torch.topk(scores, K, dim=-1).indices
    if drop:
        idx = idx.masked_fill(torch.rand(idx.shape, generator=g) < drop, -1)
    return idx.contiguous()


@pytest.mark.parametrize('alignment', [16, 64, 128])
@pytest.mark.parametrize('T,K,E', [(4001, 8, 256), (4001, 6, 72), (4001, 2, 9), (513, 9, 32), (7, 1, 1), (1, 2, 384), (64, 8, 1024),
                                   (20001, 8, 256), (33000, 4, 9), (16384, 8, 64), (4001, 8, 768)])
def test_get_fused_mapping(T, K, E, alignment):
    tk = _tk()
    topk_idx = _topk_idx(T, K, E, seed=T + K)
    want = torch_ref.get_fused_mapping(topk_idx, E, alignment)
    got = tk.moe.get_fused_mapping(topk_idx.cuda(), E, 0, alignment)
    names = ['pos_to_expert', 'pos_to_token', 'pos_to_token_topk', 'token_topk_to_pos', 'expert_start', 'expert_end', 'num_tokens_per_expert']
    for n, g, w in zip(names, got[:7], want):
        assert_same(g, w, n)
    assert got[7] == want[6].tolist()
    # fixed-size buffer, no host sync: same content, untouched tail marked as padding
    R = want[0].numel() + 3 * alignment
    got2 = tk.moe.get_fused_mapping(topk_idx.cuda(), E, R, alignment)
    assert got2[7] == [] and got2[0].numel() == R
    assert torch.equal(got2[0].cpu()[: want[0].numel()], want[0]) and torch.all(got2[0].cpu()[want[0].numel():] == -1)
    assert_same(got2[3], want[3], 'token_topk_to_pos')


def test_get_fused_mapping_no_tokens():
    tk = _tk()
    got = tk.moe.get_fused_mapping(torch.empty((0, 4), dtype=torch.int64, device='cuda'), 8, 0, 16)
    assert got[0].numel() == 0 and got[7] == [0] * 8 and torch.all(got[4].cpu() == 0)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float8_e4m3fn])
@pytest.mark.parametrize('hidden', [128, 576, 2048, 7168])
@pytest.mark.parametrize('T,K,E', [(1001, 8, 64), (257, 2, 9), (3, 1, 4), (9, 3, 5)])
def test_expand_to_fused(T, K, E, hidden, dtype):
    tk = _tk()
    topk_idx = _topk_idx(T, K, E, seed=hidden)
    p2e, _, _, t2p, *_ = torch_ref.get_fused_mapping(topk_idx, E, 16)
    x = torch.randn((T, hidden)).to(dtype)
    want = torch_ref.expand_to_fused(x, t2p, p2e)
    got = tk.moe.expand_to_fused(x.cuda(), t2p.cuda(), p2e.cuda())
    assert_same(got, want, 'expanded')


@pytest.mark.parametrize('mode', [(False, True, False), (True, True, True), (True, False, False), (False, False, False)],
                         ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('num_per_channels', [32, 128])
@pytest.mark.parametrize('hidden', [576, 4096])
def test_expand_to_fused_with_sf(hidden, num_per_channels, mode):
    tk = _tk()
    col, rnd, packed = mode
    T, K, E = 777, 6, 72
    topk_idx = _topk_idx(T, K, E, seed=hidden + num_per_channels)
    p2e, _, _, t2p, *_ = torch_ref.get_fused_mapping(topk_idx, E, 16)
    x = torch.randn((T, hidden)).to(torch.bfloat16)
    codes, sf = torch_ref.cast(x, 'e4m3', (1, num_per_channels), round_sf=rnd, use_tma_aligned_col_major_sf=col, use_packed_ue8m0=packed)
    sf = torch.empty(sf.shape, dtype=sf.dtype).copy_(sf)
    want = torch_ref.expand_to_fused_with_sf((codes, sf), num_per_channels, t2p, p2e, col)
    got = tk.moe.expand_to_fused_with_sf((codes.cuda(), sf.cuda()), num_per_channels, t2p.cuda(), p2e.cuda(), col)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'sf')


def test_moe_chain_mapping_expand_swiglu_cast():
    """The three steps as an MoE layer runs them, all on the GPU, against the same chain on the CPU."""
    tk = _tk()
    T, K, E, H = 1024, 8, 64, 1024
    g = torch.Generator().manual_seed(3)
    logits = torch.randn((T, E), generator=g)
    w, idx = torch.topk(torch.softmax(logits, -1), K, dim=-1)
    x = torch.randn((T, 2 * H), generator=g).to(torch.bfloat16)
    p2e, _, p2tk, t2p, *_ = torch_ref.get_fused_mapping(idx, E, 128)
    want = torch_ref.swiglu_forward_and_per_token_cast(torch_ref.expand_to_fused(x, t2p, p2e), 'e4m3', 128, p2tk, w.contiguous(), p2e)
    m = tk.moe.get_fused_mapping(idx.cuda().contiguous(), E, 0, 128)
    xe = tk.moe.expand_to_fused(x.cuda(), m[3], m[0])
    got = tk.quant.swiglu_forward_and_per_token_cast(xe, 'e4m3', 128, m[2], w.cuda().contiguous(), m[0])
    check_fused(got, want, H // 128, False, 'chain')
