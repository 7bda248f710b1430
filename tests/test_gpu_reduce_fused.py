"""GPU parity of reduce_fused against the CPU oracle, bit for bit (the reference compares its kernel and its torch
statement the same way, tests/moe/test_reduce_fused.py:66-81): every term is one fused multiply-add in fp32, added in
the order of k."""
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _case(T, K, E, hidden, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < 0.1, -1).contiguous()
    _, _, _, t2p, *_ = torch_ref.get_fused_mapping(topk_idx, E, 16)
    R = int(t2p.max()) + 17 if T else 16
    x = torch.randn((R, hidden), generator=g).to(dtype)
    w = torch.rand((T, K), generator=g)
    x_sf = torch.randn((R,), generator=g)
    return x, t2p, w, x_sf


@pytest.mark.parametrize('with_x_sf', [False, True])
@pytest.mark.parametrize('with_weights', [False, True])
@pytest.mark.parametrize('fp8', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16], ids=['f32', 'bf16'])
@pytest.mark.parametrize('T,K,E,hidden', [(301, 8, 32, 2048), (97, 6, 16, 7168), (64, 2, 9, 256), (33, 9, 16, 2304), (1, 1, 3, 512), (0, 4, 8, 256)])
def test_reduce_fused(T, K, E, hidden, dtype, fp8, with_weights, with_x_sf):
    tk = _tk()
    x, t2p, w, x_sf = _case(T, K, E, hidden, dtype, seed=hidden + T + K)
    sf = torch.randn((1,), generator=torch.Generator().manual_seed(T)) if fp8 else None
    xin = (x, x_sf) if with_x_sf else x
    want = torch_ref.reduce_fused(xin, w if with_weights else None, t2p, 'e4m3' if fp8 else '', sf)
    xg = (x.cuda(), x_sf.cuda()) if with_x_sf else x.cuda()
    got = tk.moe.reduce_fused(xg, w.cuda() if with_weights else None, t2p.cuda(), 'e4m3' if fp8 else '', None if sf is None else sf.cuda())
    assert_same(got, want, 'reduced')


def test_reduce_fused_into_a_given_buffer_and_without_scale():
    tk = _tk()
    x, t2p, w, _ = _case(130, 4, 8, 1024, torch.bfloat16, seed=5)
    out = torch.full((130, 1024), 7.0, dtype=torch.float8_e4m3fn, device='cuda')
    got = tk.moe.reduce_fused(x.cuda(), w.cuda(), t2p.cuda(), 'e4m3', None, out)
    assert got.data_ptr() == out.data_ptr()
    assert_same(got, torch_ref.reduce_fused(x, w, t2p, 'e4m3'), 'reduced')


def test_expand_then_reduce_is_the_weighted_identity():
    """expand_to_fused followed by reduce_fused with weights summing to one over the kept copies gives the input back."""
    tk = _tk()
    T, K, E, hidden = 257, 4, 16, 1024
    g = torch.Generator().manual_seed(9)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices.contiguous().cuda()
    p2e, _, _, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, E, 0, 64)
    x = torch.randn((T, hidden), generator=g).cuda()
    w = torch.full((T, K), 0.25, device='cuda')
    back = tk.moe.reduce_fused(tk.moe.expand_to_fused(x, t2p, p2e), w, t2p)
    assert torch.equal(back, x)          # four exact quarters of the same value


def test_reduce_fused_without_any_live_position():
    """Every (token, k) pair dropped: the expanded tensor has no rows; the result is zeros, as the oracle's."""
    tk = _tk()
    t2p = torch.full((5, 3), -1, dtype=torch.int32)
    for dtype in (torch.bfloat16, torch.float32):
        x = torch.empty((0, 512), dtype=dtype)
        for fp8 in ('', 'e4m3'):
            got = tk.moe.reduce_fused(x.cuda(), torch.rand((5, 3)).cuda(), t2p.cuda(), fp8_format=fp8)
            want = torch_ref.reduce_fused(x, torch.rand((5, 3)), t2p, fp8_format=fp8)
            assert_same(got, want, f'{dtype} {fp8}')


def test_reduce_fused_e4m3_output_beyond_the_format_range():
    """Scaled sums beyond +-448 are not saturated: they become NaN codes, as in the oracle (torch's conversion)."""
    tk = _tk()
    x = torch.tensor([[300.0, -300.0, 100.0, 447.0, 465.0, -480.0, 1.0, 0.0]] * 2, dtype=torch.float32).repeat(1, 32)
    t2p = torch.tensor([[0, 1]], dtype=torch.int32)
    w = torch.ones((1, 2))
    want = torch_ref.reduce_fused(x, w, t2p, 'e4m3')
    got = tk.moe.reduce_fused(x.cuda(), w.cuda(), t2p.cuda(), 'e4m3')
    assert_same(got, want, 'codes')
    codes = want.view(torch.uint8)[0, :8].tolist()
    assert codes[0] == 0x7F and codes[1] == 0xFF and codes[3] == 0x7F and codes[2] != 0x7F      # 600, -600, 894 -> NaN; 200 is finite
