"""GPU parity of the fused SwiGLU backward + per-token FP8 cast against the CPU oracle.

Tolerance (floating point: exp and the two divisions round differently on CPU and GPU, everything
after them is the same sequence of single roundings):
  * bf16 outputs (out, x_grad): at most 0.01 % of the values differ, each by one bf16 step
  * FP8 codes of the gradient: at most 0.01 % differ, each by one E4M3 step
  * scales: within 1e-6 relative (round_sf: identical up to 0.01 % that moved one power of two)
  * weight_grad: atol = rtol = 1e-4, the reference's own tolerance for it
The reference's test (tests/quant/test_swiglu_backward_and_per_token_cast.py:57-103) is the model:
mapping -> expansion -> per-token cast build the input, the oracle composition is the expectation.
"""
import pytest
import torch

from oracle import torch_ref
from tests._util import dense_bytes, fp8_code_report, mismatch_within

pytestmark = pytest.mark.gpu

BF16_MISMATCH_MAX = 1e-4
CODE_MISMATCH_MAX = 1e-4
SCALE_RTOL = 1e-6


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def make_inputs(T, K, E, H, N, seed, scale=1.0, drop=0.1, alignment=16):
    """CPU tensors: quantised expanded input, grad_out, weights and the two index maps."""
    g = torch.Generator().manual_seed(seed)
    scores = torch.rand((T, E), generator=g)
    topk_idx = torch.topk(scores, K, dim=-1).indices
    if drop:
        topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < drop, -1)
    p2e, _, ptt, t2p, *_ = torch_ref.get_fused_mapping(topk_idx.contiguous(), E, alignment)
    x = (torch.randn((T, 2 * H), generator=g) * scale).to(torch.bfloat16)
    xe = torch_ref.expand_to_fused(x, t2p, p2e)
    xq = torch_ref.cast(xe, 'e4m3', (1, N))
    R = xe.shape[0]
    go = torch.randn((R, H), generator=g).to(torch.bfloat16)
    w = torch.rand((T, K), generator=g)
    return xq, go, w, ptt, t2p


def bf16_report(got: torch.Tensor, want: torch.Tensor):
    """(fraction of differing values, all differences are one bf16 step or a signed-zero pair)."""
    g = got.cpu().contiguous().view(torch.int16).flatten().to(torch.int32)
    w = want.contiguous().view(torch.int16).flatten().to(torch.int32)
    diff = g != w
    n = int(diff.sum())
    if n == 0:
        return 0.0, True
    gd, wd = g[diff], w[diff]
    one = ((gd & 0x8000) == (wd & 0x8000)) & (((gd & 0x7FFF) - (wd & 0x7FFF)).abs() == 1)
    zeros = ((gd & 0x7FFF) == 0) & ((wd & 0x7FFF) == 0)
    return n / g.numel(), bool((one | zeros).all())


def check_backward(got, want, round_sf, what=''):
    out, (codes, sf), xg, wg = got
    out_ref, (codes_ref, sf_ref), xg_ref, wg_ref = want
    for a, b, name in ((out, out_ref, 'out'), (xg, xg_ref, 'x_grad')):
        assert a.dtype == b.dtype == torch.bfloat16 and tuple(a.shape) == tuple(b.shape), name
        frac, one = bf16_report(a, b)
        assert mismatch_within(frac, a.numel(), BF16_MISMATCH_MAX) and one, f'{what} {name}: {frac * 100:.5f}% differ, one-step={one}'
    assert codes.dtype == torch.float8_e4m3fn and tuple(codes.shape) == tuple(codes_ref.shape)
    assert sf.dtype == torch.float32 and tuple(sf.shape) == tuple(sf_ref.shape) and sf.is_contiguous()
    a, b = sf.cpu(), sf_ref
    if round_sf:
        moved = a != b
        assert moved.float().mean().item() <= 1e-4, f'{what}: {int(moved.sum())} rounded scales differ'
        ratio = a[moved] / b[moved]
        assert bool(((ratio == 2) | (ratio == 0.5)).all())
        keep = ~moved.repeat_interleave(codes.shape[1] // sf.shape[1], dim=1).flatten()
    else:
        rel = ((a - b).abs() / b.abs().clamp(min=1e-30)).max().item() if a.numel() else 0.0
        assert rel <= SCALE_RTOL, f'{what}: scale rel err {rel}'
        keep = None
    gc, wc = dense_bytes(codes.cpu()), dense_bytes(codes_ref)
    if keep is not None:
        gc, wc = gc[keep], wc[keep]
    frac, one = fp8_code_report(gc, wc)
    assert mismatch_within(frac, gc.numel(), CODE_MISMATCH_MAX) and one, f'{what}: {frac * 100:.5f}% codes differ, one-step={one}'
    assert wg.dtype == torch.float32 and tuple(wg.shape) == tuple(wg_ref.shape)
    torch.testing.assert_close(wg.cpu(), wg_ref, atol=1e-4, rtol=1e-4)


def run_gpu(tk, xq, go, w, ptt, t2p, N, round_sf, clamp):
    return tk.quant.swiglu_backward_and_per_token_cast(
        (xq[0].cuda(), xq[1].cuda()), go.cuda(), w.cuda(), ptt.cuda(), t2p.cuda(),
        num_per_channels=N, round_sf=round_sf, swiglu_clamp_value=clamp)


@pytest.mark.parametrize('clamp', [None, 10.0, 0.5])
@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('N', [32, 128])
@pytest.mark.parametrize('H', [256, 512, 1024 + 256, 2048, 3584, 4096 + 512, 7168])
def test_swiglu_backward_and_per_token_cast(H, N, round_sf, clamp):
    tk = _tk()
    xq, go, w, ptt, t2p = make_inputs(301, 4, 12, H, N, seed=H + N)
    want = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, N, round_sf, clamp)
    got = run_gpu(tk, xq, go, w, ptt, t2p, N, round_sf, clamp)
    check_backward(got, want, round_sf, f'H={H} N={N}')


@pytest.mark.parametrize('N', [32, 128])
@pytest.mark.parametrize('T,K,E', [(4001, 8, 64), (1, 1, 1), (5, 3, 7)])
def test_swiglu_backward_reference_sized_batches(T, K, E, N):
    tk = _tk()
    xq, go, w, ptt, t2p = make_inputs(T, K, E, 512, N, seed=T, alignment=64 if T > 100 else 4)
    want = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, N, True, 10.0)
    got = run_gpu(tk, xq, go, w, ptt, t2p, N, True, 10.0)
    check_backward(got, want, True, f'T={T}')


def test_swiglu_backward_odd_row_count_and_wide_values():
    # an odd number of expanded rows (the last workgroup is half empty) and inputs wide enough for
    # the sigmoid to saturate on both sides
    tk = _tk()
    xq, go, w, ptt, t2p = make_inputs(77, 3, 5, 384, 128, seed=4, scale=12.0, alignment=1)
    assert xq[0].shape[0] % 2 == 1
    for clamp in (None, 7.0):
        want = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, 128, False, clamp)
        got = run_gpu(tk, xq, go, w, ptt, t2p, 128, False, clamp)
        check_backward(got, want, False, f'wide clamp={clamp}')


def test_swiglu_backward_no_rows():
    # every pair unrouted: no expanded rows, weight_grad is all zeros
    tk = _tk()
    T, K, H = 6, 2, 256
    x = (torch.empty((0, 2 * H), dtype=torch.float8_e4m3fn, device='cuda'), torch.empty((0, 2 * H // 128), device='cuda'))
    go = torch.empty((0, H), dtype=torch.bfloat16, device='cuda')
    w = torch.rand((T, K), device='cuda')
    ptt = torch.empty((0,), dtype=torch.int32, device='cuda')
    t2p = torch.full((T, K), -1, dtype=torch.int32, device='cuda')
    out, (codes, sf), xg, wg = tk.quant.swiglu_backward_and_per_token_cast(x, go, w, ptt, t2p, 128)
    assert out.shape == (0, H) and codes.shape == (0, 2 * H) and sf.shape == (0, 4) and xg.shape == (0, 2 * H)
    assert torch.equal(wg.cpu(), torch.zeros((T, K)))


def test_swiglu_backward_three_dimensional_input():
    tk = _tk()
    xq, go, w, ptt, t2p = make_inputs(64, 2, 4, 256, 128, seed=8, alignment=8)
    want = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, 128)
    R = go.shape[0]
    assert R % 4 == 0
    x3 = (xq[0].view(4, R // 4, -1), xq[1])
    got = run_gpu(tk, x3, go.view(4, R // 4, -1), w, ptt, t2p, 128, False, None)
    check_backward(got, want, False, '3-d')


def test_swiglu_backward_matches_forward_op():
    # the recomputed activation equals what the forward op quantises: dequantised input through the
    # fused forward, compared after both are brought to bf16 precision
    tk = _tk()
    xq, go, w, ptt, t2p = make_inputs(128, 2, 4, 512, 128, seed=21, alignment=8)
    got = run_gpu(tk, xq, go, w, ptt, t2p, 128, False, None)
    x_deq = xq[0].float() * xq[1].repeat_interleave(128, dim=1)
    fwd = torch_ref.swiglu_forward(x_deq, ptt, w)
    frac, one = bf16_report(got[0], fwd.to(torch.bfloat16))
    assert frac <= BF16_MISMATCH_MAX and one
