"""The operators either side of the hot path on the reference's own shape grids and option sets, sampled as in
tests/test_gpu_reference_grid.py: dequantisation (tests/quant/test_cast_back.py:44-110, incl. per-channel 128 x 1
scales), the per-channel casts (test_per_channel_cast.py:20-48, test_per_channel_cast_and_transpose.py:21-45,
test_per_channel_cast_fused.py:14-84, test_swiglu_forward_and_per_channel_cast_and_transpose.py), the fused SwiGLU
backward (test_swiglu_backward_and_per_token_cast.py:20-110) and the MoE layout helpers
(tests/moe/test_get_fused_mapping.py:30-78, test_expand_to_fused.py:20-125), each against the CPU oracle."""
import itertools

import pytest
import torch

from oracle import torch_ref
from tests.test_gpu_reference_grid import SF_MODES, _ids, _sample, _testing, _tk, to_host

pytestmark = pytest.mark.gpu


def cast_back_per_token_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    return _sample([
        dict(num_tokens=n, hidden=h, fmt=fmt, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed,
             num_per_channels=npc, out_dtype=dt)
        for n in generate_num_tokens() for h in generate_hidden_sizes() for fmt in ('e2m1', 'e4m3')
        for col, rnd, packed in SF_MODES for npc in (128, h) for dt in (torch.float32, torch.bfloat16)], 7, 3)


@pytest.mark.parametrize('params', cast_back_per_token_params(), ids=_ids)
def test_per_token_cast_back_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    n, h, fmt, npc = params['num_tokens'], params['hidden'], params['fmt'], params['num_per_channels']
    kw = dict(use_tma_aligned_col_major_sf=params['use_tma_aligned_col_major_sf'], round_sf=params['round_sf'],
              use_packed_ue8m0=params['use_packed_ue8m0'])
    x = torch.randn((n, h), dtype=params['out_dtype'], device='cuda')
    codes, sf = tk.quant.per_token_cast(x, fmt, npc, **kw)
    out_name = T.dtype_to_str(params['out_dtype'])
    back = tk.quant.per_token_cast_back((codes, sf), out_name, npc)
    want = torch_ref.cast_back((to_host(codes), to_host(sf)), out_name, (1, npc))
    T.assert_equal(back.cpu(), want)
    assert float(T.calc_diff(x.cpu(), back.cpu())) < (2e-2 if fmt == 'e2m1' else 1e-3)


def cast_back_block_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    return _sample([
        dict(num_tokens=n, hidden=h, round_sf=rnd, fmt='e4m3', out_dtype=dt, num_per_tokens=bm, num_per_channels=bk)
        for n in generate_num_tokens() for h in generate_hidden_sizes() for rnd in (False, True)
        for dt in (torch.bfloat16, torch.float32) for bm, bk in ((128, 1), (128, 128))], 3)


@pytest.mark.parametrize('params', cast_back_block_params(), ids=_ids)
def test_cast_back_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    blk = (params['num_per_tokens'], params['num_per_channels'])
    x = torch.randn((params['num_tokens'], params['hidden']), dtype=params['out_dtype'])
    codes, sf = torch_ref.cast(x, 'e4m3', blk, round_sf=params['round_sf'])
    out_name = T.dtype_to_str(params['out_dtype'])
    back = tk.quant.cast_back((codes.cuda(), sf.cuda()), out_name, blk)
    T.assert_equal(back.cpu(), torch_ref.cast_back((codes, sf), out_name, blk))


def per_channel_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    plain = [dict(op='plain', num_per_tokens=128, num_tokens=n, hidden=h, round_sf=rnd)
             for n in generate_num_tokens(128) for h in generate_hidden_sizes() for rnd in (False, True)]
    turned = [dict(op='transpose', num_per_tokens=npt, num_tokens=n, hidden=h, round_sf=rnd)
              for n in generate_num_tokens(128) for h in generate_hidden_sizes() for rnd in (True, False) for npt in (32, 128)]
    return _sample(plain, 3) + _sample(turned, 5, 1)


@pytest.mark.parametrize('params', per_channel_params(), ids=_ids)
def test_per_channel_casts_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    npt, rnd = params['num_per_tokens'], params['round_sf']
    x = torch.randn((params['num_tokens'], params['hidden']), dtype=torch.bfloat16, device='cuda')
    want_codes, want_sf = torch_ref.cast(x.cpu(), 'e4m3', (npt, 1), round_sf=rnd)
    if params['op'] == 'plain':
        codes, sf = tk.quant.per_channel_cast(x, 'e4m3', npt, rnd)
        T.check_bias(torch_ref.cast_back((want_codes, want_sf), 'fp32', (npt, 1)), x.cpu().float())
    else:
        codes, sf = tk.quant.per_channel_cast_and_transpose(x, 'e4m3', npt, rnd)
        want_codes = want_codes.T.contiguous()
    T.assert_equal(codes.cpu(), want_codes)
    T.assert_equal(sf.cpu(), want_sf)


def per_channel_fused_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_moe_params
    return _sample([
        dict(**moe, hidden=h, num_per_tokens=128, num_per_channels=128, is_fused_cast_back=q, round_sf=rnd)
        for moe in itertools.chain([dict(num_send_tokens=4096, num_topk=0, num_experts=0, num_ep_ranks=0)], generate_moe_params())
        for h in generate_hidden_sizes(128) for q in (False, True) for rnd in (False, True)], 9, 2)


@pytest.mark.parametrize('params', per_channel_fused_params(), ids=_ids)
def test_per_channel_cast_fused_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    h, rnd, q = params['hidden'], params['round_sf'], params['is_fused_cast_back']
    pos_to_token = None
    if params['num_topk'] > 0:
        topk_idx = T.generate_topk_idx(params)
        _, pos_to_token, _, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, params['num_experts'], 0, 128)
        x = torch.randn((topk_idx.shape[0], h), dtype=torch.bfloat16, device='cuda')
    else:
        x = torch.randn((params['num_send_tokens'], h), dtype=torch.bfloat16, device='cuda')
    # the gather is the operator's own (pos_to_token): it reads the unexpanded rows
    if q:
        xin = tk.quant.per_token_cast(x, 'e4m3', 128)
        xin_host = (to_host(xin[0]), to_host(xin[1]))
    else:
        xin, xin_host = x, x.cpu()
    got = tk.quant.per_channel_cast_fused(xin, 'e4m3', num_per_tokens=128, round_sf=rnd, num_per_channels=128 if q else None,
                                          pos_to_token=pos_to_token)
    want = torch_ref.per_channel_cast_fused(xin_host, 128, 128 if q else None, rnd, None if pos_to_token is None else pos_to_token.cpu())
    T.assert_equal(got[0].cpu(), want[0])
    T.assert_equal(got[1].cpu(), want[1])


def swiglu_per_channel_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    return _sample([
        dict(num_tokens=n, hidden=h, num_per_tokens=npt, without_transpose=wt, round_sf=rnd, swiglu_clamp_value=clamp)
        for n in generate_num_tokens(128) for h in generate_hidden_sizes() for npt in (32, 128) for wt in (True, False)
        for rnd in (True, False) for clamp in (None, 10.0, 0.5)], 11, 5)


@pytest.mark.parametrize('params', swiglu_per_channel_params(), ids=_ids)
def test_swiglu_forward_and_per_channel_cast_on_the_reference_grid(params):
    from tests.test_gpu_per_channel import check_swiglu_per_channel
    tk = _tk()
    h, npt, wt, rnd, clamp = (params[k] for k in ('hidden', 'num_per_tokens', 'without_transpose', 'round_sf', 'swiglu_clamp_value'))
    x = torch.randn((params['num_tokens'], 2 * h), dtype=torch.bfloat16, device='cuda')
    want = torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(x.cpu(), npt, rnd, wt, clamp)
    got = tk.quant.swiglu_forward_and_per_channel_cast_and_transpose(x, 'e4m3', num_per_tokens=npt, round_sf=rnd,
                                                                    without_transpose=wt, swiglu_clamp_value=clamp)
    check_swiglu_per_channel(got, want, npt, rnd, not wt, _ids(params))


def swiglu_backward_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_moe_params
    return _sample([
        dict(**moe, hidden=h, num_per_channels=npc, round_sf=rnd, swiglu_clamp_value=clamp)
        for moe in generate_moe_params() for h in generate_hidden_sizes(256) for npc in (32, 128) for rnd in (False, True)
        for clamp in (None, 10.0, 0.5)], 97, 6)


@pytest.mark.parametrize('params', swiglu_backward_params(), ids=_ids)
def test_swiglu_backward_on_the_reference_grid(params):
    from tests.test_gpu_swiglu_backward import check_backward
    tk, T = _tk(), _testing()
    h, npc, rnd, clamp = (params[k] for k in ('hidden', 'num_per_channels', 'round_sf', 'swiglu_clamp_value'))
    h //= 2           # the grid's sizes are the widths of x = gate | up
    topk_idx = T.generate_topk_idx(params)
    num_tokens = topk_idx.shape[0]
    weights = torch.rand((num_tokens, params['num_topk']), dtype=torch.float32, device='cuda')
    x = torch.randn((num_tokens, 2 * h), dtype=torch.bfloat16, device='cuda')
    _, p2t, p2tt, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, params['num_experts'], 0, npc)
    xq = tk.quant.per_token_cast(tk.moe.expand_to_fused(x, t2p, p2t), 'e4m3', npc)
    grad = torch.randn((xq[0].shape[0], h), dtype=torch.bfloat16, device='cuda')
    got = tk.quant.swiglu_backward_and_per_token_cast(xq, grad, weights, p2tt, t2p, num_per_channels=npc, round_sf=rnd,
                                                      swiglu_clamp_value=clamp)
    want = torch_ref.swiglu_backward_and_per_token_cast((to_host(xq[0]), to_host(xq[1])), grad.cpu(), weights.cpu(), p2tt.cpu(),
                                                        t2p.cpu(), num_per_channels=npc, round_sf=rnd, swiglu_clamp_value=clamp)
    check_backward(got, want, rnd, _ids(params))


def mapping_params():
    from tilekernels_amd.testing import generate_moe_params
    return [dict(**moe, alignment=a) for moe in generate_moe_params() for a in (64, 128)]


@pytest.mark.parametrize('params', mapping_params(), ids=_ids)
def test_get_fused_mapping_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    topk_idx = T.generate_topk_idx(params)
    got = tk.moe.get_fused_mapping(topk_idx, params['num_experts'], 0, params['alignment'])
    want = torch_ref.get_fused_mapping(topk_idx.cpu(), params['num_experts'], params['alignment'])
    for g, w in zip(got[:7], want):
        T.assert_equal(g.cpu(), w)
    assert got[7] == want[6].tolist()
    # the checks of the reference's test: every routed pair has a live position and back, experts are contiguous
    p2e, p2t, p2tt, t2p = (t.cpu() for t in got[:4])
    routed = topk_idx.cpu() >= 0
    assert bool(((t2p >= 0) == routed).all())
    assert torch.equal(p2tt[t2p[routed].long()], torch.nonzero(routed.flatten()).flatten().int())
    assert torch.equal(p2e[t2p[routed].long()].long(), topk_idx.cpu()[routed])
    assert torch.equal(p2t[p2tt >= 0], (p2tt[p2tt >= 0] // params['num_topk']))
    assert all(n % params['alignment'] == 0 for n in got[7])


def expand_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_moe_params
    plain = [dict(**moe, hidden=h) for moe in generate_moe_params() for h in generate_hidden_sizes()]
    with_sf = [dict(**moe, hidden=h, num_per_channels=npc, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
               for moe in generate_moe_params() for h in generate_hidden_sizes() for npc in (32, 128) for col, rnd, packed in SF_MODES]
    return _sample(plain, 5, 1) + _sample(with_sf, 13, 4)


@pytest.mark.parametrize('params', expand_params(), ids=_ids)
def test_expand_to_fused_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    topk_idx = T.generate_topk_idx(params)
    num_tokens = topk_idx.shape[0]
    x = torch.randn((num_tokens, params['hidden']), dtype=torch.bfloat16, device='cuda')
    p2e, _, _, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, params['num_experts'], 0, 16)
    if 'num_per_channels' not in params:
        got = tk.moe.expand_to_fused(x, t2p, p2e)
        T.assert_equal(got.cpu(), torch_ref.expand_to_fused(x.cpu(), t2p.cpu(), p2e.cpu()))
        return
    npc, col = params['num_per_channels'], params['use_tma_aligned_col_major_sf']
    codes, sf = tk.quant.per_token_cast(x, 'e4m3', npc, use_tma_aligned_col_major_sf=col, round_sf=params['round_sf'],
                                        use_packed_ue8m0=params['use_packed_ue8m0'])
    sf = sf.contiguous()
    got = tk.moe.expand_to_fused_with_sf((codes, sf), npc, t2p, p2e, col)
    want = torch_ref.expand_to_fused_with_sf((codes.cpu(), sf.cpu()), npc, t2p.cpu(), p2e.cpu(), col)
    T.assert_equal(got[0].cpu(), want[0])
    T.assert_equal(to_host(got[1]), want[1], check_stride=num_tokens > 0)
