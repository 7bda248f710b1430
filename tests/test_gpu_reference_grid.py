"""The reference's own shape grid (4001 / 8001 tokens x hidden 576 ... 7168, its option sets and its MoE routing
parameters), driven through the harness re-created in tilekernels_amd.testing: generators for the grid, assert_equal
after clear_unused_sf for the comparison, check_bias on the dequantised result, as the reference's tests do
(tests/quant/test_per_token_cast.py:51-166, test_per_block_cast.py:36-110,
test_swiglu_forward_and_per_token_cast.py:34-140).  The reference runs the full product of its options; here the
product is enumerated in the same order and every STRIDE-th combination is run, so that all values of all options
occur and the CPU oracle, which is the slow side, stays within a couple of minutes (TK_FULL_TEST=1 runs them all;
TK_GRID_SHIFT=n moves every sample n combinations along, so that successive runs cover other parts of the product).
"""
import os

import pytest
import torch

from oracle import torch_ref

pytestmark = pytest.mark.gpu

FULL = os.getenv('TK_FULL_TEST') in ('1', 'true', 'True')
SHIFT = int(os.getenv('TK_GRID_SHIFT', '0'))


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _testing():
    from tilekernels_amd import testing
    return testing


def _ids(params):
    return _testing().make_param_id(params)


def _sample(params, stride, offset=0):
    return params if FULL else params[(offset + SHIFT) % stride::stride]


def to_host(t: torch.Tensor) -> torch.Tensor:
    """CPU copy with the same shape and strides (assert_equal compares strides and wants one device)."""
    if t.numel() == 0:
        return torch.empty(t.shape, dtype=t.dtype)
    return torch.empty_strided(t.shape, t.stride(), dtype=t.dtype).copy_(t)


SF_MODES = [(False, True, False), (True, True, True)]     # the two option sets the reference's cast tests run


def per_token_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    plain = [
        dict(num_tokens=n, hidden=h, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed, in_dtype=dt,
             num_per_channels=npc, x_block_size=None, fmt=fmt)
        for n in generate_num_tokens() for h in generate_hidden_sizes() for col, rnd, packed in SF_MODES
        for dt in (torch.float32, torch.bfloat16) for npc in (32, 64, 128, h) for fmt in ('e4m3', 'e2m1')
    ]
    requant = [
        dict(num_tokens=n, hidden=h, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed, in_dtype=dt,
             num_per_channels=npc, x_block_size=xb, fmt=fmt)
        for n in generate_num_tokens() for h in generate_hidden_sizes() for col, rnd, packed in SF_MODES
        for dt in (torch.float8_e4m3fn, torch.int8) for npc in (32, 128) for xb in ((128, 128), (32, 32)) for fmt in ('e4m3', 'e2m1')
    ]
    return _sample(plain, 5) + _sample(requant, 9, 2)


@pytest.mark.parametrize('params', per_token_params(), ids=_ids)
def test_per_token_cast_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    n, h, npc, fmt, xb = params['num_tokens'], params['hidden'], params['num_per_channels'], params['fmt'], params['x_block_size']
    kw = dict(use_tma_aligned_col_major_sf=params['use_tma_aligned_col_major_sf'], round_sf=params['round_sf'],
              use_packed_ue8m0=params['use_packed_ue8m0'])
    quantised_input = params['in_dtype'] in (torch.float8_e4m3fn, torch.int8)
    if quantised_input:
        original = torch.randn((n, h), dtype=torch.bfloat16, device='cuda')
        in_fmt = 'e4m3' if params['in_dtype'] == torch.float8_e4m3fn else 'e2m1'
        x_host = torch_ref.cast(original.cpu(), in_fmt, xb, **kw)
        x_dev = tuple(t.cuda() for t in x_host)
    else:
        original = torch.randn((n, h), dtype=params['in_dtype'], device='cuda')
        x_host, x_dev = original.cpu(), original

    codes, sf = tk.quant.per_token_cast(x_dev, fmt, npc, x_block_size=xb, **kw)
    codes_ref, sf_ref = torch_ref.cast(x_host, fmt, (1, npc), x_block_size=xb, **kw)
    codes_h, sf_h = to_host(codes), to_host(sf)
    if params['use_packed_ue8m0']:
        T.assert_equal(T.clear_unused_sf(sf_h, h, npc), T.clear_unused_sf(sf_ref, h, npc))
        assert sf_h.stride() == sf_ref.stride() and sf_h.dtype == sf_ref.dtype
    else:
        T.assert_equal(sf_h, sf_ref)
    T.assert_equal(codes_h, codes_ref)
    T.check_bias(torch_ref.cast_back((codes_h, sf_h), 'fp32', (1, npc)), original.cpu().float())
    assert T.count_bytes(codes, sf) == codes.numel() * codes.element_size() + sf.numel() * sf.element_size()

    if not quantised_input and fmt == 'e4m3' and not params['use_packed_ue8m0']:
        # row stride larger than the row
        wide = torch.randn((n, 2 * h), dtype=params['in_dtype'], device='cuda')[:, :h]
        wide.copy_(original)
        codes2, sf2 = tk.quant.per_token_cast(wide, fmt, npc, **kw)
        T.assert_equal(codes2, codes)
        T.assert_equal(sf2, sf)
    if not quantised_input and npc != h:
        if not params['use_tma_aligned_col_major_sf']:
            given = tk.quant.per_token_cast_with_precomputed_sf(x_dev, fmt, npc, sf, **kw)
            T.assert_equal(to_host(given), torch_ref.cast(x_host, fmt, (1, npc), sf=sf_ref, **kw))
        only = to_host(tk.quant.per_token_cast_with_sf_only(x_dev, fmt, npc, **kw))
        if params['use_packed_ue8m0']:
            T.assert_equal(T.clear_unused_sf(only, h, npc), T.clear_unused_sf(sf_ref, h, npc))
        else:
            T.assert_equal(only, sf_ref)


def per_block_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_num_tokens
    params = [
        dict(num_tokens=n, hidden=h, in_dtype=dt, fmt=fmt, use_tma_aligned_col_major_sf=col, round_sf=rnd,
             use_packed_ue8m0=packed, block_size=blk)
        for n in generate_num_tokens() for h in generate_hidden_sizes() for dt in (torch.bfloat16, torch.float32)
        for fmt in ('e4m3', 'e2m1') for col, rnd, packed in SF_MODES for blk in ((128, 128), (32, 32))
    ]
    return _sample(params, 3, 1)


@pytest.mark.parametrize('params', per_block_params(), ids=_ids)
def test_per_block_cast_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    n, h, fmt, blk = params['num_tokens'], params['hidden'], params['fmt'], params['block_size']
    kw = dict(use_tma_aligned_col_major_sf=params['use_tma_aligned_col_major_sf'], round_sf=params['round_sf'],
              use_packed_ue8m0=params['use_packed_ue8m0'])
    x = torch.randn((n, h), dtype=params['in_dtype'], device='cuda')
    x_host = x.cpu()
    codes, sf = tk.quant.per_block_cast(x, fmt, blk, **kw)
    codes_ref, sf_ref = torch_ref.cast(x_host, fmt, blk, **kw)
    codes_h, sf_h = to_host(codes), to_host(sf)
    if params['use_packed_ue8m0']:
        T.assert_equal(T.clear_unused_sf(sf_h, h, blk[1]), T.clear_unused_sf(sf_ref, h, blk[1]))
        assert sf_h.stride() == sf_ref.stride() and sf_h.dtype == sf_ref.dtype
    else:
        T.assert_equal(sf_h, sf_ref)
    T.assert_equal(codes_h, codes_ref)
    T.check_bias(torch_ref.cast_back((codes_h, sf_h), 'fp32', blk), x_host.float())
    if not params['use_tma_aligned_col_major_sf']:
        given = tk.quant.per_block_cast_with_precomputed_sf(x, fmt, blk, sf, **kw)
        T.assert_equal(to_host(given), torch_ref.cast(x_host, fmt, blk, sf=sf_ref, **kw))
    only = to_host(tk.quant.per_block_cast_with_sf_only(x, fmt, blk, **kw))
    if params['use_packed_ue8m0']:
        T.assert_equal(T.clear_unused_sf(only, h, blk[1]), T.clear_unused_sf(sf_ref, h, blk[1]))
    else:
        T.assert_equal(only, sf_ref)


def swiglu_params():
    from tilekernels_amd.testing import generate_hidden_sizes, generate_moe_params
    params = [
        dict(**moe, hidden=h, enable_pos_to_expert=mask, with_weights=weights, num_per_channels=npc,
             use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed, swiglu_clamp_value=clamp)
        for moe in generate_moe_params() for h in [v // 2 for v in generate_hidden_sizes(256)]
        for mask in (True, False) for weights in (True, False) for npc in (128, h) for col, rnd, packed in SF_MODES
        if not ((packed and weights) or (col and npc == h))
        for clamp in (None, 10.0, 0.5)
    ]
    return _sample(params, 23, 4)


def _scale_per_element(sf, hidden, num_per_channels, dead):
    """The scale of every output element as fp32 [rows, hidden] (zero in padding rows), from a scale tensor in any layout."""
    T = _testing()
    if sf.dtype == torch.int32:                                     # packed UE8M0: one exponent byte per group
        scales = torch.exp2(T.clear_unused_sf(sf, hidden, num_per_channels).float() - 127.0)
    else:
        scales = torch.empty(sf.shape, dtype=torch.float32).copy_(sf)
    nk = (hidden + num_per_channels - 1) // num_per_channels
    per_element = scales[:, :nk].repeat_interleave(num_per_channels, dim=1)[:, :hidden]
    return per_element.masked_fill(dead, 0)


@pytest.mark.parametrize('params', swiglu_params(), ids=_ids)
def test_swiglu_forward_and_per_token_cast_on_the_reference_grid(params):
    tk, T = _tk(), _testing()
    from tilekernels_amd.config import get_num_sms, set_num_sms
    h, npc, clamp = params['hidden'], params['num_per_channels'], params['swiglu_clamp_value']
    kw = dict(use_tma_aligned_col_major_sf=params['use_tma_aligned_col_major_sf'], round_sf=params['round_sf'],
              use_packed_ue8m0=params['use_packed_ue8m0'])
    topk_idx = T.generate_topk_idx(params)
    num_tokens = topk_idx.shape[0]
    p2e, p2t, p2tt, t2p, *_ = tk.moe.get_fused_mapping(topk_idx, params['num_experts'], 0, 128)
    weights = torch.randn((num_tokens, params['num_topk']), dtype=torch.float32, device='cuda')
    x = tk.moe.expand_to_fused(torch.randn((num_tokens, 2 * h), dtype=torch.bfloat16, device='cuda'), t2p, p2t)
    counting = npc != h and clamp is not None
    count_ref = torch.zeros(3, dtype=torch.int64) if counting else None
    codes_ref, sf_ref = torch_ref.swiglu_forward_and_per_token_cast(
        x.cpu(), 'e4m3', npc, p2tt.cpu() if params['with_weights'] else None, weights.cpu() if params['with_weights'] else None,
        p2e.cpu() if params['enable_pos_to_expert'] else None, swiglu_clamp_value=clamp, clamped_count=count_ref, **kw)
    dead = (p2e.cpu() < 0)[:, None]
    ref_values = codes_ref.float().masked_fill(dead, 0)
    before = get_num_sms()
    try:
        for num_sms in T.generate_num_sms():
            set_num_sms(num_sms)
            count = torch.zeros(3, dtype=torch.int64, device='cuda') if counting else None
            codes, sf = tk.quant.swiglu_forward_and_per_token_cast(
                x, 'e4m3', npc, p2tt if params['with_weights'] else None, weights if params['with_weights'] else None,
                p2e if params['enable_pos_to_expert'] else None, swiglu_clamp_value=clamp, clamped_count=count, **kw)
            codes_h, sf_h = to_host(codes), to_host(sf)
            values = codes_h.float().masked_fill(dead, 0)
            # exp and the quotient differ in the last place between CPU and GPU: at most 0.01 % of the codes may differ,
            # each by one E4M3 step, scales to 1e-6 (power-of-two scales: the same share may move by one binade)
            differing = values != ref_values
            assert differing.float().mean().item() <= 1e-4, differing.float().mean().item()
            s_got, s_ref = _scale_per_element(sf_h, h, npc, dead), _scale_per_element(sf_ref, h, npc, dead)
            if differing.any():
                # under the same scale the two codes are neighbours; where a power-of-two scale itself fell on the other side
                # of a binade (see below), every code of the group moves with it and the dequantised values stay one step
                # of the coarser grid apart
                moved = s_got != s_ref
                near = differing & ~moved
                a, b = codes_h.view(torch.uint8)[near].int(), codes_ref.view(torch.uint8)[near].int()
                assert bool((((a & 0x7F) - (b & 0x7F)).abs() <= 1).all())
                far = differing & moved
                if far.any():
                    assert params['round_sf']
                    vg, vr = (values * s_got)[far], (ref_values * s_ref)[far]
                    step = torch.maximum(vg.abs(), vr.abs()) * 2.0 ** -3 + torch.maximum(s_got, s_ref)[far] * 2.0 ** -9
                    assert bool(((vg - vr).abs() <= step).all())
            assert float(T.calc_diff(values * s_got, ref_values * s_ref)) < 1e-6
            assert sf_h.dtype == sf_ref.dtype and sf_h.shape == sf_ref.shape and sf_h.stride() == sf_ref.stride()
            if params['use_packed_ue8m0']:
                got, want = T.clear_unused_sf(sf_h.masked_fill(dead, 0), h, npc), T.clear_unused_sf(sf_ref.masked_fill(dead, 0), h, npc)
                assert (got != want).float().mean().item() <= 1e-4
                assert int((got.int() - want.int()).abs().max()) <= 1
            else:
                got, want = sf_h.masked_fill(dead, 0), sf_ref.masked_fill(dead, 0)      # padding rows count on neither side
                off = (got != want)
                if params['round_sf']:
                    assert off.float().mean().item() <= 1e-4
                    assert bool(((got[off] == 2 * want[off]) | (2 * got[off] == want[off])).all())
                else:
                    assert float(((got - want).abs() / want.abs().clamp(min=1e-30)).max()) <= 1e-6
            if counting:
                T.assert_equal(count.cpu(), count_ref)
    finally:
        set_num_sms(before)


def test_unpack_from_e2m1fn_x2_on_the_gpu():
    tk, T = _tk(), _testing()
    every = torch.arange(256, dtype=torch.uint8).view(torch.int8).reshape(16, 16)
    for dtype in (torch.float32, torch.bfloat16):
        got = tk.quant.unpack_from_e2m1fn_x2(every.cuda(), dtype)
        assert got.is_cuda and got.shape == (16, 32) and got.dtype == dtype
        T.assert_equal(got.cpu(), torch_ref.unpack_from_e2m1fn_x2(every, dtype))
    # on the product's own FP4 codes: dequantising them reproduces the oracle's dequantisation
    x = T.make_baseline_input(5, scale_rows=1 / 64)['x']
    kw = dict(use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    codes, sf = tk.quant.per_token_cast(x.cuda(), 'e2m1', 32, **kw)
    values = tk.quant.unpack_from_e2m1fn_x2(codes)
    T.assert_equal(values.cpu(), torch_ref.unpack_from_e2m1fn_x2(torch_ref.cast(x, 'e2m1', (1, 32), **kw)[0]))
    back = tk.quant.cast_back((codes, sf), 'fp32', (1, 32))
    scale = torch.pow(2.0, T.clear_unused_sf(to_host(sf), x.shape[1], 32)[:, : x.shape[1] // 32].float() - 127).repeat_interleave(32, dim=1)
    T.assert_equal(back.cpu(), values.cpu() * scale)


def test_count_bytes_matches_the_benchmark_byte_counts():
    """count_bytes over (input, codes, scales) of every benchmark configuration equals the algorithmic bytes
    bench.py prices its roofline with (configuration 4: only the rows that are read count on the input side)."""
    import bench
    tk, T = _tk(), _testing()
    expect = {1: 88997888, 2: 44043776, 3: 84410368, 5: 297271296}
    for cfg in (1, 2, 3, 4, 5):
        d = T.make_baseline_input(cfg)
        x = d['x'].cuda()
        if cfg == 1:
            out = tk.quant.per_token_cast(x, 'e4m3', 128)
        elif cfg == 2:
            out = tk.quant.per_block_cast(x, 'e4m3', (128, 128))
        elif cfg == 5:
            out = tk.quant.per_token_cast(x, 'e2m1', 32, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
        else:
            out = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=d['pos_to_expert'].cuda() if cfg == 4 else None)
        if cfg == 4:
            live = int((d['pos_to_expert'] >= 0).sum())
            total = live * x.shape[1] * 2 + T.count_bytes(d['pos_to_expert']) + T.count_bytes(out)
        else:
            total = T.count_bytes(x, out)
        assert total == bench.algorithmic_bytes(cfg, d), cfg
        if cfg in expect:
            assert total == expect[cfg], (cfg, total)
        del x, out
