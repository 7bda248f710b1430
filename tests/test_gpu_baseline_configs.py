"""The five benchmark configurations at full size: GPU results against the CPU oracle on the same
seeded inputs (casts bit-exact, fused SwiGLU within its tolerance), plus size-independent
properties (repeatability, scale-only == cast scales, dequantisation error bound, zeroed padding)."""
import pytest
import torch

from oracle import cref, torch_ref
from tests._util import assert_same, dense_bytes, fp8_code_report, packed_sf_bytes
from tests.test_gpu_swiglu import check_fused

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    torch.set_num_threads(min(16, torch.get_num_threads()))
    return tilekernels_amd


def test_config1_per_token_fp8():
    tk = _tk()
    x = tk.testing.make_baseline_input(1)['x']
    assert x.shape == (4096, 7168)
    xg = x.cuda()
    codes, sf = tk.quant.per_token_cast(xg, 'e4m3', 128)
    codes_ref, sf_ref = torch_ref.cast(x, 'e4m3', (1, 128))
    assert sf.shape == (4096, 56)
    assert_same(codes, codes_ref, 'codes')
    assert_same(sf, sf_ref, 'sf')
    # second, independent statement of the algorithm
    c2, s2 = cref.cast(x, 'e4m3', (1, 128))
    assert torch.equal(codes.cpu().view(torch.uint8), c2) and torch.equal(sf.cpu(), s2)
    # properties
    assert torch.equal(sf.cpu(), (x.float().abs().view(4096, 56, 128).amax(-1).clamp(min=1e-4) / torch.full((4096, 56), 448.0)))
    assert_same(tk.quant.per_token_cast_with_sf_only(xg, 'e4m3', 128), sf_ref, 'sf only')
    again, _ = tk.quant.per_token_cast(xg, 'e4m3', 128)
    assert torch.equal(again.view(torch.uint8), codes.view(torch.uint8))
    back = torch_ref.cast_back((codes.cpu(), sf.cpu()), 'fp32', (1, 128))
    err = (back - x.float()).abs()
    bound = sf.cpu().repeat_interleave(128, 1) * 16.01       # half an E4M3 step at the top binade (32 * sf / 2) plus fp32 slack
    assert (err <= bound).all()
    tk.testing.check_bias(back, x.float())


def test_config2_per_block_fp8():
    tk = _tk()
    w = tk.testing.make_baseline_input(2)['x']
    assert w.shape == (7168, 2048)
    codes, sf = tk.quant.per_block_cast(w.cuda(), 'e4m3', (128, 128))
    codes_ref, sf_ref = torch_ref.cast(w, 'e4m3', (128, 128))
    assert sf.shape == (56, 16)
    assert_same(sf, sf_ref, 'sf')
    assert_same(codes, codes_ref, 'codes')
    c2, s2 = cref.cast(w, 'e4m3', (128, 128))
    assert torch.equal(codes.cpu().view(torch.uint8), c2) and torch.equal(sf.cpu(), s2)
    assert_same(tk.quant.per_block_cast_with_sf_only(w.cuda(), 'e4m3', (128, 128)), sf_ref, 'sf only')
    # every block's largest element maps to +-448
    mags = (codes.cpu().view(torch.uint8) & 0x7F).view(56, 128, 16, 128).amax(dim=(1, 3))
    assert torch.all(mags == 0x7E)


def test_config3_swiglu_fp8():
    tk = _tk()
    x = tk.testing.make_baseline_input(3)['x']
    assert x.shape == (8192, 4096)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128)
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    assert got[0].shape == (8192, 2048) and got[1].shape == (8192, 16)
    frac = check_fused(got, want, 16, False, 'config 3')
    print(f'config 3: {frac * 100:.6f}% codes differ')
    again = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128)
    assert torch.equal(again[0].view(torch.uint8), got[0].view(torch.uint8)) and torch.equal(again[1], got[1])
    # the fused op equals "SwiGLU then per-token cast" up to the activation's rounding: feeding the
    # oracle's fp32 activation through the GPU cast reproduces the oracle exactly
    v = torch_ref.swiglu_forward(x)
    c2, s2 = tk.quant.per_token_cast(v.cuda(), 'e4m3', 128)
    assert_same(c2, want[0], 'cast of the oracle activation')
    assert_same(s2, want[1], 'scales of the oracle activation')


def test_config4_moe_expanded_swiglu_fp8():
    tk = _tk()
    d = tk.testing.make_baseline_input(4)
    x, pe, ptt, w = d['x'], d['pos_to_expert'], d['pos_to_token_topk'], d['topk_weights']
    R = x.shape[0]
    assert int((pe >= 0).sum()) == 4096 * 8 and R % 128 == 0 and R >= 32768
    # layout invariants of the expansion: expert-major, every expert padded to a multiple of 128
    live = pe >= 0
    assert torch.all(pe[live][1:] >= pe[live][:-1])
    assert torch.equal(torch.sort(ptt[live]).values, torch.arange(4096 * 8, dtype=torch.int32))
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128, pos_to_expert=pe.cuda())
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pe)
    check_fused(got, want, 16, False, 'config 4')
    assert torch.all(got[0].cpu().view(torch.uint8)[~live] == 0) and torch.all(got[1].cpu()[~live] == 0)
    # padding rows are never read: poison them and the result must not change
    xp = x.clone()
    xp[~live] = float('nan')
    got_p = tk.quant.swiglu_forward_and_per_token_cast(xp.cuda(), 'e4m3', 128, pos_to_expert=pe.cuda())
    assert torch.equal(got_p[0].view(torch.uint8), got[0].view(torch.uint8)) and torch.equal(got_p[1], got[1])
    # weighted variant
    got_w = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128, ptt.cuda(), w.cuda(), pe.cuda())
    want_w = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, ptt, w, pe)
    check_fused(got_w, want_w, 16, False, 'config 4 weighted')


def test_config5_fp4_packed_ue8m0():
    tk = _tk()
    x = tk.testing.make_baseline_input(5)['x']
    assert x.shape == (16384, 7168)
    kw = dict(use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    codes, sf = tk.quant.per_token_cast(x.cuda(), 'e2m1', 32, **kw)
    codes_ref, sf_ref = torch_ref.cast(x, 'e2m1', (1, 32), **kw)
    assert codes.shape == (16384, 3584) and codes.dtype == torch.int8
    assert sf.shape == (16384, 56) and sf.dtype == torch.int32 and sf.stride() == (1, 16384)
    assert_same(codes, codes_ref, 'codes')
    assert_same(sf, sf_ref, 'sf')
    c2, s2 = cref.cast(x, 'e2m1', (1, 32), round_sf=True)
    assert torch.equal(codes.cpu().view(torch.uint8), c2)
    by = packed_sf_bytes(sf, 224)
    assert torch.equal((by.to(torch.int32) << 23).view(torch.float32), s2)
    # the other legal spelling: power-of-two fp32 scales, row-major
    c3, s3 = tk.quant.per_token_cast(x.cuda(), 'e2m1', 32, round_sf=True)
    assert torch.equal(c3.view(torch.uint8), codes.view(torch.uint8)) and torch.equal(s3.cpu(), s2)
    # power-of-two scales make the quantisation multiply exact: decoded values times scale never
    # exceed 6 * scale and every group's largest code is at least 4 (the scale is the next power of two)
    mag = torch_ref.unpack_from_e2m1fn_x2(codes.cpu()[:2048]).abs().view(2048, 224, 32).amax(-1)
    assert torch.all(mag <= 6.0) and torch.all(mag >= 3.0)
