"""GPU parity of the fused SwiGLU + per-token FP8 cast against the CPU oracle.

Tolerance (floating point, exp/divide rounding differs between CPU and GPU): scales within 1e-6
relative, at most 0.01 % of the codes differ and each by one E4M3 step; clamp counters and the
zeros of padding rows are exact.  Structure follows the reference's
tests/quant/test_swiglu_forward_and_per_token_cast.py."""
import pytest
import torch

from oracle import torch_ref
from tests._util import dense_bytes, fp8_code_report, mismatch_within, packed_sf_bytes

pytestmark = pytest.mark.gpu

SCALE_RTOL = 1e-6
CODE_MISMATCH_MAX = 1e-4


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def check_fused(got, want, nk, packed, what=''):
    codes, sf = got
    codes_ref, sf_ref = want
    assert codes.dtype == codes_ref.dtype and tuple(codes.shape) == tuple(codes_ref.shape)
    assert sf.dtype == sf_ref.dtype and tuple(sf.shape) == tuple(sf_ref.shape), (sf.shape, sf_ref.shape)
    if sf.numel():
        assert sf.stride() == sf_ref.stride(), f'{what} sf stride {sf.stride()} != {sf_ref.stride()}'
    if packed:
        a, b = packed_sf_bytes(sf, nk), packed_sf_bytes(sf_ref, nk)
        assert torch.equal(a, b), f'{what}: {(a != b).sum().item()} packed scale bytes differ'
    else:
        a = torch.empty(sf.shape).copy_(sf.cpu())
        b = torch.empty(sf.shape).copy_(sf_ref)
        rel = ((a - b).abs() / b.abs().clamp(min=1e-30)).max().item() if a.numel() else 0.0
        assert rel <= SCALE_RTOL, f'{what}: scale rel err {rel}'
        assert torch.equal(a == 0, b == 0)
    frac, one_step = fp8_code_report(dense_bytes(codes.cpu()), dense_bytes(codes_ref))
    assert mismatch_within(frac, codes_ref.numel(), CODE_MISMATCH_MAX) and one_step, f'{what}: {frac * 100:.5f}% codes differ, one-step={one_step}'
    return frac


@pytest.mark.parametrize('clamp', [None, 10.0, 0.5])
@pytest.mark.parametrize('mode', [(False, False, False), (False, True, False), (True, True, False), (True, True, True)],
                         ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('with_weights', [False, True])
@pytest.mark.parametrize('with_mask', [False, True])
@pytest.mark.parametrize('H,N', [(2048, 128), (288 * 4 + 128, 128), (1024, 1024), (3584, 128), (384, 384),
                                 (512, 128), (896, 128), (5632, 128),    # one, two and eleven 512-column strips
                                 (2560, 2560), (4224, 4224), (8192, 8192), (8320, 8320),    # whole-row groups: 2, 3, 4 register pieces, two passes
                                 (768, 128), (256, 128)])   # short rows: laid end to end over the lanes
def test_swiglu_forward_and_per_token_cast(H, N, with_mask, with_weights, mode, clamp):
    tk = _tk()
    col, rnd, packed = mode
    if N == H and col:
        pytest.skip('one scale per row is row-major only')
    g = torch.Generator().manual_seed(H + 7 * N + int(with_mask) + 2 * int(with_weights))
    pe, ptt, w = tk.testing.generate_moe_layout(97, 12, 3, 16, g, drop_fraction=0.1)
    R = pe.numel()
    x = torch.randn((R, 2 * H), generator=g) * 2
    x[pe < 0] = 0
    x = x.to(torch.bfloat16)
    count = torch.tensor([3, 1, 4], dtype=torch.int64) if (clamp is not None and N != H) else None
    count_ref = None if count is None else count.clone()
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed, swiglu_clamp_value=clamp)
    want = torch_ref.swiglu_forward_and_per_token_cast(
        x, 'e4m3', N, ptt if with_weights else None, w if with_weights else None, pe if with_mask else None,
        clamped_count=count_ref, **kw)
    for num_sms in (tk.get_device_num_sms(), 7):
        tk.set_num_sms(num_sms)
        cg = None if count is None else count.cuda()
        got = tk.quant.swiglu_forward_and_per_token_cast(
            x.cuda(), 'e4m3', N, ptt.cuda() if with_weights else None, w.cuda() if with_weights else None,
            pe.cuda() if with_mask else None, clamped_count=cg, **kw)
        codes, sf = got
        if not with_mask:
            # the reference compares padding rows as zeros on both sides (they hold silu(0)*0 = 0 anyway)
            pass
        check_fused(got, want, H // N, packed, f'num_sms={num_sms}')
        if with_mask:
            dead = pe < 0
            assert torch.all(codes.cpu().view(torch.uint8)[dead] == 0)
            assert torch.all(torch.empty(sf.shape, dtype=sf.dtype).copy_(sf.cpu())[dead] == 0)
        if count is not None:
            assert cg.cpu().tolist() == count_ref.tolist()
    tk.set_num_sms(tk.get_device_num_sms())


@pytest.mark.parametrize('mode', [(False, False, False), (True, False, False), (True, True, True)],
                         ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('with_mask', [False, True])
@pytest.mark.parametrize('H', [1024, 2048, 1536, 896, 3584])   # row-wise, wide and stacked tiles of the fp32 kernel (2 pieces per wave)
def test_swiglu_fp32_input_tiles(H, with_mask, mode):
    tk = _tk()
    col, rnd, packed = mode
    g = torch.Generator().manual_seed(H + int(with_mask))
    pe, ptt, w = tk.testing.generate_moe_layout(61, 8, 2, 16, g, drop_fraction=0.1)
    R = pe.numel()
    x = torch.randn((R, 2 * H), generator=g) * 2
    x[pe < 0] = 0
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, ptt, w, pe if with_mask else None, **kw)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128, ptt.cuda(), w.cuda(), pe.cuda() if with_mask else None, **kw)
    check_fused(got, want, H // 128, packed, f'fp32 H={H}')


@pytest.mark.parametrize('clamp', [None, 0.5])
@pytest.mark.parametrize('rnd', [False, True])
@pytest.mark.parametrize('with_weights', [False, True])
@pytest.mark.parametrize('layout', ['row', 'col', 'packed'])
@pytest.mark.parametrize('R,H', [(6144, 2048), (3076, 4096), (8192, 2048), (1600, 8192), (10912, 1536), (5456, 2560), (32768, 512), (4096, 3584)])
def test_swiglu_launches_that_end_in_smaller_waves(R, H, layout, with_weights, rnd, clamp):
    """Unmasked bf16 batches of about one to three times the GPU's wave slots, H a multiple of 512: the last rows are
    handled by waves of two pieces and of one piece (a different kernel path with its own argument handling; with the
    column-major layouts the four waves of a workgroup take four rows of the same pieces and store their scales together;
    where H is no multiple of 2048 a wave's two pieces lie one below the other).
    Rows, weights, clamp and the power-of-two scales must come out as from the one-row waves."""
    if layout == 'packed' and not rnd:
        pytest.skip('packed scales are powers of two')
    tk = _tk()
    g = torch.Generator().manual_seed(R + H + int(with_weights))
    x = (torch.randn((R, 2 * H), generator=g) * 1.5).to(torch.bfloat16)
    ptt = w = None
    if with_weights:
        ptt = torch.randperm(R, generator=g).to(torch.int32)
        ptt[torch.rand(R, generator=g) < 0.05] = -1                 # rows without a routing slot get weight 0
        w = torch.rand(((R + 7) // 8, 8), generator=g) + 0.25
    kw = dict(round_sf=rnd, swiglu_clamp_value=clamp, use_tma_aligned_col_major_sf=layout != 'row', use_packed_ue8m0=layout == 'packed')
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, ptt, w, None, **kw)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128, None if ptt is None else ptt.cuda(),
                                                     None if w is None else w.cuda(), None, **kw)
    check_fused(got, want, H // 128, layout == 'packed', f'R={R} H={H} {layout}')


def test_swiglu_smaller_waves_with_padded_scale_rows():
    """Through the C ABI: scale rows with a leading dimension larger than the number of groups (the tail waves take it from a
    different kernel argument than the one-row waves)."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    R, H, ld = 8192, 2048, 24
    g = torch.Generator().manual_seed(5)
    x = torch.randn((R, 2 * H), generator=g).to(torch.bfloat16)
    want_codes, want_sf = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    xg = x.cuda()
    codes = torch.empty((R, H), dtype=torch.uint8, device='cuda')
    sf = torch.full((R, ld), -1.0, dtype=torch.float32, device='cuda')
    rc = lib.tk_swiglu_per_token_cast(xg.data_ptr(), _ffi.TK_BF16, R, H, codes.data_ptr(), sf.data_ptr(), ld, 128, _ffi.TK_SF_ROW_F32, 0, -1.0,
                                      0, 0, 0, 0, 0, 0.0, 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check_fused((codes.view(torch.float8_e4m3fn), sf[:, :16].contiguous()), (want_codes, want_sf), 16, False, 'padded scale rows')
    assert torch.all(sf[:, 16:].cpu() == -1.0)


def test_swiglu_fp32_input_and_custom_floor():
    tk = _tk()
    x = torch.randn((50, 512)) * 3
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, sf_clamp_min=0.05)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128, sf_clamp_min=0.05)
    check_fused(got, want, 2, False)
    z = torch.zeros((4, 256), dtype=torch.bfloat16)
    c, s = tk.quant.swiglu_forward_and_per_token_cast(z.cuda(), 'e4m3', 128, sf_clamp_min=448.0)
    assert torch.all(s.cpu() == 1.0) and torch.all(c.cpu().view(torch.uint8) == 0)


def test_swiglu_extreme_gate_values():
    """exp(-g) overflow / underflow must give the oracle's zeros and identities, not NaN."""
    tk = _tk()
    x = torch.randn((8, 256))
    x[:, 0] = -200.0
    x[:, 1] = 200.0
    x[:, 2] = -88.0
    x[:, 3] = -1e30
    x[:, 4] = 0.0
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128)
    check_fused(got, want, 1, False)
    assert (got[0].cpu().view(torch.uint8) & 0x7F).max() < 0x7F


def test_swiglu_empty():
    tk = _tk()
    x = torch.empty((0, 512), dtype=torch.bfloat16, device='cuda')
    c, s = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    assert c.shape == (0, 256) and s.shape == (0, 2)
    c, s = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    assert c.shape == (0, 256) and s.shape == (0, 1) and s.dtype == torch.int32


@pytest.mark.parametrize('gate', [0.5, 3.0, -1.0])
def test_swiglu_rows_that_share_one_gate_value(gate):
    """Every element of a group is the same factor silu(gate) times its up value, so 448 * v / amax falls on exact rounding
    boundaries of E4M3 for many elements, and the last bit of the factor decides which way they go: the quotient
    gate / (1 + exp(-gate)) has to be the correctly rounded one (an uncorrected reciprocal-multiply puts 1e-3 of the codes on
    the other side for gates 0.5 and 3.0, ten times the budget)."""
    tk = _tk()
    R, H = 2048, 2048
    g = torch.Generator().manual_seed(5)
    x = torch.cat([torch.full((R, H), gate), torch.randn((R, H), generator=g)], 1).to(torch.bfloat16)
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', 128)
    check_fused(got, want, H // 128, False, f'gate {gate} everywhere')
