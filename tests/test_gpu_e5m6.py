"""GPU parity of the E5M6 cast and its dequantisation against the CPU oracle, bit for bit (integer /
bit-pattern work after one fp32 product).  Structure follows the reference's
tests/quant/test_per_token_cast_to_e5m6.py and tests/quant/test_cast_back_e5m6.py, including its
special inputs (smallest and largest subnormal, smallest normal; tile_kernels/testing/generator.py:70-89)."""
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same

pytestmark = pytest.mark.gpu

SF_MODES = [(False, False, False), (False, True, False), (True, False, False), (True, True, False), (True, True, True)]
SPECIAL = (2.0 ** -20, 2.0 ** -14 * 63 / 64, 2.0 ** -14)


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _inputs(num_tokens, hidden, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    yield torch.randn((num_tokens, hidden), generator=g).to(dtype)
    # a wide spread of magnitudes inside a row: most elements land in the subnormal range of the format
    wide = torch.randn((num_tokens, hidden), generator=g) * torch.exp2(torch.randint(-30, 4, (num_tokens, hidden), generator=g).float())
    yield wide.to(dtype)
    for value in SPECIAL:
        x = torch.full((num_tokens, hidden), value, dtype=dtype)
        if num_tokens:
            x[:, -1] = 65024.0
        yield x


@pytest.mark.parametrize('mode', SF_MODES, ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'f32'])
@pytest.mark.parametrize('num_tokens,hidden', [(401, 576), (401, 2048), (130, 2560), (67, 7168), (5, 8), (3, 4104), (0, 512), (9, 11008), (7, 16384), (3, 16392)])
def test_per_token_cast_to_e5m6(num_tokens, hidden, dtype, mode):
    tk = _tk()
    col, rnd, packed = mode
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    for i, x in enumerate(_inputs(num_tokens, hidden, dtype, seed=hidden + num_tokens)):
        got = tk.quant.per_token_cast(x.cuda(), 'e5m6', hidden, **kw)
        want = torch_ref.cast_to_e5m6(x, hidden, **kw)
        assert got[0].dtype == torch.uint8 and tuple(got[0].shape) == (num_tokens, hidden * 3 // 2)
        assert_same(got[0], want[0], f'input {i}: codes')
        assert_same(got[1], want[1], f'input {i}: scales')


def test_per_token_cast_to_e5m6_strided_rows():
    tk = _tk()
    x = torch.randn((64, 2 * 1024), dtype=torch.bfloat16)
    got = tk.quant.per_token_cast(x.cuda()[:, :1024], 'e5m6', 1024, round_sf=True)
    want = torch_ref.cast_to_e5m6(x[:, :1024].contiguous(), 1024, round_sf=True)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


@pytest.mark.parametrize('out_fmt', ['bf16', 'fp32'])
@pytest.mark.parametrize('mode', [(False, True, False), (True, True, True), (False, False, False)],
                         ids=lambda m: 'col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('num_tokens,hidden', [(401, 576), (130, 2560), (67, 7168), (5, 8), (0, 512)])
def test_cast_back_e5m6(num_tokens, hidden, mode, out_fmt):
    tk = _tk()
    col, rnd, packed = mode
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    for i, x in enumerate(_inputs(num_tokens, hidden, torch.float32, seed=7 * hidden + num_tokens)):
        xq = torch_ref.cast_to_e5m6(x, hidden, **kw)
        want = torch_ref.cast_back_from_e5m6(xq, out_fmt, (1, hidden))
        got = tk.quant.cast_back((xq[0].cuda(), xq[1].cuda()), out_fmt, (1, hidden), x_special_fmt='e5m6')
        assert_same(got, want, f'input {i}')
        if num_tokens and i == 0:
            # 7 significant bits: the round trip stays within 2^-7 relative of the row's largest value
            err = (got.cpu().float() - x).abs().amax(dim=1)
            assert torch.all(err <= x.abs().amax(dim=1) * 2.0 ** -7)


def test_cast_back_e5m6_every_code_and_finer_scale_blocks():
    """All 4096 codes (infinities and NaNs included) through the unpacker, with 1 x 128 and 128 x 128 scale blocks."""
    tk = _tk()
    codes = torch.arange(4096, dtype=torch.int32).repeat(256, 1)[:, torch.randperm(4096, generator=torch.Generator().manual_seed(0))]
    packed = torch_ref.pack_e5m6(codes.contiguous())
    for blk in ((1, 128), (128, 128), (1, 4096)):
        sf = torch.exp2(torch.randint(-8, 8, (-(-256 // blk[0]), 4096 // blk[1]), generator=torch.Generator().manual_seed(blk[0])).float())
        want = torch_ref.cast_back_from_e5m6((packed, sf), 'fp32', blk)
        got = tk.quant.cast_back((packed.cuda(), sf.cuda()), 'fp32', blk, x_special_fmt='e5m6').cpu()
        same = (got.view(torch.int32) == want.view(torch.int32)) | (got.isnan() & want.isnan())
        assert bool(same.all()), f'block {blk}: {(~same).sum().item()} values differ'


def test_e5m6_round_trip_through_the_public_api():
    tk = _tk()
    x = torch.randn((512, 4096), dtype=torch.bfloat16, device='cuda')
    xq = tk.quant.per_token_cast(x, 'e5m6', 4096, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    back = tk.quant.per_token_cast_back(xq, 'bf16', 4096, x_special_fmt='e5m6')
    assert back.dtype == torch.bfloat16 and back.shape == x.shape
    tk.testing.check_bias(back.float().cpu(), x.float().cpu())
