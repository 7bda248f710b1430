"""GPU parity of the per-channel cast family against the CPU oracle.

The plain, gathering, dequantising and transposing casts are integer-exact: codes, scales, dtype
and shape must match bit for bit.  The SwiGLU variant rounds the activation to bf16 before the cast,
so the CPU/GPU difference in exp shows only where a value sits on a bf16 rounding boundary: at most
0.01 % of the scales may differ (by one bf16 step of the column maximum, or one power of two with
round_sf), and outside those blocks at most 0.01 % of the codes, each by one E4M3 step.
Structure follows the reference's tests/quant/test_per_channel_cast*.py and
test_swiglu_forward_and_per_channel_cast_and_transpose.py.
"""
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same, dense_bytes, fp8_code_report

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    return tilekernels_amd


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('hidden', [576, 2048, 2560, 7168])
@pytest.mark.parametrize('num_tokens', [128, 4096])
def test_per_channel_cast(num_tokens, hidden, round_sf):
    tk = _tk()
    g = torch.Generator().manual_seed(hidden + num_tokens)
    x = torch.randn((num_tokens, hidden), generator=g).to(torch.bfloat16)
    want = torch_ref.cast(x, 'e4m3', (128, 1), round_sf=round_sf)
    got = tk.quant.per_channel_cast(x.cuda(), 'e4m3', 128, round_sf)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


def _moe_case(T, K, E, hidden, seed, alignment=128):
    g = torch.Generator().manual_seed(seed)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < 0.1, -1).contiguous()
    _, pos_to_token, *_ = torch_ref.get_fused_mapping(topk_idx, E, alignment)
    x = torch.randn((T, hidden), generator=g).to(torch.bfloat16)
    return x, pos_to_token


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('quantised', [False, True])
@pytest.mark.parametrize('hidden', [256, 2048, 7168])
@pytest.mark.parametrize('moe', [None, (1001, 6, 16, 128), (513, 2, 9, 16), (64, 1, 3, 16)])
def test_per_channel_cast_fused(moe, hidden, quantised, round_sf):
    tk = _tk()
    if moe is None:
        g = torch.Generator().manual_seed(hidden)
        x, pos = torch.randn((1024, hidden), generator=g).to(torch.bfloat16), None
    else:
        T, K, E, alignment = moe
        x, pos = _moe_case(T, K, E, hidden, seed=hidden + T, alignment=alignment)
        assert pos.numel() % 16 == 0
    xin = torch_ref.cast(x, 'e4m3', (1, 128)) if quantised else x
    want = torch_ref.per_channel_cast_fused(xin, 128, 128 if quantised else None, round_sf, pos)
    xg = (xin[0].cuda(), xin[1].cuda()) if quantised else xin.cuda()
    got = tk.quant.per_channel_cast_fused(xg, 'e4m3', num_per_tokens=128, round_sf=round_sf,
                                          num_per_channels=128 if quantised else None,
                                          pos_to_token=None if pos is None else pos.cuda())
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('num_per_tokens', [32, 128])
@pytest.mark.parametrize('hidden', [576, 2048, 3072, 7168])
@pytest.mark.parametrize('num_tokens', [128, 4096])
def test_per_channel_cast_and_transpose(num_tokens, hidden, num_per_tokens, round_sf):
    tk = _tk()
    g = torch.Generator().manual_seed(hidden + num_tokens + num_per_tokens)
    x = torch.randn((num_tokens, hidden), generator=g).to(torch.bfloat16)
    want = torch_ref.per_channel_cast_and_transpose(x, num_per_tokens, round_sf)
    got = tk.quant.per_channel_cast_and_transpose(x.cuda(), 'e4m3', num_per_tokens, round_sf)
    assert tuple(got[0].shape) == (hidden, num_tokens)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('hidden', [256, 2048, 7168])
@pytest.mark.parametrize('moe', [None, (513, 2, 9, 16)])
def test_per_channel_cast_fused_fp32_input(moe, hidden, round_sf):
    """fp32 input (tile_kernels/quant/common.py:84-88 admits it for the plain and the gathered cast)."""
    tk = _tk()
    if moe is None:
        g = torch.Generator().manual_seed(hidden + 1)
        x, pos = torch.randn((1024, hidden), generator=g), None
    else:
        T, K, E, alignment = moe
        x, pos = _moe_case(T, K, E, hidden, seed=hidden + T + 1, alignment=alignment)
        x = torch.randn(x.shape, generator=torch.Generator().manual_seed(hidden))      # full fp32 mantissas
    x[3, 5] = 3.0e38
    want = torch_ref.per_channel_cast_fused(x, 128, None, round_sf, pos)
    got = tk.quant.per_channel_cast_fused(x.cuda(), 'e4m3', num_per_tokens=128, round_sf=round_sf,
                                          pos_to_token=None if pos is None else pos.cuda())
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')
    if moe is None:
        got = tk.quant.per_channel_cast(x.cuda(), 'e4m3', 128, round_sf)
        assert_same(got[0], want[0], 'codes')
        assert_same(got[1], want[1], 'scales')


def check_swiglu_per_channel(got, want, npt, round_sf, transposed, what=''):
    codes, sf = got
    codes_ref, sf_ref = want
    assert codes.dtype == torch.float8_e4m3fn and tuple(codes.shape) == tuple(codes_ref.shape) and codes.is_contiguous()
    assert sf.dtype == torch.float32 and tuple(sf.shape) == tuple(sf_ref.shape) and sf.is_contiguous()
    a, b = sf.cpu(), sf_ref
    moved = a != b
    assert moved.float().mean().item() <= 1e-4, f'{what}: {int(moved.sum())} of {moved.numel()} scales differ'
    if moved.any():
        ratio = a[moved] / b[moved]
        if round_sf:
            assert bool(((ratio == 2) | (ratio == 0.5)).all())
        else:
            assert bool(((ratio - 1).abs() <= 2.0 ** -7).all())
    gc = codes.cpu().view(torch.uint8)
    wc = codes_ref.view(torch.uint8)
    if transposed:
        gc, wc = gc.T, wc.T                     # back to [tokens, hidden]
    keep = ~moved.repeat_interleave(npt, dim=0)
    frac, one = fp8_code_report(gc[keep], wc[keep])
    assert frac <= 1e-4 and one, f'{what}: {frac * 100:.5f}% codes differ, one-step={one}'


@pytest.mark.parametrize('clamp', [None, 10.0, 0.5])
@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('without_transpose', [False, True])
@pytest.mark.parametrize('num_per_tokens', [32, 128])
@pytest.mark.parametrize('hidden', [576, 2048, 7168])
def test_swiglu_forward_and_per_channel_cast_and_transpose(hidden, num_per_tokens, without_transpose, round_sf, clamp):
    tk = _tk()
    num_tokens = 1024 if hidden > 4096 else 4096
    g = torch.Generator().manual_seed(hidden + num_per_tokens)
    x = torch.randn((num_tokens, 2 * hidden), generator=g).to(torch.bfloat16)
    want = torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(x, num_per_tokens, round_sf, without_transpose, clamp)
    got = tk.quant.swiglu_forward_and_per_channel_cast_and_transpose(
        x.cuda(), 'e4m3', num_per_tokens=num_per_tokens, round_sf=round_sf, without_transpose=without_transpose,
        swiglu_clamp_value=clamp)
    check_swiglu_per_channel(got, want, num_per_tokens, round_sf, not without_transpose, f'hidden={hidden}')


def test_per_channel_cast_round_trip_bias():
    # dequantised per-channel codes stay within one E4M3 step of the input (the reference's check_bias idea)
    tk = _tk()
    x = torch.randn((256, 512), generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    codes, sf = tk.quant.per_channel_cast(x.cuda(), 'e4m3', 128)
    back = codes.cpu().float() * sf.cpu().repeat_interleave(128, dim=0)
    err = (back - x.float()).abs()
    assert bool((err <= 16.01 * sf.cpu().repeat_interleave(128, dim=0)).all())
    assert abs((back - x.float()).mean().item()) < 1e-3


def test_per_channel_no_rows():
    tk = _tk()
    x = torch.empty((0, 256), dtype=torch.bfloat16, device='cuda')
    codes, sf = tk.quant.per_channel_cast_fused(x, 'e4m3', 128)
    assert tuple(codes.shape) == (0, 256) and tuple(sf.shape) == (0, 256)
    codes, sf = tk.quant.per_channel_cast_and_transpose(x, 'e4m3', 32)
    assert tuple(codes.shape) == (256, 0) and tuple(sf.shape) == (0, 256)


@pytest.mark.parametrize('transpose', [False, True])
@pytest.mark.parametrize('quantised', [False, True])
def test_c_abi_combinations_the_wrappers_do_not_use(quantised, transpose):
    """tk_per_channel_cast takes every combination of its flags; the Python wrappers only use the ones the
    reference offers.  Here: 32 tokens per scale together with a gather whose length is 16 mod 32 (the
    last scale block is half full), with and without FP8 input and transposed output."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K, M = 200, 384, 16 * 21
    g = torch.Generator().manual_seed(11)
    x = torch.randn((T, K), generator=g).to(torch.bfloat16)
    pos = torch.randint(-1, T, (M,), generator=g, dtype=torch.int32)
    xin = torch_ref.cast(x, 'e4m3', (1, 128)) if quantised else x
    want_codes, want_sf = torch_ref.per_channel_cast_fused(xin, 32, 128 if quantised else None, False, pos)
    if transpose:
        want_codes = want_codes.T.contiguous()
    xd = xin[0].cuda() if quantised else xin.cuda()
    sfd = xin[1].cuda() if quantised else None
    posd = pos.cuda()
    out = torch.empty(tuple(want_codes.shape), dtype=torch.float8_e4m3fn, device='cuda')
    out_sf = torch.empty(tuple(want_sf.shape), dtype=torch.float32, device='cuda')
    rc = lib.tk_per_channel_cast(xd.data_ptr(), 0, _ffi.ptr(sfd), T, K, posd.data_ptr(), M, out.data_ptr(), out_sf.data_ptr(),
                                 32, 0, int(transpose), 0, 0, 0.0, _ffi.current_stream(out.device))
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert_same(out, want_codes, 'codes')
    assert_same(out_sf, want_sf, 'scales')


@pytest.mark.parametrize('x_shift,out_shift', [(0, 0), (8, 0), (0, 8), (8, 8)])
def test_fp8_input_with_buffers_that_are_only_8_byte_aligned(x_shift, out_shift):
    """The FP8-input cast moves 16 bytes per lane where its buffers allow it and 8 bytes otherwise: both give the oracle's result."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    T, K = 272, 1152
    g = torch.Generator().manual_seed(5)
    x = torch.randn((T, K), generator=g).to(torch.bfloat16)
    xin = torch_ref.cast(x, 'e4m3', (1, 128))
    want_codes, want_sf = torch_ref.per_channel_cast_fused(xin, 128, 128, True, None)
    xbuf = torch.zeros(T * K + 16, dtype=torch.uint8, device='cuda')
    xbuf[x_shift:x_shift + T * K].copy_(xin[0].view(torch.uint8).flatten().cuda())
    obuf = torch.zeros(T * K + 16, dtype=torch.uint8, device='cuda')
    sfd = xin[1].cuda()
    out_sf = torch.empty(tuple(want_sf.shape), dtype=torch.float32, device='cuda')
    rc = lib.tk_per_channel_cast(xbuf.data_ptr() + x_shift, 0, sfd.data_ptr(), T, K, None, T, obuf.data_ptr() + out_shift, out_sf.data_ptr(),
                                 128, 1, 0, 0, 0, 0.0, _ffi.current_stream(obuf.device))
    assert rc == 0, rc
    torch.cuda.synchronize()
    got = obuf[out_shift:out_shift + T * K].view(torch.float8_e4m3fn).reshape(T, K)
    assert_same(got, want_codes, 'codes')
    assert_same(out_sf, want_sf, 'scales')
    assert int(obuf[:out_shift].sum()) == 0 and int(obuf[out_shift + T * K:].sum()) == 0
