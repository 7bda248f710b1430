"""GPU parity of the per-token and per-block casts against the CPU oracle: codes and scales are
bit-exact, scale tensors have the reference's dtype/shape/strides.  Structure follows the
reference's tests/quant/test_per_token_cast.py and tests/quant/test_per_block_cast.py."""
import numpy as np
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same, packed_sf_bytes

pytestmark = pytest.mark.gpu

SF_MODES = [(False, False, False), (False, True, False), (True, False, False), (True, True, False), (True, True, True)]


def _mode_id(m):
    return 'col%d-round%d-packed%d' % tuple(int(v) for v in m)


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _rand(shape, dtype, outliers=True):
    x = torch.randn(shape, dtype=torch.float32)
    if outliers and x.numel():
        x[torch.rand(shape) < 0.002] *= 100
        x[x.shape[0] // 2] = 0              # an all-zero row: amax floor
    return x.to(dtype)


@pytest.mark.parametrize('mode', SF_MODES, ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'f32'])
@pytest.mark.parametrize('M,K,N', [
    (401, 7168, 128), (401, 7168, 32), (37, 576, 128), (37, 576, 64), (37, 576, 32), (37, 576, 16), (37, 576, 576),
    (1, 128, 128), (5, 64, 64), (16, 2048, 2048), (130, 2560, 128), (19, 3072, 3072), (64, 512, 128), (3, 4096, 16), (70, 5632, 128), (70, 6656, 32),
])
def test_per_token_cast(M, K, N, dtype, fmt, mode):
    tk = _tk()
    col, rnd, packed = mode
    x = _rand((M, K), dtype)
    xg = x.cuda()
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    codes, sf = tk.quant.per_token_cast(xg, fmt, N, **kw)
    codes_ref, sf_ref = torch_ref.cast(x, fmt, (1, N), **kw)
    assert_same(codes, codes_ref, 'codes')
    assert_same(sf, sf_ref, 'sf')

    # dequantised values are unbiased around the input
    back = torch_ref.cast_back((codes.cpu(), sf.cpu()), 'fp32', (1, N))
    if fmt == 'e4m3' and M * K >= 4096:
        tk.testing.check_bias(back, x.float())

    whole_row = N == K and N not in (16, 32, 64, 128)
    # row stride larger than K
    if not packed:
        wide = torch.randn((M, 2 * K), dtype=dtype, device='cuda')[:, :K]
        wide.copy_(xg)
        c2, s2 = tk.quant.per_token_cast(wide, fmt, N, **kw)
        assert_same(c2, codes_ref, 'codes (strided input)')
        assert_same(s2, sf_ref, 'sf (strided input)')
    if not whole_row:
        only = tk.quant.per_token_cast_with_sf_only(xg, fmt, N, **kw)
        assert_same(only, sf_ref, 'sf-only')
        if not col:
            c3 = tk.quant.per_token_cast_with_precomputed_sf(xg, fmt, N, sf=sf, **kw)
            c3_ref = torch_ref.cast(x, fmt, (1, N), sf=sf_ref, **kw)
            assert_same(c3, c3_ref, 'codes from given sf')


@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
def test_per_token_cast_given_sf_saturates(fmt):
    """Scales that are too small push values past the format's maximum: they clamp, never NaN."""
    tk = _tk()
    x = _rand((33, 512), torch.float32)
    _, sf_ref = torch_ref.cast(x, fmt, (1, 128))
    small = sf_ref * torch.where(torch.rand_like(sf_ref) < 0.5, 0.125, 1.0)
    got = tk.quant.per_token_cast_with_precomputed_sf(x.cuda(), fmt, 128, sf=small.cuda())
    assert_same(got, torch_ref.cast(x, fmt, (1, 128), sf=small), 'saturating codes')


@pytest.mark.parametrize('mode', SF_MODES, ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'f32'])
@pytest.mark.parametrize('M,K,block', [
    (401, 2048, (128, 128)), (401, 576, (128, 128)), (401, 576, (32, 32)), (130, 7168, (32, 32)), (1, 64, (128, 128)),
    (257, 2560, (32, 128)), (257, 2560, (128, 32)), (128, 128, (128, 128)), (33, 64, (32, 32)),
])
def test_per_block_cast(M, K, block, dtype, fmt, mode):
    tk = _tk()
    col, rnd, packed = mode
    x = _rand((M, K), dtype)
    xg = x.cuda()
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    codes, sf = tk.quant.per_block_cast(xg, fmt, block, **kw)
    codes_ref, sf_ref = torch_ref.cast(x, fmt, block, **kw)
    assert_same(sf, sf_ref, 'sf')
    assert_same(codes, codes_ref, 'codes')
    if fmt == 'e4m3' and M * K >= 4096:
        tk.testing.check_bias(torch_ref.cast_back((codes.cpu(), sf.cpu()), 'fp32', block), x.float())
    only = tk.quant.per_block_cast_with_sf_only(xg, fmt, block, **kw)
    assert_same(only, sf_ref, 'sf-only')
    if not col:
        c3 = tk.quant.per_block_cast_with_precomputed_sf(xg, fmt, block, sf=sf, **kw)
        assert_same(c3, torch_ref.cast(x, fmt, block, sf=sf_ref, **kw), 'codes from given sf')


@pytest.mark.parametrize('mode', [(False, False, False), (True, True, True)], ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize('M,K,block', [(4096, 2048, (128, 128)), (3968, 2560, (32, 32)), (4230, 2048, (128, 32)), (2048, 4096, (32, 128))])
def test_per_block_cast_wide_tiles(M, K, block, dtype, fmt, mode):
    """Matrices of 512 to 1280 tiles of 128 x 128 whose width is a multiple of 512 take tiles of 128 x 512, whose lane
    pairs exchange codes and store 16 consecutive ones (8 bytes of FP4) each; a ragged last row of tiles takes the other path."""
    tk = _tk()
    col, rnd, packed = mode
    x = _rand((M, K), dtype)
    xg = x.cuda()
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    codes, sf = tk.quant.per_block_cast(xg, fmt, block, **kw)
    codes_ref, sf_ref = torch_ref.cast(x, fmt, block, **kw)
    assert_same(sf, sf_ref, 'sf')
    assert_same(codes, codes_ref, 'codes')
    if not col:
        c3 = tk.quant.per_block_cast_with_precomputed_sf(xg, fmt, block, sf=sf * 0.5, **kw)     # half the scale: values saturate
        assert_same(c3, torch_ref.cast(x, fmt, block, sf=sf_ref * 0.5, **kw), 'codes from given sf')


def _all_bf16_as_f32():
    v = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    return torch.from_numpy(v[np.isfinite(v)].copy())


@pytest.mark.parametrize('scale', [1.0, 448.0 / 3.7, 37.3, 2.0 ** -7, 1.0 / 448.0])
def test_device_e4m3_conversion_over_every_bf16_value(scale):
    """The hardware fp32 -> E4M3 conversion (with the clamp) against the oracle for every finite bf16
    value times a scale, plus every rounding boundary of the format and its fp32 neighbours."""
    tk = _tk()
    tab = torch.arange(127, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    mids = (tab[:-1] + tab[1:]) / 2
    pts = torch.cat([tab, mids])
    pts = torch.cat([pts, torch.nextafter(pts, torch.tensor(float('inf'))), torch.nextafter(pts, torch.tensor(-1.0)),
                     torch.tensor([448.0 * (1 + 2 ** -23), 463.9, 464.0, 465.0, 1e30, 3e38])])
    v = torch.cat([_all_bf16_as_f32() * scale, pts, -pts])
    v = v[torch.isfinite(v)]
    n = (v.numel() + 127) // 128 * 128
    x = torch.zeros(n)
    x[: v.numel()] = v
    x = x.view(-1, 128)
    ones = torch.ones((x.shape[0], 1))
    got = tk.quant.per_token_cast_with_precomputed_sf(x.cuda(), 'e4m3', 128, sf=ones.cuda())
    assert_same(got, torch_ref.cast(x, 'e4m3', (1, 128), sf=ones), 'e4m3 codes')


def test_device_e2m1_conversion_at_every_boundary():
    tk = _tk()
    tab = torch.tensor(torch_ref.E2M1_VALUES)
    mids = (tab[:-1] + tab[1:]) / 2
    pts = torch.cat([tab, mids, torch.tensor([6.5, 7.0, 100.0, 1e30, 1e-30, 1e-40, 0.1, 0.2499])])
    pts = torch.cat([pts, torch.nextafter(pts, torch.tensor(float('inf'))), torch.nextafter(pts, torch.tensor(-1.0))])
    v = torch.cat([pts, -pts, _all_bf16_as_f32() * 0.37, torch.empty(100000).uniform_(-7, 7)])
    v = v[torch.isfinite(v)]
    n = (v.numel() + 31) // 32 * 32
    x = torch.zeros(n)
    x[: v.numel()] = v
    x = x.view(-1, 32)
    ones = torch.ones((x.shape[0], 1))
    got = tk.quant.per_token_cast_with_precomputed_sf(x.cuda(), 'e2m1', 32, sf=ones.cuda())
    assert_same(got, torch_ref.cast(x, 'e2m1', (1, 32), sf=ones), 'e2m1 codes')


@pytest.mark.parametrize('rnd', [False, True], ids=['exact_sf', 'round_sf'])
@pytest.mark.parametrize('fmt,N', [('e4m3', 128), ('e2m1', 32), ('e4m3', 32)])
def test_group_maxima_over_the_whole_exponent_range(fmt, N, rnd):
    """Group maxima from 2^-126 to 2^126: the scale divisions take their short forms between 2^-60 and 2^60 and the
    general ones outside, decided per wave, so groups of both kinds share waves here; codes and scales stay bit-exact."""
    tk = _tk()
    g = torch.Generator().manual_seed(11)
    K = 2048
    exps = torch.arange(-126, 127)
    rows = []
    for rep in range(3):
        k = exps[torch.randint(0, exps.numel(), (12, K // N), generator=g)]
        x = torch.randn((12, K), generator=g).clamp(-3, 3) * torch.exp2(k.float() - 2).repeat_interleave(N, dim=1)
        rows.append(x)
    # rows that stay inside the short-form range, rows that stay outside, and mixed ones (above)
    rows.append(torch.randn((8, K), generator=g) * 2.0 ** 40)
    rows.append(torch.randn((8, K), generator=g) * 2.0 ** -70)
    rows.append(torch.randn((8, K), generator=g).clamp(-3, 3) * 2.0 ** 100)
    x = torch.cat(rows)
    assert torch.isfinite(x).all()
    codes, sf = tk.quant.per_token_cast(x.cuda(), fmt, N, round_sf=rnd)
    codes_ref, sf_ref = torch_ref.cast(x, fmt, (1, N), round_sf=rnd)
    assert_same(sf, sf_ref, 'sf')
    assert_same(codes, codes_ref, 'codes')
    if N == 128 or fmt == 'e2m1':
        xb = x[: x.shape[0] // 128 * 128] if x.shape[0] >= 128 else torch.cat([x] * 4)[:128]
        cb, sb = tk.quant.per_block_cast(xb.cuda(), fmt, (N, N) if N == 128 else (32, 32), round_sf=rnd)
        cbr, sbr = torch_ref.cast(xb, fmt, (N, N) if N == 128 else (32, 32), round_sf=rnd)
        assert_same(sb, sbr, 'block sf')
        assert_same(cb, cbr, 'block codes')


def test_empty_inputs():
    tk = _tk()
    x = torch.empty((0, 256), dtype=torch.bfloat16)
    for kw in (dict(), dict(use_tma_aligned_col_major_sf=True), dict(use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)):
        for fmt in ('e4m3', 'e2m1'):
            c, s = tk.quant.per_token_cast(x.cuda(), fmt, 128, **kw)
            cr, sr = torch_ref.cast(x, fmt, (1, 128), **kw)
            assert c.shape == cr.shape and c.dtype == cr.dtype
            assert s.shape == sr.shape and s.dtype == sr.dtype
            c, s = tk.quant.per_block_cast(x.cuda(), fmt, (128, 128), **kw)
            cr, sr = torch_ref.cast(x, fmt, (128, 128), **kw)
            assert c.shape == cr.shape and s.shape == sr.shape and s.dtype == sr.dtype


def test_cpu_tensor_is_rejected_loudly():
    tk = _tk()
    with pytest.raises(Exception):
        tk.quant.per_token_cast(torch.zeros((4, 128), dtype=torch.bfloat16), 'e4m3', 128)


def test_packed_scales_read_back():
    """Packed UE8M0 words decode to the same powers of two as the fp32 rounded scales."""
    tk = _tk()
    x = _rand((70, 1536), torch.bfloat16).cuda()
    _, pk = tk.quant.per_token_cast(x, 'e2m1', 32, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    _, f = tk.quant.per_token_cast(x, 'e2m1', 32, round_sf=True)
    by = packed_sf_bytes(pk, 48)
    assert torch.equal((by.to(torch.int32) << 23).view(torch.float32), f.cpu())


def _to_gpu_like(t: torch.Tensor) -> torch.Tensor:
    """Copy to the GPU keeping the strides (column-major scale views are not dense)."""
    g = torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device='cuda')
    g.copy_(t)
    return g


@pytest.mark.parametrize('mode', [(False, True, False), (True, True, True), (True, True, False), (False, False, False)], ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('in_fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('x_block', [(128, 128), (32, 32), (1, 128), (1, 32)])
@pytest.mark.parametrize('M,K,N', [(401, 7168, 128), (401, 7168, 32), (37, 576, 128), (37, 576, 32), (130, 2048, 64), (131, 4096, 32),
                                   (7, 6144, 128)])
def test_per_token_cast_of_quantised_input(M, K, N, x_block, in_fmt, fmt, mode):
    """Input = (codes, scales) of an earlier cast, in every scale layout; same structure as the
    quantised-input cases of the reference's tests/quant/test_per_token_cast.py:25-36."""
    tk = _tk()
    col, rnd, packed = mode
    kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    x = torch.randn((M, K)).to(torch.bfloat16)
    q = torch_ref.cast(x, in_fmt, x_block, **kw)
    want_codes, want_sf = torch_ref.cast(q, fmt, (1, N), x_block_size=x_block, **kw)
    qg = (q[0].cuda(), _to_gpu_like(q[1]))
    codes, sf = tk.quant.per_token_cast(qg, fmt, N, x_block_size=x_block, **kw)
    assert_same(codes, want_codes, 'codes')
    assert_same(sf, want_sf, 'sf')


@pytest.mark.parametrize('fmt,N', [('e2m1', 32), ('e4m3', 128), ('e4m3', 32), ('e2m1', 64)])
@pytest.mark.parametrize('pad,shift', [(0, 0), (16, 0), (8, 0), (16, 8), (32, 16)])
def test_per_token_cast_of_strided_e4m3_codes(pad, shift, fmt, N):
    """E4M3 codes handed over as a view with a row stride of K + pad bytes starting `shift` bytes into the row: rows
    that are 16-byte aligned take the kernel with one 16-byte load per lane, the others the 8-byte one."""
    tk = _tk()
    M, K = 67, 4096
    x = torch.randn((M, K)).to(torch.bfloat16)
    q = torch_ref.cast(x, 'e4m3', (1, 128), round_sf=True)
    want_codes, want_sf = torch_ref.cast(q, fmt, (1, N), x_block_size=(1, 128), round_sf=True)
    wide = torch.zeros((M, K + pad), dtype=torch.uint8, device='cuda')
    view = wide[:, shift:shift + K].view(torch.float8_e4m3fn)
    view.view(torch.uint8).copy_(q[0].view(torch.uint8).cuda())
    assert view.stride(0) == K + pad and view.data_ptr() % 16 == shift % 16
    codes, sf = tk.quant.per_token_cast((view, q[1].cuda()), fmt, N, x_block_size=(1, 128), round_sf=True)
    assert_same(codes, want_codes, 'codes')
    assert_same(sf, want_sf, 'sf')


@pytest.mark.parametrize('out_fmt', ['bf16', 'fp32'])
@pytest.mark.parametrize('mode', [(False, False, False), (False, True, False), (True, True, False), (True, True, True)], ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('M,K,block', [(401, 7168, (1, 128)), (401, 7168, (1, 32)), (37, 576, (1, 64)), (130, 2048, (128, 128)),
                                       (257, 2560, (32, 32)), (19, 3072, (1, 3072)), (4096, 512, (1, 128)), (1, 64, (1, 64))])
def test_cast_back(M, K, block, fmt, mode, out_fmt):
    """Dequantisation against the oracle, bit for bit, every scale layout; structure follows the
    reference's tests/quant/test_cast_back.py."""
    tk = _tk()
    col, rnd, packed = mode
    x = _rand((M, K), torch.bfloat16)
    q = torch_ref.cast(x, fmt, block, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    want = torch_ref.cast_back(q, out_fmt, block)
    got = tk.quant.cast_back((q[0].cuda(), _to_gpu_like(q[1])), out_fmt, block)
    assert_same(got, want, 'dequantised')
    if block[0] == 1:
        assert_same(tk.quant.per_token_cast_back((q[0].cuda(), _to_gpu_like(q[1])), out_fmt, block[1]), want, 'per-token back')


@pytest.mark.parametrize('out_fmt', ['bf16', 'fp32'])
@pytest.mark.parametrize('mode', [(False, False, False), (True, False, False), (True, True, True)], ids=_mode_id)
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('M,K,block', [(257, 512, (128, 1)), (130, 192, (32, 2)), (64, 1088, (128, 4)), (300, 64, (1, 4)), (129, 2048, (128, 1))])
def test_cast_back_with_scale_blocks_narrower_than_a_lane(M, K, block, fmt, mode, out_fmt):
    """Scale blocks of 1, 2 or 4 columns (the per-channel 128 x 1 scales among them): a lane's 8 codes then carry 8, 4 or 2
    different scales, which a kernel of its own fetches; both code formats, every scale layout."""
    tk = _tk()
    col, rnd, packed = mode
    x = _rand((M, K), torch.bfloat16)
    q = torch_ref.cast(x, fmt, block, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=packed)
    want = torch_ref.cast_back(q, out_fmt, block)
    got = tk.quant.cast_back((q[0].cuda(), _to_gpu_like(q[1])), out_fmt, block)
    assert_same(got, want, 'dequantised')


def test_cast_then_cast_back_round_trip_on_device():
    tk = _tk()
    x = _rand((512, 4096), torch.bfloat16).cuda()
    q = tk.quant.per_token_cast(x, 'e4m3', 128, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    back = tk.quant.per_token_cast_back(q, 'fp32', 128)
    tk.testing.check_bias(back.cpu(), x.float().cpu())
    # with power-of-two scales the dequantised values are exact, so re-encoding them with the same
    # scales gives the same codes
    codes, sf = tk.quant.per_token_cast(x, 'e4m3', 128, round_sf=True)
    back = tk.quant.per_token_cast_back((codes, sf), 'fp32', 128)
    again = tk.quant.per_token_cast_with_precomputed_sf(back, 'e4m3', 128, sf=sf, round_sf=True)
    assert torch.equal(again.view(torch.uint8), codes.view(torch.uint8))
