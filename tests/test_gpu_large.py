"""Tensors with more than 2^31 elements (and more than 4 GiB): every operator's element offsets must be
64-bit.  The CPU oracle cannot evaluate such sizes in seconds, but all these operators are independent
from row to row (or from one 128-row block to the next), so windows of rows at the start, in the
middle and at the very end of the tensor are compared with the oracle run on just those rows, to the
same bar as the small cases (casts bit-exact, SwiGLU within its stated tolerance)."""
import pytest
import torch

from oracle import torch_ref
from tests._util import dense_bytes
from tests.test_gpu_swiglu import check_fused
from tests.test_gpu_swiglu_backward import check_backward

pytestmark = pytest.mark.gpu

LIMIT = 2 ** 31


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _windows(M, rows):
    """Row ranges of `rows` rows: first, one straddling the 2^31-element mark region (middle), last."""
    mid = (M // 2) // rows * rows
    return [(0, rows), (mid, mid + rows), (M - rows, M)]


def _randn_bf16(shape, seed):
    g = torch.Generator(device='cuda').manual_seed(seed)
    return torch.randn(shape, generator=g, device='cuda', dtype=torch.bfloat16)


def _same_bytes(got, want, what):
    g, w = dense_bytes(got.cpu()), dense_bytes(want)
    assert got.dtype == want.dtype and tuple(got.shape) == tuple(want.shape), what
    assert torch.equal(g, w), f'{what}: {(g != w).sum().item()} of {g.numel()} bytes differ'


@pytest.fixture(autouse=True)
def _release():
    yield
    torch.cuda.empty_cache()


def test_per_token_cast_and_cast_back_beyond_2g_elements():
    tk = _tk()
    M, K = 36000, 61440
    assert M * K > LIMIT
    x = _randn_bf16((M, K), 1)
    codes, sf = tk.quant.per_token_cast(x, 'e4m3', 128)
    back = tk.quant.cast_back((codes, sf), 'bf16', (1, 128))
    codes4, sf4 = tk.quant.per_token_cast(x, 'e2m1', 32, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    assert sf4.shape == (M, K // 128) and sf4.stride() == (1, M)
    for a, b in _windows(M, 16):
        xw = x[a:b].cpu()
        c_ref, s_ref = torch_ref.cast(xw, 'e4m3', (1, 128))
        _same_bytes(codes[a:b], c_ref, f'codes[{a}:{b}]')
        _same_bytes(sf[a:b], s_ref, f'sf[{a}:{b}]')
        _same_bytes(back[a:b], torch_ref.cast_back((c_ref, s_ref), 'bf16', (1, 128)), f'cast_back[{a}:{b}]')
        c_ref, s_ref = torch_ref.cast(xw, 'e2m1', (1, 32), use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
        _same_bytes(codes4[a:b], c_ref, f'e2m1 codes[{a}:{b}]')
        _same_bytes(sf4[a:b], s_ref, f'packed sf[{a}:{b}]')


def test_per_block_cast_beyond_2g_elements():
    tk = _tk()
    M, K = 282 * 128, 61440
    assert M * K > LIMIT
    x = _randn_bf16((M, K), 2)
    codes, sf = tk.quant.per_block_cast(x, 'e4m3', (128, 128))
    for a, b in _windows(M, 128):
        c_ref, s_ref = torch_ref.cast(x[a:b].cpu(), 'e4m3', (128, 128))
        _same_bytes(codes[a:b], c_ref, f'codes[{a}:{b}]')
        _same_bytes(sf[a // 128:b // 128], s_ref, f'sf[{a // 128}]')


def test_swiglu_forward_beyond_2g_elements():
    tk = _tk()
    R, H = 131200, 8192
    assert R * 2 * H > LIMIT
    x = _randn_bf16((R, 2 * H), 3)
    pe = torch.zeros((R,), dtype=torch.int32, device='cuda')
    pe[5::7] = -1
    codes, sf = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pe)
    for a, b in _windows(R, 32):
        xw, pw = x[a:b].cpu(), pe[a:b].cpu()
        want = torch_ref.swiglu_forward_and_per_token_cast(xw, 'e4m3', 128, pos_to_expert=pw)
        # padding rows: zeros on both sides (the oracle leaves them unwritten; its helper clears them)
        dead = pw < 0
        assert torch.all(codes[a:b].cpu().view(torch.uint8)[dead] == 0) and torch.all(sf[a:b].cpu()[dead] == 0)
        live = ~dead
        check_fused((codes[a:b][live.cuda()], sf[a:b][live.cuda()].contiguous()),
                    (want[0][live], want[1][live].contiguous()), H // 128, False, f'rows[{a}:{b}]')


def test_swiglu_backward_beyond_2g_elements():
    tk = _tk()
    R, H, N = 131200, 8192, 128
    assert R * 2 * H > LIMIT
    xq = tk.quant.per_token_cast(_randn_bf16((R, 2 * H), 4), 'e4m3', N)
    go = _randn_bf16((R, H), 5)
    # one routed copy per token: position r belongs to (token r, k = 0), so rows stay independent
    w = torch.rand((R, 1), device='cuda')
    ptt = torch.arange(R, dtype=torch.int32, device='cuda')
    t2p = ptt.view(R, 1).clone()
    out, xg_q, xg, wg = tk.quant.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, N)
    for a, b in _windows(R, 32):
        n = b - a
        idx = torch.arange(n, dtype=torch.int32)
        want = torch_ref.swiglu_backward_and_per_token_cast((xq[0][a:b].cpu(), xq[1][a:b].cpu()), go[a:b].cpu(), w[a:b].cpu(),
                                                            idx, idx.view(n, 1).clone(), N)
        got = (out[a:b], (xg_q[0][a:b], xg_q[1][a:b].contiguous()), xg[a:b], wg[a:b])
        check_backward(got, want, False, f'rows[{a}:{b}]')


@pytest.mark.parametrize('transpose', [False, True])
def test_per_channel_cast_beyond_2g_elements(transpose):
    tk = _tk()
    M, K = 282 * 128, 61440
    assert M * K > LIMIT
    x = _randn_bf16((M, K), 6)
    if transpose:
        codes, sf = tk.quant.per_channel_cast_and_transpose(x, 'e4m3', 128)
        assert codes.shape == (K, M)
        codes = codes.t()
    else:
        codes, sf = tk.quant.per_channel_cast(x, 'e4m3', 128)
    for a, b in _windows(M, 128):
        c_ref, s_ref = torch_ref.cast(x[a:b].cpu(), 'e4m3', (128, 1))
        _same_bytes(codes[a:b].contiguous(), c_ref, f'codes[{a}:{b}]')
        _same_bytes(sf[a // 128:b // 128], s_ref, f'sf[{a // 128}]')


def test_casts_of_e4m3_codes_beyond_2g_elements():
    """The two kernels that take E4M3 codes 16 to a lane: the re-quantisation to E2M1 and the per-channel cast."""
    tk = _tk()
    M, K = 282 * 128, 61440
    assert M * K > LIMIT
    x = _randn_bf16((M, K), 8)
    q = tk.quant.per_token_cast(x, 'e4m3', 128, round_sf=True)
    del x
    codes4, sf4 = tk.quant.per_token_cast(q, 'e2m1', 32, x_block_size=(1, 128), round_sf=True)
    codes8, sf8 = tk.quant.per_channel_cast_fused(q, 'e4m3', num_per_tokens=128, round_sf=True, num_per_channels=128)
    for a, b in _windows(M, 128):
        qw = (q[0][a:b].cpu(), q[1][a:b].cpu())
        c_ref, s_ref = torch_ref.cast(qw, 'e2m1', (1, 32), x_block_size=(1, 128), round_sf=True)
        _same_bytes(codes4[a:b], c_ref, f'e2m1 codes[{a}:{b}]')
        _same_bytes(sf4[a:b], s_ref, f'e2m1 sf[{a}:{b}]')
        c_ref, s_ref = torch_ref.per_channel_cast_fused(qw, 128, 128, True, None)
        _same_bytes(codes8[a:b], c_ref, f'per-channel codes[{a}:{b}]')
        _same_bytes(sf8[a // 128:b // 128], s_ref, f'per-channel sf[{a // 128}]')


def test_expand_to_fused_beyond_4_gib():
    tk = _tk()
    T, K, E, hidden = 36000, 8, 64, 8192
    g = torch.Generator().manual_seed(7)
    topk_idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
    topk_idx = topk_idx.masked_fill(torch.rand(topk_idx.shape, generator=g) < 0.05, -1).contiguous()
    p2e, p2t, _, t2p, *_ = tk.moe.get_fused_mapping(topk_idx.cuda(), E, 0, 16)
    x = _randn_bf16((T, hidden), 8)
    out = tk.moe.expand_to_fused(x, t2p, p2e)
    R = p2e.numel()
    assert out.shape == (R, hidden) and R * hidden * 2 > 2 ** 32
    # the mapping kernels are checked against the oracle elsewhere; here they define the expectation
    live = p2t >= 0
    want = x[p2t.clamp(min=0).long()]
    want[~live] = 0
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_more_row_tiles_than_one_grid_plane():
    """Wide and row-wise tiles put their row tiles on grid.y and grid.z, 32768 per plane: matrices with more row tiles
    than that (and a last plane that is not full) must give the same result as their halves cast separately, and the
    oracle's result on windows of rows."""
    tk = _tk()
    # per-token cast and its inverse: 2 rows per tile, two column tiles of 7 strips
    M, K = 2 * 32768 + 2 * 1200 + 1, 7168
    x = _randn_bf16((M, K), 11)
    codes, sf = tk.quant.per_token_cast(x, 'e4m3', 128)
    back = tk.quant.cast_back((codes, sf), 'bf16', (1, 128))
    h = 32768
    for a, b in [(0, h), (h, M)]:
        c2, s2 = tk.quant.per_token_cast(x[a:b], 'e4m3', 128)
        assert torch.equal(dense_bytes(codes[a:b].cpu()), dense_bytes(c2.cpu())) and torch.equal(sf[a:b], s2)
        assert torch.equal(back[a:b], tk.quant.cast_back((c2, s2), 'bf16', (1, 128)))
    for a, b in _windows(M, 9):
        c_ref, s_ref = torch_ref.cast(x[a:b].cpu(), 'e4m3', (1, 128))
        _same_bytes(codes[a:b], c_ref, f'codes[{a}:{b}]')
        _same_bytes(sf[a:b], s_ref, f'sf[{a}:{b}]')
        _same_bytes(back[a:b], torch_ref.cast_back((c_ref, s_ref), 'bf16', (1, 128)), f'back[{a}:{b}]')
    del x, codes, sf, back
    torch.cuda.empty_cache()
    # SwiGLU cast: 4 rows per tile, two column tiles of 2048 outputs; row-major and packed column-major scales
    R, H = 4 * 32768 + 4 * 700 + 3, 4096
    x = _randn_bf16((R, 2 * H), 12)
    for kw in (dict(), dict(use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)):
        got = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, **kw)
        for a, b in _windows(R, 8):
            want = torch_ref.swiglu_forward_and_per_token_cast(x[a:b].cpu(), 'e4m3', 128, **kw)
            part = tk.quant.swiglu_forward_and_per_token_cast(x[a:b].contiguous(), 'e4m3', 128, **kw)
            check_fused(part, want, H // 128, bool(kw), f'window [{a}:{b}] alone')
            assert torch.equal(dense_bytes(got[0][a:b].cpu()), dense_bytes(part[0].cpu())), f'codes[{a}:{b}] {kw}'


@pytest.mark.parametrize('dtype,H', [(torch.bfloat16, 4096), (torch.float32, 2048)], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('clamp', [None, 0.75])
def test_masked_swiglu_with_more_rows_than_one_grid_plane(dtype, H, clamp):
    """A masked batch in row-wise tiles runs one row per workgroup: with two columns of tiles and more than 32768 rows the
    grid gets a second, partly empty plane, whose surplus workgroups must leave without touching anything."""
    tk = _tk()
    R = 32768 + 1203
    g = torch.Generator(device='cuda').manual_seed(13)
    x = (torch.randn((R, 2 * H), generator=g, device='cuda') * 2).to(dtype)
    pe = torch.zeros((R,), dtype=torch.int32, device='cuda')
    pe[3::5] = -1
    guard = 64
    codes_buf = torch.full((R + guard, H), 0x5A, dtype=torch.uint8, device='cuda')
    kw = dict(swiglu_clamp_value=clamp)
    codes, sf = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pe, **kw)
    for a, b in [(0, 16), (32768 - 8, 32768 + 8), (R - 16, R)]:
        xw, pw = x[a:b].cpu(), pe[a:b].cpu()
        want = torch_ref.swiglu_forward_and_per_token_cast(xw, 'e4m3', 128, pos_to_expert=pw, **kw)
        dead = pw < 0
        assert torch.all(codes[a:b].cpu().view(torch.uint8)[dead] == 0) and torch.all(sf[a:b].cpu()[dead] == 0)
        live = ~dead
        check_fused((codes[a:b][live.cuda()], sf[a:b][live.cuda()].contiguous()),
                    (want[0][live], want[1][live].contiguous()), H // 128, False, f'rows[{a}:{b}]')
    # the same call through the C ABI into a buffer with guard rows behind it: nothing beyond row R is written
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    sf2 = torch.empty_like(sf)
    rc = lib.tk_swiglu_per_token_cast(x.data_ptr(), _ffi.dtype_code(x), R, H, codes_buf.data_ptr(), sf2.data_ptr(), H // 128, 128, 0, 0, -1.0,
                                      0, 0, 0, pe.data_ptr(), int(clamp is not None), float(clamp or 0.0), 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.equal(codes_buf[:R], codes.view(torch.uint8)) and torch.equal(sf2, sf)
    assert bool((codes_buf[R:] == 0x5A).all()), 'rows beyond the batch were written'
