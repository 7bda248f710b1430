"""Pins for the oracle's per-channel casts (oracle/torch_ref.per_channel_cast_fused and the two
transposing compositions).  The arithmetic of a block is the already pinned ``cast``; what is new
is the (N, 1) block geometry, the gather and the transposition, checked here against a naive
column loop, the scalar C restatement and hand-built index lists."""
import pytest
import torch

from oracle import cref, torch_ref


def _naive_per_channel(x: torch.Tensor, n: int, round_sf: bool):
    """Column by column, block by block, with scalar Python control flow."""
    xf = x.float()
    M, K = xf.shape
    nb = -(-M // n)
    codes = torch.zeros((M, K), dtype=torch.float8_e4m3fn)
    sf = torch.zeros((nb, K))
    for k in range(K):
        for b in range(nb):
            col = xf[b * n:(b + 1) * n, k]
            amax = max(float(col.abs().max()), 1e-4)
            a = torch.tensor(amax, dtype=torch.float32)
            s = a / torch.tensor(448.0)
            if round_sf:
                bits = (s.view(torch.int32) + 0x7FFFFF) & 0x7F800000
                s = bits.view(torch.float32)
                inv = 1.0 / s
            else:
                inv = torch.tensor(448.0) / a
            sf[b, k] = s
            codes[b * n:(b + 1) * n, k] = (col * inv).clamp(-448, 448).to(torch.float8_e4m3fn)
    return codes, sf


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('M,K,n', [(8, 5, 4), (12, 3, 4), (10, 4, 4), (64, 6, 32)])
def test_geometry_against_naive_column_loop(M, K, n, round_sf):
    g = torch.Generator().manual_seed(M * 31 + K)
    x = (torch.randn((M, K), generator=g) * torch.logspace(-2, 2, K)[None, :]).to(torch.bfloat16)
    codes, sf = torch_ref.cast(x, 'e4m3', (n, 1), round_sf=round_sf)
    codes_n, sf_n = _naive_per_channel(x, n, round_sf)
    assert tuple(sf.shape) == (-(-M // n), K)
    assert torch.equal(sf, sf_n)
    assert torch.equal(codes.view(torch.uint8), codes_n.view(torch.uint8))


@pytest.mark.parametrize('round_sf', [False, True])
@pytest.mark.parametrize('n', [32, 128])
def test_per_channel_torch_and_c_restatements_agree(n, round_sf):
    g = torch.Generator().manual_seed(n)
    x = (torch.randn((256, 192), generator=g) * 3).to(torch.bfloat16)
    x[:, 7] = 0                                   # an all-zero column: scale = floor / 448
    codes, sf = torch_ref.cast(x, 'e4m3', (n, 1), round_sf=round_sf)
    codes_c, sf_c = cref.cast(x, 'e4m3', (n, 1), round_sf=round_sf)
    assert torch.equal(codes.view(torch.uint8), codes_c)
    assert torch.equal(sf.view(torch.int32), sf_c.view(torch.int32))
    assert torch.all(codes.view(torch.uint8)[:, 7] == 0)


def test_gather_rows_and_zero_rows():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((6, 8), generator=g).to(torch.bfloat16)
    pos = torch.tensor([3, -1, 0, 0, 5, -1, 2, 1, -1, -1, -1, -1, 4, 4, 4, 4], dtype=torch.int32)
    codes, sf = torch_ref.per_channel_cast_fused(x, 128, None, False, pos)
    assert tuple(codes.shape) == (16, 8) and tuple(sf.shape) == (1, 8)
    rows = torch.stack([x[i] if i >= 0 else torch.zeros(8, dtype=torch.bfloat16) for i in pos.tolist()])
    want_codes, want_sf = torch_ref.cast(rows, 'e4m3', (128, 1))
    assert torch.equal(codes.view(torch.uint8), want_codes.view(torch.uint8)) and torch.equal(sf, want_sf)
    assert torch.all(codes.view(torch.uint8)[pos < 0] == 0)
    # the column maximum only sees the gathered rows: row 5's value never appears when it is not gathered
    pos2 = torch.tensor([0, 1, 2, 3] * 4, dtype=torch.int32)
    _, sf2 = torch_ref.per_channel_cast_fused(x, 128, None, False, pos2)
    assert torch.equal(sf2[0], x[:4].float().abs().amax(0).clamp(min=1e-4) / 448.0)


def test_gather_of_quantised_input():
    g = torch.Generator().manual_seed(2)
    x = torch.randn((8, 256), generator=g).to(torch.bfloat16)
    xq = torch_ref.cast(x, 'e4m3', (1, 128))
    pos = torch.tensor([7, 6, -1, 0, 1, 1, -1, 3] * 2, dtype=torch.int32)
    codes, sf = torch_ref.per_channel_cast_fused(xq, 128, 128, True, pos)
    deq = xq[0].float() * xq[1].repeat_interleave(128, dim=1)
    rows = torch.stack([deq[i] if i >= 0 else torch.zeros(256) for i in pos.tolist()])
    want_codes, want_sf = torch_ref.cast(rows, 'e4m3', (128, 1), round_sf=True)
    assert torch.equal(codes.view(torch.uint8), want_codes.view(torch.uint8)) and torch.equal(sf, want_sf)


def test_transposing_compositions():
    g = torch.Generator().manual_seed(3)
    x = torch.randn((128, 64), generator=g).to(torch.bfloat16)
    codes_t, sf_t = torch_ref.per_channel_cast_and_transpose(x, 32, False)
    codes, sf = torch_ref.cast(x, 'e4m3', (32, 1))
    assert tuple(codes_t.shape) == (64, 128) and codes_t.is_contiguous()
    assert torch.equal(codes_t.view(torch.uint8), codes.view(torch.uint8).T) and torch.equal(sf, sf_t)

    x2 = torch.randn((128, 128), generator=g).to(torch.bfloat16) * 3
    a, sa = torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(x2, 128, True, False, 0.5)
    b, sb = torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(x2, 128, True, True, 0.5)
    assert tuple(a.shape) == (64, 128) and tuple(b.shape) == (128, 64)
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8).T) and torch.equal(sa, sb)
    # the activation is rounded to bf16 before the cast: the scale is amax of the bf16 values
    act = torch_ref.swiglu_forward(x2, swiglu_clamp_value=0.5).to(torch.bfloat16).float()
    assert act.abs().max() <= 0.5 * 0.5 + 1e-6          # silu(g <= .5) * |u| <= .5 stays small
    want = act.abs().amax(0).clamp(min=1e-4) / 448.0
    bits = (want.view(torch.int32) + 0x7FFFFF) & 0x7F800000
    assert torch.equal(sa[0], bits.view(torch.float32))
