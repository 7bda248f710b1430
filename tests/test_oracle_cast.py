"""Pins block geometry, partial blocks, scale layouts and the SwiGLU formula of the CPU oracle,
and cross-checks its two independent statements (torch and scalar C) bit for bit.  No GPU."""
import itertools

import numpy as np
import pytest
import torch

from oracle import cref, torch_ref

F32 = np.float32


def naive_cast(x: torch.Tensor, fmt: str, bm: int, bk: int, round_sf: bool):
    """Double loop over blocks with numpy float32 scalars; encoders by table search."""
    xf = x.to(torch.float32).numpy()
    M, K = xf.shape
    qmax, floor = (F32(448), F32(1e-4)) if fmt == 'e4m3' else (F32(6), F32(6.0 * 2.0 ** -126))
    table = (torch.arange(127, dtype=torch.uint8).view(torch.float8_e4m3fn).double().numpy()
             if fmt == 'e4m3' else np.array(torch_ref.E2M1_VALUES))
    nm, nk = -(-M // bm), -(-K // bk)
    sf = np.zeros((nm, nk), F32)
    code = np.zeros((M, K), np.uint8)
    for i in range(nm):
        for j in range(nk):
            blk = xf[i * bm:(i + 1) * bm, j * bk:(j + 1) * bk]
            a = max(F32(np.abs(blk).max()), floor)
            s = F32(a) / qmax
            if round_sf:
                m, e = np.frexp(np.float64(s))        # s = m * 2^e, m in [0.5, 1)
                s = F32(2.0 ** (e - 1 if m == 0.5 else e))
                inv = F32(1) / s
            else:
                inv = qmax / F32(a)
            sf[i, j] = s
            q = (blk * inv).astype(F32)
            aq = np.minimum(np.abs(q.astype(np.float64)), float(qmax))
            d = np.abs(aq[..., None] - table)
            lo = d.argmin(-1)
            hi = table.size - 1 - d[..., ::-1].argmin(-1)
            c = np.where(lo % 2 == 0, lo, hi).astype(np.uint8)
            c |= (np.signbit(q).astype(np.uint8) << (7 if fmt == 'e4m3' else 3))
            code[i * bm:(i + 1) * bm, j * bk:(j + 1) * bk] = c
    if fmt == 'e2m1':
        code = code[:, 0::2] | (code[:, 1::2] << 4)
    return code, sf


@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('shape,blk', [((5, 192), (1, 128)), ((5, 192), (128, 128)), ((70, 96), (32, 32)),
                                        ((3, 64), (1, 64)), ((130, 192), (128, 128)), ((7, 48), (1, 16))])
@pytest.mark.parametrize('round_sf', [False, True])
def test_cast_matches_naive_loop_on_tiny_inputs(fmt, shape, blk, round_sf):
    x = (torch.randn(shape) * 3).to(torch.bfloat16)
    x[0, 0] = 0
    want_c, want_s = naive_cast(x, fmt, blk[0], blk[1], round_sf)
    c, s = torch_ref.cast(x, fmt, blk, round_sf=round_sf)
    assert np.array_equal(c.view(torch.uint8).numpy(), want_c)
    assert np.array_equal(s.numpy(), want_s)
    c2, s2 = cref.cast(x, fmt, blk, round_sf=round_sf)
    assert np.array_equal(c2.numpy(), want_c) and np.array_equal(s2.numpy(), want_s)


@pytest.mark.parametrize('fmt,blk,dtype,round_sf', [
    (f, b, d, r) for f, b, d, r in itertools.product(
        ['e4m3', 'e2m1'], [(1, 128), (1, 32), (1, 64), (1, 16), (128, 128), (32, 32), (1, 576)],
        [torch.bfloat16, torch.float32], [False, True])])
def test_torch_and_c_statements_agree_bitwise(fmt, blk, dtype, round_sf):
    x = torch.randn((301, 576), dtype=torch.float32)
    x[torch.rand_like(x) < 0.002] *= 100
    x[17] = 0
    x = (x * 10.0 ** float(torch.randint(-6, 6, (1,)))).to(dtype)
    c, s = torch_ref.cast(x, fmt, blk, round_sf=round_sf)
    c2, s2 = cref.cast(x, fmt, blk, round_sf=round_sf)
    assert torch.equal(c.view(torch.uint8), c2)
    assert torch.equal(s.view(torch.int32), s2.view(torch.int32))
    # caller-supplied scales, including ones that force saturation
    given = s * torch.where(torch.rand_like(s) < 0.3, 0.25, 1.0)
    g1 = torch_ref.cast(x, fmt, blk, sf=given)
    g2 = cref.cast(x, fmt, blk, sf=given)
    assert torch.equal(g1.view(torch.uint8), g2)
    if fmt == 'e4m3':
        assert (g1.view(torch.uint8) & 0x7F).max() <= 0x7E      # clamp, never NaN


def test_row_stride_is_honoured_by_the_c_statement():
    big = torch.randn((33, 512)).to(torch.bfloat16)
    x = big[:, :256]
    c, s = torch_ref.cast(x, 'e4m3', (1, 128))
    c2, s2 = cref.cast(x, 'e4m3', (1, 128))
    assert torch.equal(c.view(torch.uint8), c2) and torch.equal(s, s2)


@pytest.mark.parametrize('M,K,blk', [(5, 640, (1, 128)), (8, 576, (1, 128)), (130, 256, (128, 128)), (4001 // 40, 576, (32, 32)),
                                     (7, 7168, (1, 32))])
def test_scale_layouts(M, K, blk):
    x = torch.randn((M, K)).to(torch.bfloat16)
    nm, nk = -(-M // blk[0]), -(-K // blk[1])
    ld = -(-nm // 4) * 4
    _, row = torch_ref.cast(x, 'e4m3', blk, round_sf=True)
    assert row.shape == (nm, nk) and row.is_contiguous() and row.dtype == torch.float32
    _, col = torch_ref.cast(x, 'e4m3', blk, round_sf=True, use_tma_aligned_col_major_sf=True)
    assert col.shape == (nm, nk) and col.stride() == (1, ld) and torch.equal(col, row)
    _, pk = torch_ref.cast(x, 'e4m3', blk, round_sf=True, use_tma_aligned_col_major_sf=True, use_packed_ue8m0=True)
    nw = -(-nk // 4)
    assert pk.dtype == torch.int32 and pk.shape == (nm, nw) and pk.stride() == (1, ld)
    by = torch.empty((nm, nw), dtype=torch.int32).copy_(pk).view(torch.uint8).reshape(nm, nw * 4)
    assert torch.equal(by[:, :nk].to(torch.int32), row.view(torch.int32) >> 23)
    assert torch.all(by[:, nk:] == 0)
    # round trip through the dequantiser in all three layouts
    codes, _ = torch_ref.cast(x, 'e4m3', blk, round_sf=True)
    a = torch_ref.cast_back((codes, row), 'fp32', blk)
    assert torch.equal(a, torch_ref.cast_back((codes, col), 'fp32', blk))
    assert torch.equal(a, torch_ref.cast_back((codes, pk), 'fp32', blk))
    assert (a - x.float()).abs().max() <= x.float().abs().max() * 2 ** -3


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('M', [1, 6, 37])
def test_single_column_of_column_major_scales_keeps_the_kernel_path_strides(M, packed):
    """One block along the row: the scale tensor is [M, 1] with strides (1, round_up(M, 4)), as the reference's kernel
    path returns it (a transposed view of [1, round_up(M, 4)] storage), not the (1, 1) that its torch statement's
    `.T.contiguous().T` leaves for a single column."""
    x = torch.randn((M, 128)).to(torch.bfloat16)
    _, sf = torch_ref.cast(x, 'e4m3', (1, 128), round_sf=True, use_tma_aligned_col_major_sf=True, use_packed_ue8m0=packed)
    assert tuple(sf.shape) == (M, 1) and sf.stride() == (1, (M + 3) // 4 * 4)
    assert sf.dtype == (torch.int32 if packed else torch.float32)
    _, row = torch_ref.cast(x, 'e4m3', (1, 128), round_sf=True)
    if packed:
        assert torch.equal(sf.flatten() & 0xFF, (row.view(torch.int32).flatten() >> 23))
    else:
        assert torch.equal(sf.flatten(), row.flatten())


def test_empty_input_shapes():
    x = torch.empty((0, 256), dtype=torch.bfloat16)
    c, s = torch_ref.cast(x, 'e4m3', (1, 128))
    assert c.shape == (0, 256) and c.dtype == torch.float8_e4m3fn and s.shape == (0, 2)
    c, s = torch_ref.cast(x, 'e2m1', (1, 32), round_sf=True, use_tma_aligned_col_major_sf=True, use_packed_ue8m0=True)
    assert c.shape == (0, 128) and c.dtype == torch.int8 and s.shape == (0, 2) and s.dtype == torch.int32
    c, s = torch_ref.cast(x, 'e4m3', (1, 128), use_tma_aligned_col_major_sf=True)
    assert s.shape == (0, 2) and s.dtype == torch.float32


def test_requantising_a_quantised_input():
    x = torch.randn((64, 256)).to(torch.bfloat16)
    q = torch_ref.cast(x, 'e4m3', (32, 32), round_sf=True)
    deq = torch_ref.cast_back(q, 'fp32', (32, 32))
    a = torch_ref.cast(q, 'e2m1', (1, 32), x_block_size=(32, 32), round_sf=True)
    b = torch_ref.cast(deq, 'e2m1', (1, 32), round_sf=True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


# ---------------------------------------------------------------- SwiGLU

def test_swiglu_formula_against_float64_and_silu():
    x = torch.randn((64, 512)).to(torch.bfloat16)
    v = torch_ref.swiglu_forward(x)
    g, u = x[:, :256].double(), x[:, 256:].double()
    exact = g / (1 + torch.exp(-g)) * u
    assert v.dtype == torch.float32 and v.shape == (64, 256)
    rel = ((v.double() - exact).abs() / exact.abs().clamp(min=1e-30)).max()
    assert rel < 4 * 2 ** -23
    alt = torch.nn.functional.silu(x[:, :256].float()) * x[:, 256:].float()
    assert ((v - alt).abs() <= 4 * 2 ** -23 * alt.abs() + 1e-30).all()
    # gate and up are not interchangeable: catches a swapped operand
    assert not torch.allclose(v, torch_ref.swiglu_forward(torch.cat([x[:, 256:], x[:, :256]], 1)))
    # C statement: same formula, libm exp instead of torch's vectorised exp
    vc = cref.swiglu_forward(x)
    assert ((v - vc).abs() <= 2 * 2 ** -23 * v.abs()).all()


def test_swiglu_special_values():
    x = torch.tensor([[0.0, -200.0, 200.0, 1.0, 3.0, 3.0, 3.0, -2.0]], dtype=torch.float32)
    v = torch_ref.swiglu_forward(x)
    assert v[0, 0] == 0 and v[0, 1] == 0 and torch.signbit(v[0, 1] * -1) is not None
    assert v[0, 2] == 600.0                                  # exp(-200) underflows: silu(200) = 200
    assert abs(v[0, 3].item() - (-2.0 / (1 + np.exp(-1.0)))) < 1e-6
    vc = cref.swiglu_forward(x)
    assert torch.equal(vc[0, :3], v[0, :3])


def test_swiglu_clamp_counts_and_weights():
    x = (torch.randn((40, 256)) * 4).to(torch.bfloat16)
    cnt = torch.tensor([5, 6, 7], dtype=torch.int64)
    cnt_c = cnt.clone()
    pos = torch.arange(40, dtype=torch.int32) * 2 % 24
    pos[3] = -1
    pos[11] = -1
    w = torch.rand((6, 4))
    v = torch_ref.swiglu_forward(x, pos, w, 2.0, cnt)
    g, u = x[:, :128].float(), x[:, 128:].float()
    assert cnt.tolist() == [5 + int((g > 2).sum()), 6 + int((u > 2).sum()), 7 + int((u < -2).sum())]
    gc, uc = g.clamp(max=2.0), u.clamp(-2.0, 2.0)
    want = gc / (1 + torch.exp(-gc)) * uc
    wr = torch.where(pos >= 0, w.reshape(-1)[pos.clamp(min=0).long()], torch.zeros(()))
    assert torch.equal(v, want * wr[:, None])
    assert torch.all(v[3] == 0) and torch.all(v[11] == 0)
    vc = cref.swiglu_forward(x, pos, w, 2.0, cnt_c)
    assert cnt_c.tolist() == cnt.tolist()
    assert ((v - vc).abs() <= 2 * 2 ** -23 * v.abs()).all()


def test_fused_composition_masks_rows_and_keeps_layout():
    x = torch.randn((37, 512)).to(torch.bfloat16)
    pe = torch.randint(0, 4, (37,), dtype=torch.int32)
    pe[[2, 9, 36]] = -1
    c, s = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pe)
    assert c.shape == (37, 256) and s.shape == (37, 2)
    assert torch.all(c.view(torch.uint8)[pe < 0] == 0) and torch.all(s[pe < 0] == 0)
    live = pe >= 0
    c0, s0 = torch_ref.cast(torch_ref.swiglu_forward(x), 'e4m3', (1, 128))
    assert torch.equal(c.view(torch.uint8)[live], c0.view(torch.uint8)[live]) and torch.equal(s[live], s0[live])
    c, s = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pe, round_sf=True,
                                                       use_tma_aligned_col_major_sf=True, use_packed_ue8m0=True)
    assert s.dtype == torch.int32 and s.stride() == (1, 40) and torch.all(s[pe < 0] == 0)
    # custom amax floor
    c, s = torch_ref.swiglu_forward_and_per_token_cast(torch.zeros((2, 256), dtype=torch.bfloat16), 'e4m3', 128, sf_clamp_min=448.0)
    assert torch.all(s == 1.0)
