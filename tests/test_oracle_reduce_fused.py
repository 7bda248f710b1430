"""Pins of the oracle's reduce_fused (no GPU needed)."""
import numpy as np
import pytest
import torch

from oracle import cref, torch_ref


def _case(T, K, hidden, dtype, seed, drop=0.2):
    g = torch.Generator().manual_seed(seed)
    R = T * K + 5
    x = torch.randn((R, hidden), generator=g).to(dtype)
    perm = torch.randperm(R, generator=g)[: T * K].to(torch.int32).view(T, K)
    pos = torch.where(torch.rand((T, K), generator=g) < drop, torch.full_like(perm, -1), perm)
    w = torch.rand((T, K), generator=g)
    x_sf = torch.randn((R,), generator=g)
    return x, pos, w, x_sf


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_against_float64(dtype):
    x, pos, w, x_sf = _case(40, 6, 256, dtype, seed=0)
    got = torch_ref.reduce_fused((x, x_sf), w, pos).double()
    want = torch.zeros((40, 256), dtype=torch.float64)
    for k in range(6):
        live = (pos[:, k] >= 0).double().unsqueeze(1)
        src = pos[:, k].clamp(min=0).long()
        want += live * x[src].double() * (w[:, k].double() * x_sf[src].double()).unsqueeze(1)
    scale = (x.double().abs().max() * 6 * x_sf.abs().max()).item()
    tol = scale * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -20)
    assert (got - want).abs().max().item() <= tol


def test_order_and_single_rounding_against_libm_fmaf():
    """A naive loop: per token, per term in order, one fmaf per element (the C library's) -- same bits."""
    x, pos, w, x_sf = _case(9, 5, 256, torch.float32, seed=1)
    got = torch_ref.reduce_fused((x, x_sf), w, pos)
    want = torch.zeros((9, 256))
    for t in range(9):
        acc = np.zeros(256, dtype=np.float32)
        for k in range(5):
            p = int(pos[t, k])
            if p < 0:
                continue
            s = (w[t, k] * x_sf[p]).expand(256).contiguous()      # one fp32 product
            acc = cref.fmaf(x[p].numpy(), s.numpy(), acc)
        want[t] = torch.from_numpy(acc)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    # the order matters: accumulating the terms backwards gives other bits somewhere
    back = torch_ref.reduce_fused((x, x_sf), w.flip(1), pos.flip(1))
    assert not torch.equal(got, back)


def test_hand_cases():
    x = torch.tensor([[1.0] * 256, [2.0] * 256, [4.0] * 256])
    pos = torch.tensor([[0, 2], [-1, 1], [-1, -1]], dtype=torch.int32)
    w = torch.tensor([[0.5, 0.25], [8.0, 3.0], [1.0, 1.0]])
    assert torch_ref.reduce_fused(x, w, pos)[:, 0].tolist() == [1.5, 6.0, 0.0]                 # skipped positions add nothing
    assert torch_ref.reduce_fused(x, None, pos)[:, 0].tolist() == [5.0, 2.0, 0.0]              # no weights: factor 1
    x_sf = torch.tensor([2.0, 10.0, -1.0])
    assert torch_ref.reduce_fused((x, x_sf), w, pos)[:, 0].tolist() == [0.0, 60.0, 0.0]        # 1*0.5*2 + 4*0.25*(-1)
    out = torch_ref.reduce_fused(x, w, pos, 'e4m3', torch.tensor([100.0]))
    assert out.dtype == torch.float8_e4m3fn and out.float()[[0, 2], 0].tolist() == [144.0, 0.0]     # 150 -> nearest E4M3 (144, step 16)
    assert torch_ref.reduce_fused(x.bfloat16(), w, pos).dtype == torch.bfloat16
    assert torch_ref.reduce_fused(x, w, pos[:0]).shape == (0, 256)


def test_rounding_to_the_output_types():
    x = torch.tensor([[1.0 + 2.0 ** -9] * 256])                 # not a bf16 number, not an E4M3 number
    pos = torch.tensor([[0]], dtype=torch.int32)
    assert torch_ref.reduce_fused(x.bfloat16(), None, pos).float()[0, 0].item() == 1.0       # input rounding
    assert torch_ref.reduce_fused(x, None, pos, 'e4m3').float()[0, 0].item() == 1.0
    # the E4M3 neighbours of 1 are 1.0 and 1.125, midpoint 1.0625: 1.00195 * 1.06 = 1.06207 goes down, * 1.0625 = 1.06458 goes up
    assert torch_ref.reduce_fused(x, None, pos, 'e4m3', torch.tensor([1.06])).float()[0, 0].item() == 1.0
    assert torch_ref.reduce_fused(x, None, pos, 'e4m3', torch.tensor([1.0625])).float()[0, 0].item() == 1.125


def test_no_live_position_at_all():
    """Every pair dropped: the expanded tensor has no rows and the result is zeros."""
    x = torch.empty((0, 256), dtype=torch.bfloat16)
    t2p = torch.full((3, 2), -1, dtype=torch.int32)
    out = torch_ref.reduce_fused(x, torch.rand((3, 2)), t2p)
    assert out.shape == (3, 256) and out.dtype == torch.bfloat16 and torch.all(out == 0)
