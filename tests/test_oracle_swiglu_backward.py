"""Pins for the oracle's SwiGLU backward (oracle/torch_ref.swiglu_backward, oracle/quant_ref.c).

None of these retypes the oracle's formula: the gradients are checked against float64 autograd of
``silu(g) * u * w``, the clamp rules against hand-built cases, the fused multiply-add helper against
the C library's ``fmaf`` on operands chosen to trigger double rounding, and the two independently
written restatements (torch, scalar C) against each other.
"""
import numpy as np
import pytest
import torch

from oracle import cref, torch_ref


def _make_case(seed, tokens=23, experts=6, topk=3, H=256, N=128, drop=0.2, scale=2.0):
    import tilekernels_amd as tk
    g = torch.Generator().manual_seed(seed)
    pe, ptt, w = tk.testing.generate_moe_layout(tokens, experts, topk, 8, g, drop_fraction=drop)
    R = pe.numel()
    x = torch.randn((R, 2 * H), generator=g) * scale
    x[pe < 0] = 0
    xq = torch_ref.cast(x.to(torch.bfloat16), 'e4m3', (1, N))
    go = torch.randn((R, H), generator=g).to(torch.bfloat16)
    t2p = torch.full((tokens * topk,), -1, dtype=torch.int32)
    live = ptt >= 0
    t2p[ptt[live].long()] = torch.arange(R, dtype=torch.int32)[live]
    return xq, go, w, ptt, t2p.view(tokens, topk)


def _autograd(xq, go, w, ptt, N, clamp):
    """float64 autograd of sum(grad_out * silu(g) * u * w_row) with torch's own clamp/sigmoid."""
    codes, sf = xq
    H = codes.shape[1] // 2
    xf = (codes.to(torch.float32) * sf.repeat_interleave(N, dim=1)).double()
    gate = xf[:, :H].clone().requires_grad_(True)
    up = xf[:, H:].clone().requires_grad_(True)
    wd = w.double().clone().requires_grad_(True)
    live = ptt >= 0
    w_row = torch.zeros(codes.shape[0], dtype=torch.float64)
    w_row = w_row.index_put((live.nonzero().squeeze(1),), wd.reshape(-1)[ptt[live].long()])
    gc, uc = gate, up
    if clamp is not None:
        gc = torch.clamp(gate, max=clamp)
        uc = torch.clamp(up, min=-clamp, max=clamp)
    act = torch.nn.functional.silu(gc) * uc
    out = act * w_row[:, None]
    (out * go.double()).sum().backward()
    return out.detach(), torch.cat([gate.grad, up.grad], dim=1), wd.grad


@pytest.mark.parametrize('clamp', [None, 10.0, 0.5])
@pytest.mark.parametrize('N', [32, 128])
def test_backward_matches_float64_autograd(N, clamp):
    xq, go, w, ptt, t2p = _make_case(11 + N, N=N)
    out, xg, wg = torch_ref.swiglu_backward(xq, go, w, ptt, t2p, N, clamp)
    out64, xg64, wg64 = _autograd(xq, go, w, ptt, N, clamp)
    assert out.dtype == xg.dtype == wg.dtype == torch.float32
    torch.testing.assert_close(out.double(), out64, rtol=2e-6, atol=1e-7)
    torch.testing.assert_close(xg.double(), xg64, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(wg.double(), wg64, rtol=1e-5, atol=1e-5)
    # the halves are not interchangeable and the gradient is not trivially zero
    H = go.shape[1]
    assert xg[:, :H].abs().max() > 0 and xg[:, H:].abs().max() > 0
    assert not torch.allclose(xg[:, :H], xg[:, H:])


def test_clamp_rules_on_hand_built_values():
    # one row, H = 128: gate/up values placed by hand around clamp = 2
    H, N, clamp = 128, 128, 2.0
    vals = torch.zeros((1, 2 * H))
    vals[0, 0], vals[0, H + 0] = 3.0, 1.0        # gate above the clamp: gate gradient 0, up gradient uses gate = 2
    vals[0, 1], vals[0, H + 1] = 1.0, 3.0        # up above: up gradient 0, up used as 2
    vals[0, 2], vals[0, H + 2] = 1.0, -3.0       # up below: up gradient 0, up used as -2
    vals[0, 3], vals[0, H + 3] = -3.0, 1.5       # gate far below: NOT clamped (one-sided)
    vals[0, 4], vals[0, H + 4] = 2.0, -2.0       # exactly at the clamp: not clamped, gradients flow
    sf = torch.full((1, 2), 2.0 ** -6)           # codes = vals * 64, all exactly representable
    codes = (vals * 64).to(torch.float8_e4m3fn)
    assert torch.equal(codes.float() * 2.0 ** -6, vals)
    go = torch.ones((1, H), dtype=torch.bfloat16)
    w = torch.tensor([[0.5]])
    ptt = torch.tensor([0], dtype=torch.int32)
    t2p = torch.tensor([[0]], dtype=torch.int32)
    out, xg, wg = torch_ref.swiglu_backward((codes, sf), go, w, ptt, t2p, N, clamp)

    def silu(v):
        return v / (1 + np.exp(-v))

    def dsilu(v):
        s = 1 / (1 + np.exp(-v))
        return s * (1 + v * (1 - s))

    want_out = [silu(2.0) * 1.0, silu(1.0) * 2.0, silu(1.0) * -2.0, silu(-3.0) * 1.5, silu(2.0) * -2.0]
    np.testing.assert_allclose(out[0, :5].numpy(), 0.5 * np.array(want_out), rtol=1e-6)
    want_gate_grad = [0.0, 0.5 * dsilu(1.0) * 2.0, 0.5 * dsilu(1.0) * -2.0, 0.5 * dsilu(-3.0) * 1.5, 0.5 * dsilu(2.0) * -2.0]
    want_up_grad = [0.5 * silu(2.0), 0.0, 0.0, 0.5 * silu(-3.0), 0.5 * silu(2.0)]
    np.testing.assert_allclose(xg[0, :5].numpy(), want_gate_grad, rtol=1e-6)
    np.testing.assert_allclose(xg[0, H:H + 5].numpy(), want_up_grad, rtol=1e-6)
    # zeros elsewhere contribute nothing; weight gradient = sum(grad_out * act)
    np.testing.assert_allclose(wg.item(), sum(want_out), rtol=1e-6)


def test_padding_rows_and_unrouted_pairs():
    xq, go, w, ptt, t2p = _make_case(5, drop=0.4)
    out, xg, wg = torch_ref.swiglu_backward(xq, go, w, ptt, t2p, 128, None)
    dead = ptt < 0
    assert dead.any() and (t2p < 0).any()
    assert torch.equal(out[dead], torch.zeros_like(out[dead]))
    assert torch.equal(xg[dead], torch.zeros_like(xg[dead]))
    assert torch.equal(wg[t2p < 0], torch.zeros_like(wg[t2p < 0]))
    assert (wg[t2p >= 0] != 0).all()


def test_fma_helper_is_single_rounding():
    rng = np.random.default_rng(3)
    n = 200000
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    c = np.ones(n, dtype=np.float32)
    # Engineered cases: c = base and a * b = half an ulp of base times (1 + d) with |d| <= 2^-24, so the
    # exact sum sits a hair off an fp32 rounding boundary.  Where |d| < 2^-29 the float64 sum cannot
    # hold the offset and lands on the boundary itself: rounding twice then goes the wrong way.
    m = 20000
    base = np.abs(rng.standard_normal(m).astype(np.float32)) + np.float32(0.5)
    half_ulp = (np.spacing(base).astype(np.float64) / 2)
    a2 = (1.0 + rng.random(m)).astype(np.float32)
    b2 = (half_ulp / a2.astype(np.float64)).astype(np.float32)
    A = np.concatenate([a, a2])
    B = np.concatenate([b, b2])
    C = np.concatenate([c, base])
    want = cref.fmaf(A, B, C)
    got = torch_ref.fma_f32(torch.from_numpy(A), torch.from_numpy(B), torch.from_numpy(C)).numpy()
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    # the naive float64 route does get some of the engineered cases wrong, so the check has teeth
    naive = (A.astype(np.float64) * B.astype(np.float64) + C.astype(np.float64)).astype(np.float32)
    assert (naive.view(np.uint32) != want.view(np.uint32)).any()


@pytest.mark.parametrize('clamp', [None, 0.5])
@pytest.mark.parametrize('N', [32, 128])
def test_torch_and_c_restatements_agree(N, clamp):
    xq, go, w, ptt, t2p = _make_case(40 + N, N=N, H=512)
    out, xg, wg = torch_ref.swiglu_backward(xq, go, w, ptt, t2p, N, clamp)
    out_c, xg_c, wg_c = cref.swiglu_backward(xq, go, w, ptt, N, clamp)
    # the two differ only in exp (vectorised vs libm), so almost every value is bit-identical
    for a, b, name in ((out, out_c, 'out'), (xg, xg_c, 'x_grad')):
        same = (a.view(torch.int32) == b.view(torch.int32)).float().mean().item()
        assert same > 0.95, (name, same)
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-30)
    torch.testing.assert_close(wg, wg_c, rtol=1e-5, atol=1e-5)


def test_composition_shapes_and_dtypes():
    xq, go, w, ptt, t2p = _make_case(9, N=32)
    out, (codes, sf), xg, wg = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, 32, round_sf=True)
    R, H = go.shape
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (R, H)
    assert xg.dtype == torch.bfloat16 and tuple(xg.shape) == (R, 2 * H)
    assert codes.dtype == torch.float8_e4m3fn and tuple(codes.shape) == (R, 2 * H)
    assert sf.dtype == torch.float32 and tuple(sf.shape) == (R, 2 * H // 32)
    assert torch.equal(sf, torch.exp2(torch.log2(sf).round()))       # powers of two
    assert wg.dtype == torch.float32 and wg.shape == w.shape
