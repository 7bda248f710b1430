"""The re-created test harness (tilekernels_amd.testing) and the FP4 decoder of the quant package on the CPU:
comparators against hand-built cases, generators against the reference's grid
(tile_kernels/testing/generator.py:10-69, numeric.py:5-65, quant.py:6-21, bench.py:59-118)."""
import pytest
import torch

from oracle import torch_ref
from tilekernels_amd import testing as T
from tilekernels_amd.quant.common import unpack_from_e2m1fn_x2


def test_unpack_from_e2m1fn_x2_over_every_byte():
    every = torch.arange(256, dtype=torch.uint8).view(torch.int8).reshape(4, 64)
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for dtype in (torch.float32, torch.bfloat16):
        got = unpack_from_e2m1fn_x2(every, dtype)
        assert got.shape == (4, 128) and got.dtype == dtype
        assert torch.equal(got, torch_ref.unpack_from_e2m1fn_x2(every, dtype))
        flat = got.flatten().float()
        for byte in range(256):
            lo, hi = byte & 0xF, byte >> 4
            for k, nib in enumerate((lo, hi)):        # the even element sits in the low nibble
                want = table[nib & 7] * (-1.0 if nib & 8 else 1.0)
                assert flat[2 * byte + k].item() == want
                if want == 0:
                    assert bool(torch.signbit(flat[2 * byte + k])) == bool(nib & 8)


def test_assert_equal_checks_dtype_shape_stride_and_bytes():
    a = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    T.assert_equal(a, a.clone())
    with pytest.raises(AssertionError):
        T.assert_equal(a, a.double())
    with pytest.raises(AssertionError):
        T.assert_equal(a, a.reshape(4, 3))
    with pytest.raises(AssertionError):
        T.assert_equal(a.T.contiguous().T, a)                    # same values, other strides
    T.assert_equal(a.T.contiguous().T, a, check_stride=False)
    b = a.clone()
    b[1, 2] = -0.0 if a[1, 2] == 0 else a[1, 2] + 1
    with pytest.raises(AssertionError):
        T.assert_equal(a, b)
    z = torch.zeros(2)
    with pytest.raises(AssertionError):                            # bytes, not values: -0.0 is not +0.0
        T.assert_equal(z, -z)
    T.assert_equal(torch.empty((0, 5)), torch.empty((0, 5)))


def test_calc_diff_and_count_bytes():
    x = torch.randn(1000)
    assert T.calc_diff(x, x) < 1e-15
    assert abs(float(T.calc_diff(x, -x)) - 2.0) < 1e-12
    assert T.calc_diff(torch.zeros(4), torch.zeros(4)) == 0
    assert abs(float(T.calc_diff(x, 2 * x)) - 0.2) < 1e-12      # 1 - 2*2/(1+4)
    q = (torch.zeros((3, 8), dtype=torch.float8_e4m3fn), torch.zeros((3, 2), dtype=torch.float32))
    assert T.count_bytes(torch.zeros((3, 8), dtype=torch.bfloat16), q, None) == 48 + 24 + 24


def test_check_bias_accepts_unbiased_and_rejects_biased_rounding():
    x = torch.randn(200000)
    step = 2.0 ** -4
    nearest = torch.round(x / step) * step
    T.check_bias(nearest, x)
    with pytest.raises(AssertionError):
        T.check_bias(torch.floor(x / step) * step, x)            # always rounds down
    T.check_bias(torch.empty(0), torch.empty(0))


def test_clear_unused_sf_zeroes_only_the_tail_bytes():
    rows, hidden, npc = 6, 576, 32                                # 18 blocks: 5 words, the last with 2 unused bytes
    nk, words = 18, 5
    storage = torch.randint(1, 255, (words, 8 * 4), dtype=torch.uint8)     # [words, align(4 * rows, 16)] bytes
    sf = storage.view(torch.int32).T[:rows]                                # the packed layout's int32 view
    flat = T.clear_unused_sf(sf, hidden, npc)
    assert flat.shape == (rows, 20) and flat.dtype == torch.uint8
    assert torch.all(flat[:, nk:] == 0) and torch.all(flat[:, :nk] != 0)
    want = torch.empty((rows, words), dtype=torch.int32).copy_(sf).view(torch.uint8).reshape(rows, 20)[:, :nk]
    assert torch.equal(flat[:, :nk], want)


def test_grid_generators_follow_the_reference():
    assert T.generate_num_tokens() == [4001, 8001]
    assert T.generate_num_tokens(alignment=128) == [4096, 8064]
    assert T.generate_hidden_sizes() == [576, 2048, 2560, 3072, 4096, 6144, 7168]
    assert T.generate_hidden_sizes(256) == [2048, 2560, 3072, 4096, 6144, 7168]
    moe = list(T.generate_moe_params())
    assert len(moe) == 12 and all(p['num_send_tokens'] == 4001 for p in moe)
    assert {(p['num_topk']) for p in moe} == {2, 6, 8, 9}
    assert {(p['num_experts'], p['num_ep_ranks']) for p in moe} == {(9, 8), (32, 8), (4, 64)}
    params = dict(num_send_tokens=50, num_topk=4, num_experts=3, num_ep_ranks=8)
    idx = T.generate_topk_idx(params, device='cpu')
    assert idx.dtype == torch.int64 and idx.shape[1] == 4 and idx.is_contiguous()
    assert int(idx.max()) < 3 and int(idx.min()) >= -1 and bool((idx >= 0).any(dim=1).all())
    for row in idx.tolist():                                       # an expert at most once per token
        live = [e for e in row if e >= 0]
        assert len(live) == len(set(live))
    assert T.generate_topk_idx(dict(num_send_tokens=0, num_topk=2, num_experts=1, num_ep_ranks=1), device='cpu').shape == (0, 2)
    r = T.generate_rand_float((64, 64), device='cpu')
    assert r.dtype == torch.float32 and bool(torch.isfinite(r).all()) and float(r.abs().max()) <= torch.finfo(torch.float32).max / 8


def test_parameter_naming():
    p = dict(num_tokens=4001, in_dtype=torch.bfloat16, block_size=(128, 128), round_sf=True, x_block_size=None)
    assert T.make_param_id(p) == 'num_tokens=4001-in_dtype=bf16-block_size=128x128-round_sf=1-x_block_size=None'
    assert T.make_param_key(p) == 'num_tokens=4001,in_dtype=bf16,block_size=128x128,round_sf=1'
    assert T.make_param_id({}) == 'default'
    assert T.dtype_to_str(torch.float8_e4m3fn) == 'e4m3' and T.dtype_to_str(torch.float32) == 'fp32'
