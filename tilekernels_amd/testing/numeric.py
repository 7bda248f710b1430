"""Comparators used by the parity tests and the benchmark (the reference keeps their counterparts
in tile_kernels/testing/numeric.py:5-65)."""
import math

import torch


def _bytes_of(t: torch.Tensor) -> torch.Tensor:
    # a [n, 1] tensor with strides (1, n) counts as contiguous yet cannot be viewed; flatten first
    return t.contiguous().flatten().view(torch.uint8)


def assert_equal(x: torch.Tensor, y: torch.Tensor, check_dtype: bool = True, check_shape: bool = True,
                 check_stride: bool = True) -> None:
    """Same dtype, shape, strides, device and bytes."""
    if check_dtype:
        assert x.dtype == y.dtype, f'dtype {x.dtype} != {y.dtype}'
    if check_shape:
        assert x.shape == y.shape, f'shape {tuple(x.shape)} != {tuple(y.shape)}'
    if check_stride and x.numel() > 0:
        assert x.stride() == y.stride(), f'stride {x.stride()} != {y.stride()}'
    assert x.device == y.device, f'device {x.device} != {y.device}'
    if not torch.equal(_bytes_of(x), _bytes_of(y)):
        where = torch.nonzero(x != y)
        raise AssertionError(f'values differ at {where.shape[0]} positions, first {where[:8].tolist()}:\n'
                             f'{x[x != y][:8]}\nvs\n{y[x != y][:8]}')


def calc_diff(x: torch.Tensor, y: torch.Tensor):
    """1 - cosine-style similarity 2<x,y>/(|x|^2+|y|^2), in float64."""
    x, y = x.double(), y.double()
    den = (x * x + y * y).sum()
    return 0 if den == 0 else 1 - 2 * (x * y).sum() / den


def check_bias(x: torch.Tensor, ref_x: torch.Tensor) -> None:
    """Rounding must not lean to one side: the share of values that got smaller (ties split) has
    to stay within 10/sqrt(n) of one half (binomial bound, far beyond 6 sigma)."""
    n = x.numel()
    if n == 0:
        return
    below = (x < ref_x).sum().item()
    same = (x == ref_x).sum().item()
    ratio = (below + same / 2) / n
    assert abs(ratio - 0.5) < 10 / math.sqrt(n), \
        f'biased rounding: share below = {ratio:.5f} over {n} values ({below} below, {same} equal)'


def count_bytes(*tensors) -> int:
    total = 0
    for t in tensors:
        if isinstance(t, (tuple, list)):
            total += count_bytes(*t)
        elif t is not None:
            total += t.numel() * t.element_size()
    return total
