"""Shared helpers of the GPU parity tests."""
import torch

E4M3_ABS = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().abs()


def assert_same(got: torch.Tensor, want: torch.Tensor, what: str = '') -> None:
    """dtype, shape, strides and bytes of a GPU result against the CPU oracle's tensor."""
    assert got.dtype == want.dtype, f'{what} dtype {got.dtype} != {want.dtype}'
    assert tuple(got.shape) == tuple(want.shape), f'{what} shape {tuple(got.shape)} != {tuple(want.shape)}'
    if got.numel() > 0:
        assert got.stride() == want.stride(), f'{what} stride {got.stride()} != {want.stride()}'
    g = dense_bytes(got.cpu())
    w = dense_bytes(want)
    if not torch.equal(g, w):
        bad = torch.nonzero(g != w).flatten()
        raise AssertionError(f'{what}: {bad.numel()} of {g.numel()} bytes differ, first at {bad[:8].tolist()}: '
                             f'{g[bad[:8]].tolist()} vs {w[bad[:8]].tolist()}')


def dense_bytes(t: torch.Tensor) -> torch.Tensor:
    return torch.empty(t.shape, dtype=t.dtype).copy_(t).flatten().view(torch.uint8)


def packed_sf_bytes(sf: torch.Tensor, nk: int) -> torch.Tensor:
    """int32 [nm, ceil(nk/4)] packed scales -> uint8 [nm, nk] (drops the unused tail bytes)."""
    nm, nw = sf.shape
    return torch.empty((nm, nw), dtype=torch.int32).copy_(sf.cpu()).view(torch.uint8).reshape(nm, nw * 4)[:, :nk]


def fp8_code_report(got: torch.Tensor, want: torch.Tensor):
    """(fraction of differing codes, all differences are one E4M3 step) for two uint8 code tensors."""
    g, w = got.flatten().to(torch.int16), want.flatten().to(torch.int16)
    diff = g != w
    n = int(diff.sum())
    if n == 0:
        return 0.0, True
    gd, wd = g[diff], w[diff]
    same_sign = (gd & 0x80) == (wd & 0x80)
    one_step = same_sign & (((gd & 0x7F) - (wd & 0x7F)).abs() == 1)
    both_zero = ((gd & 0x7F) == 0) & ((wd & 0x7F) == 0)
    return n / g.numel(), bool((one_step | both_zero).all())


def mismatch_within(frac: float, numel: int, budget: float) -> bool:
    """The share of differing elements against a budget that is a rate.  Only on a tensor so small that the budget
    is less than two elements (fewer than 20 000 elements at 1e-4) are up to two differing elements accepted; the
    tensor must still hold enough elements (1024) for two of them to be a small share."""
    if frac <= budget:
        return True
    return budget * numel < 2 and numel >= 1024 and round(frac * numel) <= 2
