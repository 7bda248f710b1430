"""Per-block (bm x bk) FP8 E4M3 / FP4 E2M1 cast: host side of tk_per_block_cast.

Signatures, defaults, asserts and return conventions follow
tile_kernels/quant/per_block_cast_kernel.py:141-276.
"""
from typing import Optional

import torch

from .. import _ffi
from .common import alloc_scaling_factors, cast_epilogue, get_cast_output_config, sf_leading_dim
from .types import QuantTensor


def per_block_cast_impl(x, fmt, block_size, use_tma_aligned_col_major_sf=False, round_sf=False,
                        use_packed_ue8m0=False, sf_only=False, sf=None):
    assert isinstance(x, torch.Tensor) and x.is_contiguous() and x.dim() == 2
    assert x.dtype in (torch.bfloat16, torch.float32)
    num_tokens, hidden = x.shape
    assert hidden % 64 == 0
    if sf is not None:
        assert not sf_only and not use_tma_aligned_col_major_sf and not use_packed_ue8m0
    out_config = get_cast_output_config(fmt, block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)
    bm, bk = out_config.sf_block
    assert bm in (32, 128) and bk in (32, 128)
    dev = _ffi.require_gpu(x, sf)
    lib = _ffi.load()

    out = torch.empty((num_tokens, hidden if fmt == 'e4m3' else hidden // 2), dtype=out_config.torch_dtype, device=dev)
    if sf is not None:
        assert sf.dtype == torch.float32 and sf.dim() == 2
        assert tuple(sf.shape) == (-(-num_tokens // bm), hidden // bk if hidden % bk == 0 else hidden // bk + 1)
        assert sf.stride(1) == 1 or sf.shape[1] == 1
        out_sf = sf
    else:
        out_sf = alloc_scaling_factors((num_tokens, hidden), out_config, dev)

    if num_tokens > 0:
        mode = _ffi.TK_SF_ONLY if sf_only else (_ffi.TK_CAST_GIVEN_SF if sf is not None else _ffi.TK_CAST_AND_SF)
        with _ffi.on_device(dev):
            rc = lib.tk_per_block_cast(
                x.data_ptr(), _ffi.dtype_code(x), num_tokens, hidden, 0 if sf_only else out.data_ptr(),
                out_sf.data_ptr(), sf_leading_dim(out_sf), out_config.fmt_code, bm, bk, out_config.layout_code,
                int(round_sf), mode, _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_per_block_cast')

    if sf is not None:
        return out
    out_sf = cast_epilogue(out_sf, num_tokens, hidden, out_config)
    return out_sf if sf_only else (out, out_sf)


def per_block_cast(
    x: torch.Tensor,
    fmt: str,
    block_size: tuple,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> QuantTensor:
    """Cast contiguous ``x[num_tokens, hidden]`` to FP8/FP4 with one scale per ``block_size`` block.
    Returns ``(out, out_sf)``."""
    return per_block_cast_impl(x, fmt, block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)


def per_block_cast_with_sf_only(
    x: torch.Tensor,
    fmt: str,
    block_size: tuple,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> torch.Tensor:
    """Same as :func:`per_block_cast` but computes and returns only the scale factors."""
    return per_block_cast_impl(x, fmt, block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0, sf_only=True)


def per_block_cast_with_precomputed_sf(
    x: torch.Tensor,
    fmt: str,
    block_size: tuple,
    sf: torch.Tensor,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> torch.Tensor:
    """Cast with caller-supplied row-major fp32 block scales; returns the codes only."""
    return per_block_cast_impl(x, fmt, block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0,
                               sf_only=False, sf=sf)
