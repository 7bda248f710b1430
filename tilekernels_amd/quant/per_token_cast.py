"""Per-token (1 x N) FP8 E4M3 / FP4 E2M1 cast and the per-row E5M6 cast: host side of tk_per_token_cast.

Signatures, defaults, asserts and return conventions follow
tile_kernels/quant/per_token_cast_kernel.py:159-302.
"""
from typing import Optional, Union

import torch

from .. import _ffi
from .common import (alloc_scaling_factors, cast_epilogue, get_cast_output_config, sf_leading_dim)
from .types import QuantTensor


def per_token_cast_impl(x, fmt, num_per_channels, x_block_size=None, use_tma_aligned_col_major_sf=False,
                        round_sf=False, use_packed_ue8m0=False, sf_only=False, sf=None):
    assert fmt in ('e5m6', 'e4m3', 'e2m1')
    if isinstance(x, tuple):
        assert not sf_only and sf is None
        return _per_token_cast_quantised_input(x, fmt, num_per_channels, x_block_size, use_tma_aligned_col_major_sf,
                                               round_sf, use_packed_ue8m0)
    assert x_block_size is None
    assert isinstance(x, torch.Tensor) and x.dtype in (torch.bfloat16, torch.float32)
    out_config = get_cast_output_config(fmt, (1, num_per_channels), use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)
    assert x.dim() == 2 and (x.stride(1) == 1 or x.shape[1] <= 1)
    num_tokens, hidden = x.shape
    if fmt == 'e5m6':
        # whole rows share one scale and only the full cast exists (tile_kernels/quant/per_token_cast_to_e5m6_kernel.py:172-196)
        assert num_per_channels == hidden and hidden % 8 == 0 and not sf_only and sf is None
    else:
        assert num_per_channels in (16, 32, 64, 128) or (num_per_channels == hidden and hidden % 64 == 0)
        if num_per_channels == hidden and hidden not in (16, 32, 64, 128):
            assert not sf_only and sf is None
    dev = _ffi.require_gpu(x, sf)
    lib = _ffi.load()

    out_cols = {'e4m3': hidden, 'e2m1': hidden // 2, 'e5m6': hidden // 8 * 3}[fmt]
    out = torch.empty((num_tokens, out_cols), dtype=out_config.torch_dtype, device=dev)
    if sf is not None:
        assert not sf_only
        assert not use_tma_aligned_col_major_sf and not use_packed_ue8m0, 'precomputed sf must be row-major fp32'
        assert sf.dtype == torch.float32 and sf.dim() == 2
        assert tuple(sf.shape) == (num_tokens, -(-hidden // num_per_channels)), f'sf shape {tuple(sf.shape)}'
        assert sf.stride(1) == 1 or sf.shape[1] == 1
        out_sf = sf
    else:
        out_sf = alloc_scaling_factors((num_tokens, hidden), out_config, dev)

    if num_tokens > 0:
        mode = _ffi.TK_SF_ONLY if sf_only else (_ffi.TK_CAST_GIVEN_SF if sf is not None else _ffi.TK_CAST_AND_SF)
        with _ffi.on_device(dev):
            rc = lib.tk_per_token_cast(
                x.data_ptr(), _ffi.dtype_code(x), num_tokens, hidden, x.stride(0) if num_tokens > 1 else hidden,
                0 if sf_only else out.data_ptr(), out_sf.data_ptr(), sf_leading_dim(out_sf),
                out_config.fmt_code, num_per_channels, out_config.layout_code, int(round_sf), mode,
                _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_per_token_cast')

    if sf is not None:
        return out
    if fmt == 'e5m6':
        out = out.view(torch.uint8)
    out_sf = cast_epilogue(out_sf, num_tokens, hidden, out_config)
    return out_sf if sf_only else (out, out_sf)


def _input_sf_storage(x_sf: torch.Tensor):
    """(storage tensor, layout code, leading dimension) of the scale tensor of a quantised input, told
    apart the way the reference does (tile_kernels/quant/common.py:72-82): unit stride along the rows
    means the column-major layout, int32 elements mean packed UE8M0 bytes."""
    assert x_sf.dim() == 2
    if x_sf.stride(0) == 1:
        store = x_sf.T
        if x_sf.dtype == torch.int32:
            store = store.view(torch.uint8)
            return store, _ffi.TK_SF_COL_UE8M0, sf_leading_dim(store)
        assert x_sf.dtype == torch.float32
        return store, _ffi.TK_SF_COL_F32, sf_leading_dim(store)
    assert x_sf.stride(1) == 1 and x_sf.dtype == torch.float32
    return x_sf, _ffi.TK_SF_ROW_F32, sf_leading_dim(x_sf)


def _per_token_cast_quantised_input(x, fmt, num_per_channels, x_block_size, use_tma_aligned_col_major_sf, round_sf,
                                    use_packed_ue8m0):
    """``x = (data, sf)``: FP8 / packed FP4 codes with one scale per ``x_block_size`` block are
    dequantised and re-quantised in one pass (tile_kernels/quant/per_token_cast_kernel.py:87-126)."""
    assert isinstance(x_block_size, tuple) and len(x_block_size) == 2
    data, x_sf = x
    assert isinstance(data, torch.Tensor) and isinstance(x_sf, torch.Tensor)
    assert data.dtype in (torch.float8_e4m3fn, torch.int8, torch.uint8)
    assert data.dim() == 2 and (data.stride(1) == 1 or data.shape[1] <= 1)
    in_fp4 = data.dtype != torch.float8_e4m3fn
    num_tokens = data.shape[0]
    hidden = data.shape[1] * (2 if in_fp4 else 1)                    # logical width
    token_stride = data.stride(0) * (2 if in_fp4 else 1) if num_tokens > 1 else hidden
    out_config = get_cast_output_config(fmt, (1, num_per_channels), use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)
    assert num_per_channels in (16, 32, 64, 128)
    dev = _ffi.require_gpu(data, x_sf)
    lib = _ffi.load()
    out = torch.empty((num_tokens, hidden if fmt == 'e4m3' else hidden // 2), dtype=out_config.torch_dtype, device=dev)
    out_sf = alloc_scaling_factors((num_tokens, hidden), out_config, dev)
    if num_tokens > 0:
        store, layout, ld = _input_sf_storage(x_sf)
        with _ffi.on_device(dev):
            rc = lib.tk_per_token_cast_quantized(
                data.data_ptr(), _ffi.TK_E2M1 if in_fp4 else _ffi.TK_E4M3, num_tokens, hidden, token_stride,
                store.data_ptr(), ld, layout, x_block_size[0], x_block_size[1],
                out.data_ptr(), out_sf.data_ptr(), sf_leading_dim(out_sf), out_config.fmt_code, num_per_channels,
                out_config.layout_code, int(round_sf), _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_per_token_cast_quantized')
    return out, cast_epilogue(out_sf, num_tokens, hidden, out_config)


def per_token_cast(
    x: torch.Tensor,
    fmt: str,
    num_per_channels: int,
    x_block_size: Optional[tuple] = None,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> QuantTensor:
    """Cast ``x[num_tokens, hidden]`` to FP8 (``'e4m3'``) or packed FP4 (``'e2m1'``) with one scale per
    ``num_per_channels`` consecutive channels of a token, or to packed 12-bit ``'e5m6'`` (uint8
    ``[num_tokens, hidden * 3 // 2]``) with one scale per token.  Returns ``(out, out_sf)``."""
    return per_token_cast_impl(x, fmt, num_per_channels, x_block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)


def per_token_cast_with_sf_only(
    x: torch.Tensor,
    fmt: str,
    num_per_channels: int,
    x_block_size: Optional[tuple] = None,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> torch.Tensor:
    """Same as :func:`per_token_cast` but computes and returns only the scale factors."""
    return per_token_cast_impl(x, fmt, num_per_channels, x_block_size, use_tma_aligned_col_major_sf, round_sf,
                               use_packed_ue8m0, sf_only=True)


def per_token_cast_with_precomputed_sf(
    x: torch.Tensor,
    fmt: str,
    num_per_channels: int,
    sf: torch.Tensor,
    x_block_size: Optional[tuple] = None,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> torch.Tensor:
    """Cast with caller-supplied row-major fp32 scales ``sf[num_tokens, ceil(hidden / N)]``; returns
    the codes only."""
    return per_token_cast_impl(x, fmt, num_per_channels, x_block_size, use_tma_aligned_col_major_sf, round_sf,
                               use_packed_ue8m0, sf_only=False, sf=sf)
