"""Dequantisation of FP8 / packed FP4 / packed E5M6 codes with block scales: host side of tk_cast_back.

Signatures follow tile_kernels/quant/cast_back_kernel.py:77-143 and cast_back_e5m6_kernel.py:141-176.
"""
from typing import Optional

import torch

from .. import _ffi
from .per_token_cast import _input_sf_storage
from .types import QuantTensor


def cast_back(x: QuantTensor, fmt: str, x_block_size: tuple, x_special_fmt: Optional[str] = None) -> torch.Tensor:
    """Dequantise ``(data, sf)`` to ``'bf16'`` or ``'fp32'``; ``x_block_size`` is the
    ``(rows, channels)`` extent that shares one scale."""
    assert fmt in ('bf16', 'fp32')
    out_dtype = torch.bfloat16 if fmt == 'bf16' else torch.float32
    data, x_sf = x
    assert x_special_fmt in (None, 'e5m6'), f'Unsupported special format: {x_special_fmt}'
    assert data.dim() == 2 and data.is_contiguous()
    num_tokens, hidden = data.shape
    assert x_sf.dim() == 2
    assert x_sf.dtype in (torch.int32, torch.float32)
    if x_special_fmt == 'e5m6':
        # eight 12-bit codes per 12 bytes, handed over as uint8 (tile_kernels/quant/cast_back_e5m6_kernel.py:159-166)
        assert data.dtype == torch.uint8
        hidden = hidden * 2 // 3
        assert hidden % 8 == 0
        in_fmt = _ffi.TK_E5M6
    else:
        assert data.dtype in (torch.float8_e4m3fn, torch.int8, torch.uint8)
        in_fp4 = data.dtype != torch.float8_e4m3fn
        if in_fp4:
            hidden *= 2
        assert hidden % 64 == 0
        in_fmt = _ffi.TK_E2M1 if in_fp4 else _ffi.TK_E4M3
    dev = _ffi.require_gpu(data, x_sf)
    lib = _ffi.load()
    out = torch.empty((num_tokens, hidden), dtype=out_dtype, device=dev)
    if num_tokens > 0:
        store, layout, ld = _input_sf_storage(x_sf)
        with _ffi.on_device(dev):
            rc = lib.tk_cast_back(data.data_ptr(), in_fmt, num_tokens, hidden,
                                  store.data_ptr(), ld, layout, x_block_size[0], x_block_size[1], out.data_ptr(),
                                  _ffi.TK_F32 if fmt == 'fp32' else _ffi.TK_BF16, _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_cast_back')
    return out


def per_token_cast_back(x: QuantTensor, fmt: str, num_per_channels: int, x_special_fmt: Optional[str] = None) -> torch.Tensor:
    """:func:`cast_back` for per-token (1 x ``num_per_channels``) scales."""
    return cast_back(x, fmt, (1, num_per_channels), x_special_fmt=x_special_fmt)
