"""Per-channel (N tokens x 1 column) FP8 E4M3 casts: host side of tk_per_channel_cast.

Signatures, defaults and asserts follow tile_kernels/quant/per_channel_cast_kernel.py:8-28,
per_channel_cast_fused_kernel.py:130-203, per_channel_cast_and_transpose_kernel.py:84-123 and
swiglu_forward_and_per_channel_cast_and_transpose_kernel.py:178-231.
"""
from typing import Optional, Union

import torch

from .. import _ffi
from ..utils import ceil_div
from .types import QuantTensor


def _launch(x, x_sf, num_tokens, hidden, pos_to_token, num_tokens_out, num_per_tokens, round_sf, transpose,
            swiglu=False, swiglu_clamp_value=None):
    dev = _ffi.require_gpu(x, x_sf, pos_to_token)
    lib = _ffi.load()
    out_shape = (hidden, num_tokens_out) if transpose else (num_tokens_out, hidden)
    out = torch.empty(out_shape, dtype=torch.float8_e4m3fn, device=dev)
    out_sf = torch.empty((ceil_div(num_tokens_out, num_per_tokens), hidden), dtype=torch.float32, device=dev)
    if num_tokens_out > 0:
        with _ffi.on_device(dev):
            rc = lib.tk_per_channel_cast(
                x.data_ptr(), _ffi.TK_F32 if x.dtype == torch.float32 else _ffi.TK_BF16, _ffi.ptr(x_sf), num_tokens, hidden, _ffi.ptr(pos_to_token), num_tokens_out,
                out.data_ptr(), out_sf.data_ptr(), num_per_tokens, int(round_sf), int(transpose), int(swiglu),
                int(swiglu_clamp_value is not None), 0.0 if swiglu_clamp_value is None else float(swiglu_clamp_value),
                _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_per_channel_cast')
    return out, out_sf


def per_channel_cast_fused(
    x: Union[torch.Tensor, QuantTensor],
    fmt: str,
    num_per_tokens: int,
    round_sf: bool = False,
    num_per_channels: Optional[int] = None,
    pos_to_token: Optional[torch.Tensor] = None,
) -> QuantTensor:
    """Cast ``x[num_tokens, hidden]`` to FP8 with one scale per 128 tokens of a column, optionally
    dequantising an FP8 ``(data, sf)`` input with 1 x 128 scales first and gathering rows through
    ``pos_to_token`` (negative entries give zero rows).  Returns ``(out, out_sf)``."""
    x_sf = None
    if isinstance(x, tuple):
        assert num_per_channels is not None
        x, x_sf = x
    else:
        assert num_per_channels is None

    assert fmt == 'e4m3'
    assert x.dim() == 2 and x.is_contiguous()
    num_tokens, hidden = x.shape
    num_tokens_out = num_tokens

    if pos_to_token is not None:
        assert pos_to_token.dim() == 1 and pos_to_token.is_contiguous()
        assert pos_to_token.dtype == torch.int32
        num_tokens_out = pos_to_token.size(0)
        # Alignment requirement for expanded tokens
        assert num_tokens_out % 16 == 0
    else:
        assert num_tokens_out % 128 == 0

    assert num_per_tokens == 128
    if x_sf is not None:
        assert num_per_channels == 128
        assert x.dtype == torch.float8_e4m3fn
        assert x_sf.dim() == 2 and x_sf.is_contiguous() and x_sf.dtype == torch.float32
        assert x_sf.size(0) == num_tokens and x_sf.size(1) * 128 == hidden
    else:
        assert x.dtype in (torch.bfloat16, torch.float32)
    assert hidden % 8 == 0

    return _launch(x, x_sf, num_tokens, hidden, pos_to_token, num_tokens_out, num_per_tokens, round_sf, False)


def per_channel_cast(x: torch.Tensor, fmt: str, num_per_tokens: int, round_sf: bool = False) -> QuantTensor:
    """Cast ``x[num_tokens, hidden]`` to FP8 with per-channel (column-wise) scales, one per 128 tokens."""
    assert x.is_contiguous() and x.dim() == 2
    assert fmt == 'e4m3'
    num_tokens, hidden = x.shape
    assert num_tokens % 128 == 0 and hidden % 64 == 0
    assert num_per_tokens == 128
    return per_channel_cast_fused(x, 'e4m3', num_per_tokens=num_per_tokens, round_sf=round_sf)


def per_channel_cast_and_transpose(x: torch.Tensor, fmt: str, num_per_tokens: int, round_sf: bool = False) -> QuantTensor:
    """Cast bf16 ``x[num_tokens, hidden]`` to FP8 with per-channel scales (32 or 128 tokens) and return
    the codes transposed: ``out[hidden, num_tokens]``, ``out_sf[num_tokens // num_per_tokens, hidden]``."""
    assert x.dim() == 2 and x.is_contiguous()
    assert x.dtype == torch.bfloat16
    num_tokens, hidden = x.shape
    assert fmt == 'e4m3'
    assert num_tokens % 128 == 0 and hidden % 64 == 0
    assert num_per_tokens in [32, 128]
    return _launch(x, None, num_tokens, hidden, None, num_tokens, num_per_tokens, round_sf, True)


def swiglu_forward_and_per_channel_cast_and_transpose(
    x: torch.Tensor,
    fmt: str,
    num_per_tokens: int,
    round_sf: bool = False,
    without_transpose: bool = False,
    swiglu_clamp_value: Optional[float] = None,
) -> QuantTensor:
    """SwiGLU on bf16 ``x[num_tokens, 2 * hidden]``, rounded to bf16, then the per-channel FP8 cast
    (32 or 128 tokens per scale).  ``out`` is ``[hidden, num_tokens]``, or ``[num_tokens, hidden]`` with
    ``without_transpose``; ``out_sf[num_tokens // num_per_tokens, hidden]``."""
    assert fmt == 'e4m3'
    assert x.dim() == 2 and x.is_contiguous()
    assert x.dtype == torch.bfloat16
    num_tokens, hidden = x.shape
    # Swiglu forward : hidden -> hidden // 2
    assert num_tokens % 128 == 0 and hidden % 128 == 0
    assert num_per_tokens in (32, 128)
    hidden = hidden // 2
    return _launch(x, None, num_tokens, hidden, None, num_tokens, num_per_tokens, round_sf, not without_transpose,
                   swiglu=True, swiglu_clamp_value=swiglu_clamp_value)
