"""Weighted reduction of expanded rows back to tokens: host side of tk_reduce_fused.

Signature, asserts and return convention follow tile_kernels/moe/reduce_fused_kernel.py:70-135.
"""
from typing import Optional, Union

import torch

from .. import _ffi
from ..quant.types import QuantTensor


def reduce_fused(
    x: Union[torch.Tensor, QuantTensor],
    topk_weights: Optional[torch.Tensor],
    token_topk_to_pos: torch.Tensor,
    fp8_format: str = '',
    sf: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``out[t] = sum_k x[token_topk_to_pos[t, k]] * topk_weights[t, k]`` (positions < 0 skipped), accumulated in
    fp32; ``x`` may be ``(data, x_sf)`` with one fp32 factor per expanded row.  ``fp8_format='e4m3'`` gives an FP8
    result, scaled by the one-element tensor ``sf`` if given; otherwise the result has the dtype of ``x``."""
    x_sf = None
    if isinstance(x, tuple):
        x, x_sf = x
    num_expanded_tokens, hidden = x.shape
    num_tokens, num_topk = token_topk_to_pos.shape
    assert hidden % 256 == 0
    assert x.dtype in (torch.bfloat16, torch.float32) and x.is_contiguous()
    assert token_topk_to_pos.dtype == torch.int32 and token_topk_to_pos.is_contiguous()

    out_dtype = x.dtype
    if fp8_format != '':
        assert fp8_format == 'e4m3'
        out_dtype = torch.float8_e4m3fn
    else:
        assert sf is None, 'Only FP8 output supports sf.'
    dev = _ffi.require_gpu(x, x_sf, topk_weights, token_topk_to_pos, sf, out)
    if out is not None:
        assert tuple(out.shape) == (num_tokens, hidden) and out.dtype == out_dtype and out.is_contiguous()
    else:
        out = torch.empty((num_tokens, hidden), dtype=out_dtype, device=dev)
    if x_sf is not None:
        assert x_sf.shape[0] == num_expanded_tokens and x_sf.dtype == torch.float32 and x_sf.is_contiguous()
    if topk_weights is not None:
        assert tuple(topk_weights.shape) == (num_tokens, num_topk) and topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()
    if sf is not None:
        assert sf.numel() >= 1 and sf.dtype == torch.float32

    if num_tokens > 0:
        lib = _ffi.load()
        out_code = _ffi.TK_OUT_E4M3 if out_dtype == torch.float8_e4m3fn else _ffi.dtype_code(x)
        with _ffi.on_device(dev):
            rc = lib.tk_reduce_fused(x.data_ptr(), _ffi.dtype_code(x), num_expanded_tokens, hidden, _ffi.ptr(x_sf), _ffi.ptr(topk_weights),
                                     token_topk_to_pos.data_ptr(), num_tokens, num_topk, out.data_ptr(), out_code, _ffi.ptr(sf),
                                     _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_reduce_fused')
    return out
