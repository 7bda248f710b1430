"""Fused SwiGLU + per-token FP8 quantisation: host side of tk_swiglu_per_token_cast.

Signature, defaults and asserts follow
tile_kernels/quant/swiglu_forward_and_per_token_cast_kernel.py:175-260.
"""
from typing import Optional

import torch

from .. import _ffi
from ..config import get_num_sms
from .common import alloc_scaling_factors, cast_epilogue, get_cast_output_config, sf_leading_dim
from .types import QuantTensor


def swiglu_forward_and_per_token_cast(
    x: torch.Tensor,
    fmt: str,
    num_per_channels: int,
    pos_to_token_topk: Optional[torch.Tensor] = None,
    topk_weights: Optional[torch.Tensor] = None,
    pos_to_expert: Optional[torch.Tensor] = None,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
    swiglu_clamp_value: Optional[float] = None,
    clamped_count: Optional[torch.Tensor] = None,
    sf_clamp_min: Optional[float] = None,
) -> QuantTensor:
    """``silu(x[:, :H]) * x[:, H:]`` (optionally clamped, optionally times the row's routing weight)
    quantised to FP8 E4M3 with one scale per ``num_per_channels`` (128 or H) outputs, in one pass.

    Rows whose ``pos_to_expert`` entry is negative are padding: their codes and scales are zeros.
    ``clamped_count`` (int64[3]) is incremented in place.  Returns ``(out, out_sf)``.
    """
    assert x.dim() == 2 and x.is_contiguous()
    assert x.dtype in (torch.bfloat16, torch.float32)
    num_expanded_tokens, hidden = x.shape
    assert hidden % 2 == 0
    hidden //= 2

    if pos_to_token_topk is not None:
        assert pos_to_token_topk.dim() == 1 and pos_to_token_topk.shape[0] == num_expanded_tokens
        assert pos_to_token_topk.dtype == torch.int32 and pos_to_token_topk.is_contiguous()
        assert topk_weights is not None and topk_weights.dim() == 2
        assert topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()
    if pos_to_expert is not None:
        assert pos_to_expert.dim() == 1 and pos_to_expert.shape[0] == num_expanded_tokens
        assert pos_to_expert.dtype == torch.int32 and pos_to_expert.is_contiguous()
    if clamped_count is not None:
        assert swiglu_clamp_value is not None
        assert clamped_count.dim() == 1 and clamped_count.shape[0] == 3
        assert clamped_count.dtype == torch.int64 and clamped_count.is_contiguous()

    assert hidden % 128 == 0
    assert num_per_channels == 128 or num_per_channels == hidden
    assert num_per_channels == 128 or (not use_tma_aligned_col_major_sf)
    assert fmt == 'e4m3'

    out_config = get_cast_output_config(fmt, (1, num_per_channels), use_tma_aligned_col_major_sf, round_sf,
                                        use_packed_ue8m0, custom_clamp_min_value=sf_clamp_min)
    dev = _ffi.require_gpu(x, pos_to_token_topk, topk_weights, pos_to_expert, clamped_count)
    lib = _ffi.load()

    out = torch.empty((num_expanded_tokens, hidden), dtype=torch.float8_e4m3fn, device=dev)
    out_sf = alloc_scaling_factors((num_expanded_tokens, hidden), out_config, dev)
    if num_expanded_tokens > 0:
        with _ffi.on_device(dev):
            # the counting variant: at most 8 workgroups per compute unit, which then loop over tiles (every workgroup that
            # clamped anything sends one atomic request to the counters, and those are served one at a time)
            max_blocks = get_num_sms() * 8 if clamped_count is not None else 0
            rc = lib.tk_swiglu_per_token_cast(
                x.data_ptr(), _ffi.dtype_code(x), num_expanded_tokens, hidden, out.data_ptr(), out_sf.data_ptr(),
                sf_leading_dim(out_sf), num_per_channels, out_config.layout_code, int(round_sf),
                -1.0 if sf_clamp_min is None else float(sf_clamp_min),
                _ffi.ptr(pos_to_token_topk), _ffi.ptr(topk_weights),
                0 if topk_weights is None else topk_weights.numel(), _ffi.ptr(pos_to_expert),
                int(swiglu_clamp_value is not None), 0.0 if swiglu_clamp_value is None else float(swiglu_clamp_value),
                _ffi.ptr(clamped_count), max_blocks, _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_swiglu_per_token_cast')
    return out, cast_epilogue(out_sf, num_expanded_tokens, hidden, out_config)
