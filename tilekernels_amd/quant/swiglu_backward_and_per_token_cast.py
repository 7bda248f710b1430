"""Fused SwiGLU backward + per-token FP8 quantisation of the input gradient: host side of
tk_swiglu_backward_per_token_cast.

Signature, defaults and asserts follow
tile_kernels/quant/swiglu_backward_and_per_token_cast_kernel.py:166-244.
"""
from typing import Optional

import torch

from .. import _ffi
from .types import QuantTensor


def swiglu_backward_and_per_token_cast(
    x: QuantTensor,
    grad_out: torch.Tensor,
    weight: torch.Tensor,
    pos_to_token_topk: torch.Tensor,
    token_topk_to_pos: torch.Tensor,
    num_per_channels: int,
    round_sf: bool = False,
    swiglu_clamp_value: Optional[float] = None,
) -> tuple[torch.Tensor, QuantTensor, torch.Tensor, torch.Tensor]:
    """Backward of ``out = silu(g) * u * w`` on the FP8 forward input ``x = (data, sf)`` with
    data ``[num_expand_tokens, 2 * hidden]`` and sf ``[num_expand_tokens, 2 * hidden // num_per_channels]``.

    Returns ``(out, (x_grad_fp8, x_grad_fp8_sf), x_grad, weight_grad)``: the bf16 forward output, the
    input gradient quantised per token in groups of ``num_per_channels`` (32 or 128), the same gradient
    in bf16, and the fp32 gradient of the routing weights ``[num_tokens, num_topk]``.
    """
    assert num_per_channels in (32, 128)
    x, x_sf = x

    assert x.dtype == torch.float8_e4m3fn
    assert (x.dim() == 2 or x.dim() == 3) and x.is_contiguous()
    assert x_sf.dim() == 2 and x_sf.is_contiguous() and x_sf.dtype == torch.float32
    assert grad_out.dtype == torch.bfloat16 and grad_out.is_contiguous()
    assert weight.dim() == 2 and weight.is_contiguous() and weight.dtype == torch.float32
    assert pos_to_token_topk.dim() == 1 and pos_to_token_topk.is_contiguous() and pos_to_token_topk.dtype == torch.int32
    assert token_topk_to_pos.dim() == 2 and token_topk_to_pos.is_contiguous() and token_topk_to_pos.dtype == torch.int32

    assert x.size(-1) % (2 * num_per_channels) == 0
    hidden = x.size(-1) // 2

    x = x.view(-1, hidden * 2)
    grad_out = grad_out.view(-1, hidden)
    num_expand_tokens = x.size(0)
    num_tokens, num_topk = token_topk_to_pos.shape

    assert x_sf.shape == (num_expand_tokens, 2 * hidden // num_per_channels)
    assert grad_out.shape == (num_expand_tokens, hidden)
    assert weight.shape == (num_tokens, num_topk)
    assert pos_to_token_topk.shape == (num_expand_tokens,)

    dev = _ffi.require_gpu(x, x_sf, grad_out, weight, pos_to_token_topk, token_topk_to_pos)
    lib = _ffi.load()

    out = torch.empty((num_expand_tokens, hidden), dtype=grad_out.dtype, device=dev)
    x_grad_fp8 = torch.empty((num_expand_tokens, hidden * 2), dtype=x.dtype, device=dev)
    x_grad_fp8_sf = torch.empty((num_expand_tokens, 2 * hidden // num_per_channels), dtype=torch.float32, device=dev)
    x_grad = torch.empty((num_expand_tokens, hidden * 2), dtype=grad_out.dtype, device=dev)
    weight_grad = torch.empty((num_tokens, num_topk), dtype=torch.float32, device=dev)

    # also launched without rows: weight_grad of unrouted pairs is still defined (zero)
    if num_expand_tokens > 0 or weight.numel() > 0:
        with _ffi.on_device(dev):
            rc = lib.tk_swiglu_backward_per_token_cast(
                x.data_ptr(), x_sf.data_ptr(), num_expand_tokens, hidden, num_per_channels, grad_out.data_ptr(),
                weight.data_ptr(), pos_to_token_topk.data_ptr(), token_topk_to_pos.data_ptr(), weight.numel(),
                out.data_ptr(), x_grad_fp8.data_ptr(), x_grad_fp8_sf.data_ptr(), x_grad.data_ptr(),
                weight_grad.data_ptr(), int(round_sf), int(swiglu_clamp_value is not None),
                0.0 if swiglu_clamp_value is None else float(swiglu_clamp_value), _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_swiglu_backward_per_token_cast')
    return out, (x_grad_fp8, x_grad_fp8_sf), x_grad, weight_grad
