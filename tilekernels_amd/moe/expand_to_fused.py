"""Host side of tk_expand_to_fused; signatures follow tile_kernels/moe/expand_to_fused_kernel.py:94-200."""
import torch

from .. import _ffi
from ..quant.types import QuantTensor
from ..utils import align, ceil_div


def expand_to_fused(x: torch.Tensor, token_topk_to_pos: torch.Tensor, pos_to_expert: torch.Tensor) -> torch.Tensor:
    """Copy row ``t`` of ``x`` to every expanded position ``token_topk_to_pos[t, k] >= 0``; padding rows
    (``pos_to_expert < 0``) are zero."""
    assert x.is_contiguous() and token_topk_to_pos.is_contiguous()
    assert x.dim() == 2 and token_topk_to_pos.dim() == 2
    assert token_topk_to_pos.dtype == torch.int32 and pos_to_expert.dtype == torch.int32 and pos_to_expert.is_contiguous()
    num_tokens, hidden = x.shape
    num_tokens_, num_topk = token_topk_to_pos.shape
    num_expanded_tokens = pos_to_expert.shape[0]
    assert num_tokens == num_tokens_
    dev = _ffi.require_gpu(x, token_topk_to_pos, pos_to_expert)
    lib = _ffi.load()
    out = torch.empty((num_expanded_tokens, hidden), dtype=x.dtype, device=dev)
    if num_tokens > 0:
        with _ffi.on_device(dev):
            rc = lib.tk_expand_to_fused(x.data_ptr(), num_tokens, hidden * x.element_size(), token_topk_to_pos.data_ptr(), num_topk,
                                        pos_to_expert.data_ptr(), num_expanded_tokens, out.data_ptr(), 0, 0, 0, 0, 0,
                                        _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_expand_to_fused')
    return out


def expand_to_fused_with_sf(x: QuantTensor, num_per_channels: int, token_topk_to_pos: torch.Tensor,
                            pos_to_expert: torch.Tensor, use_tma_aligned_col_major_sf: bool = False):
    """:func:`expand_to_fused` for codes plus their (contiguous, row-per-token) scale rows; the expanded
    scales are row-major or, with ``use_tma_aligned_col_major_sf``, column-major over a 4-row-aligned buffer."""
    x, x_sf = x
    assert x.is_contiguous() and x_sf.is_contiguous() and token_topk_to_pos.is_contiguous() and pos_to_expert.is_contiguous()
    assert x.dim() == 2 and token_topk_to_pos.dim() == 2 and pos_to_expert.dim() == 1
    assert x_sf.dtype in (torch.float32, torch.int32)
    assert token_topk_to_pos.dtype == torch.int32 and pos_to_expert.dtype == torch.int32
    assert num_per_channels in [32, 128]

    num_tokens, hidden = x.shape
    num_topk = token_topk_to_pos.shape[1]
    num_expanded_tokens = pos_to_expert.shape[0]
    assert num_tokens == token_topk_to_pos.shape[0]
    assert num_tokens == x_sf.shape[0]
    num_expanded_sf_tokens = align(num_expanded_tokens, 4) if use_tma_aligned_col_major_sf else num_expanded_tokens
    hidden_sf = ceil_div(hidden, num_per_channels)
    if x_sf.dtype == torch.int32:
        hidden_sf = ceil_div(hidden_sf, 4)
        assert use_tma_aligned_col_major_sf
    assert hidden_sf == x_sf.shape[1]
    dev = _ffi.require_gpu(x, x_sf, token_topk_to_pos, pos_to_expert)
    lib = _ffi.load()

    out = torch.empty((num_expanded_tokens, hidden), dtype=x.dtype, device=dev)
    shape = (hidden_sf, num_expanded_sf_tokens) if use_tma_aligned_col_major_sf else (num_expanded_tokens, hidden_sf)
    out_sf = torch.empty(shape, dtype=x_sf.dtype, device=dev)
    ld = shape[1]
    out_sf = out_sf[:, :num_expanded_tokens] if use_tma_aligned_col_major_sf else out_sf
    if num_tokens > 0:
        with _ffi.on_device(dev):
            rc = lib.tk_expand_to_fused(x.data_ptr(), num_tokens, hidden * x.element_size(), token_topk_to_pos.data_ptr(), num_topk,
                                        pos_to_expert.data_ptr(), num_expanded_tokens, out.data_ptr(), x_sf.data_ptr(), hidden_sf,
                                        out_sf.data_ptr(), ld, int(use_tma_aligned_col_major_sf), _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_expand_to_fused')
    return out, (out_sf.T if use_tma_aligned_col_major_sf else out_sf)
