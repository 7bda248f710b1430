"""Lossless FP4 (E2M1) -> FP8 (E4M3) re-blocking: host side of tk_per_block_cast_lossless.

Signature, asserts and return convention follow
tile_kernels/quant/per_block_cast_lossless_kernel.py:150-209.
"""
import torch

from .. import _ffi
from .common import alloc_scaling_factors, cast_epilogue, get_cast_output_config, sf_leading_dim
from .per_token_cast import _input_sf_storage
from .types import QuantTensor


def per_block_cast_lossless(
    x: QuantTensor,
    fmt: str,
    x_block_size: tuple,
    out_block_size: tuple,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
) -> QuantTensor:
    """Re-quantise packed FP4 codes with power-of-two scales per ``x_block_size`` block to FP8 codes with
    power-of-two scales per ``out_block_size`` block without changing any value.  Returns ``(out, out_sf)``."""
    assert isinstance(x, tuple) and isinstance(x_block_size, tuple)
    data, x_sf = x
    assert fmt == 'e4m3' and data.dtype == torch.int8, 'lossless cast only supports e2m1 -> e4m3 input'
    assert data.is_contiguous() and data.dim() == 2
    num_tokens, hidden = data.shape[0], data.shape[1] * 2
    assert hidden % 32 == 0
    out_config = get_cast_output_config(fmt, out_block_size, use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0)
    assert out_block_size[0] % x_block_size[0] == 0 and out_block_size[1] % x_block_size[1] == 0, \
        'Output block size must be multiple of input block size'
    dev = _ffi.require_gpu(data, x_sf)
    lib = _ffi.load()
    out = torch.empty((num_tokens, hidden), dtype=out_config.torch_dtype, device=dev)
    out_sf = alloc_scaling_factors((num_tokens, hidden), out_config, dev)
    if num_tokens > 0:
        store, layout, ld = _input_sf_storage(x_sf)
        with _ffi.on_device(dev):
            rc = lib.tk_per_block_cast_lossless(
                data.data_ptr(), num_tokens, hidden, store.data_ptr(), ld, layout, x_block_size[0], x_block_size[1],
                out.data_ptr(), out_sf.data_ptr(), sf_leading_dim(out_sf), out_config.layout_code,
                out_block_size[0], out_block_size[1], _ffi.current_stream(dev))
        _ffi.check(rc, 'tk_per_block_cast_lossless')
    return out, cast_epilogue(out_sf, num_tokens, hidden, out_config)
