"""Host-side cast configuration and scale-factor ("sf") tensor geometry.

Mirrors what the reference keeps in tile_kernels/quant/common.py:20-193: the output dtype per
format, the three sf layouts and how the sf tensor handed back to the caller is shaped/strided.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from .. import _ffi
from ..utils import align, ceil_div


@dataclass(frozen=True)
class CastOutputConfig:
    fmt: str                                  # 'e4m3' | 'e2m1' | 'e5m6'
    sf_block: tuple                           # (rows, cols) sharing one scale
    use_tma_aligned_col_major_sf: bool = False
    round_sf: bool = False
    use_packed_ue8m0: bool = False
    custom_clamp_min_value: Optional[float] = None

    @property
    def torch_dtype(self) -> torch.dtype:
        # int8 = two E2M1 codes; uint32 = a third of eight packed E5M6 codes (handed back as uint8)
        return {'e4m3': torch.float8_e4m3fn, 'e2m1': torch.int8, 'e5m6': torch.uint32}[self.fmt]

    @property
    def sf_torch_dtype(self) -> torch.dtype:
        return torch.uint8 if self.use_packed_ue8m0 else torch.float32

    @property
    def fmt_code(self) -> int:
        return {'e4m3': _ffi.TK_E4M3, 'e2m1': _ffi.TK_E2M1, 'e5m6': _ffi.TK_E5M6}[self.fmt]

    @property
    def layout_code(self) -> int:
        if self.use_packed_ue8m0:
            return _ffi.TK_SF_COL_UE8M0
        return _ffi.TK_SF_COL_F32 if self.use_tma_aligned_col_major_sf else _ffi.TK_SF_ROW_F32


def get_cast_output_config(fmt, sf_block, use_tma_aligned_col_major_sf=False, round_sf=False,
                           use_packed_ue8m0=False, custom_clamp_min_value=None) -> CastOutputConfig:
    assert fmt in ('e5m6', 'e4m3', 'e2m1')
    # one UE8M0 byte per block only exists as a power-of-two scale in the column-major packed layout
    assert not use_packed_ue8m0 or (use_tma_aligned_col_major_sf and round_sf), \
        'use_packed_ue8m0 needs use_tma_aligned_col_major_sf=True and round_sf=True'
    return CastOutputConfig(fmt, tuple(sf_block), use_tma_aligned_col_major_sf, round_sf, use_packed_ue8m0,
                            custom_clamp_min_value)


def get_sf_shape(shape, config: CastOutputConfig):
    """Storage shape of the sf tensor (before the epilogue's transpose)."""
    nm = ceil_div(shape[0], config.sf_block[0])
    nk = ceil_div(shape[1], config.sf_block[1])
    if config.use_packed_ue8m0:           # 4 exponent bytes of one row sit next to each other
        nm, nk = nm * 4, ceil_div(nk, 4)
    return (nk, nm) if config.use_tma_aligned_col_major_sf else (nm, nk)


def alloc_scaling_factors(shape, out_config: CastOutputConfig, device) -> torch.Tensor:
    """Uninitialised sf storage; column-major rows are padded to 16 bytes."""
    rows, cols = get_sf_shape(shape, out_config)
    padded = cols
    if out_config.use_tma_aligned_col_major_sf:
        padded = align(cols, 16 if out_config.use_packed_ue8m0 else 4)
    buf = torch.empty((rows, padded), dtype=out_config.sf_torch_dtype, device=device)
    return buf[:, :cols] if out_config.use_tma_aligned_col_major_sf else buf


def sf_leading_dim(storage: torch.Tensor) -> int:
    """Distance between storage rows, in elements of the storage dtype (bytes when packed)."""
    if storage.shape[0] == 1:          # a single row's stride is arbitrary; any value >= the row length works
        return max(storage.stride(0), storage.shape[1])
    return storage.stride(0)


def cast_epilogue(out_sf: torch.Tensor, num_tokens: int, hidden: int, config: CastOutputConfig) -> torch.Tensor:
    """Storage -> the tensor handed to the caller: packed bytes viewed as int32 words, column-major
    storage transposed, rows cut to the number of row blocks."""
    if config.use_packed_ue8m0:
        if num_tokens == 0:
            out_sf = torch.empty((out_sf.shape[0], out_sf.shape[1] // 4), dtype=torch.int32, device=out_sf.device)
        else:
            out_sf = out_sf.view(torch.int32)
    if config.use_tma_aligned_col_major_sf:
        out_sf = out_sf.T
    rows = ceil_div(num_tokens, config.sf_block[0])
    return out_sf if out_sf.shape[0] == rows else out_sf[:rows, :]


def unpack_from_e2m1fn_x2(x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Decode packed E2M1 pairs (int8/uint8, even element in the low nibble) to floats; the last
    dimension doubles.  Debug helper, plain torch ops on the tensor's own device."""
    assert x.dtype in (torch.int8, torch.uint8)
    if x.ndim == 0:
        raise ValueError('x must have at least 1 dimension so the last dim can be doubled')
    mags = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
    table = torch.tensor(mags + tuple(-m for m in mags), dtype=torch.float32, device=x.device)
    b = x.view(torch.uint8).to(torch.int64)
    both = torch.stack((table[b & 0xF], table[b >> 4]), dim=-1)
    return both.reshape(*x.shape[:-1], x.shape[-1] * 2).to(out_dtype)
