import torch

from ..utils import align, ceil_div


def clear_unused_sf(sf: torch.Tensor, hidden: int, num_per_channels: int) -> torch.Tensor:
    """Packed UE8M0 scales as a byte matrix [rows, align(nk, 4)] with the bytes past the last real
    channel block zeroed (they are unspecified in the reference, tile_kernels/testing/quant.py:6-21)."""
    nk = ceil_div(hidden, num_per_channels)
    flat = sf.contiguous().flatten().view(torch.uint8).view(-1, align(nk, 4))
    flat[:, nk:] = 0
    return flat
