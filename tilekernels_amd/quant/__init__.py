from .cast_back import cast_back, per_token_cast_back
from .common import unpack_from_e2m1fn_x2
from .per_block_cast import per_block_cast, per_block_cast_with_precomputed_sf, per_block_cast_with_sf_only
from .per_block_cast_lossless import per_block_cast_lossless
from .per_channel_cast import (per_channel_cast, per_channel_cast_and_transpose, per_channel_cast_fused,
                               swiglu_forward_and_per_channel_cast_and_transpose)
from .per_token_cast import per_token_cast, per_token_cast_with_precomputed_sf, per_token_cast_with_sf_only
from .swiglu_backward_and_per_token_cast import swiglu_backward_and_per_token_cast
from .swiglu_forward_and_per_token_cast import swiglu_forward_and_per_token_cast
from .types import QuantTensor

__all__ = [
    'QuantTensor', 'per_token_cast', 'per_token_cast_with_sf_only', 'per_token_cast_with_precomputed_sf',
    'per_block_cast', 'per_block_cast_with_sf_only', 'per_block_cast_with_precomputed_sf', 'per_block_cast_lossless',
    'swiglu_forward_and_per_token_cast', 'swiglu_backward_and_per_token_cast', 'unpack_from_e2m1fn_x2', 'cast_back', 'per_token_cast_back',
    'per_channel_cast', 'per_channel_cast_fused', 'per_channel_cast_and_transpose',
    'swiglu_forward_and_per_channel_cast_and_transpose',
]
