"""Expert-major MoE layout helpers on either side of the fused SwiGLU op (the reference keeps them in
``tile_kernels.moe``): the mapping, the expansion and its inverse, the weighted reduction."""
from .expand_to_fused import expand_to_fused, expand_to_fused_with_sf
from .get_fused_mapping import get_fused_mapping
from .reduce_fused import reduce_fused

__all__ = ['get_fused_mapping', 'expand_to_fused', 'expand_to_fused_with_sf', 'reduce_fused']
