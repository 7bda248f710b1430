"""Expert-major MoE layout helpers on either side of the fused SwiGLU op (the reference keeps them in
``tile_kernels.moe``): only the mapping and the expansion are provided."""
from .expand_to_fused import expand_to_fused, expand_to_fused_with_sf
from .get_fused_mapping import get_fused_mapping

__all__ = ['get_fused_mapping', 'expand_to_fused', 'expand_to_fused_with_sf']
