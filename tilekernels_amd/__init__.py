"""tilekernels_amd: MI355X (gfx950) implementation of the tile_kernels.quant FP8/FP4 cast path.

Hand-written HIP kernels behind a C ABI (include/tk_quant.h, lib/libtk_quant.so); this package is
the thin host side with the reference's Python signatures.  GPU only.
"""
from . import config, moe, quant, testing, utils  # noqa: F401
from .config import get_device_num_sms, get_num_sms, set_num_sms  # noqa: F401

__version__ = '0.1.0'
