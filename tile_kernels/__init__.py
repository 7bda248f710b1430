"""Import-path alias: ``import tile_kernels`` resolves to the MI355X implementation.

Code written against the reference's ``tile_kernels.quant`` / ``tile_kernels.config`` /
``tile_kernels.testing`` finds the same names here.  The quantisation package and the MoE layout
helpers next to it (mapping, expansion, weighted reduction) exist; the other sub-packages of the
reference (engram, mhc, transpose, modeling, torch, the rest of moe) are not provided.
"""
import sys

import tilekernels_amd as _impl
from tilekernels_amd import config, moe, quant, testing, utils  # noqa: F401
from tilekernels_amd.config import get_device_num_sms, get_num_sms, set_num_sms  # noqa: F401

for _name in ('config', 'moe', 'quant', 'testing', 'utils'):
    sys.modules[f'{__name__}.{_name}'] = getattr(_impl, _name)
for _name in ('common', 'types'):
    sys.modules[f'{__name__}.quant.{_name}'] = sys.modules[f'tilekernels_amd.quant.{_name}']
for _name in ('numeric', 'quant', 'generator', 'bench'):
    sys.modules[f'{__name__}.testing.{_name}'] = sys.modules[f'tilekernels_amd.testing.{_name}']
