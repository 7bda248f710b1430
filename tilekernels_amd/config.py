"""Compute-unit knob, with the reference's names (tile_kernels/config.py:7-23): a "SM" here is a
CDNA compute unit.  It only caps the workgroup count of the clamp-counting SwiGLU variant."""
import functools

import torch

_num_sms = 0


@functools.lru_cache(maxsize=None)
def get_device_num_sms() -> int:
    return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count


def set_num_sms(num_sms: int) -> None:
    global _num_sms
    assert 0 < num_sms <= get_device_num_sms()
    _num_sms = num_sms


def get_num_sms() -> int:
    return _num_sms if _num_sms else get_device_num_sms()
