"""Naming helpers for parametrised tests and benchmark records (tile_kernels/testing/bench.py:59-118)."""
import torch


def dtype_to_str(dtype: torch.dtype) -> str:
    return {torch.bfloat16: 'bf16', torch.float32: 'fp32', torch.float16: 'fp16', torch.float8_e4m3fn: 'e4m3',
            torch.int8: 'int8', torch.int32: 'int32'}.get(dtype, str(dtype).replace('torch.', ''))


def _format_value(value) -> str:
    if isinstance(value, torch.dtype):
        return dtype_to_str(value)
    if isinstance(value, bool):
        return str(int(value))
    if isinstance(value, (tuple, list)):
        return 'x'.join(_format_value(v) for v in value)
    return str(value)


def make_param_id(params: dict) -> str:
    """pytest id of one parameter dict: ``key=value`` pairs joined by dashes."""
    return '-'.join(f'{k}={_format_value(v)}' for k, v in params.items()) if params else 'default'


def make_param_key(params: dict) -> str:
    """Key of a benchmark record: the non-None parameters, comma separated."""
    return ','.join(f'{k}={_format_value(v)}' for k, v in params.items() if v is not None)
