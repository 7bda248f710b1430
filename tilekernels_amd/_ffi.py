"""ctypes binding of libtk_quant.so (the C ABI declared in include/tk_quant.h).

There is deliberately no fallback: if the library has not been built, importing the ops raises.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library links against before the library itself)

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, 'lib', 'libtk_quant.so')

TK_BF16, TK_F32, TK_OUT_E4M3 = 0, 1, 2
TK_E4M3, TK_E2M1, TK_E5M6 = 0, 1, 2
TK_SF_ROW_F32, TK_SF_COL_F32, TK_SF_COL_UE8M0 = 0, 1, 2
TK_CAST_AND_SF, TK_SF_ONLY, TK_CAST_GIVEN_SF = 0, 1, 2

_i64, _i32, _vp, _f32 = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_float

# name -> (restype, argtypes); must list every symbol declared in include/tk_quant.h
SIGNATURES = {
    'tk_per_token_cast': (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    'tk_check_per_token_cast': (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32]),
    'tk_per_token_cast_quantized': (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64, _i32,
                                           _i32, _i32, _i32, _vp]),
    'tk_check_per_token_cast_quantized': (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64,
                                                 _i32, _i32, _i32, _i32]),
    'tk_per_block_cast': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    'tk_check_per_block_cast': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _i32]),
    'tk_swiglu_per_token_cast': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _f32, _vp, _vp, _i64,
                                        _vp, _i32, _f32, _vp, _i32, _vp]),
    'tk_check_swiglu_per_token_cast': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _f32, _vp, _vp,
                                              _i64, _vp, _i32, _f32, _vp]),
    'tk_cast_back': (_i32, [_vp, _i32, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _i32, _vp]),
    'tk_check_cast_back': (_i32, [_vp, _i32, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _i32]),
    'tk_per_block_cast_lossless': (_i32, [_vp, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64, _i32, _i32, _i32, _vp]),
    'tk_check_per_block_cast_lossless': (_i32, [_vp, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64, _i32, _i32, _i32]),
    'tk_reduce_fused': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _vp, _i64, _i32, _vp, _i32, _vp, _vp]),
    'tk_check_reduce_fused': (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _vp, _i64, _i32, _vp, _i32, _vp]),
    'tk_fused_mapping_workspace_bytes': (_i64, [_i64, _i32, _i32]),
    'tk_get_fused_mapping': (_i32, [_vp, _i64, _i32, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    'tk_get_fused_mapping_static': (_i32, [_vp, _i64, _i32, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    'tk_check_get_fused_mapping': (_i32, [_vp, _i64, _i32, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64]),
    'tk_expand_to_fused': (_i32, [_vp, _i64, _i64, _vp, _i32, _vp, _i64, _vp, _vp, _i32, _vp, _i64, _i32, _vp]),
    'tk_check_expand_to_fused': (_i32, [_vp, _i64, _i64, _vp, _i32, _vp, _i64, _vp, _vp, _i32, _vp, _i64, _i32]),
    'tk_swiglu_backward_per_token_cast': (_i32, [_vp, _vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp,
                                                 _i32, _i32, _f32, _vp]),
    'tk_check_swiglu_backward_per_token_cast': (_i32, [_vp, _vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp,
                                                       _vp, _i32, _i32, _f32]),
    'tk_per_channel_cast': (_i32, [_vp, _i32, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _vp]),
    'tk_check_per_channel_cast': (_i32, [_vp, _i32, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32]),
    'tk_stream_floor': (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    'tk_stream_floor_timeline': (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp]),
    'tk_stream_floor_stamp_words': (_i64, [_i64, _i64]),
    'tk_stream_floor_tailed': (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _i64, _i64, _vp]),
    'tk_stream_floor_flat': (_i32, [_vp, _i64, _i32, _vp, _i32, _i32, _vp]),
    'tk_swiglu_cast_variant': (_i32, [_vp, _i64, _i64, _vp, _vp, _i32, _i32, _vp]),
    'tk_strerror': (ctypes.c_char_p, [_i32]),
    'tk_version': (_i32, []),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raises if it has not been built (python -m tilekernels_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f'{LIB_PATH} not found: build it with `python -m tilekernels_amd.build` '
                '(hipcc, gfx950). tilekernels_amd has no CPU or PyTorch fallback.')
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class TkError(RuntimeError):
    pass


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().tk_strerror(status).decode()
        raise TkError(f'{what}: {msg} (status {status})')


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return TK_BF16
    if t.dtype == torch.float32:
        return TK_F32
    raise AssertionError(f'unsupported input dtype {t.dtype}')


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# torch's own accessor of the raw stream handle (what its compiled extensions use): no Stream object per call
_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def current_stream(device: torch.device) -> int:
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _SameDevice:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_SAME_DEVICE = _SameDevice()


def on_device(device: torch.device):
    """Context in which `device` is the current one: a switch only where it is not already."""
    if device.index is not None and device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(device)


def require_gpu(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise TkError('tilekernels_amd runs on the GPU only (got a CPU tensor); there is no CPU path')
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise TkError(f'tensors on different devices: {dev} and {t.device}')
    return dev
