"""ctypes access to the scalar C checker in oracle/quant_ref.c (TEST INFRASTRUCTURE).

Numpy/torch-facing wrappers around ``tkref_cast`` / ``tkref_swiglu`` and the two encoders.  Only
tests, the smoke check and the benchmark's CPU-baseline leg may import this module.
"""
import ctypes
import os
import subprocess
from typing import Optional

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, '_build', 'libtkref.so')
_lib = None


def build(force: bool = False) -> str:
    """Compile the checker with gcc (seconds).  Returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(['make', '-C', _HERE] + (['-B'] if force else []), check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, f32, i32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
        L.tkref_cast.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, f32, vp, vp, vp]
        L.tkref_cast.restype = i32
        L.tkref_swiglu.argtypes = [vp, i32, i64, i64, vp, vp, vp, i32, f32, vp, vp]
        L.tkref_swiglu.restype = i32
        L.tkref_e4m3_encode_n.argtypes = [vp, i64, vp]
        L.tkref_e2m1_encode_n.argtypes = [vp, i64, vp]
        L.tkref_swiglu_backward.argtypes = [vp, vp, i64, i64, i32, vp, vp, i64, vp, i32, f32, vp, vp, vp]
        L.tkref_swiglu_backward.restype = i32
        L.tkref_fmaf_n.argtypes = [vp, vp, vp, i64, vp]
        L.tkref_count_div_mismatches.argtypes = [f32, ctypes.c_uint32, ctypes.c_uint32, i32]
        L.tkref_count_div_mismatches.restype = i64
        _lib = L
    return _lib


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def e4m3_encode(v: np.ndarray) -> np.ndarray:
    v = np.ascontiguousarray(v, dtype=np.float32)
    out = np.empty(v.shape, dtype=np.uint8)
    lib().tkref_e4m3_encode_n(v.ctypes.data, v.size, out.ctypes.data)
    return out


def e2m1_encode(v: np.ndarray) -> np.ndarray:
    v = np.ascontiguousarray(v, dtype=np.float32)
    out = np.empty(v.shape, dtype=np.uint8)
    lib().tkref_e2m1_encode_n(v.ctypes.data, v.size, out.ctypes.data)
    return out


def cast(x: torch.Tensor, fmt: str, block_size, sf: Optional[torch.Tensor] = None, round_sf: bool = False,
         amax_floor: Optional[float] = None):
    """Returns (codes uint8 [M, K or K/2], scales fp32 [nm, nk] row-major) or codes alone when
    ``sf`` is given.  ``x`` may have a row stride larger than K."""
    assert x.device.type == 'cpu' and x.dim() == 2 and x.stride(1) == 1
    assert x.dtype in (torch.bfloat16, torch.float32)
    M, K = x.shape
    bm, bk = block_size
    fp4 = fmt == 'e2m1'
    nm, nk = -(-M // bm), -(-K // bk)
    codes = torch.zeros((M, K // 2 if fp4 else K), dtype=torch.uint8)
    sf_out = torch.zeros((nm, nk), dtype=torch.float32)
    given = None
    if sf is not None:
        given = sf.to(torch.float32).contiguous()
        assert tuple(given.shape) == (nm, nk)
    rc = lib().tkref_cast(_ptr(x), int(x.dtype == torch.float32), M, K, x.stride(0) if M > 1 else max(K, 1), bm, bk,
                          int(fp4), int(round_sf), -1.0 if amax_floor is None else float(amax_floor),
                          _ptr(given), _ptr(codes), _ptr(sf_out))
    assert rc == 0
    return codes if sf is not None else (codes, sf_out)


def swiglu_forward(x: torch.Tensor, pos_to_token_topk=None, topk_weights=None, swiglu_clamp_value=None,
                   clamped_count=None, pos_to_expert=None) -> torch.Tensor:
    assert x.device.type == 'cpu' and x.dim() == 2 and x.is_contiguous()
    R, H2 = x.shape
    H = H2 // 2
    out = torch.empty((R, H), dtype=torch.float32)
    w = None if topk_weights is None else topk_weights.to(torch.float32).contiguous()
    p = None if pos_to_token_topk is None else pos_to_token_topk.to(torch.int32).contiguous()
    e = None if pos_to_expert is None else pos_to_expert.to(torch.int32).contiguous()
    if clamped_count is not None:
        assert clamped_count.dtype == torch.int64 and clamped_count.is_contiguous()
    rc = lib().tkref_swiglu(_ptr(x), int(x.dtype == torch.float32), R, H, _ptr(p), _ptr(w), _ptr(e),
                            int(swiglu_clamp_value is not None),
                            0.0 if swiglu_clamp_value is None else float(swiglu_clamp_value),
                            _ptr(clamped_count), _ptr(out))
    assert rc == 0
    return out


def count_div_mismatches(c: float, lo_bits: int, hi_bits: int, uncorrected: bool = False) -> int:
    """Positive floats in [lo_bits, hi_bits) (bit patterns) where a*y + fma(-c, a*y, a)*y != a/c
    (``uncorrected``: where a*y alone != a/c)."""
    return int(lib().tkref_count_div_mismatches(c, lo_bits, hi_bits, int(uncorrected)))


def swiglu_backward(x, grad_out: torch.Tensor, weight: torch.Tensor, pos_to_token_topk: torch.Tensor,
                    num_per_channels: int, swiglu_clamp_value=None):
    """Returns fp32 ``(out [R, H], x_grad [R, 2H], weight_grad like weight)``."""
    codes, sf = x
    codes = codes.view(torch.uint8).contiguous()
    R, H2 = codes.shape
    H = H2 // 2
    sf = sf.to(torch.float32).contiguous()
    assert grad_out.dtype == torch.bfloat16 and grad_out.is_contiguous() and tuple(grad_out.shape) == (R, H)
    w = weight.to(torch.float32).contiguous()
    p = pos_to_token_topk.to(torch.int32).contiguous()
    out = torch.empty((R, H), dtype=torch.float32)
    x_grad = torch.empty((R, H2), dtype=torch.float32)
    w_grad = torch.empty_like(w)
    rc = lib().tkref_swiglu_backward(_ptr(codes), _ptr(sf), R, H, num_per_channels, _ptr(grad_out), _ptr(w), w.numel(),
                                     _ptr(p), int(swiglu_clamp_value is not None),
                                     0.0 if swiglu_clamp_value is None else float(swiglu_clamp_value),
                                     _ptr(out), _ptr(x_grad), _ptr(w_grad))
    assert rc == 0
    return out, x_grad, w_grad


def fmaf(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    a, b, c = (np.ascontiguousarray(t, dtype=np.float32) for t in (a, b, c))
    out = np.empty(a.shape, dtype=np.float32)
    lib().tkref_fmaf_n(a.ctypes.data, b.ctypes.data, c.ctypes.data, a.size, out.ctypes.data)
    return out
