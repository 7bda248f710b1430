"""CPU oracle for the FP8/FP4 quantisation path (TEST INFRASTRUCTURE, not product code).

This module restates, with plain PyTorch CPU ops, the arithmetic of the reference's
pure-torch implementations:

* ``cast`` / ``cast_back``      <- tile_kernels/torch/cast.py:62-221 and :40-59
* ``swiglu_forward``            <- tile_kernels/torch/swiglu.py:9-88
* ``swiglu_backward``           <- tile_kernels/torch/swiglu.py:90-227
* ``per_channel_cast_fused``    <- tile_kernels/torch/per_channel_cast_fused.py:9-46
* ``unpack_from_e2m1fn_x2``     <- tile_kernels/quant/common.py:247-295
* ``encode_e2m1``               <- tile_kernels/torch/cast.py:224-252 (same result, closed form)
* ``cast_to_e5m6`` / ``cast_back_from_e5m6`` <- tile_kernels/torch/cast_e5m6.py:145-258
* ``reduce_fused``              <- tile_kernels/torch/reduce_fused.py:14-72
* ``per_block_cast_lossless``   <- tile_kernels/quant/per_block_cast_lossless_kernel.py:20-147 (the reference has no
  torch statement of it; its test states the property, tests/quant/test_per_block_cast_lossless.py:90-104)

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
it.  The shipped package never does: it has no CPU path at all.

How each function is pinned (all pins live in tests/test_oracle_*.py and run without a GPU):

* E4M3 encoding goes through ``Tensor.to(torch.float8_e4m3fn)``; it is checked against an
  independent nearest-ties-to-even search over the 256-entry OCP E4M3FN value table for every
  bf16 bit pattern and for fp32 midpoints/neighbours, plus hand known answers.
* ``encode_e2m1`` is a threshold formula; it is checked against a brute-force nearest/ties-to-
  even-code search over the 16-entry E2M1 table and against hand known answers.
* scale arithmetic is checked against closed forms (amax 448 -> 1.0, zero group -> clamp/448,
  the integer identity for power-of-two rounding over every exponent).
* block geometry / partial blocks / scale layouts are checked against a naive Python double
  loop on tiny inputs and against stride/shape invariants.
* the whole of ``cast`` is cross-checked bit-for-bit against the independent scalar C
  restatement in oracle/quant_ref.c.
* ``swiglu_forward`` is checked against float64 evaluation and ``torch.nn.functional.silu``.
* ``per_channel_cast_fused`` and the two transposing compositions reduce to ``cast`` with block
  (N, 1); that geometry is checked against a naive column loop and the C restatement, the gather
  against hand-built index lists.
* ``swiglu_backward`` is checked against float64 autograd of ``silu(g) * u * w`` (a dropped term,
  a wrong sign or swapped halves fails it), against hand-set clamp cases, and its ``fma_f32`` helper
  against the C library's correctly rounded ``fmaf`` on operands built to hit double rounding.
* the E5M6 pair: the fp32 -> fp16 round-toward-zero step against a brute-force "largest fp16 magnitude
  not above |x|" search, the 12-bit rounding against an independent nearest-ties-to-even search over
  all 4096 codes for values whose fp16 form is normal, the 96-bit packing against a Python big-integer
  concatenation and hand-built words, the round trip through ``cast_back_from_e5m6``, and the
  reference's three special inputs.  Below the smallest normal fp16 the reference does NOT round to
  nearest (it rounds on bits of the fp32 pattern that are not the ones dropped; cast_e5m6.py:75-81,
  per_token_cast_to_e5m6_kernel.py:49-56): that range is restated from those lines and covered only by
  hand-computed cases, so parity with the reference is unpinned there beyond those cases.
* ``per_block_cast_lossless``: the property the reference tests (dequantising the result equals dequantising
  the input, exactly, on its own kind of data), the closed form of the output exponent (block maximum minus 6, not
  below 0) on hand-built inputs, and the exactness bound (a span of 11 binades) at and beyond its edge.
* ``reduce_fused``: a float64 evaluation (bounds the whole sum), a naive Python loop over tokens and terms built on
  the C library's ``fmaf`` (fixes the order of accumulation and the single rounding per term), hand cases for
  skipped positions, missing weights, row factors, the final scale and each output type.
"""
from typing import Optional, Tuple, Union

import torch

QuantTensor = Tuple[torch.Tensor, torch.Tensor]

E4M3_MAX = 448.0
E2M1_MAX = 6.0
E4M3_AMAX_FLOOR = 1e-4
E2M1_AMAX_FLOOR = 6.0 * 2.0 ** -126
E5M6_MAX = 65024.0            # (2 - 2^-6) * 2^15: the largest fp16 whose low four mantissa bits are zero
E5M6_AMAX_FLOOR = 1e-4

# magnitudes of the eight E2M1 codes, index = 3-bit code (exp:2 | mant:1)
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def _round_up(a: int, b: int) -> int:
    return _ceil_div(a, b) * b


def _fmt_constants(fmt: str):
    if fmt == 'e4m3':
        return torch.float8_e4m3fn, E4M3_MAX, E4M3_AMAX_FLOOR
    if fmt == 'e2m1':
        return torch.int8, E2M1_MAX, E2M1_AMAX_FLOOR
    raise AssertionError(f'unsupported format {fmt}')


def unpack_from_e2m1fn_x2(x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Decode bytes holding two E2M1 codes (even element in the low nibble) to floats.

    Follows tile_kernels/quant/common.py:247-295: code = s(1) e(2) m(1), bias 1.
    """
    assert x.dtype in (torch.int8, torch.uint8) and x.ndim >= 1
    table = torch.tensor(E2M1_VALUES + tuple(-v for v in E2M1_VALUES), dtype=torch.float32, device=x.device)
    b = x.view(torch.uint8).to(torch.int64)
    pair = torch.stack((table[b & 0xF], table[(b >> 4) & 0xF]), dim=-1)
    return pair.reshape(*x.shape[:-1], x.shape[-1] * 2).to(out_dtype)


def encode_e2m1(q: torch.Tensor) -> torch.Tensor:
    """fp32 -> 4-bit E2M1 code (uint8, sign in bit 3), round-to-nearest, ties to the even code,
    saturating at 6.  Same mapping as tile_kernels/torch/cast.py:224-252.

    The seven decision points between neighbouring magnitudes are .25 .75 1.25 1.75 2.5 3.5 5;
    a tie moves up exactly when the upper neighbour has an even code (.75 1.75 3.5).
    """
    assert q.dtype == torch.float32
    a = q.abs()
    code = ((a > 0.25).to(torch.uint8) + (a >= 0.75).to(torch.uint8) + (a > 1.25).to(torch.uint8)
            + (a >= 1.75).to(torch.uint8) + (a > 2.5).to(torch.uint8) + (a >= 3.5).to(torch.uint8)
            + (a > 5.0).to(torch.uint8))
    code = torch.where(torch.isnan(q), torch.full_like(code, 7), code)  # exponent 255 saturates (cast.py:247-249)
    return code | (torch.signbit(q).to(torch.uint8) << 3)


def _sf_as_fp32(sf: torch.Tensor) -> torch.Tensor:
    """Scale tensor in any of the three layouts -> dense row-major fp32 (cast.py:27-37)."""
    if sf.dtype == torch.float32:
        return sf
    assert sf.dtype == torch.int32
    rows, words = sf.shape
    # a [rows, 1] view with strides (1, ld) passes for contiguous, so copy into fresh storage instead
    dense = torch.empty((rows, words), dtype=torch.int32).copy_(sf).view(torch.uint8).reshape(rows, words * 4)
    return (dense.to(torch.int32) << 23).view(torch.float32)


def _dequantise(x: QuantTensor, blk: Tuple[int, int]) -> torch.Tensor:
    codes, sf = x
    assert codes.dtype in (torch.float8_e4m3fn, torch.int8)
    vals = unpack_from_e2m1fn_x2(codes) if codes.dtype == torch.int8 else codes.to(torch.float32)
    scale = _sf_as_fp32(sf).repeat_interleave(blk[0], 0).repeat_interleave(blk[1], 1)
    return vals * scale[: vals.shape[0], : vals.shape[1]]


def cast_back(x: QuantTensor, fmt: str, block_size: Tuple[int, int] = (32, 32)) -> torch.Tensor:
    """Dequantise ``(codes, scales)`` to fp32 or bf16 (tile_kernels/torch/cast.py:40-59)."""
    out = _dequantise(x, block_size)
    return out.to(torch.float32 if fmt == 'fp32' else torch.bfloat16)


def _block_amax(xf: torch.Tensor, bh: int, bw: int) -> torch.Tensor:
    """max |x| over every (bh x bw) block, partial edge blocks over their in-range part only."""
    h, w = xf.shape
    nm, nk = _ceil_div(h, bh), _ceil_div(w, bw)
    canvas = xf.new_zeros((nm * bh, nk * bw))   # |x| >= 0, so zero fill never wins a max it should lose
    canvas[:h, :w] = xf.abs()
    return canvas.view(nm, bh, nk, bw).amax(dim=(1, 3))


def _expand_blocks(t: torch.Tensor, bh: int, bw: int, h: int, w: int) -> torch.Tensor:
    return t.repeat_interleave(bh, 0).repeat_interleave(bw, 1)[:h, :w]


def _format_sf(sf_bits: torch.Tensor, col_major: bool, packed: bool) -> torch.Tensor:
    """int32 bit patterns of the per-block dequant scales [nm, nk] -> returned scale tensor.

    Layouts (tile_kernels/torch/cast.py:201-219, tile_kernels/quant/common.py:130-193):
      row-major : fp32 [nm, nk] contiguous
      col-major : fp32 [nm, nk], strides (1, round_up(nm, 4))
      packed    : int32 [nm, ceil(nk/4)], strides (1, round_up(nm, 4)); byte t of word [m, j] is the
                  biased exponent of group 4j+t, zero beyond nk

    One deliberate deviation from the torch statement this file restates: for a single column (nk == 1, or one
    packed word) tile_kernels/torch/cast.py:216 returns strides (1, 1), because ``.T.contiguous().T`` of a
    one-column tensor keeps row-major strides, while the reference's kernel path returns a transposed view of its
    ``[nk, round_up(nm, 4)]`` storage, i.e. (1, round_up(nm, 4)) (tile_kernels/quant/common.py:141-165, 186-193).
    This function returns the kernel path's strides for every nk, so that one rule describes the layout; values
    and shape are the same either way, and the reference's tests flatten both sides before they compare.
    """
    nm, nk = sf_bits.shape
    if not col_major:
        return sf_bits.view(torch.float32)
    ld = _round_up(nm, 4)
    if packed:
        nw = _ceil_div(nk, 4)
        expo = torch.zeros((ld, nw * 4), dtype=torch.uint8)
        expo[:nm, :nk] = (sf_bits >> 23).to(torch.uint8)
        words = expo.view(torch.int32)                       # [ld, nw], little endian byte t = group 4j+t
        store = torch.zeros((nw, ld), dtype=torch.int32)
        store.copy_(words.T)
        return store.T[:nm]
    store = torch.zeros((nk, ld), dtype=torch.float32)
    store[:, :nm] = sf_bits.view(torch.float32).T
    return store.T[:nm]


def cast(
    x: Union[torch.Tensor, QuantTensor],
    fmt: str,
    block_size: Tuple[int, int] = (32, 32),
    sf: Optional[torch.Tensor] = None,
    x_block_size: Optional[Tuple[int, int]] = None,
    round_sf: bool = False,
    use_tma_aligned_col_major_sf: bool = False,
    use_packed_ue8m0: bool = False,
    amax_floor: Optional[float] = None,
) -> Union[torch.Tensor, QuantTensor]:
    """Quantise a 2-D tensor to E4M3 or packed E2M1 with one scale per (bh x bw) block.

    Same arguments and results as the reference's ``tile_kernels.torch.cast``
    (tile_kernels/torch/cast.py:62-221).  ``amax_floor`` additionally lets a caller override the
    lower clamp of the block amax, which the fused SwiGLU op exposes as ``sf_clamp_min``
    (tile_kernels/quant/swiglu_forward_and_per_token_cast_kernel.py:234-236).
    """
    requant = isinstance(x, tuple)
    if requant:
        assert x_block_size is not None
        xf = _dequantise(x, x_block_size)
    else:
        assert x.dtype in (torch.bfloat16, torch.float32)
        xf = x.to(torch.float32)
    assert xf.ndim == 2
    h, w = xf.shape
    bh, bw = block_size
    code_dtype, qmax, floor = _fmt_constants(fmt)
    if amax_floor is not None:
        floor = amax_floor
    fp4 = fmt == 'e2m1'
    nm, nk = _ceil_div(h, bh), _ceil_div(w, bw)

    if h == 0:   # cast.py:110-123
        codes = torch.empty((0, w // 2 if fp4 else w), dtype=code_dtype)
        if sf is not None:
            return codes
        if use_packed_ue8m0:
            return codes, torch.empty((_ceil_div(nk, 4), 0), dtype=torch.int32).T
        if use_tma_aligned_col_major_sf:
            return codes, torch.empty((nk, 0), dtype=torch.float32).T
        return codes, torch.empty((0, nk), dtype=torch.float32)

    if fp4:
        assert w % 2 == 0

    if sf is None:
        amax = _block_amax(xf, bh, bw).clamp(min=floor)
        qmax_t = torch.full_like(amax, qmax)
        dq = amax / qmax_t                                   # one correctly rounded division (cast.py:151-154)
        if round_sf:
            # next power of two >= dq, by carrying the mantissa into the exponent (cast.py:158-161)
            bits = (dq.view(torch.int32) + 0x007FFFFF) & 0x7F800000
            dq_r = bits.view(torch.float32)
            inv = torch.where(dq_r == 0, torch.zeros_like(dq_r), 1.0 / dq_r)
        else:
            bits = dq.view(torch.int32)
            inv = torch.where(bits == 0, torch.zeros_like(dq), qmax_t / amax)   # cast.py:163-164
    else:
        assert not use_packed_ue8m0 and not use_tma_aligned_col_major_sf
        assert sf.ndim == 2 and tuple(sf.shape) == (nm, nk), f'scale shape {tuple(sf.shape)} != {(nm, nk)}'
        inv = sf.reciprocal()                                # cast.py:165-170

    q = xf * _expand_blocks(inv, bh, bw, h, w)

    if fp4:
        nib = encode_e2m1(q).view(h, w // 2, 2)
        codes = (nib[..., 0] | (nib[..., 1] << 4)).view(torch.int8)     # cast.py:192-196
    else:
        codes = q.clamp(-qmax, qmax).to(code_dtype)                      # cast.py:188-190

    if sf is not None:
        return codes
    return codes, _format_sf(bits, use_tma_aligned_col_major_sf, use_packed_ue8m0)


def swiglu_forward(
    x: torch.Tensor,
    pos_to_token_topk: Optional[torch.Tensor] = None,
    topk_weights: Optional[torch.Tensor] = None,
    swiglu_clamp_value: Optional[float] = None,
    clamped_count: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """fp32 ``silu(x[:, :H]) * x[:, H:]`` with optional clamp, clamp counters and per-row routing
    weight; padding rows (``pos_to_token_topk < 0``) get weight 0.

    Same arguments and results as ``tile_kernels.torch.swiglu_forward``
    (tile_kernels/torch/swiglu.py:9-88); the operation order ``g / (1 + exp(-g)) * u * w`` is kept
    because it fixes the fp32 roundings.
    """
    assert x.dim() == 2 and x.is_contiguous()
    assert x.dtype in (torch.bfloat16, torch.float32)
    rows, two_h = x.shape
    assert two_h % 2 == 0
    hid = two_h // 2
    xf = x.to(torch.float32)
    gate, up = xf[:, :hid], xf[:, hid:]

    if swiglu_clamp_value is not None:
        c = swiglu_clamp_value
        if clamped_count is not None:   # counted before clamping, over every row (swiglu.py:66-70)
            clamped_count += torch.stack(((gate > c).sum(), (up > c).sum(), (up < -c).sum())).to(clamped_count.dtype)
        gate = gate.clamp(max=c)
        up = up.clamp(min=-c, max=c)

    out = gate / (1.0 + torch.exp(-gate)) * up

    if pos_to_token_topk is not None:
        assert pos_to_token_topk.dim() == 1 and pos_to_token_topk.shape[0] == rows
        assert topk_weights is not None and topk_weights.dim() == 2
        flat_w = topk_weights.reshape(-1).to(torch.float32)
        live = pos_to_token_topk >= 0
        w = torch.zeros(rows, dtype=torch.float32)
        w[live] = flat_w[pos_to_token_topk[live].long()]
        out = out * w[:, None]
    return out


def swiglu_forward_and_per_token_cast(
    x: torch.Tensor,
    fmt: str,
    num_per_channels: int,
    pos_to_token_topk: Optional[torch.Tensor] = None,
    topk_weights: Optional[torch.Tensor] = None,
    pos_to_expert: Optional[torch.Tensor] = None,
    use_tma_aligned_col_major_sf: bool = False,
    round_sf: bool = False,
    use_packed_ue8m0: bool = False,
    swiglu_clamp_value: Optional[float] = None,
    clamped_count: Optional[torch.Tensor] = None,
    sf_clamp_min: Optional[float] = None,
):
    """Composition the reference's own test uses as ground truth for the fused op
    (tests/quant/test_swiglu_forward_and_per_token_cast.py:91-128): SwiGLU, zero the rows whose
    ``pos_to_expert`` is -1, per-token cast, then codes and scales of those rows forced to zero.

    Returns ``(codes, scales)`` with masked rows zeroed, i.e. what the device op must produce.
    """
    v = swiglu_forward(x, pos_to_token_topk, topk_weights, swiglu_clamp_value, clamped_count)
    dead = None
    if pos_to_expert is not None:
        dead = (pos_to_expert < 0)[:, None]
        v = v.masked_fill(dead, 0)
    codes, sf = cast(v, fmt, (1, num_per_channels), round_sf=round_sf,
                     use_tma_aligned_col_major_sf=use_tma_aligned_col_major_sf,
                     use_packed_ue8m0=use_packed_ue8m0, amax_floor=sf_clamp_min)
    if dead is not None:
        codes.view(torch.uint8).masked_fill_(dead, 0)
        sf.masked_fill_(dead, 0)          # in place: keeps the column-major strides
    return codes, sf


def fma_f32(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """Correctly rounded fp32 ``a * b + c`` (one rounding), elementwise.

    The reference evaluates ``x * (1 - s) + 1`` through a compiled helper so that it becomes a single
    fused multiply-add (tile_kernels/torch/swiglu.py:90-95).  Here the product of two fp32 values is
    exact in float64 (48 significant bits); the float64 sum is then forced to round-to-odd with the
    error term of a TwoSum, which makes the final rounding to fp32 the rounding of the exact value.
    """
    p = a.to(torch.float64) * b.to(torch.float64)
    c = c.to(torch.float64).expand_as(p)
    s = p + c
    bb = s - p
    err = (p - (s - bb)) + (c - bb)
    bits = s.contiguous().view(torch.int64).clone()
    fix = (err != 0) & torch.isfinite(s) & ((bits & 1) == 0) & (s != 0)
    grow = (err > 0) == (s > 0)            # the exact value lies further from zero than s
    bits = torch.where(fix, torch.where(grow, bits + 1, bits - 1), bits)
    return bits.view(torch.float64).to(torch.float32)


def swiglu_backward(
    x: QuantTensor,
    grad_out: torch.Tensor,
    weight: torch.Tensor,
    pos_to_token_topk: torch.Tensor,
    token_topk_to_pos: torch.Tensor,
    num_per_channels: int,
    swiglu_clamp_value: Optional[float] = None,
):
    """Backward of ``out = silu(g) * u * w`` on the dequantised forward input, in fp32.

    Same arguments and results as ``tile_kernels.torch.swiglu_backward``
    (tile_kernels/torch/swiglu.py:98-227): ``(out, x_grad_full, weight_grad)`` with
    ``x_grad_full = [d/dgate | d/dup]``.  Every product below is one fp32 rounding, in the
    reference's order; the only fused operation is ``fma(g, 1 - s, 1)``.
    """
    codes, sf = x
    assert num_per_channels in (32, 128)
    assert codes.dtype == torch.float8_e4m3fn and codes.is_contiguous()
    assert sf.dim() == 2 and sf.is_contiguous() and sf.dtype == torch.float32
    assert weight.dim() == 2 and weight.is_contiguous()
    assert pos_to_token_topk.dim() == 1
    assert token_topk_to_pos.dim() == 2 and token_topk_to_pos.is_contiguous()
    assert codes.size(-1) % (2 * num_per_channels) == 0
    hid = codes.size(-1) // 2
    codes = codes.view(-1, 2 * hid)
    grad_out = grad_out.view(-1, hid)
    rows = codes.size(0)
    num_tokens, num_topk = token_topk_to_pos.shape
    assert sf.shape == (rows, 2 * hid // num_per_channels)
    assert grad_out.shape == (rows, hid)
    assert weight.shape == (num_tokens, num_topk)
    assert pos_to_token_topk.shape == (rows,)

    xf = codes.to(torch.float32) * sf.repeat_interleave(num_per_channels, dim=1)
    gate, up = xf[:, :hid].clone(), xf[:, hid:].clone()

    gate_clamped = up_clamped = None
    if swiglu_clamp_value is not None:
        c = swiglu_clamp_value
        gate_clamped = gate > c
        up_hi, up_lo = up > c, up < -c
        up_clamped = up_hi | up_lo
        gate[gate_clamped] = c
        up[up_hi] = c
        up[up_lo] = -c

    denom = 1.0 + torch.exp(-gate)
    sig = torch.ones_like(gate) / denom

    live = pos_to_token_topk >= 0
    idx = pos_to_token_topk[live].long()
    w = torch.zeros(rows, dtype=torch.float32)
    w[live] = weight.reshape(-1).to(torch.float32)[idx]

    go = grad_out.to(torch.float32)
    go_ws = go * w[:, None] * sig
    gate_grad = go_ws * up * fma_f32(gate, 1.0 - sig, torch.ones((), dtype=torch.float32))
    up_grad = go_ws * gate
    if swiglu_clamp_value is not None:
        gate_grad[gate_clamped] = 0.0
        up_grad[up_clamped] = 0.0

    act = gate / denom * up
    out = act * w[:, None]

    weight_grad = torch.zeros_like(weight)
    dots = (go * act).sum(dim=1)
    weight_grad.view(-1)[idx] = dots[live]
    return out, torch.cat([gate_grad, up_grad], dim=1), weight_grad


def swiglu_backward_and_per_token_cast(
    x: QuantTensor,
    grad_out: torch.Tensor,
    weight: torch.Tensor,
    pos_to_token_topk: torch.Tensor,
    token_topk_to_pos: torch.Tensor,
    num_per_channels: int,
    round_sf: bool = False,
    swiglu_clamp_value: Optional[float] = None,
):
    """Composition the reference's own test uses as ground truth for the fused backward op
    (tests/quant/test_swiglu_backward_and_per_token_cast.py:78-97): fp32 backward, per-token
    1 x N E4M3 cast of the fp32 input gradient, and bf16 roundings of the output and the gradient.

    Returns ``(out_bf16, (x_grad_codes, x_grad_sf), x_grad_bf16, weight_grad)``.
    """
    out, x_grad, weight_grad = swiglu_backward(x, grad_out, weight, pos_to_token_topk, token_topk_to_pos,
                                               num_per_channels, swiglu_clamp_value)
    q = cast(x_grad, 'e4m3', (1, num_per_channels), round_sf=round_sf)
    return out.to(grad_out.dtype), q, x_grad.to(grad_out.dtype), weight_grad


def per_channel_cast_fused(
    x: Union[torch.Tensor, QuantTensor],
    num_per_tokens: int,
    num_per_channels: Optional[int],
    round_sf: bool,
    pos_to_token: Optional[torch.Tensor],
) -> QuantTensor:
    """Per-channel cast (one scale per ``num_per_tokens`` tokens of a column) with the optional row
    gather and the optional dequantisation of an FP8 input with 1 x ``num_per_channels`` scales.

    Same arguments and results as the reference's torch statement
    (tile_kernels/torch/per_channel_cast_fused.py:9-46): gathered rows with a negative index are
    zero rows (zero codes and zero scales for a quantised input), then ``cast`` with block
    ``(num_per_tokens, 1)``.
    """
    quantised = isinstance(x, tuple)
    if pos_to_token is not None:
        data = x[0] if quantised else x
        idx = pos_to_token.clamp(min=0).long()
        live = (pos_to_token >= 0)[:, None]
        rows = torch.where(live, data[idx].to(torch.float32), torch.zeros((), dtype=torch.float32)).to(data.dtype)
        if quantised:
            sf_rows = torch.where(live, x[1][idx], torch.zeros((), dtype=x[1].dtype))
            x = (rows, sf_rows)
        else:
            x = rows
    return cast(x, 'e4m3', block_size=(num_per_tokens, 1),
                x_block_size=(1, num_per_channels) if quantised else None, round_sf=round_sf)


def per_channel_cast_and_transpose(x: torch.Tensor, num_per_tokens: int, round_sf: bool) -> QuantTensor:
    """What the reference's test expects of the transposing variant
    (tests/quant/test_per_channel_cast_and_transpose.py:45-48): the per-channel cast, codes transposed."""
    codes, sf = cast(x, 'e4m3', block_size=(num_per_tokens, 1), round_sf=round_sf)
    return codes.T.contiguous(), sf


def swiglu_forward_and_per_channel_cast_and_transpose(x: torch.Tensor, num_per_tokens: int, round_sf: bool = False,
                                                      without_transpose: bool = False,
                                                      swiglu_clamp_value: Optional[float] = None) -> QuantTensor:
    """Composition the reference's test uses as ground truth
    (tests/quant/test_swiglu_forward_and_per_channel_cast_and_transpose.py:62-75): SwiGLU in fp32,
    rounded to bf16, per-channel cast, codes transposed unless ``without_transpose``."""
    act = swiglu_forward(x, swiglu_clamp_value=swiglu_clamp_value).to(torch.bfloat16)
    codes, sf = cast(act, 'e4m3', block_size=(num_per_tokens, 1), round_sf=round_sf)
    if not without_transpose:
        codes = codes.T.contiguous()
    return codes, sf


# --------------------------------------------------------------------------------------------------
# MoE expert-major ("fused") layout: the callers on either side of the fused SwiGLU op.

def get_fused_mapping(topk_idx: torch.Tensor, num_experts: int, alignment: int):
    """Maps between the (token, k) list and the expert-major expanded layout.

    Contract of tile_kernels.moe.get_fused_mapping (tile_kernels/moe/get_fused_mapping_kernel.py:166-250)
    as its test states it (tests/moe/test_get_fused_mapping.py:54-78): experts occupy consecutive
    segments, each padded to a multiple of ``alignment`` rows; padding positions hold -1.  The
    reference leaves the order inside a segment unspecified; this statement fixes it as the order of
    the flat (token, k) index (a stable counting sort).

    Returns (pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
    num_tokens_per_expert), all int32; num_tokens_per_expert holds the padded segment lengths.
    """
    assert topk_idx.dim() == 2
    num_tokens, num_topk = topk_idx.shape
    flat = topk_idx.reshape(-1).to(torch.int64)
    live = flat >= 0
    counts = torch.bincount(flat[live], minlength=num_experts)
    padded = (counts + alignment - 1) // alignment * alignment
    ends = torch.cumsum(padded, 0)
    starts = ends - padded
    total = int(ends[-1]) if num_experts else 0
    pos_to_expert = torch.full((total,), -1, dtype=torch.int32)
    pos_to_token = torch.full((total,), -1, dtype=torch.int32)
    pos_to_token_topk = torch.full((total,), -1, dtype=torch.int32)
    token_topk_to_pos = torch.full((num_tokens * num_topk,), -1, dtype=torch.int32)
    idx = torch.nonzero(live).flatten()
    order = idx[torch.argsort(flat[idx], stable=True)]          # grouped by expert, flat index ascending inside
    experts = flat[order]
    rank = torch.arange(order.numel()) - (torch.cumsum(counts, 0) - counts)[experts]
    pos = starts[experts] + rank
    pos_to_expert[pos] = experts.to(torch.int32)
    pos_to_token[pos] = (order // num_topk).to(torch.int32)
    pos_to_token_topk[pos] = order.to(torch.int32)
    token_topk_to_pos[order] = pos.to(torch.int32)
    return (pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos.view(num_tokens, num_topk),
            starts.to(torch.int32), ends.to(torch.int32), padded.to(torch.int32))


def expand_to_fused(x: torch.Tensor, token_topk_to_pos: torch.Tensor, pos_to_expert: torch.Tensor) -> torch.Tensor:
    """Row t of ``x`` is copied to every position token_topk_to_pos[t, k] >= 0; all other rows of the
    expanded tensor are zero (tile_kernels/torch/expand_to_fused.py:6-39)."""
    num_tokens, hidden = x.shape
    out = torch.zeros((pos_to_expert.shape[0], hidden), dtype=x.dtype)
    num_topk = token_topk_to_pos.shape[1]
    pos = token_topk_to_pos.reshape(-1).long()
    src = torch.arange(num_tokens).repeat_interleave(num_topk)
    keep = pos >= 0
    as_bytes = out.view(torch.uint8)                 # index_copy on raw bytes: works for fp8 / int8 alike
    as_bytes[pos[keep]] = x.view(torch.uint8)[src[keep]]
    return out


def expand_to_fused_with_sf(x: QuantTensor, num_per_channels: int, token_topk_to_pos: torch.Tensor,
                            pos_to_expert: torch.Tensor, use_tma_aligned_col_major_sf: bool = False):
    """Same expansion for codes and their row-major scale rows; the expanded scales come back
    row-major, or column-major over a 4-row-aligned buffer (tile_kernels/torch/expand_to_fused.py:42-91)."""
    data, sf = x
    out = expand_to_fused(data, token_topk_to_pos, pos_to_expert)
    num_expanded = pos_to_expert.shape[0]
    cols = sf.shape[1]
    if use_tma_aligned_col_major_sf:
        store = torch.zeros((cols, _round_up(num_expanded, 4)), dtype=sf.dtype)
        out_sf = store[:, :num_expanded].T
    else:
        out_sf = torch.zeros((num_expanded, cols), dtype=sf.dtype)
    num_topk = token_topk_to_pos.shape[1]
    pos = token_topk_to_pos.reshape(-1).long()
    src = torch.arange(data.shape[0]).repeat_interleave(num_topk)
    keep = pos >= 0
    out_sf[pos[keep]] = sf[src[keep]]
    return out, out_sf


# ------------------------------------------------------------------------------------------------
# E5M6: a 12-bit float (sign, 5 exponent bits, 6 mantissa bits) = the top 12 bits of an IEEE fp16.
# Eight codes are stored as three 32-bit words.

def fp16_bits_toward_zero(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> the bit pattern (int32, 0..0xFFFF) of the fp16 nearest to zero-ward of it: finite values
    beyond the fp16 range become infinity, NaNs 0x7FFF (tile_kernels/torch/cast_e5m6.py:37-62)."""
    bits = x.contiguous().view(torch.int32)
    mag = bits & 0x7FFFFFFF
    e, m = mag >> 23, mag & 0x7FFFFF
    sig = m | 0x800000                                          # significand with its leading one
    out = torch.zeros_like(mag)
    normal = (e >= 113) & (e <= 142)
    out = torch.where(normal, ((e - 112) << 10) | (m >> 13), out)
    sub = (e >= 103) & (e <= 112)                               # fp16 subnormals: 2^-24 .. 2^-14
    out = torch.where(sub, sig >> (126 - e).clamp(0, 31), out)
    out = torch.where(e > 142, torch.full_like(out, 0x7C00), out)
    out = torch.where(mag > 0x7F800000, torch.full_like(out, 0x7FFF), out)
    return out | ((bits >> 16) & 0x8000)


def encode_e5m6(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> 12-bit E5M6 codes (int32).  The fp16 pattern is cut to 12 bits and bumped when
    (kept lsb) + (low 17 bits of the fp32 pattern) exceeds 0x10000 (cast_e5m6.py:75-81): round to
    nearest, ties to even, wherever the fp16 form is normal."""
    bits = x.contiguous().view(torch.int32)
    kept = fp16_bits_toward_zero(x) >> 4
    bump = ((kept & 1) + (bits & 0x1FFFF)) > 0x10000
    return (kept + bump.to(torch.int32)) & 0xFFF


def pack_e5m6(codes: torch.Tensor) -> torch.Tensor:
    """[M, K] codes -> uint8 [M, K * 3 // 2]: each 8 codes form a 96-bit string, first code in the
    most significant bits, stored as three little-endian 32-bit words from the high word down
    (cast_e5m6.py:83-101)."""
    m, k = codes.shape
    c = codes.to(torch.int64).view(m, k // 8, 8)
    hi = (c[..., 0] << 36) | (c[..., 1] << 24) | (c[..., 2] << 12) | c[..., 3]      # 48 bits
    lo = (c[..., 4] << 36) | (c[..., 5] << 24) | (c[..., 6] << 12) | c[..., 7]
    words = torch.stack([hi >> 16, ((hi & 0xFFFF) << 16) | (lo >> 32), lo & 0xFFFFFFFF], dim=-1)
    signed = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)
    return signed.view(m, k // 8 * 3).view(torch.uint8)


def unpack_e5m6(packed: torch.Tensor) -> torch.Tensor:
    """uint8 [M, K * 3 // 2] -> int32 codes [M, K] (cast_e5m6.py:104-133)."""
    m = packed.shape[0]
    w = packed.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    w = w.view(m, w.shape[1] // 3, 3)
    hi = (w[..., 0] << 16) | (w[..., 1] >> 16)
    lo = ((w[..., 1] & 0xFFFF) << 32) | w[..., 2]
    cols = [(hi >> 36) & 0xFFF, (hi >> 24) & 0xFFF, (hi >> 12) & 0xFFF, hi & 0xFFF,
            (lo >> 36) & 0xFFF, (lo >> 24) & 0xFFF, (lo >> 12) & 0xFFF, lo & 0xFFF]
    return torch.stack(cols, dim=-1).view(m, w.shape[1] * 8).to(torch.int32)


def decode_e5m6(codes: torch.Tensor) -> torch.Tensor:
    """12-bit codes -> fp32 values (the fp16 whose top 12 bits they are)."""
    h = (codes.to(torch.int32) << 4) & 0xFFFF
    h = torch.where(h >= 0x8000, h - 0x10000, h).to(torch.int16)
    return h.view(torch.float16).to(torch.float32)


def cast_to_e5m6(x: torch.Tensor, num_per_channels: int, use_tma_aligned_col_major_sf: bool = False,
                 round_sf: bool = False, use_packed_ue8m0: bool = False) -> QuantTensor:
    """Per-token E5M6 cast with one scale per ``num_per_channels`` channels (the reference's kernel
    takes whole rows only): amax floored at 1e-4, scale = amax / 65024, multiplier 65024 / amax or,
    with ``round_sf``, the inverse of the scale rounded up to a power of two
    (tile_kernels/torch/cast_e5m6.py:145-222).  Returns ``(uint8 [M, K*3/2], scales)``."""
    assert x.ndim == 2 and x.dtype in (torch.float32, torch.bfloat16)
    xf = x.to(torch.float32)
    h, w = xf.shape
    assert w % num_per_channels == 0 and w % 8 == 0
    amax = _block_amax(xf, 1, num_per_channels).clamp(min=E5M6_AMAX_FLOOR)
    qmax = torch.full_like(amax, E5M6_MAX)
    dq = amax / qmax
    if round_sf:
        bits = (dq.view(torch.int32) + 0x007FFFFF) & 0x7F800000
        inv = ((254 - (bits >> 23)).clamp(min=0) << 23).view(torch.float32)      # 2^-(e-127), exactly
    else:
        bits = dq.view(torch.int32)
        inv = qmax / amax
    codes = encode_e5m6(xf * _expand_blocks(inv, 1, num_per_channels, h, w))
    return pack_e5m6(codes), _format_sf(bits.contiguous(), use_tma_aligned_col_major_sf, use_packed_ue8m0)


def cast_back_from_e5m6(x: QuantTensor, fmt: str, block_size: Tuple[int, int]) -> torch.Tensor:
    """``(uint8 [M, K*3/2], scales)`` -> bf16 / fp32 [M, K]: code value times its block's scale, one
    fp32 product (tile_kernels/torch/cast_e5m6.py:225-258)."""
    packed, sf = x
    assert packed.ndim == 2 and packed.dtype == torch.uint8 and fmt in ('bf16', 'fp32')
    h, w = packed.shape[0], packed.shape[1] * 2 // 3
    bh, bw = block_size
    scales = _sf_as_fp32(sf)[:_ceil_div(h, bh), :_ceil_div(w, bw)]
    out = decode_e5m6(unpack_e5m6(packed)) * _expand_blocks(scales, bh, bw, h, w)
    return out.to(torch.float32 if fmt == 'fp32' else torch.bfloat16)


def per_block_cast_lossless(x: QuantTensor, fmt: str, x_block_size: Tuple[int, int], out_block_size: Tuple[int, int],
                            use_tma_aligned_col_major_sf: bool = False, round_sf: bool = False,
                            use_packed_ue8m0: bool = False) -> QuantTensor:
    """Packed E2M1 codes with power-of-two scales per ``x_block_size`` block -> E4M3 codes with power-of-two
    scales per ``out_block_size`` block, every value unchanged: the output exponent is the largest input
    exponent in the block minus 6 (not below 0), each value is shifted by the difference
    (tile_kernels/quant/per_block_cast_lossless_kernel.py:104-134)."""
    codes, sf = x
    assert fmt == 'e4m3' and codes.dtype == torch.int8
    vals = unpack_from_e2m1fn_x2(codes)
    h, w = vals.shape
    (ibm, ibk), (obm, obk) = x_block_size, out_block_size
    assert obm % ibm == 0 and obk % ibk == 0
    e_in = (_sf_as_fp32(sf).contiguous().view(torch.int32) >> 23)[:_ceil_div(h, ibm), :_ceil_div(w, ibk)]
    e_elem = _expand_blocks(e_in, ibm, ibk, h, w)
    top = _block_amax(e_elem.to(torch.float32), obm, obk).to(torch.int32)        # exponents are small non-negative integers
    e_out = (top - 6).clamp(min=0)
    shift = e_elem - _expand_blocks(e_out, obm, obk, h, w)
    out = (vals * torch.exp2(shift.to(torch.float32))).to(torch.float8_e4m3fn)
    return out, _format_sf((e_out << 23).contiguous(), use_tma_aligned_col_major_sf, use_packed_ue8m0)


def reduce_fused(x: Union[torch.Tensor, QuantTensor], topk_weights: Optional[torch.Tensor], token_topk_to_pos: torch.Tensor,
                 fp8_format: str = '', sf: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t] = sum_k x[pos[t, k]] * (w[t, k] * x_sf[pos[t, k]])`` over the positions >= 0, accumulated in fp32 with one
    fused multiply-add per term in the order of k, times ``sf[0]``, rounded to the dtype of ``x`` or to E4M3
    (tile_kernels/torch/reduce_fused.py:14-72)."""
    x_sf = None
    if isinstance(x, tuple):
        x, x_sf = x
    hidden = x.shape[1]
    num_tokens, num_topk = token_topk_to_pos.shape
    out_dtype = torch.float8_e4m3fn if fp8_format == 'e4m3' else x.dtype
    if num_tokens == 0:
        return torch.empty((0, hidden), dtype=out_dtype)
    acc = torch.zeros((num_tokens, hidden), dtype=torch.float32)
    for k in range(num_topk):
        pos = token_topk_to_pos[:, k].long()
        live = pos >= 0
        if not bool(live.any()):
            continue      # nothing to add (and x may have no rows at all)
        src = pos.clamp(min=0)
        s = topk_weights[:, k].clone() if topk_weights is not None else torch.ones(num_tokens, dtype=torch.float32)
        if x_sf is not None:
            s = s * x_sf[src]
        term = fma_f32(x[src].to(torch.float32), s.unsqueeze(1), acc)
        acc = torch.where(live.unsqueeze(1), term, acc)
    if sf is not None:
        acc = acc * sf[0]
    return acc.to(out_dtype)
