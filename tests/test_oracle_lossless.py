"""Pins of the oracle's lossless FP4 -> FP8 re-blocking (no GPU needed): the property the reference's own test
states (tests/quant/test_per_block_cast_lossless.py:90-104: dequantising the result equals dequantising the
input), the closed form of the output exponents, and the edge of exactness."""
import pytest
import torch

from oracle import torch_ref

OUT_BLOCKS = [(1, 128), (32, 32), (128, 128)]
SF_MODES = [(False, True, False), (True, True, True)]


def reference_style_input(num_tokens, hidden, seed):
    """Random data as the reference's test builds it: one random binade for the tensor, magnitudes clamped to a
    ratio of 2^9 (generator.py:92-105, test_per_block_cast_lossless.py:15-20)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((num_tokens, hidden), generator=g) * 2.0 ** int(torch.randint(-100, 100, (1,), generator=g))
    if x.numel():
        floor = x.abs().max() / 2 ** 9
        x = torch.sign(x) * torch.max(x.abs(), floor)
    return x


@pytest.mark.parametrize('out_mode', SF_MODES)
@pytest.mark.parametrize('in_mode', SF_MODES)
@pytest.mark.parametrize('out_block', OUT_BLOCKS)
@pytest.mark.parametrize('num_tokens,hidden', [(130, 576), (37, 2048), (0, 256)])
def test_dequantised_values_are_unchanged(num_tokens, hidden, out_block, in_mode, out_mode):
    x = reference_style_input(num_tokens, hidden, seed=hidden + num_tokens)
    x_fp4 = torch_ref.cast(x, 'e2m1', (1, 32), use_tma_aligned_col_major_sf=in_mode[0], round_sf=in_mode[1], use_packed_ue8m0=in_mode[2])
    out = torch_ref.per_block_cast_lossless(x_fp4, 'e4m3', (1, 32), out_block, *out_mode)
    assert out[0].dtype == torch.float8_e4m3fn and tuple(out[0].shape) == (num_tokens, hidden)
    # the scale tensor has the layout a plain E4M3 cast gives for the same block and arguments
    _, like = torch_ref.cast(x, 'e4m3', out_block, use_tma_aligned_col_major_sf=out_mode[0], round_sf=out_mode[1], use_packed_ue8m0=out_mode[2])
    assert out[1].dtype == like.dtype and tuple(out[1].shape) == tuple(like.shape) and (num_tokens == 0 or out[1].stride() == like.stride())
    before = torch_ref.cast_back(x_fp4, 'fp32', (1, 32))
    after = torch_ref.cast_back(out, 'fp32', out_block)
    assert torch.equal(before.view(torch.int32), after.view(torch.int32))


def _fp4_rows(codes_per_block, exps):
    """One row: block b holds the 32 codes `codes_per_block[b]` (E2M1 nibble values) with scale 2^(exps[b]-127)."""
    nib = torch.tensor(codes_per_block, dtype=torch.uint8).view(1, -1)
    packed = (nib[:, 0::2] | (nib[:, 1::2] << 4)).view(torch.int8)
    sf = (torch.tensor(exps, dtype=torch.int32).view(1, -1) << 23).view(torch.float32)
    return packed, sf


def test_output_exponent_closed_form():
    # four input blocks of 32 with exponents 130, 127, 121, 125 in one 1 x 128 output block:
    # e_out = 130 - 6 = 124, shifts +6, +3, -3, +1
    six, half = 0x7, 0x1                     # nibbles of +6.0 and +0.5
    packed, sf = _fp4_rows([[six] * 32, [half] * 32, [six] * 32, [0x9] * 32], [130, 127, 121, 125])   # 0x9 = -0.5
    out, out_sf = torch_ref.per_block_cast_lossless((packed, sf), 'e4m3', (1, 32), (1, 128))
    assert out_sf.view(torch.int32).tolist() == [[124 << 23]]
    want = [6.0 * 64] * 32 + [0.5 * 8] * 32 + [6.0 / 8] * 32 + [-0.5 * 2] * 32
    assert out.float().tolist() == [want]
    # as four 1 x 32 output blocks each keeps its own exponent minus 6 and every code is shifted by 6
    out, out_sf = torch_ref.per_block_cast_lossless((packed, sf), 'e4m3', (1, 32), (1, 32))
    assert (out_sf.view(torch.int32) >> 23).tolist() == [[124, 121, 115, 119]]
    assert out.float().tolist() == [[384.0] * 32 + [32.0] * 32 + [384.0] * 32 + [-32.0] * 32]


def test_output_exponent_does_not_go_below_zero():
    packed, sf = _fp4_rows([[0x2] * 32, [0x2] * 32], [3, 5])      # 1.0 with scales 2^-124 and 2^-122
    out, out_sf = torch_ref.per_block_cast_lossless((packed, sf), 'e4m3', (1, 32), (1, 64))
    assert (out_sf.view(torch.int32) >> 23).tolist() == [[0]]
    assert out.float().tolist() == [[8.0] * 32 + [32.0] * 32]     # shifted by 3 and 5


def test_edge_of_exactness():
    # a span of 11 binades inside one output block is still exact for the smallest magnitude (0.5 -> 2^-6, the
    # smallest normal E4M3 number) ...
    packed, sf = _fp4_rows([[0x7] * 32, [0x1] * 32], [140, 129])
    out = torch_ref.per_block_cast_lossless((packed, sf), 'e4m3', (1, 32), (1, 64))
    assert torch.equal(torch_ref.cast_back(out, 'fp32', (1, 64)), torch_ref.cast_back((packed, sf), 'fp32', (1, 32)))
    assert out[0].float()[0, 32].item() == 2.0 ** -6
    # ... and E4M3's subnormals carry 0.5 (one bit) exactly for three binades more
    packed, sf = _fp4_rows([[0x7] * 32, [0x1] * 32], [140, 126])
    out = torch_ref.per_block_cast_lossless((packed, sf), 'e4m3', (1, 32), (1, 64))
    assert out[0].float()[0, 32].item() == 2.0 ** -9
