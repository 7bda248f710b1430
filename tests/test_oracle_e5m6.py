"""Pins of the E5M6 part of the CPU oracle (no GPU needed).

E5M6 is the top 12 bits of an IEEE fp16.  What the mathematics fixes is checked by independent means:
the round-toward-zero fp16 step by a brute-force search, the 12-bit rounding (for values whose fp16
form is normal) by a nearest-ties-to-even search over all 4096 codes, the packing by big-integer
concatenation, the scales by closed forms, plus hand-worked answers including the reference's own
special inputs (tile_kernels/testing/generator.py:70-89).  Below the smallest normal fp16 the
reference's rule is not round-to-nearest; there only hand-computed cases apply.
"""
import numpy as np
import pytest
import torch

from oracle import torch_ref


def _f32(values):
    return torch.tensor(values, dtype=torch.float32)


def _sample_values(seed=0, n=20000):
    g = torch.Generator().manual_seed(seed)
    # magnitudes spread over the exponent range an E5M6 input can have after scaling, both signs
    expo = torch.randint(-26, 17, (n,), generator=g).float()
    x = (torch.rand((n,), generator=g) + 1.0) * torch.exp2(expo) * torch.where(torch.rand((n,), generator=g) < 0.5, -1.0, 1.0)
    return x


# ---- fp32 -> fp16, rounded toward zero

def test_fp16_toward_zero_is_the_largest_fp16_not_above():
    x = torch.cat([_sample_values(), _f32([0.0, -0.0, 65504.0, 65519.9, 2.0 ** -24, 2.0 ** -25, 1.9999 * 2.0 ** -25, 2.0 ** -14])])
    bits = torch_ref.fp16_bits_toward_zero(x)
    assert int(bits.min()) >= 0 and int(bits.max()) <= 0xFFFF
    got = bits.to(torch.int32).numpy().astype(np.uint16).view(np.float16).astype(np.float64)
    xv = x.double().numpy()
    finite = np.abs(xv) < 65536.0
    # same sign (or zero), magnitude not above |x|, and the next fp16 away from zero is above |x|
    assert np.all(np.signbit(got) == np.signbit(xv))
    assert np.all(np.abs(got[finite]) <= np.abs(xv[finite]))
    mag = np.abs(got[finite]).astype(np.float16)
    with np.errstate(over='ignore'):
        nxt = np.nextafter(mag, np.float16(np.inf)).astype(np.float64)      # 65504 -> inf
    assert np.all(nxt > np.abs(xv[finite]))


def test_fp16_toward_zero_beyond_the_range():
    bits = torch_ref.fp16_bits_toward_zero(_f32([65536.0, -1e9, float('inf'), float('-inf'), float('nan'), 1e-30, -1e-30]))
    assert bits.tolist()[:4] == [0x7C00, 0xFC00, 0x7C00, 0xFC00]
    assert bits[4].item() & 0x7FFF == 0x7FFF
    assert bits.tolist()[5:] == [0x0000, 0x8000]


# ---- 12-bit rounding

def _code_table():
    """value of each non-negative finite code, float64"""
    codes = torch.arange(0, 0x7C0, dtype=torch.int32)
    return torch_ref.decode_e5m6(codes).double().numpy()


def test_decode_known_codes():
    got = torch_ref.decode_e5m6(torch.tensor([0x000, 0x001, 0x03F, 0x040, 0x3C0, 0x7BF, 0x800 | 0x3C0, 0x7C0], dtype=torch.int32))
    want = [0.0, 2.0 ** -20, 2.0 ** -14 * 63 / 64, 2.0 ** -14, 1.0, 65024.0, -1.0, float('inf')]
    assert got.tolist() == want


def test_encode_is_nearest_even_where_fp16_is_normal():
    x = _sample_values(seed=1)
    x = x[(x.abs() >= 2.0 ** -14) & (x.abs() <= 65024.0)]
    table = _code_table()
    # add exact midpoints and their fp32 neighbours between random adjacent codes
    idx = np.random.RandomState(0).randint(0x040, 0x7BF, size=2000)
    mid = (table[idx] + table[idx + 1]) / 2                     # exactly representable in fp32
    mids = torch.from_numpy(np.concatenate([mid, np.nextafter(mid.astype(np.float32), np.float32(0)),
                                            np.nextafter(mid.astype(np.float32), np.float32(1e9))]).astype(np.float32))
    x = torch.cat([x, mids, -mids])
    got = torch_ref.encode_e5m6(x).numpy()
    a = x.abs().double().numpy()
    hi = np.searchsorted(table, a, side='left').clip(1, len(table) - 1)        # table[hi-1] <= a <= table[hi] (or a == table[hi])
    lo = hi - 1
    dl, dh = a - table[lo], table[hi] - a
    want = np.where(dl < dh, lo, np.where(dh < dl, hi, np.where(lo % 2 == 0, lo, hi)))
    want = want | np.where(np.signbit(x.numpy()), 0x800, 0)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (x[bad[:5]].tolist(), got[bad[:5]].tolist(), want[bad[:5]].tolist())


def test_encode_hand_cases_below_the_normal_range():
    # worked by hand from the rule "fp16 toward zero, keep 12 bits, bump when lsb + (fp32 bits & 0x1FFFF) > 0x10000":
    #   2^-20            fp32 0x35800000: fp16 0x0010, kept 0x001, low bits 0      -> 0x001
    #   1.5 * 2^-20      fp32 0x35C00000: fp16 0x0018, kept 0x001, low bits 0      -> 0x001 (a tie a nearest-even rule would send to 0x002)
    #   (1+2^-7) * 2^-20 fp32 0x35810000: fp16 0x0010, kept 0x001, low bits 0x10000 -> 1 + 0x10000 > 0x10000 -> 0x002 (not the nearest)
    #   63/64 * 2^-14    fp32 0x387C0000: fp16 0x03F0, kept 0x03F, low bits 0      -> 0x03F
    #   2^-25            below half the smallest fp16 subnormal: fp16 0, kept 0, low bits 0 -> 0x000
    x = _f32([2.0 ** -20, 1.5 * 2.0 ** -20, (1 + 2.0 ** -7) * 2.0 ** -20, 63 / 64 * 2.0 ** -14, 2.0 ** -25, -(2.0 ** -20)])
    assert x.view(torch.int32).tolist()[:4] == [0x35800000, 0x35C00000, 0x35810000, 0x387C0000]
    assert torch_ref.encode_e5m6(x).tolist() == [0x001, 0x001, 0x002, 0x03F, 0x000, 0x801]


def test_encode_rounds_up_into_the_next_binade_and_to_infinity():
    # 1.9999 rounds to 2.0 (mantissa carry into the exponent); above 65024 + 256 the code becomes infinity's
    x = _f32([1.9999, 65024.0, 65024.0 + 255.9, 65024.0 + 256.1])
    assert torch_ref.encode_e5m6(x).tolist() == [0x400, 0x7BF, 0x7BF, 0x7C0]


# ---- packing

def test_pack_matches_big_integer_concatenation():
    g = torch.Generator().manual_seed(2)
    codes = torch.randint(0, 4096, (5, 48), generator=g, dtype=torch.int32)
    packed = torch_ref.pack_e5m6(codes)
    assert packed.dtype == torch.uint8 and tuple(packed.shape) == (5, 72)
    words = packed.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    for r in range(5):
        for gidx in range(6):
            big = 0
            for c in codes[r, 8 * gidx: 8 * gidx + 8].tolist():
                big = (big << 12) | c
            want = [(big >> 64) & 0xFFFFFFFF, (big >> 32) & 0xFFFFFFFF, big & 0xFFFFFFFF]
            assert words[r, 3 * gidx: 3 * gidx + 3].tolist() == want
    assert torch.equal(torch_ref.unpack_e5m6(packed), codes)


def test_pack_hand_built_words():
    codes = torch.tensor([[1, 2, 3, 4, 5, 6, 7, 8]], dtype=torch.int32)
    words = torch_ref.pack_e5m6(codes).view(torch.int32).tolist()[0]
    assert words == [0x00100200, 0x30040050, 0x06007008]
    # byte order inside a word is the machine's (little endian)
    assert torch_ref.pack_e5m6(codes)[0, :4].tolist() == [0x00, 0x02, 0x10, 0x00]


# ---- the whole cast

@pytest.mark.parametrize('round_sf', [False, True])
def test_cast_scale_closed_forms(round_sf):
    x = torch.zeros((3, 64))
    x[0, 5] = 65024.0            # amax 65024 -> scale 1
    x[1, 7] = -130048.0          # amax 2 * 65024 -> scale 2
    # row 2 all zero: amax floored at 1e-4
    packed, sf = torch_ref.cast_to_e5m6(x, 64, round_sf=round_sf)
    floor_sf = torch.tensor(1e-4, dtype=torch.float32) / torch.tensor(65024.0)
    if round_sf:
        floor_sf = torch.exp2(torch.ceil(torch.log2(floor_sf.double()))).float()
    assert sf[:, 0].tolist() == [1.0, 2.0, floor_sf.item()]
    codes = torch_ref.unpack_e5m6(packed)
    assert codes[0, 5].item() == 0x7BF and codes[1, 7].item() == 0x800 | 0x7BF
    assert int(codes.abs().sum()) == 0x7BF + (0x800 | 0x7BF)


def test_cast_reference_special_inputs():
    # tile_kernels/testing/generator.py:76-89: a constant row whose last element is 65024, so the scale is 1
    for value, code in ((2.0 ** -20, 0x001), (2.0 ** -14 * 63 / 64, 0x03F), (2.0 ** -14, 0x040)):
        for dtype in (torch.float32, torch.bfloat16):
            x = torch.full((4, 64), value, dtype=dtype)
            x[:, -1] = 65024.0
            if dtype == torch.bfloat16 and x[0, 0].float().item() != value:
                continue                                   # not a bf16 number (63/64 * 2^-14 is: 6 mantissa bits)
            packed, sf = torch_ref.cast_to_e5m6(x, 64, round_sf=True)
            codes = torch_ref.unpack_e5m6(packed)
            assert torch.all(sf == 1.0)
            assert torch.all(codes[:, :-1] == code) and torch.all(codes[:, -1] == 0x7BF)
            back = torch_ref.cast_back_from_e5m6((packed, sf), 'fp32', (1, 64))
            assert torch.equal(back, x.float())


@pytest.mark.parametrize('mode', [(False, False, False), (False, True, False), (True, True, False), (True, True, True)])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_cast_round_trip_and_layouts(dtype, mode):
    col, rnd, packed_sf = mode
    g = torch.Generator().manual_seed(3)
    x = (torch.randn((37, 576), generator=g) * 3).to(dtype)
    packed, sf = torch_ref.cast_to_e5m6(x, 576, col, rnd, packed_sf)
    assert packed.dtype == torch.uint8 and tuple(packed.shape) == (37, 864)
    # the scale tensor has the layout the E4M3 cast gives for the same arguments
    _, sf_like = torch_ref.cast(x, 'e4m3', (1, 576), round_sf=rnd, use_tma_aligned_col_major_sf=col, use_packed_ue8m0=packed_sf)
    assert sf.dtype == sf_like.dtype and tuple(sf.shape) == tuple(sf_like.shape) and sf.stride() == sf_like.stride()
    back = torch_ref.cast_back_from_e5m6((packed, sf), 'fp32', (1, 576))
    amax = x.float().abs().amax(dim=1, keepdim=True)
    # 7 significant bits: relative error at most 2^-7 of the value, plus the grid of the subnormal range
    err = (back - x.float()).abs()
    assert torch.all(err <= x.float().abs() * 2.0 ** -7 + amax * 2.0 ** -20 / 65024 * 64)
    assert torch.equal(torch_ref.cast_back_from_e5m6((packed, sf), 'bf16', (1, 576)), back.to(torch.bfloat16))
