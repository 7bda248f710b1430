"""Pins the two encoders and the scale arithmetic of the CPU oracle (both the torch and the C
statement) against value tables, brute force and hand known answers.  No GPU needed."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import cref, torch_ref

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'known_answers.json')))
E4M3_TABLE = np.array(GOLD['e4m3_values'], dtype=np.float64)          # index = code 0..0x7E
E2M1_TABLE = np.array(torch_ref.E2M1_VALUES, dtype=np.float64)


def brute_nearest(v32: np.ndarray, table: np.ndarray, sat: float) -> np.ndarray:
    """Nearest table entry of clamp(|v|), ties to the even index, sign in the top bit position."""
    a = np.minimum(np.abs(v32.astype(np.float64)), sat)
    d = np.abs(a[:, None] - table[None, :])
    best = d.min(axis=1)
    cand = d == best[:, None]
    lo = cand.argmax(axis=1)                                   # lowest index at minimum distance
    hi = table.size - 1 - cand[:, ::-1].argmax(axis=1)         # highest
    code = np.where(lo % 2 == 0, lo, hi)                       # a tie has two neighbours: take the even one
    return code.astype(np.uint8), np.signbit(v32)


def torch_e4m3(v32: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(v32.copy())
    return t.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def all_bf16_finite() -> np.ndarray:
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    v = bits.view(np.float32)
    return v[np.isfinite(v)]


def midpoints_and_neighbours(table: np.ndarray) -> np.ndarray:
    mids = ((table[:-1] + table[1:]) / 2).astype(np.float32)
    pts = np.concatenate([table.astype(np.float32), mids])
    up = np.nextafter(pts, np.float32(np.inf))
    dn = np.nextafter(pts, np.float32(-np.inf))
    allp = np.concatenate([pts, up, dn, np.float32([448.0 * (1 + 2 ** -23), 463.9, 464.0, 465.0, 1e30])])
    allp = allp[allp >= 0]
    return np.concatenate([allp, -allp]).astype(np.float32)


def test_e4m3_table_is_the_ocp_format():
    assert E4M3_TABLE.size == 127 and E4M3_TABLE[0x7E] == 448.0 and E4M3_TABLE[1] == 2.0 ** -9
    assert E4M3_TABLE[0x08] == 2.0 ** -6 and np.all(np.diff(E4M3_TABLE) > 0)
    # torch decodes the same table
    dec = torch.arange(127, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float64).numpy()
    assert np.array_equal(dec, E4M3_TABLE)


@pytest.mark.parametrize('scale', [1.0, 448.0 / 3.7, 1.0 / 448.0, 37.3, 2.0 ** -7])
def test_e4m3_encoders_vs_brute_force_all_bf16(scale):
    v = (all_bf16_finite() * np.float32(scale)).astype(np.float32)
    code, sign = brute_nearest(v, E4M3_TABLE, 448.0)
    want = code | (sign.astype(np.uint8) << 7)
    assert np.array_equal(torch_e4m3(v), want)
    assert np.array_equal(cref.e4m3_encode(v), want)


def test_e4m3_encoders_at_every_rounding_boundary():
    v = midpoints_and_neighbours(E4M3_TABLE)
    code, sign = brute_nearest(v, E4M3_TABLE, 448.0)
    want = code | (sign.astype(np.uint8) << 7)
    assert np.array_equal(torch_e4m3(v), want)
    assert np.array_equal(cref.e4m3_encode(v), want)


def test_e4m3_known_answers():
    v = np.float32([k[0] for k in GOLD['e4m3_kat']])
    want = np.uint8([k[1] for k in GOLD['e4m3_kat']])
    assert np.array_equal(torch_e4m3(v), want)
    assert np.array_equal(cref.e4m3_encode(v), want)
    nan = np.float32([np.nan])
    assert cref.e4m3_encode(nan)[0] & 0x7F == 0x7F and torch_e4m3(nan)[0] & 0x7F == 0x7F


def test_e2m1_encoders_vs_brute_force():
    rng = np.random.default_rng(7)
    v = np.concatenate([
        midpoints_and_neighbours(E2M1_TABLE),
        (all_bf16_finite() * np.float32(0.37)).astype(np.float32),
        rng.standard_normal(200000).astype(np.float32) * 3,
        rng.uniform(-7, 7, 200000).astype(np.float32),
    ])
    code, sign = brute_nearest(v, E2M1_TABLE, 6.0)
    want = code | (sign.astype(np.uint8) << 3)
    got_t = torch_ref.encode_e2m1(torch.from_numpy(v.copy())).numpy()
    assert np.array_equal(got_t, want)
    assert np.array_equal(cref.e2m1_encode(v), want)


def test_e2m1_known_answers_and_roundtrip():
    v = np.float32([k[0] for k in GOLD['e2m1_kat']])
    want = np.uint8([k[1] for k in GOLD['e2m1_kat']])
    assert np.array_equal(torch_ref.encode_e2m1(torch.from_numpy(v)).numpy(), want)
    assert np.array_equal(cref.e2m1_encode(v), want)
    # every code decodes to its table value and re-encodes to itself; low nibble = even element
    packed = torch.arange(256, dtype=torch.uint8).view(1, 256)
    dec = torch_ref.unpack_from_e2m1fn_x2(packed)
    assert dec.shape == (1, 512)
    lo, hi = dec[0, 0::2], dec[0, 1::2]
    tab = torch.tensor(list(torch_ref.E2M1_VALUES) + [-x for x in torch_ref.E2M1_VALUES])
    assert torch.equal(lo, tab[torch.arange(256) & 15]) and torch.equal(hi, tab[torch.arange(256) >> 4])
    re = torch_ref.encode_e2m1(dec[0])
    # -0 does not survive a value round trip through the decoder's table (-0.0 entry keeps its sign)
    assert torch.equal(re[0::2], (torch.arange(256) & 15).to(torch.uint8))


def test_power_of_two_rounding_identity_over_every_exponent():
    """(b + 0x7FFFFF) & 0x7F800000 (cast.py:159) == ((b - 1) >> 23) + 1 as biased exponent
    (common.py:211) == 2^ceil(log2 s), for every positive normal exponent."""
    rng = np.random.default_rng(3)
    for e in range(1, 254):
        mant = np.concatenate([[0, 1, 2, 0x400000, 0x7FFFFE, 0x7FFFFF], rng.integers(0, 1 << 23, 20)]).astype(np.int64)
        b = (e << 23) | mant
        a = (b + 0x7FFFFF) & 0x7F800000
        k = ((b - 1) >> 23) + 1
        assert np.array_equal(a >> 23, k)
        s = b.astype(np.uint32).view(np.float32).astype(np.float64)
        want = np.array([math.ceil(math.log2(x)) if m else e - 127 for x, m in zip(s, mant)])
        assert np.array_equal((a >> 23) - 127, want)


@pytest.mark.parametrize('fmt,round_sf,amax,sf_hex,inv_hex', GOLD['scale_kat'])
def test_scale_known_answers(fmt, round_sf, amax, sf_hex, inv_hex):
    n = 128 if fmt == 'e4m3' else 32
    x = torch.zeros((1, n), dtype=torch.float32)
    x[0, 5] = -amax
    x[0, 9] = amax / 2
    sf_want, inv_want = float.fromhex(sf_hex), float.fromhex(inv_hex)
    for impl in ('torch', 'c'):
        if impl == 'torch':
            codes, sf = torch_ref.cast(x, fmt, (1, n), round_sf=round_sf)
            codes = codes.view(torch.uint8)
        else:
            codes, sf = cref.cast(x, fmt, (1, n), round_sf=round_sf)
        assert sf.item() == sf_want
        # the element holding -amax encodes fl(-amax * inv)
        q = np.float32(-amax) * np.float32(inv_want)
        if fmt == 'e4m3':
            assert codes[0, 5].item() == cref.e4m3_encode(np.float32([q]))[0]
        else:
            assert (codes[0, 2].item() >> 4) == cref.e2m1_encode(np.float32([q]))[0]
    if amax == 0.0 and fmt == 'e4m3':
        assert sf.item() == float(np.float32(1e-4) / np.float32(448))


def test_zero_group_gets_floor_scale_and_zero_codes():
    x = torch.zeros((2, 256), dtype=torch.bfloat16)
    codes, sf = torch_ref.cast(x, 'e4m3', (1, 128))
    assert torch.all(codes.view(torch.uint8) == 0)
    assert torch.all(sf == float(np.float32(1e-4) / np.float32(448)))


def test_division_is_not_a_reciprocal_multiply():
    """Most amax values separate fl(a/448) from fl(a*fl(1/448)); the oracle must be the former."""
    a = all_bf16_finite()
    a = a[(a > 1e-3) & (a < 1e4)]
    x = torch.zeros((a.size, 128), dtype=torch.float32)
    x[:, 0] = torch.from_numpy(a)
    _, sf = torch_ref.cast(x, 'e4m3', (1, 128))
    true_div = (a.astype(np.float32) / np.float32(448)).astype(np.float32)
    recip = (a.astype(np.float32) * (np.float32(1) / np.float32(448))).astype(np.float32)
    assert np.array_equal(sf[:, 0].numpy(), true_div)
    assert (true_div != recip).mean() > 0.3
    _, sf_c = cref.cast(x, 'e4m3', (1, 128))
    assert np.array_equal(sf_c[:, 0].numpy(), true_div)
