"""Writes known_answers.json from the format definitions alone (no oracle, no reference import)."""
import json
import os
from fractions import Fraction


def e4m3_magnitudes():
    vals = []
    for code in range(0x7F):                      # 0x7F is NaN
        e, m = code >> 3, code & 7
        v = Fraction(m, 8) * Fraction(1, 64) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
        vals.append(float(v))                     # all exactly representable in binary32
    return vals


def main():
    data = {
        'e4m3_values': e4m3_magnitudes(),
        # [input, expected byte]
        'e4m3_kat': [
            [0.0, 0x00], [-0.0, 0x80], [448.0, 0x7E], [-448.0, 0xFE], [449.0, 0x7E], [464.0, 0x7E], [1e9, 0x7E],
            [-1e9, 0xFE], [1.0, 0x38], [1.0625, 0x38], [1.1875, 0x3A], [1.125, 0x39], [0.015625, 0x08],
            [2.0 ** -9, 0x01], [2.0 ** -10, 0x00], [1.5 * 2.0 ** -9, 0x02], [2.5 * 2.0 ** -9, 0x02],
            [7.5 * 2.0 ** -9, 0x08], [-1e-6, 0x80], [240.0, 0x77], [232.0, 0x76], [248.0, 0x78], [432.0, 0x7E],
            [416.0, 0x7D], [424.0, 0x7D], [440.0, 0x7E],
        ],
        # [input, expected nibble]
        'e2m1_kat': [
            [0.0, 0], [-0.0, 8], [0.25, 0], [0.2500001, 1], [0.5, 1], [0.75, 2], [0.7499999, 1], [1.0, 2],
            [1.25, 2], [1.2500001, 3], [1.5, 3], [1.75, 4], [2.0, 4], [2.5, 4], [2.5000002, 5], [3.0, 5], [3.5, 6],
            [4.0, 6], [5.0, 6], [5.0000005, 7], [6.0, 7], [7.0, 7], [1e30, 7], [-0.25, 8], [-0.75, 10], [-3.5, 14],
            [-7.0, 15], [1e-40, 0], [-1e-40, 8],
        ],
        # [fmt, round_sf, amax, expected scale, expected inverse]; floats given as hex strings
        'scale_kat': [
            ['e4m3', False, 448.0, (1.0).hex(), (1.0).hex()],
            ['e4m3', False, 224.0, (0.5).hex(), (2.0).hex()],
            ['e4m3', True, 448.0, (1.0).hex(), (1.0).hex()],
            ['e4m3', True, 449.0, (2.0).hex(), (0.5).hex()],
            ['e4m3', True, 224.0, (0.5).hex(), (2.0).hex()],
            ['e4m3', True, 225.0, (1.0).hex(), (1.0).hex()],
            ['e2m1', False, 6.0, (1.0).hex(), (1.0).hex()],
            ['e2m1', True, 6.0, (1.0).hex(), (1.0).hex()],
            ['e2m1', True, 6.5, (2.0).hex(), (0.5).hex()],
            ['e2m1', True, 0.0, (2.0 ** -126).hex(), (2.0 ** 126).hex()],
            ['e2m1', False, 0.0, (2.0 ** -126).hex(), (2.0 ** 126).hex()],
        ],
    }
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'known_answers.json'), 'w') as f:
        json.dump(data, f, indent=1)


if __name__ == '__main__':
    main()
