"""Writes bmm_literal_16x16.json: the one literal input the upstream tests hold
(upstream tests/test_bmm.py:36-98: A 16x16 int8, B 16x16 int8, scale 0.0186,
expected = round(A.B*scale).clamp(-128,127), :99-101) together with the
expected output.

The matrices below are data transcribed from that test.  The expected output is
computed here by two routes that share no code with the oracle: exact integer
matmul in Python ints followed by (a) the fp32 expression the upstream test
uses and (b) exact rational arithmetic with round-half-even; the script refuses
to write the fixture unless both agree (no product lands close enough to a .5
tie for fp32 rounding to matter).

Run: python tests/golden/make_bmm_literal.py
"""
import json
import os
from fractions import Fraction

import numpy as np

A = [[7, 8, 6, 16, 3, 7, 10, 4, 11, 5, 4, 11, 11, 7, 6, 9],
     [7, 7, 9, 8, 9, 9, 6, 6, 6, 9, 10, 10, 8, 9, 9, 6],
     [7, 9, 8, 9, 7, 7, 6, 5, 7, 7, 8, 10, 11, 8, 9, 8],
     [9, 7, 6, 12, 5, 7, 12, 6, 12, 6, 4, 9, 9, 8, 7, 10],
     [7, 6, 6, 10, 10, 9, 12, 7, 8, 9, 7, 7, 5, 8, 8, 8],
     [6, 9, 9, 6, 10, 9, 8, 9, 9, 6, 10, 8, 8, 6, 6, 9],
     [6, 8, 7, 9, 12, 7, 7, 10, 10, 7, 8, 9, 5, 7, 8, 7],
     [6, 9, 9, 7, 12, 9, 4, 5, 7, 5, 13, 10, 13, 4, 6, 9],
     [8, 10, 11, 8, 12, 7, 5, 8, 6, 7, 9, 7, 11, 5, 7, 7],
     [5, 9, 8, 8, 5, 8, 6, 4, 12, 5, 8, 10, 15, 6, 7, 11],
     [7, 8, 8, 5, 7, 10, 7, 6, 7, 8, 11, 7, 10, 8, 8, 9],
     [7, 7, 9, 5, 6, 11, 7, 8, 7, 9, 11, 7, 11, 8, 7, 8],
     [9, 8, 7, 9, 3, 9, 10, 4, 9, 5, 5, 9, 13, 9, 8, 9],
     [5, 8, 9, 8, 8, 8, 7, 8, 9, 9, 10, 9, 7, 9, 8, 7],
     [6, 7, 7, 13, 3, 6, 11, 7, 12, 8, 4, 8, 8, 10, 9, 8],
     [8, 7, 6, 14, 6, 6, 11, 5, 9, 7, 4, 10, 6, 10, 9, 9]]

# B as written upstream: [K, N]; the kernel takes its transpose [N, K] (test_bmm.py:103)
B = [[-37, 19, 26, -45, -6, -3, 10, 97, 80, 4, -31, -51, 58, -83, 31, -100],
     [-16, 10, -9, -24, 15, -39, 22, 26, -10, 50, -38, 1, -25, -26, 5, -15],
     [-76, -19, 44, -56, -13, -12, 21, 51, 77, -8, -28, 14, -12, -6, 15, -5],
     [-53, 2, -11, -42, 26, 10, -82, 43, 25, 54, 69, -25, 70, -2, -37, -71],
     [15, -119, 2, -66, -54, -64, 115, 112, -95, -75, 7, 44, 8, -74, 110, -52],
     [-53, -16, 38, -35, 16, -98, 35, 93, 7, 14, -53, -90, 47, -54, 48, -11],
     [-23, 10, -74, -30, 18, -85, 45, 61, 35, 57, 17, -98, -16, -19, -67, 63],
     [-78, -55, 44, -105, -25, -89, 80, 81, 71, 3, 29, 8, -19, 44, 7, -55],
     [-36, -56, 62, -13, 50, -21, -63, 12, -58, -2, -19, 39, -4, 104, 26, -96],
     [-73, -37, 4, -94, -7, -24, 24, 23, 29, -40, 7, 5, 1, 1, 0, -6],
     [-28, -44, 70, -63, -8, -102, 107, 59, 6, -51, -47, -10, 47, -37, 98, -32],
     [-3, 3, 67, 3, 56, -52, -20, -10, -24, 75, -26, -11, 87, 53, 23, -60],
     [-67, 38, 27, -80, 56, -75, -18, 76, 48, -8, -105, -94, 80, -127, 51, -88],
     [-8, 41, -5, 0, 86, -21, 44, -21, -20, 80, -21, -30, 4, 29, -38, 55],
     [-47, 32, 53, -54, -4, 58, 9, 28, 6, -32, -11, 13, 51, -33, 75, -1],
     [63, -60, -74, -27, 22, -55, 16, 51, -5, -54, 1, -101, 2, -58, 1, -45]]

SCALE = 0.0186


def round_half_even(fr):
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        return fl + 1
    return fl


def main():
    n = 16
    acc = [[sum(A[i][k] * B[k][j] for k in range(n)) for j in range(n)] for i in range(n)]
    s32 = np.float32(SCALE)
    route_a = [[int(np.clip(np.rint(np.float32(acc[i][j]) * s32), -128, 127)) for j in range(n)] for i in range(n)]
    sfr = Fraction(float(s32))
    route_b = [[max(-128, min(127, round_half_even(Fraction(acc[i][j]) * sfr))) for j in range(n)] for i in range(n)]
    assert route_a == route_b, "fp32 and exact routes disagree: a product sits on a rounding boundary"
    out = {"source": "upstream tests/test_bmm.py:36-106", "scale": SCALE, "a": A, "b_kn": B,
           "acc": acc, "expected_s8": route_a}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bmm_literal_16x16.json")
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path)


if __name__ == "__main__":
    main()
