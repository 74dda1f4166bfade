"""Independent evaluation of the reference's DFT checksum table builder
(include/utils/abft.h:21-61) for the tests.

The builder evaluates cos/sin of the angle  -(float)(2*pi*i*j) / float(N):  the
product is formed in double, rounded to float, and only then divided by N.
Here that angle is produced with struct (IEEE single rounding of a Python
float) and cos/sin are evaluated by mpmath in 40-digit arithmetic and summed
exactly, so nothing of numpy's or libm's float32 code paths is shared with the
implementations under test.  `variant` selects deliberately wrong readings of
the same source lines; the tests require that each of them is told apart.
"""
import math
import struct

import mpmath as mp

SQRT3_2_LITERAL = 0.8660253882408142


def _f32(v: float) -> float:
    return struct.unpack("f", struct.pack("f", v))[0]


def checksum_rows(N: int, rows, variant: str = "reference"):
    """{i: c_N[i]} for the requested rows, as Python complex numbers."""
    mp.mp.dps = 40
    s3 = mp.sqrt(3) / 2 if variant == "exact_sqrt3" else mp.mpf(SQRT3_2_LITERAL)   # the literal is float-rounded
    r = [mp.mpc(1, 0), mp.mpc(-0.5, -s3), mp.mpc(-0.5, s3)]
    out = {}
    for i in rows:
        acc = mp.mpc(0)
        for j in range(N):
            if variant in ("reference", "exact_sqrt3", "r_shifted"):
                a = -_f32(2 * math.pi * i * j) / N              # power-of-two division is exact
            elif variant == "unrounded_angle":                  # angle kept in double
                a = -(2 * math.pi * i * j) / N
            elif variant == "float_two_pi":                     # 2*pi rounded before the product
                a = -_f32(_f32(2 * math.pi) * i * j) / N
            elif variant == "float_index_product":              # i*j rounded to float first
                a = -_f32(2 * math.pi * _f32(float(i * j))) / N
            elif variant == "positive_angle":                   # sign of the exponent
                a = _f32(2 * math.pi * i * j) / N
            else:
                raise ValueError(variant)
            k = (j + 1) % 3 if variant == "r_shifted" else j % 3
            acc += mp.mpc(mp.cos(a), mp.sin(a)) * r[k]
        out[i] = complex(acc)
    return out
