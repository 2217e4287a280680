"""Writes fp8_decode_tables.json: the value of each of the 256 codes of OCP float8 e4m3fn and e5m2, from the
closed form of the format specification (sign, biased exponent, mantissa; e4m3fn has no infinities and a single
NaN mantissa pattern per sign, e5m2 is IEEE-like), evaluated with exact rational arithmetic.  No library float8
implementation takes part, so the table pins torch-CPU's and the C oracle's decoders independently.

Run from the repository root:  python tests/golden/make_fp8_tables.py
"""

import json
from fractions import Fraction
from pathlib import Path


def decode(code: int, exp_bits: int, man_bits: int, bias: int, fn: bool):
    sign = -1 if code >> 7 else 1
    e = (code >> man_bits) & ((1 << exp_bits) - 1)
    m = code & ((1 << man_bits) - 1)
    top = (1 << exp_bits) - 1
    if fn:  # e4m3fn: only S.1111.111 is NaN, there is no infinity
        if e == top and m == (1 << man_bits) - 1:
            return "nan"
    elif e == top:  # IEEE-like: infinities and NaNs
        return "nan" if m else ("inf" if sign > 0 else "-inf")
    if e == 0:
        v = Fraction(m, 1 << man_bits) * Fraction(2) ** (1 - bias)
    else:
        v = (1 + Fraction(m, 1 << man_bits)) * Fraction(2) ** (e - bias)
    f = float(sign * v)
    assert Fraction(f) == sign * v  # every fp8 value is exactly representable in binary64
    if f == 0.0 and sign < 0:
        return "-0.0"
    return f.hex()


def main():
    tables = {
        "float8_e4m3fn": [decode(c, 4, 3, 7, True) for c in range(256)],
        "float8_e5m2": [decode(c, 5, 2, 15, False) for c in range(256)],
    }
    out = Path(__file__).with_name("fp8_decode_tables.json")
    out.write_text(json.dumps(tables, indent=0) + "\n")
    print(f"wrote {out}")


if __name__ == "__main__":
    main()
