"""Writes the committed fixtures of tests/golden/ from first principles (no reference code is
imported or run; the reference holds no reproducible vectors for this path).

  e4m3fn_table.json : the 256 OCP e4m3fn code points decoded from the format definition
                      (1 sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities,
                      S.1111.111 = NaN) with exact rational arithmetic.
  awq_kat.json      : hand-built AWQ words: for a packed int32 the eight logical columns it must
                      unpack to (nibble i holds logical column {0,2,4,6,1,3,5,7}[i]).
  int8_quant_kat.json : small per-token int8 quantization cases worked out by hand in exact
                      arithmetic (values chosen to be exactly representable, ties included).
"""
import json
import pathlib
from fractions import Fraction

HERE = pathlib.Path(__file__).resolve().parent


def e4m3fn_table():
    out = []
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 0xF, c & 7
        if e == 15 and m == 7:
            out.append("nan")
            continue
        v = Fraction(m, 8) * Fraction(1, 64) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
        out.append(float(-v if s else v))
    return out


def awq_kat():
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    cases = []
    for cols in ([0, 1, 2, 3, 4, 5, 6, 7], [15, 0, 15, 0, 15, 0, 15, 0], [8, 9, 10, 11, 12, 13, 14, 15],
                 [1, 0, 0, 0, 0, 0, 0, 0], [0, 1, 0, 0, 0, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 15]):
        word = 0
        for i in range(8):
            word |= cols[order[i]] << (4 * i)
        if word >= 2 ** 31:
            word -= 2 ** 32
        cases.append({"word": word, "columns": cols})
    return cases


def int8_quant_kat():
    # absmax 127 -> scale exactly 1: q = round-half-even(x)
    return [
        {"dtype": "bfloat16", "x": [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.0],
         "scale": 1.0, "q": [127, 0, 2, 2, 0, -2, -2, 3]},
        # absmax 63.5 -> scale exactly 0.5: q = round-half-even(2x)
        {"dtype": "bfloat16", "x": [63.5, 0.25, 0.75, 1.25, -63.5, 10.0, -0.25, 0.0],
         "scale": 0.5, "q": [127, 0, 2, 2, -127, 20, 0, 0]},
        {"dtype": "float16", "x": [254.0, 1.0, 3.0, 5.0, -1.0, -3.0, 7.0, -254.0],
         "scale": 2.0, "q": [127, 0, 2, 2, 0, -2, 4, -127]},
    ]


if __name__ == "__main__":
    (HERE / "e4m3fn_table.json").write_text(json.dumps(e4m3fn_table()))
    (HERE / "awq_kat.json").write_text(json.dumps(awq_kat(), indent=1))
    (HERE / "int8_quant_kat.json").write_text(json.dumps(int8_quant_kat(), indent=1))
    print("wrote fixtures to", HERE)
