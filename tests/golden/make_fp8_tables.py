"""Writes fp8_tables.json: the value of every byte of OCP e4m3fn and e5m2, decoded from the bit fields by the
format definition (sign, exponent bias 7 / 15, 3 / 2 mantissa bits, subnormals; e4m3fn has no infinity and one NaN
pattern per sign, e5m2 follows IEEE). Independent of torch; the tests use it to pin torch's casts, the oracle's
fp8 rounding and the HIP conversion kernels. Run: python tests/golden/make_fp8_tables.py"""
import json
import os


def decode(byte, ebits, mbits, bias, fn):
    s = -1.0 if byte >> 7 else 1.0
    e = (byte >> mbits) & ((1 << ebits) - 1)
    m = byte & ((1 << mbits) - 1)
    if fn:
        if e == (1 << ebits) - 1 and m == (1 << mbits) - 1:
            return None  # NaN
    elif e == (1 << ebits) - 1:
        return None if m else (s * float("inf"))
    if e == 0:
        return s * m * 2.0 ** (1 - bias - mbits)
    return s * (1 + m / (1 << mbits)) * 2.0 ** (e - bias)


def main():
    out = {"e4m3fn": [decode(b, 4, 3, 7, True) for b in range(256)],
           "e5m2": [decode(b, 5, 2, 15, False) for b in range(256)]}
    for k in out:
        out[k] = ["nan" if v is None else ("inf" if v == float("inf") else ("-inf" if v == float("-inf") else v))
                  for v in out[k]]
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "fp8_tables.json"), "w") as f:
        json.dump(out, f)


if __name__ == "__main__":
    main()
