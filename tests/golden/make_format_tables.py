"""Writes tests/golden/format_tables.json: the e4m3fn and e2m1 value tables, computed from the
format definitions (OCP FP8: bias 7, no infinities, NaN = S.1111.111; OCP MX e2m1) without
importing the oracle, so that the oracle's own tables can be checked against them."""
import json
import os

e4 = []
for c in range(256):
    sgn = -1.0 if c & 0x80 else 1.0
    e, m = (c >> 3) & 15, c & 7
    if e == 15 and m == 7:
        e4.append(None)
    elif e == 0:
        e4.append(sgn * m / 512.0)
    else:
        e4.append(sgn * (8 + m) / 8.0 * 2.0 ** (e - 7))
e2 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
e2 = e2 + [-v for v in e2]
out = {"e4m3_decode": e4, "e2m1_decode": e2,
       "note": "OCP FP8 e4m3fn (bias 7, no inf, NaN=S.1111.111) and OCP MX e2m1 value tables"}
json.dump(out, open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "format_tables.json"), "w"))
