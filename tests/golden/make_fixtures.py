"""Writes tests/golden/fixtures.json: small known-answer vectors computed without the oracle and without the library.

* rng: the counter-based generator, restated with Python integers: z = seed * 0x9E3779B97F4A7C15 + idx +
  0x632BE59BD9B4E019 (mod 2^64), splitmix64 finaliser, top 24 bits -> (v - 2^23) / 2^23.
* saxpy: fused multiply-add cases evaluated in exact rational arithmetic and rounded once to float32
  (round-to-nearest-even), including cases where an unfused a*x + y differs.
* abft: the one fault experiment the reference holds: +1.0 at tile-local (0, 1), threshold 0.1 ->
  row 0 / column 1 flagged, 1.0 removed (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:30,40,145,263,358).

Run from the repository root: python tests/golden/make_fixtures.py
"""
import json
import os
import struct
from fractions import Fraction

MASK = (1 << 64) - 1


def mix64(z):
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def uniform(seed, idx):
    z = mix64((seed * 0x9E3779B97F4A7C15 + idx + 0x632BE59BD9B4E019) & MASK)
    return ((z >> 40) - (1 << 23)) / float(1 << 23)


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def round_to_f32(q):
    """Nearest float32 (ties to even) of a Fraction, by bisection on the float32 grid around float(q)."""
    guess = f32(float(q))
    bits = struct.unpack("<I", struct.pack("<f", guess))[0]
    cands = []
    for d in (-1, 0, 1):
        b = bits + d
        if 0 <= b < 0x7F800000 or 0x80000000 <= b < 0xFF800000:
            cands.append((struct.unpack("<f", struct.pack("<I", b & 0xFFFFFFFF))[0], b))
    best = min(cands, key=lambda c: (abs(Fraction(c[0]) - q), c[1] & 1))
    return best[0]


def main():
    rng = [{"seed": s, "idx": i, "value": uniform(s, i)}
           for s in (0, 1, 31, 2 ** 40 + 7) for i in (0, 1, 2, 1023, 2 ** 31 + 5, 2 ** 40)]
    saxpy = []
    for a, x, y in [(2.5, 0.1, -0.25), (1.0 + 2.0 ** -12, 1.0 + 2.0 ** -12, -1.0), (3.0, 1.0 / 3.0, -1.0),
                    (-7.25e4, 1.2345678e-3, 89.5), (2.5, 0.33333334, 1e-8), (1e-20, 1e-20, 1e-30)]:
        a, x, y = f32(a), f32(x), f32(y)
        fused = round_to_f32(Fraction(a) * Fraction(x) + Fraction(y))
        unfused = f32(f32(a * x) + y)
        saxpy.append({"a": a, "x": x, "y": y, "fused": fused, "unfused": unfused})
    abft = {"tile_m": 128, "tile_n": 128, "fault": {"row": 0, "col": 1, "delta": 1.0}, "threshold": 0.1,
            "expect": {"flag": 1, "row": 0, "col": 1, "n_bad_rows": 1, "n_bad_cols": 1, "correction": -1.0}}
    out = {"rng": rng, "saxpy": saxpy, "abft": abft}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
