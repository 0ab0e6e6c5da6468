"""Writes tests/golden/minstd_uniform.json: known answers for the Uniform initialiser (reference:
csrc/utils/initializer.cu:72-88, thrust::minstd_rand + uniform_real_distribution), computed from the published
definition of the engine with python integers and exact rationals.  Nothing of the reference is imported or run.

    python tests/golden/make_vectors.py
"""
import json
import os
from fractions import Fraction

import numpy as np

M, A = 2**31 - 1, 48271


def round_f32(fr):
    c = np.float32(float(fr))
    cands = [np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))]
    return min(cands, key=lambda v: (abs(Fraction(float(v)) - fr), int(v.view(np.uint32)) & 1))


def uniform(n, a, b, seed):
    s = seed % M or 1
    x = s * pow(A, n + 1, M) % M                     # state after n + 1 steps: element n discards n draws
    r = np.float32(np.float32(x - 1)) / (np.float32(1.0) + np.float32(M - 2))
    width = np.float32(b) - np.float32(a)
    return round_f32(Fraction(float(r)) * Fraction(float(width)) + Fraction(float(np.float32(a))))


def main():
    offsets = list(range(32)) + [63, 64, 1000, 4095, 65536, 1_000_003, 33_762_576]
    cases = []
    for seed in (0, 1, 7, 12345, M, M + 7):
        for a, b in ((-0.01, 0.01), (0.0, 1.0), (-1.0, 1.0)):
            bits = [int(np.float32(uniform(n, a, b, seed)).view(np.uint32)) for n in offsets]
            cases.append({"seed": seed, "a": a, "b": b, "offsets": offsets, "f32_bits": bits})
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "minstd_uniform.json")
    with open(out, "w") as f:
        json.dump({"engine": "minstd_rand: x <- 48271 x mod (2^31 - 1); value n uses the state after n + 1 steps",
                   "cases": cases}, f, indent=0)
    print("wrote", out, len(cases), "cases")


if __name__ == "__main__":
    main()
