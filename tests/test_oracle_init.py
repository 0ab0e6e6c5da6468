"""Pins the oracle's table initialisers (reference: csrc/utils/initializer.cu:11-103).

* Zero / Uniform: closed form of the minstd engine, computed here with python integers and exact
  rationals (independent of the oracle's C++): this is the pin.
* Normal / TruncatedNormal: the inverse normal CDF of python's statistics.NormalDist in float64 (the pin of
  the formula) + distribution moments + determinism.
* The two *_vs_reference_build tests compare with the reference's own initializer.cu compiled against the
  image's rocThrust (oracle/_ref), when that library is present.  rocThrust stands in for the CUDA Thrust the
  reference is built with, so these are cross-checks that pin nothing.
"""
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle as orc

M = 2**31 - 1
A = 48271


def _state(seed):
    s = seed % M
    return 1 if s == 0 else s


def _round_f32(fr):
    """Exact rational -> nearest float32 (ties to even) via numpy on an exactly representable double pair."""
    # float(Fraction) is correctly rounded to double; a second rounding to f32 could double-round, so
    # check the two neighbouring floats exactly instead.
    c = np.float32(float(fr))
    cands = [np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))]
    best = min(cands, key=lambda v: (abs(Fraction(float(v)) - fr), int(v.view(np.uint32)) & 1))
    return best


def _uniform_closed_form(n, a, b, seed):
    x = _state(seed) * pow(A, n + 1, M) % M
    r = np.float32(x - 1)                                  # exact conversion rounds to f32
    r = np.float32(r) / (np.float32(1.0) + np.float32(M - 2))
    width = np.float32(b) - np.float32(a)
    return _round_f32(Fraction(float(r)) * Fraction(float(width)) + Fraction(float(np.float32(a))))


@pytest.mark.parametrize("seed", [0, 1, 12345, M, M + 7])
def test_uniform_closed_form(seed):
    a, b = -0.01, 0.01
    got = orc.init_values(4096, "Uniform", a, b, seed)
    idx = list(range(64)) + [100, 1000, 4095]
    for n in idx:
        assert got[n] == _uniform_closed_form(n, a, b, seed), (n, seed)
    assert got.min() >= a and got.max() < b


def test_uniform_far_offsets_match_sequential():
    # discard(n) for huge n equals n single steps: check the skip-ahead against a running product
    seed, a, b = 3, 0.0, 1.0
    n0 = 5_000_000
    big = orc.init_values(n0 + 16, "Uniform", a, b, seed)[n0:]
    for k in range(16):
        assert big[k] == _uniform_closed_form(n0 + k, a, b, seed)


def test_zero():
    assert not orc.init_values(1000, "Zero", 1.0, 2.0, 5).any()


def _ref(n, kind, a, b, seed):
    l = orc.ref_lib()
    if l is None:
        pytest.skip("oracle/_ref not built (reference tree absent at build time)")
    out = np.empty(n, dtype=np.float32)
    l.ref_initialize_host(out.ctypes.data, n, orc.INIT[kind], a, b, seed)
    return out


@pytest.mark.parametrize("seed", [0, 7])
def test_uniform_vs_reference_build(seed):
    a, b = -0.01, 0.01
    ref = _ref(20000, "Uniform", a, b, seed)
    got = orc.init_values(20000, "Uniform", a, b, seed)
    # the host build of the reference has no fused multiply-add: allow one ulp of the range
    assert np.max(np.abs(ref - got)) <= 2e-9
    assert _ref(1000, "Zero", a, b, seed).tolist() == [0.0] * 1000


@pytest.mark.parametrize("kind", ["Normal", "TruncatedNormal"])
def test_normal_vs_reference_build(kind):
    ref = _ref(20000, kind, 0.5, 2.0, 11)
    got = orc.init_values(20000, kind, 0.5, 2.0, 11)
    # same uniform draws, same formula; erfcinv implementations differ in the last bits
    assert np.max(np.abs(ref - got)) <= 2e-5 * 2.0


def _normal_by_inverse_cdf(n, mean, stddev, seed):
    """Element n of the Normal initialiser from the definitions alone: the engine's draw x, thrust's direct sampling
    (csrc/utils/initializer.cu:29-46 -> thrust::normal_distribution, device branch): u = x - 1 in [0, m - 2]; the
    lower half maps to mean - stddev * sqrt(2) * erfcinv(2p), p = (u + 1/2) / (m - 2), the upper half is mirrored
    (u -> m - 2 - u, sign flipped).  -sqrt(2) * erfcinv(2p) is the inverse normal CDF at p: python's own."""
    from statistics import NormalDist
    rng_range = M - 2
    u = _state(seed) * pow(A, n + 1, M) % M - 1
    if u > rng_range // 2:
        return mean - stddev * NormalDist().inv_cdf((rng_range - u + 0.5) / rng_range), u
    return mean + stddev * NormalDist().inv_cdf((u + 0.5) / rng_range), u


@pytest.mark.parametrize("mean,stddev,seed", [(0.0, 1.0, 0), (0.5, 2.0, 11), (-3.0, 0.1, 12345)])
def test_normal_against_the_inverse_normal_cdf(mean, stddev, seed):
    # pins sign, scale and the mirror of the upper half independently of any erfcinv implementation
    got = orc.init_values(3000, "Normal", mean, stddev, seed)
    lower = upper = 0
    for n in list(range(200)) + [777, 1500, 2999]:
        want, u = _normal_by_inverse_cdf(n, mean, stddev, seed)
        lower += u <= (M - 2) // 2
        upper += u > (M - 2) // 2
        assert abs(float(got[n]) - want) <= 1e-6 * stddev + 1.2e-7 * abs(want), (n, got[n], want)
        # the lower half of the draws gives values below the mean, the upper half above
        assert (got[n] < mean) == (u <= (M - 2) // 2) or abs(got[n] - mean) < 1e-6 * stddev
    assert lower > 50 and upper > 50                       # both branches were exercised
    # truncation: the first draw that lies within two sigma, redrawn from the engine reseeded with its own next
    # output (initializer.cu:60-67)
    t = orc.init_values(3000, "TruncatedNormal", mean, stddev, seed)
    redrawn = 0
    for n in range(300):
        x = _state(seed) * pow(A, n + 1, M) % M
        while True:
            rng_range = M - 2
            u = x - 1
            from statistics import NormalDist
            if u > rng_range // 2:
                v = mean - stddev * NormalDist().inv_cdf((rng_range - u + 0.5) / rng_range)
            else:
                v = mean + stddev * NormalDist().inv_cdf((u + 0.5) / rng_range)
            x = x * A % M                                  # rng(): the next output ...
            x = 1 if x % M == 0 else x % M                 # ... becomes the seed
            if not (v > mean + 2 * stddev or v < mean - 2 * stddev):
                break
            redrawn += 1
            x = x * A % M                                  # the next dist(rng) draws from the reseeded engine
        assert abs(float(t[n]) - v) <= 1e-6 * stddev + 1.2e-7 * abs(v), (n, t[n], v)
    assert redrawn >= 5                                    # ~4.6 % of the draws fall outside two sigma


def test_normal_moments_and_determinism():
    x = orc.init_values(400000, "Normal", 1.0, 3.0, 2)
    assert abs(x.mean() - 1.0) < 0.03 and abs(x.std() - 3.0) < 0.03
    y = orc.init_values(1000, "Normal", 1.0, 3.0, 2)
    assert np.array_equal(x[:1000], y)
    t = orc.init_values(200000, "TruncatedNormal", 0.0, 1.0, 9)
    assert t.min() >= -2.0 and t.max() <= 2.0 and abs(t.mean()) < 0.02
    # a truncated draw equals the plain draw wherever the plain draw is already inside 2 sigma
    n = orc.init_values(200000, "Normal", 0.0, 1.0, 9)
    inside = np.abs(n) <= 2.0
    assert np.array_equal(t[inside], n[inside])


def test_uniform_golden_vectors():
    # known answers committed under tests/golden (made by tests/golden/make_vectors.py from the engine's definition)
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "minstd_uniform.json")
    cases = json.load(open(path))["cases"]
    for c in cases:
        small = [(n, b) for n, b in zip(c["offsets"], c["f32_bits"]) if n < 70000]
        got = orc.init_values(70000, "Uniform", c["a"], c["b"], c["seed"]).view(np.uint32)
        for n, bits in small:
            assert int(got[n]) == bits, (c["seed"], c["a"], c["b"], n)
    c = cases[0]
    n_far = c["offsets"][-1]
    far = orc.init_values(n_far + 1, "Uniform", c["a"], c["b"], c["seed"]).view(np.uint32)
    for n, bits in zip(c["offsets"], c["f32_bits"]):
        assert int(far[n]) == bits
