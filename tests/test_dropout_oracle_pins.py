"""Pins of oracle/dropout_oracle.py (CPU only).

* ``philox4x32_10`` against the known-answer vectors that the Random123 distribution ships for philox4x32 with 10
  rounds (kat_vectors: counter / key of zeros, of ones, and of the digits of pi).
* ``randint`` / ``rand`` bit for bit against tests/golden/dropout_golden.npz, which holds what Triton's ``tl.randint``
  / ``tl.rand`` return for the same seeds and offsets (32-bit offsets up to 2^31 - 1 and 64-bit offsets).
* ``dropout``: the closed forms (kept entries are x / (1 - p) in float32, dropped ones 0, the mask depends on seed and
  position only) and the keep rate against the binomial bound.
"""
import os

import numpy as np
import pytest

from oracle import dropout_oracle as do

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dropout_golden.npz"))


def test_philox_known_answers():
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for counter, key, expect in kat:
        got = do.philox4x32_10(counter, key)
        assert tuple(int(g) for g in got) == expect, [hex(int(g)) for g in got]


def cases(prefix):
    for name in GOLDEN.files:
        if name.startswith(prefix + "_s"):
            seed, first = name[len(prefix) + 2:].split("_o")
            yield name, int(seed), int(first), GOLDEN[name]


def test_randint_matches_triton_bit_for_bit():
    n = 0
    for prefix in ("randint", "randint64"):
        for name, seed, first, expect in cases(prefix):
            offs = np.arange(expect.size, dtype=np.uint64) + np.uint64(first)
            assert np.array_equal(do.randint(seed, offs), expect), name
            n += 1
    assert n == 8


def test_rand_matches_triton_bit_for_bit():
    n = 0
    for prefix in ("rand", "rand64"):
        for name, seed, first, expect in cases(prefix):
            offs = np.arange(expect.size, dtype=np.uint64) + np.uint64(first)
            got = do.rand(seed, offs)
            assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), expect.view(np.uint32)), name
            assert (got >= 0).all() and (got < 1).all()
            n += 1
    assert n == 8


def test_rand_extremes():
    # the fold maps int32 -1 and 0 to 0 and both ends of the range to the largest value, which stays below 1
    assert np.float32(2 ** 31 - 1) * do.RAND_SCALE < np.float32(1.0)
    v = np.array([-2 ** 31, -1, 0, 2 ** 31 - 1], dtype=np.int64)
    folded = np.where(v < 0, -v - 1, v)
    assert folded.tolist() == [2 ** 31 - 1, 0, 0, 2 ** 31 - 1]


@pytest.mark.parametrize("p", [0.1, 0.5, 0.9])
def test_dropout_closed_forms_and_keep_rate(p):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 1000)).astype(np.float32)
    y = do.dropout(x, p, seed=1234)
    r = do.rand(1234, np.arange(x.size, dtype=np.uint64)).reshape(x.shape)
    dropped = r < np.float32(p)
    assert (y[dropped] == 0).all()
    assert np.array_equal(y[~dropped], x[~dropped] / (np.float32(1) - np.float32(p)))
    n = x.size
    rate = dropped.mean()
    assert abs(rate - p) < 5 * np.sqrt(p * (1 - p) / n), rate           # five standard deviations
    # the mask is a function of (seed, position): another input, the same mask; another seed, another mask
    y2 = do.dropout(np.ones_like(x), p, seed=1234)
    assert np.array_equal(y2 == 0, dropped)
    y3 = do.dropout(np.ones_like(x), p, seed=1235)
    assert 0.2 * min(p, 1 - p) < ((y3 == 0) != dropped).mean() < 2.5 * min(p, 1 - p) + 0.3
    # float64 storage: the float64 quotient by the float32 (1 - p)
    y64 = do.dropout(x.astype(np.float64), p, seed=1234)
    keep = np.float64(np.float32(1) - np.float32(p))
    assert y64.dtype == np.float64 and np.array_equal(y64[~dropped], x.astype(np.float64)[~dropped] / keep)


def test_float64_product_rounds_like_the_float32_division():
    """The kernel divides by the shared float32 (1 - p) as float32(float64(x) * (1 / float64(1 - p))).  That equals the
    correctly rounded float32 quotient for every x (the quotient of two float32 values stays 2^-49 away from any
    rounding boundary, the product is within 2^-52 of it): checked here on 6 million (x, p) pairs, including
    subnormal and huge x, p next to 0 and 1, and every float32 x of one binade."""
    rng = np.random.default_rng(17)
    n = 2_000_000
    xs = [rng.standard_normal(n).astype(np.float32) * np.float32(10.0) ** rng.integers(-44, 38, n).astype(np.float32),
          rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32),
          (np.arange(n, dtype=np.uint32) * np.uint32(4) + np.uint32(0x3F800000)).view(np.float32)]
    ps = [rng.random(n).astype(np.float32), np.float32(1.0) - np.float32(2.0) ** -rng.integers(1, 25, n).astype(np.float32),
          rng.random(n).astype(np.float32) * np.float32(1e-3)]
    with np.errstate(all="ignore"):
        for x, p in zip(xs, ps):
            keep = np.float32(1.0) - p
            ok = keep > 0
            x, keep = x[ok], keep[ok]
            want = x / keep
            got = (x.astype(np.float64) * (1.0 / keep.astype(np.float64))).astype(np.float32)
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
            assert same.all(), (x[~same][:4], keep[~same][:4])
