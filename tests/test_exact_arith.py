"""The kernels' division-free quotients (mist_amd/csrc/exact_arith.h) against IEEE division.

The row-term kernel divides by a handful of constants (interference factors, link bandwidths)
about a hundred times per candidate row; it multiplies by the constant's reciprocal and repairs
the quotient with two residual steps.  Here the same header is built for the host and held
against numpy's ``/`` and ``//`` bit for bit, on operands chosen to stress rounding: significands
of all ones, powers of two and their neighbours, few-bit significands, exact multiples, values
an ulp either side of a multiple, signed zeros, infinities and NaN.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("exact_arith") / "libexact_arith_shim.so"
    cmd = ["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fPIC", "-shared",
           "-I" + os.path.join(REPO, "mist_amd", "csrc"), os.path.join(HERE, "exact_arith_shim.cpp"),
           "-o", str(out)]
    subprocess.run(cmd, check=True)
    lib = ctypes.CDLL(str(out))
    ptr = ctypes.c_void_p
    for name in ("quotients_by_reciprocal", "quotients_by_reciprocal_no_negative_zero", "floor_divides"):
        getattr(lib, name).argtypes = [ptr, ptr, ptr, ptr, ctypes.c_long]
        getattr(lib, name).restype = None
    return lib


def _call(fn, a, b):
    a = np.ascontiguousarray(a, dtype=np.float64)
    b = np.ascontiguousarray(b, dtype=np.float64)
    out = np.full(a.shape, np.nan)
    tame = np.zeros(a.shape, dtype=np.uint8)
    fn(a.ctypes.data, b.ctypes.data, out.ctypes.data, tame.ctypes.data, a.size)
    return out, tame.astype(bool)


def _doubles(rng, n, emin, emax):
    """Doubles with exponents in [emin, emax] and significands that stress rounding."""
    mant = rng.integers(0, 1 << 52, n, dtype=np.uint64)
    kind = rng.integers(0, 8, n)
    mant = np.where(kind == 0, (1 << 52) - 1 - rng.integers(0, 4, n, dtype=np.uint64), mant)
    mant = np.where(kind == 1, rng.integers(0, 4, n, dtype=np.uint64), mant)
    keep = ~((np.uint64(1) << rng.integers(0, 52, n, dtype=np.uint64)) - np.uint64(1))
    mant = np.where(kind == 2, mant & keep, mant)
    exp = rng.integers(emin + 1023, emax + 1024, n, dtype=np.uint64)
    return ((exp << np.uint64(52)) | mant).view(np.float64)


def _same_bits(x, y):
    return np.array_equal(x.view(np.uint64), y.view(np.uint64))


def test_quotient_by_reciprocal_is_the_ieee_quotient(shim):
    rng = np.random.default_rng(11)
    n = 4_000_000
    a = _doubles(rng, n, -120, 120) * rng.choice([1.0, 1.0, 1.0, -1.0], n)
    b = _doubles(rng, n, -100, 99)
    got, tame = _call(shim.quotients_by_reciprocal, a, b)
    assert tame.all()
    assert _same_bits(got, a / b)
    # quotients that are exact, or an ulp away from exact: a = q b rounded, and its neighbours
    q = _doubles(rng, n, -20, 20)
    exact = q * b
    for a in (exact, np.nextafter(exact, np.inf), np.nextafter(exact, -np.inf)):
        got, tame = _call(shim.quotients_by_reciprocal, a, b)
        assert tame.all()
        assert _same_bits(got, a / b)


def test_interference_sized_operands(shim):
    """Seconds between 1e-8 and 1e3 scaled by factors near 1, and their differences (which
    cancel to a few ulps or to zero): the operands of the interference model's peels."""
    rng = np.random.default_rng(12)
    n = 2_000_000
    f = np.round(rng.uniform(0.5, 4.0, n), rng.integers(1, 6))
    f = np.where(f <= 0, 1.0, f)
    x = 10.0 ** rng.uniform(-8, 3, n)
    other = np.where(rng.random(n) < 0.3, x * f, 10.0 ** rng.uniform(-8, 3, n))
    a = np.abs(x * f - np.minimum(x * f, other))
    assert (a == 0).sum() > n // 10
    for fn in (shim.quotients_by_reciprocal, shim.quotients_by_reciprocal_no_negative_zero):
        got, tame = _call(fn, a, f)
        assert tame.all()
        assert _same_bits(got, a / f)


def test_untamed_operands_are_sent_to_the_division(shim):
    a = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-300, 1e300, 1.0, 1.0, 1.0, 5e-324])
    b = np.array([3.0, 3.0, 3.0, 3.0, 3.0, 3.0, 3.0, 0.0, 1e-40, 1e40, 3.0])
    got, tame = _call(shim.quotients_by_reciprocal, a, b)
    assert tame.tolist() == [True, True] + [False] * 9
    assert _same_bits(got[:2], np.array([0.0, -0.0]))  # signed zeros survive


def test_floor_divide_is_numpys(shim):
    rng = np.random.default_rng(13)
    n = 4_000_000
    b = _doubles(rng, n, -30, 30)
    a = _doubles(rng, n, -30, 60)
    cases = [(a, b)]
    k = np.floor(10.0 ** rng.uniform(0, 14, n))  # exact multiples and their neighbours
    for shift in (0.0, np.inf, -np.inf):
        m = k * b
        cases.append((m if shift == 0.0 else np.nextafter(m, shift), b))
    cases.append((np.floor(rng.uniform(0, 1e6, n)), np.floor(rng.uniform(1, 64, n))))  # sizes / ranks
    cases.append((np.zeros(8), np.arange(1.0, 9.0)))
    checked = 0
    for a, b in cases:
        got, tame = _call(shim.floor_divides, a, b)
        with np.errstate(all="ignore"):
            want = np.floor_divide(a, b)
        assert _same_bits(got[tame], want[tame])
        checked += int(tame.sum())
    assert checked > 3 * n
    # what the fast path must leave to the general one
    a = np.array([-1.0, 1.0, 1.0, np.inf, np.nan, 1e80, 2.0 ** 60])
    b = np.array([2.0, 0.0, -2.0, 2.0, 2.0, 1e-30, 1.0])
    _, tame = _call(shim.floor_divides, a, b)
    assert not tame.any()
