"""Shared helpers for the test-suite (numpy only)."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# float32 parity bar: |a - b| <= RTOL * |b| + ATOL  (max relative error 1e-4 per element,
# absolute 1e-5 near zero)
RTOL = 1e-4
ATOL = 1e-5


def assert_close_f32(got, want, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + atol
    bad = np.nonzero(~(err <= bound))[0]
    if bad.size:
        i = bad[np.argmax(err[bad] - bound[bad])]
        raise AssertionError("%s: %d/%d elements outside tol; worst at %d: got %r want %r (err %g)"
                             % (what, bad.size, got.size, i, got[i], want[i], err[i]))


def assert_equal_exact(got, want, what=""):
    got = np.asarray(got).ravel()
    want = np.asarray(want).ravel()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if not np.array_equal(got, want):
        bad = np.nonzero(got != want)[0]
        raise AssertionError("%s: %d/%d mismatches; first at %d: got %r want %r"
                             % (what, bad.size, got.size, bad[0], got[bad[0]], want[bad[0]]))


def read_ref_bin(path):
    """Reference regression blob: 4-byte big-endian element count, then little-endian float32
    (test/test_utils.hpp:188-215 in the reference)."""
    with open(path, "rb") as f:
        raw = f.read()
    n = int.from_bytes(raw[:4], "big")
    a = np.frombuffer(raw, dtype="<f4", offset=4)
    assert a.size == n, (path, a.size, n)
    return a.astype(np.float32)
