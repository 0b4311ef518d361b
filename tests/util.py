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


STRICT_LOG = os.path.join(os.path.dirname(os.path.dirname(GOLDEN)), "gpurun_out", "strict_f32_bar.jsonl")


def strict_bar(got, truth, what, max_outside_frac, max_excess, reference=None):
    """The stated float32 bar without any scaling: against `truth` (the same computation with float64
    accumulation), count the elements outside |a - b| <= 1e-4 * |b| + 1e-5 and take the worst excess over that
    bound.  Prints the figures, appends them to STRICT_LOG and asserts the given limits
    (a fraction of the elements, and an absolute excess).  `reference`: the float32 sequential-order oracle's result
    for the same inputs; its own count against the same truth is recorded beside the GPU's."""
    import json
    got = np.asarray(got, np.float64).ravel()
    truth = np.asarray(truth, np.float64).ravel()
    assert got.shape == truth.shape, (what, got.shape, truth.shape)
    err = np.abs(got - truth)
    excess = err - (RTOL * np.abs(truth) + ATOL)
    outside = int((excess > 0).sum())
    rec = {"what": what, "elements": int(got.size), "outside_strict_bar": outside,
           "outside_frac": outside / max(1, got.size), "worst_excess": float(max(0.0, excess.max())),
           "max_abs_err": float(err.max()), "max_abs_value": float(np.abs(truth).max())}
    if reference is not None:
        r = np.asarray(reference, np.float64).ravel()
        rex = np.abs(r - truth) - (RTOL * np.abs(truth) + ATOL)
        rec["reference_f32_outside"] = int((rex > 0).sum())
        rec["reference_f32_worst_excess"] = float(max(0.0, rex.max()))
    print("strict float32 bar: %(what)s: %(outside_strict_bar)d of %(elements)d outside (%(outside_frac).2e), "
          "worst excess %(worst_excess).3g, max |err| %(max_abs_err).3g at max |y| %(max_abs_value).3g" % rec)
    try:
        os.makedirs(os.path.dirname(STRICT_LOG), exist_ok=True)
        with open(STRICT_LOG, "a") as f:
            f.write(json.dumps(rec) + "\n")
    except OSError:
        pass
    assert rec["outside_frac"] <= max_outside_frac, rec
    assert rec["worst_excess"] <= max_excess, rec
    return rec
