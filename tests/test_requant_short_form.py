"""The uint8 one-launch kernel's short epilogue (qmodel_u8.hip, conv_tiles): with a positive multiplier and rshift >= 2 it
takes idx = high word of (acc << lshift) * multiplier + 2^30, shifted right by rshift - 2, clamps it to 0..513 and reads the
byte from a table built as clamp((idx >> 1) - (idx & 1), 0, 255).  Checked here, on the CPU, against the oracle's
requantisation (the reference's VQRDMULH + RNDRSHIFT with its -1 rounding term) over accumulators that land below, inside
and above the byte range, at the rounding thresholds, and at the ends of the int32 range."""
import numpy as np
import pytest

from oracle.binding import quant


def _short_form(acc, mult, ls, rs):
    shifted = np.int64(np.int32(np.uint32((int(acc) << ls) & 0xffffffff)))
    prod = int(shifted) * int(mult) + (1 << 30)
    hi = prod >> 32                                   # arithmetic: the kernel reads the 64-bit product's high word
    idx = hi >> (rs - 2)
    idx = 0 if idx < 0 else (513 if idx > 513 else idx)
    r = (idx >> 1) - (idx & 1)
    return 0 if r < 0 else (255 if r > 255 else r)


@pytest.mark.parametrize("mult", [1, 3, (1 << 30) - 1, 1 << 30, (1 << 30) + 12345, 1518500250, (1 << 31) - 1])
@pytest.mark.parametrize("ls,rs", [(0, 2), (0, 3), (0, 7), (0, 9), (0, 15), (0, 31), (1, 8), (3, 12)])
def test_short_form_equals_the_oracle(oracle, mult, ls, rs):
    rng = np.random.default_rng(mult % 1000 + 37 * rs + ls)
    oq = quant(0, mult, ls, rs)
    # accumulators whose result lies around 0..255: v = acc * 2^ls * mult / 2^31 ~ r * 2^rs
    scale = (1 << 31) / (mult * (1 << ls)) * (1 << rs)
    around = (rng.uniform(-20, 300, 3000) * scale).clip(-2**31, 2**31 - 1).astype(np.int64)
    thresholds = (np.arange(0, 258, 0.5)[:, None] * scale + np.arange(-3, 4)[None, :]).ravel().clip(-2**31, 2**31 - 1).astype(np.int64)
    ends = np.array([-2**31, -2**31 + 1, -1, 0, 1, 2**31 - 1, 2**31 - 2], np.int64)
    anywhere = rng.integers(-2**31, 2**31, 2000)
    bad = []
    for acc in np.concatenate([around, thresholds, ends, anywhere]):
        if ls and not (-(1 << (31 - ls)) <= acc < (1 << (31 - ls))):
            continue                                  # the left shift would wrap: both sides wrap alike, covered by ls == 0 ends
        want = oracle.requant(int(acc), oq)
        got = _short_form(int(acc), mult, ls, rs)
        if want != got:
            bad.append((int(acc), want, got))
    assert not bad, bad[:5]
