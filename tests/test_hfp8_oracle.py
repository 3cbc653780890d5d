"""Pins the oracle's fp32 -> 8-bit float (hfp8) encoder without the GPU: against
the reference's FloatToFloat8_ref compiled from its sources, and against what
the format fixes: every code is a fixed point of decode -> encode, and any
other value goes to the nearest representable magnitude, ties to the even
code, saturating at max_pos."""
import numpy as np
import pytest

import oracle

needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref/libfbgemm_ref.so not built")
FORMATS = [(4, 7), (5, 15), (3, 3), (2, 1), (4, 4)]


def samples(rng, ebits, bias):
    mags = np.array([oracle.float8_to_float(b, ebits, bias) for b in range(128)], dtype=np.float32)
    mid = ((mags[:-1].astype(np.float64) + mags[1:]) / 2).astype(np.float32)  # exact: one more mantissa bit
    x = np.concatenate([
        mags, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
        rng.normal(size=4000).astype(np.float32) * np.float32(mags[-1] / 4),
        (rng.uniform(-1, 1, size=4000) * 2.0 ** rng.integers(-30, 20, size=4000)).astype(np.float32),
        np.array([0.0, 1e-30, 1e-45, 3e38, np.inf], dtype=np.float32)])
    return np.concatenate([x, -x]), mags


@needs_ref
@pytest.mark.parametrize("ebits,bias", FORMATS)
def test_encoder_matches_reference(ebits, bias):
    x, _ = samples(np.random.default_rng(ebits * 100 + bias), ebits, bias)
    a = oracle.float_to_hfp8(x, ebits, bias)
    r = oracle.float_to_hfp8(x, ebits, bias, impl="ref")
    assert (a == r).all()


@pytest.mark.parametrize("ebits,bias", FORMATS)
def test_encoder_is_nearest_even_and_saturates(ebits, bias):
    x, mags = samples(np.random.default_rng(ebits * 100 + bias + 1), ebits, bias)
    max_pos = oracle.hfp8_max_pos(ebits, bias)
    top = int(np.nonzero(mags <= max_pos)[0].max())
    assert mags[top] == max_pos  # the largest finite code the reference uses
    got = oracle.float_to_hfp8(x, ebits, bias)
    grid = mags[:top + 1].astype(np.float64)
    ax = np.minimum(np.abs(x).astype(np.float64), float(max_pos))
    hi = np.clip(np.searchsorted(grid, ax), 1, top)
    lo = hi - 1
    dl, dh = ax - grid[lo], grid[hi] - ax
    want = np.where(dl < dh, lo, np.where(dh < dl, hi, np.where(lo % 2 == 0, lo, hi)))
    want = want.astype(np.uint8) | (np.signbit(x).astype(np.uint8) << 7)
    assert (got == want).all(), np.nonzero(got != want)[0][:5]
    # every code at or below max_pos is a fixed point
    codes = np.arange(top + 1, dtype=np.uint8)
    assert (oracle.float_to_hfp8(mags[:top + 1], ebits, bias) == codes).all()
    assert (oracle.float_to_hfp8(-mags[:top + 1], ebits, bias) == (codes | 0x80)).all()


def test_explicit_max_pos_clamps():
    x = np.array([1.0, 3.0, 100.0, -100.0], dtype=np.float32)
    got = oracle.float_to_hfp8(x, 4, 7, max_pos=2.0)
    back = [oracle.float8_to_float(int(b), 4, 7) for b in got]
    assert back == [1.0, 2.0, 2.0, -2.0]
