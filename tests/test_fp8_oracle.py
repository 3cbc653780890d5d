"""Pins the 8-bit float (hfp8) part of the oracle without the GPU: the decode
against the format's closed form for all 256 codes and several (exponent bits,
bias) pairs, and against the reference's own Float8ToFloat_ref /
EmbeddingSpMDMFP8_ref compiled from its sources."""
import numpy as np
import pytest

import oracle
from oracle import ST_BF16, ST_FP16, ST_FP32

needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref/libfbgemm_ref.so not built")
FORMATS = [(4, 7), (4, 15), (5, 15), (5, 30), (3, 3), (2, 1)]


@pytest.mark.parametrize("ebits,bias", FORMATS)
def test_decode_is_the_formats_closed_form(ebits, bias):
    mbits = 7 - ebits
    for b in range(256):
        s, e, m = b >> 7, (b >> mbits) & ((1 << ebits) - 1), b & ((1 << mbits) - 1)
        if e == 0:
            want = 2.0 ** (1 - bias) * (m / (1 << mbits))  # subnormal
        else:
            want = 2.0 ** (e - bias) * (1 + m / (1 << mbits))
        want = -want if s else want
        got = oracle.float8_to_float(b, ebits, bias)
        assert got == np.float32(want), (b, got, want)
        assert np.signbit(got) == bool(s)


@needs_ref
@pytest.mark.parametrize("ebits,bias", FORMATS)
def test_decode_matches_reference(ebits, bias):
    for b in range(256):
        a, r = oracle.float8_to_float(b, ebits, bias), oracle.float8_to_float(b, ebits, bias, impl="ref")
        assert np.float32(a).view(np.uint32) == np.float32(r).view(np.uint32)


@needs_ref
@pytest.mark.parametrize("out_ty", [ST_FP32, ST_FP16, ST_BF16])
def test_pooled_lookup_matches_reference(out_ty):
    rng = np.random.default_rng(41)
    for D, rows, nb, weighted, normalize, use_offsets, positional in [
            (8, 50, 6, False, False, True, False), (33, 40, 9, True, True, True, False),
            (128, 100, 12, True, False, False, False), (64, 30, 5, True, True, True, True), (1, 5, 3, False, True, True, False)]:
        stride = D + int(rng.integers(0, 3))
        table = rng.integers(0, 256, size=rows * stride, dtype=np.uint8)
        lens = rng.integers(0, 9, size=nb).astype(np.int64)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        idx = rng.integers(0, rows, size=int(off[-1])).astype(np.int64)
        w = None
        if weighted:
            w = rng.normal(size=max(1, int(lens.max())) if positional else len(idx)).astype(np.float32)
        kw = dict(weights=w, normalize=normalize, out_ty=out_ty, positional=positional, use_offsets=use_offsets,
                  input_stride=stride, exponent_bits=4, exponent_bias=7, data_size=rows, output_size=nb)
        ool = off if use_offsets else lens
        ok_a, a = oracle.spmdm_fp8(D, table, idx, ool, **kw)
        ok_r, r = oracle.spmdm_fp8(D, table, idx, ool, impl="ref", **kw)
        assert ok_a and ok_r
        assert (a.view(np.uint32 if out_ty == ST_FP32 else np.uint16) == r.view(np.uint32 if out_ty == ST_FP32 else np.uint16)).all()
    # rejections: out of range, -1 (the reference's kernel does not skip it), length mismatch
    table = rng.integers(0, 256, size=10 * 4, dtype=np.uint8)
    off = np.asarray([0, 2, 3], np.int64)
    for bad_idx in ([0, 10, 1], [0, -1, 1]):
        idx = np.asarray(bad_idx, np.int64)
        for impl in ("oracle", "ref"):
            ok, _ = oracle.spmdm_fp8(4, table, idx, off, data_size=10, impl=impl)
            assert not ok
    ok, out = oracle.spmdm_fp8(4, table, np.asarray([0, -1, 1], np.int64), off, data_size=10, skip_minus_one=True)
    assert ok  # the table-batched operator's rule: -1 is a pruned row
    for impl in ("oracle", "ref"):
        ok, _ = oracle.spmdm_fp8(4, table, np.asarray([0, 1], np.int64), off, data_size=10, impl=impl)
        assert not ok
