"""Pins the C oracle against the reference's own scalar code compiled from its
sources (oracle/_ref, built by `make -C oracle ref`). Skipped where that build
is absent; tests/test_oracle_golden.py then holds the same comparison as
committed vectors.

Shapes and corner cases follow the reference's unit tests
(test/EmbeddingSpMDMNBitTest.cc:21-46,74-90, test/EmbeddingSpMDM8BitTest.cc:20-43,65-80):
odd dims, empty indices, an out-of-range index, a lengths-sum mismatch."""
import itertools

import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

pytestmark = pytest.mark.skipif(
    not __import__("oracle").have_ref(), reason="oracle/_ref not built on this machine")

# (batch, rows, D, avg_len) after the reference's list, trimmed to what runs in seconds
SHAPES = [
    (10, 400, 2, 5), (10, 400, 4, 5), (10, 400, 7, 5), (10, 400, 8, 5), (10, 400, 16, 5),
    (10, 400, 40, 5), (10, 400, 48, 5), (10, 400, 56, 5), (3, 1000, 86, 20),
    (2, 1000, 128, 50), (10, 400, 164, 5), (4, 300, 256, 10), (1, 50, 32, 100), (0, 20, 32, 5),
]


def both(o, **kw):
    ok_a, out_a = o.spmdm(impl="oracle", **kw)
    ok_b, out_b = o.spmdm(impl="ref", **kw)
    assert ok_a == ok_b, kw
    if ok_a:
        H.assert_same_bits(out_a, out_b, "oracle vs reference")
    return ok_a


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32, BF16])
@pytest.mark.parametrize("shape", SHAPES)
def test_spmdm_matches_reference(oracle, ty, shape):
    nb, rows, D, avg = shape
    if ty == INT2 and D % 4 and D > 4:
        D = (D + 3) // 4 * 4
    rng = np.random.default_rng(hash((ty, shape)) % 2**32)
    for sbl, out_ty, weighted, normalize, idx_dt, off_dt, use_offsets in itertools.product(
            (True, False), (FP32, FP16, BF16), (0, 1, 2), (False, True),
            (np.int32, np.int64), (np.int32, np.int64), (True, False)):
        if rng.random() > 0.12:  # sample the cross product; every axis still varies
            continue
        if ty in (FP16, FP32, BF16) and not sbl and rng.random() < 0.5:
            continue
        table, stride = H.make_table(rng, ty, rows, D, sbl)
        idx, off, lens = H.make_bags(rng, rows, nb, avg, idx_dt, off_dt, empty_frac=0.2)
        if not sbl and len(idx):
            idx[rng.random(len(idx)) < 0.2] = -1
        w = None
        if weighted == 1:
            w = rng.normal(size=len(idx)).astype(np.float32)
        elif weighted == 2:
            w = rng.normal(size=max(1, int(lens.max()) if len(lens) else 1)).astype(np.float32)
        both(oracle, in_ty=ty, block_size=D, table=table, indices=idx,
             offsets_or_lengths=off if use_offsets else lens, weights=w, normalize=normalize,
             out_ty=out_ty, positional=weighted == 2, use_offsets=use_offsets,
             scale_bias_last=sbl, data_size=rows, output_size=nb)


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16])
def test_strides_and_tbe_layout(oracle, ty):
    rng = np.random.default_rng(7 + ty)
    rows, D, nb = 300, 64, 12
    for align in (1, 16):
        stride = oracle.padded_row_bytes(D, ty, align)
        table, stride = H.make_table(rng, ty, rows, D, False, stride_bytes=stride)
        idx, off, _ = H.make_bags(rng, rows, nb, 6)
        idx[::5] = -1
        total_D = D + 24
        ok = both(oracle, in_ty=ty, block_size=D, table=table, indices=idx, offsets_or_lengths=off,
                  weights=rng.uniform(size=len(idx)).astype(np.float32), out_ty=FP16,
                  output_stride=total_D, input_stride=H.input_stride_elems(ty, stride),
                  scale_bias_last=False, data_size=rows)
        assert ok


@pytest.mark.parametrize("ty", [INT8, INT4, INT2])
def test_rejections_match(oracle, ty):
    rng = np.random.default_rng(11 + ty)
    rows, D, nb = 100, 32, 8
    table, _ = H.make_table(rng, ty, rows, D, True)
    idx, off, _ = H.make_bags(rng, rows, nb, 5)
    kw = dict(in_ty=ty, block_size=D, table=table, data_size=rows)
    assert both(oracle, indices=idx, offsets_or_lengths=off, **kw)
    bad = idx.copy(); bad[len(bad) // 2] = rows
    assert not both(oracle, indices=bad, offsets_or_lengths=off, **kw)
    bad = idx.copy(); bad[1] = -1  # -1 is not a skip in the trailer layout
    assert not both(oracle, indices=bad, offsets_or_lengths=off, **kw)
    assert not both(oracle, indices=idx, offsets_or_lengths=off, index_size=len(idx) - 1, **kw)
    assert not both(oracle, indices=np.concatenate([idx, idx[:1]]), offsets_or_lengths=off,
                    index_size=len(idx) + 1, **kw)
    # empty index list with non-empty bags (the reference's EMPTY_INDICES corner case)
    assert not both(oracle, indices=np.zeros(0, idx.dtype), offsets_or_lengths=off, **kw)
    zero_off = np.zeros_like(off)
    assert both(oracle, indices=np.zeros(0, idx.dtype), offsets_or_lengths=zero_off, **kw)


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32])
def test_rowwise_sparse_matches(oracle, ty):
    rng = np.random.default_rng(23 + ty)
    logical, D, nb = 500, 48, 16
    # 70% pruned mapping as test/EmbeddingSpMDMTestUtils.cc:89-109 builds it
    keep = rng.random(logical) >= 0.7
    mapping = np.full(logical, -1, np.int32)
    mapping[keep] = np.arange(int(keep.sum()), dtype=np.int32)
    rows = max(1, int(keep.sum()))
    table, _ = H.make_table(rng, ty, rows, D, True)
    for weighted, normalize, idx_dt, use_offsets in itertools.product((0, 1, 2), (False, True), (np.int32, np.int64), (True, False)):
        idx, off, lens = H.make_bags(rng, logical, nb, 8, idx_dt, np.int32)
        w = None
        if weighted == 1:
            w = rng.normal(size=len(idx)).astype(np.float32)
        elif weighted == 2:
            w = rng.normal(size=int(lens.max())).astype(np.float32)
        ok = both(oracle, in_ty=ty, block_size=D, table=table, indices=idx,
                  offsets_or_lengths=off if use_offsets else lens, weights=w, normalize=normalize,
                  positional=weighted == 2, use_offsets=use_offsets, remap=mapping,
                  data_size=logical, output_size=nb)
        assert ok
    bad = idx.copy(); bad[0] = logical
    assert not both(oracle, in_ty=ty, block_size=D, table=table, indices=bad, offsets_or_lengths=off,
                    remap=mapping, data_size=logical)


@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
def test_compressed_indices_remap_matches(oracle, idx_dt):
    rng = np.random.default_rng(5)
    logical, nb = 1000, 40
    mapping = np.where(rng.random(logical) < 0.5, -1, 0).astype(np.int32)
    mapping[mapping == 0] = np.arange(int((mapping == 0).sum()), dtype=np.int32)
    idx, off, _ = H.make_bags(rng, logical, nb, 10, idx_dt, idx_dt, empty_frac=0.1)
    for w in (None, rng.normal(size=len(idx)).astype(np.float32)):
        a = oracle.compressed_indices_remap(idx, mapping, off, w, impl="oracle")
        b = oracle.compressed_indices_remap(idx, mapping, off, w, impl="ref")
        for x, y in zip(a, b):
            if x is None:
                assert y is None
            else:
                H.assert_same_bits(x, y, "compressed_indices_remap")


def test_conversions_match(oracle):
    h = np.arange(65536, dtype=np.uint16)
    H.assert_same_bits(oracle.half2float(h), oracle.half2float(h, "ref"), "half2float")
    rng = np.random.default_rng(3)
    f = rng.integers(0, 2**32, size=1_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    edge = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e30, -1e30, 6.1e-5, 5.96e-8, 2.98e-8,
                     2.9802322e-8, 2.9802326e-8, 1e-10, np.inf, -np.inf], np.float32)
    f = np.concatenate([f, edge])
    H.assert_same_bits(oracle.float2half_rn(f), oracle.float2half_rn(f, "ref"), "float2half_rn")
    H.assert_same_bits(oracle.float2bf16(f), oracle.float2bf16(f, "ref"), "float2bf16")
