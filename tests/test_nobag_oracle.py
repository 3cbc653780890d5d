"""Pins the oracle's single-table no_bag mode (one output row per index) without
the GPU: against the no_bag branches of the reference's EmbeddingSpMDM_ref /
EmbeddingSpMDMNBit_ref compiled from its sources, against the pooled oracle on
bags of one (the reference's own identity, nbit_forward_test.py:1060-1160), and
against the closed form of a single weighted row."""
import numpy as np
import pytest

import oracle
from oracle import ST_BF16, ST_FP16, ST_FP32, ST_INT4, ST_INT8

needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref/libfbgemm_ref.so not built")


def bits(a):
    return a.view({4: np.uint32, 2: np.uint16, 1: np.uint8}[a.dtype.itemsize])


def make_table(rng, in_ty, D, rows, scale_bias_last, pad=0):
    """Returns (table array in the storage type, input_stride in storage elements)."""
    if in_ty == ST_INT8:
        sb = 8 if scale_bias_last else 4
        stride = D + sb + pad
        t = rng.integers(0, 256, size=(rows, stride), dtype=np.uint8)
        s = rng.uniform(0.01, 0.1, size=rows).astype(np.float32)
        b = rng.uniform(-1, 1, size=rows).astype(np.float32)
        if scale_bias_last:
            t[:, D:D + 4] = s.view(np.uint8).reshape(rows, 4)
            t[:, D + 4:D + 8] = b.view(np.uint8).reshape(rows, 4)
        else:
            t[:, 0:2] = s.astype(np.float16).view(np.uint8).reshape(rows, 2)
            t[:, 2:4] = b.astype(np.float16).view(np.uint8).reshape(rows, 2)
        return t.reshape(-1), stride
    if in_ty == ST_INT4:
        stride = (D + 1) // 2 + 4 + pad
        return rng.integers(0, 256, size=rows * stride, dtype=np.uint8), stride
    stride = D + pad
    if in_ty == ST_FP32:
        return rng.normal(size=rows * stride).astype(np.float32), stride
    x = rng.normal(size=rows * stride).astype(np.float32)
    if in_ty == ST_FP16:
        return x.astype(np.float16).view(np.uint16), stride
    return (x.view(np.uint32) >> 16).astype(np.uint16), stride


CASES = [(ST_INT8, ST_FP32, True), (ST_INT8, ST_FP16, True), (ST_INT8, ST_BF16, False), (ST_INT8, ST_FP32, False),
         (ST_INT8, ST_INT8, True), (ST_INT8, ST_INT8, False), (ST_INT4, ST_INT4, True), (ST_INT4, ST_INT4, False),
         (ST_FP32, ST_FP32, True), (ST_FP32, ST_FP16, True), (ST_FP16, ST_FP32, True), (ST_FP16, ST_FP16, True),
         (ST_BF16, ST_BF16, True), (ST_BF16, ST_FP32, True)]


@needs_ref
@pytest.mark.parametrize("in_ty,out_ty,sbl", CASES)
def test_matches_reference(in_ty, out_ty, sbl):
    rng = np.random.default_rng(7 + in_ty * 10 + out_ty)
    for D, rows, n, pad, weighted in [(8, 20, 13, 0, False), (33, 17, 40, 3, True), (128, 50, 64, 0, True), (1, 3, 5, 0, False), (64, 9, 0, 0, True)]:
        if in_ty == ST_INT4 and D % 2:
            D += 1
        table, stride = make_table(rng, in_ty, D, rows, sbl, pad)
        idx = rng.integers(0, rows, size=n).astype(np.int64)
        w = rng.normal(size=max(n, 1)).astype(np.float32)[:n] if weighted else None
        for ostride in ([-1, D + 5] if out_ty not in (ST_INT8, ST_INT4) else [-1, stride, stride + 3, max(1, stride - 2)]):
            kw = dict(weights=w, out_ty=out_ty, output_stride=ostride, input_stride=stride if pad else -1,
                      scale_bias_last=sbl, data_size=rows)
            ok_a, a = oracle.spmdm_nobag(in_ty, D, table, idx, **kw)
            ok_r, r = oracle.spmdm_nobag(in_ty, D, table, idx, impl="ref", **kw)
            assert ok_a and ok_r
            assert (bits(a) == bits(r)).all(), (D, rows, n, pad, ostride)


@needs_ref
@pytest.mark.parametrize("in_ty,out_ty,sbl", [(ST_INT8, ST_FP32, True), (ST_INT8, ST_INT8, False), (ST_FP16, ST_FP16, True), (ST_INT4, ST_INT4, False)])
def test_rejections_match_reference(in_ty, out_ty, sbl):
    rng = np.random.default_rng(3)
    D, rows = 16, 10
    table, stride = make_table(rng, in_ty, D, rows + 1, sbl)  # one spare row: the 4-bit copy lets idx == data_size through
    for bad in (-1, -5, rows + 1, 1 << 40):
        idx = np.array([1, 2, bad, 3], dtype=np.int64)
        ok_a, _ = oracle.spmdm_nobag(in_ty, D, table, idx, out_ty=out_ty, scale_bias_last=sbl, data_size=rows)
        ok_r, _ = oracle.spmdm_nobag(in_ty, D, table, idx, impl="ref", out_ty=out_ty, scale_bias_last=sbl, data_size=rows)
        assert not ok_a and not ok_r
    idx = np.array([1, rows, 3], dtype=np.int64)
    ok_a, _ = oracle.spmdm_nobag(in_ty, D, table, idx, out_ty=out_ty, scale_bias_last=sbl, data_size=rows)
    ok_r, _ = oracle.spmdm_nobag(in_ty, D, table, idx, impl="ref", out_ty=out_ty, scale_bias_last=sbl, data_size=rows)
    assert ok_a == ok_r == (in_ty == ST_INT4)


def test_combinations_the_reference_does_not_have():
    # 4-bit rows only copy to a 4-bit output: the reference asserts on anything else and, with asserts
    # compiled out, returns false (src/RefImplementations.cc:1466-1474). The oracle states the release behaviour.
    rng = np.random.default_rng(5)
    table, _ = make_table(rng, ST_INT4, 16, 4, True)
    idx = np.zeros(2, dtype=np.int64)
    for out_ty in (ST_FP32, ST_FP16):
        assert not oracle.spmdm_nobag(ST_INT4, 16, table, idx, out_ty=out_ty, data_size=4)[0]


@pytest.mark.parametrize("in_ty,sbl", [(ST_INT8, True), (ST_INT8, False), (ST_FP16, True), (ST_FP32, True), (ST_BF16, True)])
@pytest.mark.parametrize("out_ty", [ST_FP32, ST_FP16, ST_BF16])
def test_equals_pooling_bags_of_one(in_ty, sbl, out_ty):
    rng = np.random.default_rng(11)
    D, rows, n = 40, 30, 25
    table, _ = make_table(rng, in_ty, D, rows, sbl)
    idx = rng.integers(0, rows, size=n).astype(np.int64)
    w = rng.normal(size=n).astype(np.float32)
    ok, a = oracle.spmdm_nobag(in_ty, D, table, idx, weights=w, out_ty=out_ty, scale_bias_last=sbl, data_size=rows)
    ok2, b = oracle.spmdm(in_ty, D, table, idx, np.arange(n + 1, dtype=np.int64), weights=w, out_ty=out_ty,
                          scale_bias_last=sbl, data_size=rows)
    assert ok and ok2 and (bits(a) == bits(b)).all()


def test_single_row_closed_form():
    # one 8-bit row, weight w: out[j] = fl(fl(w*s) * q[j] + fl(w*b)) with one rounding (fma)
    D = 16
    s, b, w = np.float32(0.0371), np.float32(-0.62), np.float32(1.7)
    q = np.arange(D, dtype=np.uint8) * 13
    row = np.concatenate([q, s.reshape(1).view(np.uint8), b.reshape(1).view(np.uint8)])
    ok, out = oracle.spmdm_nobag(ST_INT8, D, row, np.zeros(1, dtype=np.int64), weights=np.array([w]), data_size=1)
    ws, wb = np.float32(w * s), np.float32(w * b)
    want = (np.float64(ws) * q.astype(np.float64) + np.float64(wb)).astype(np.float32)  # exact in float64, then one rounding
    assert ok and (out.view(np.uint32) == want.view(np.uint32)).all()
    # byte copies: the row as stored, truncated to the narrower of the two strides
    ok, raw = oracle.spmdm_nobag(ST_INT8, D, row, np.zeros(1, dtype=np.int64), out_ty=ST_INT8, output_stride=D + 8, data_size=1)
    assert ok and (raw == row).all()
    ok, raw = oracle.spmdm_nobag(ST_INT8, D, row, np.zeros(1, dtype=np.int64), out_ty=ST_INT8, output_stride=D + 11, data_size=1)
    assert ok and (raw[:D + 8] == row).all() and (raw[D + 8:] == 0).all()
