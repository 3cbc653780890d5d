"""Pins the oracle without the reference tree: committed vectors produced by the
reference's own scalar code (tests/golden/make_golden.py), closed forms, and
brute force in float64."""
import os

import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spmdm_cases.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def test_golden_spmdm_cases(oracle, gold):
    cases = gold["cases"]
    assert len(cases) >= 100
    for i, case in enumerate(cases):
        ty, D, rows, nb, avg, sbl, out_ty, weighted, normalize, idx64, off64, use_off, sparse, corner = [int(x) for x in case]
        w = gold[f"w_{i}"] if f"w_{i}" in gold else None
        remap = gold[f"remap_{i}"] if f"remap_{i}" in gold else None
        ok, out = oracle.spmdm(ty, D, gold[f"table_{i}"], gold[f"idx_{i}"], gold[f"off_{i}"] if use_off else gold[f"lens_{i}"],
                               weights=w, normalize=bool(normalize), out_ty=out_ty, positional=weighted == 2,
                               use_offsets=bool(use_off), scale_bias_last=bool(sbl), remap=remap,
                               data_size=int(gold[f"logical_{i}"]), output_size=nb, index_size=int(gold[f"index_size_{i}"]))
        assert int(ok) == int(gold[f"ok_{i}"]), f"case {i}: return value"
        if ok:
            H.assert_same_bits(out, gold[f"out_{i}"], f"golden case {i} {case}")


def test_golden_conversions(oracle, gold):
    H.assert_same_bits(oracle.half2float(gold["half_in"]), gold["half_to_float"], "half -> float")
    H.assert_same_bits(oracle.float2half_rn(gold["float_in"]), gold["float_to_half"], "float -> half")
    H.assert_same_bits(oracle.float2bf16(gold["float_in"]), gold["float_to_bf16"], "float -> bf16")


def test_conversions_against_numpy(oracle):
    h = np.arange(65536, dtype=np.uint16)
    f = oracle.half2float(h)
    ref = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(ref) | np.isinf(ref)
    assert (f.view(np.uint32)[~np.isnan(ref)] == ref.view(np.uint32)[~np.isnan(ref)]).all()
    assert np.isnan(f[np.isnan(ref)]).all() and finite.any()
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2**32, size=500_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)  # IEEE round-to-nearest-even, overflow to inf
    assert (oracle.float2half_rn(x) == want).all()
    # bf16 rule of the reference: add 0x8000, truncate (ties go up, not to even)
    u = x.view(np.uint32)
    assert (oracle.float2bf16(x) == ((u.astype(np.uint64) + 0x8000) >> 16).astype(np.uint16)).all()
    assert oracle.float2bf16(np.array([1.00390625], np.float32))[0] == 0x3F81  # a tie: RNE would give 0x3F80


@pytest.mark.parametrize("ty", [INT8, INT4, INT2])
def test_closed_forms(oracle, ty):
    """scale=1, bias=0: sums of small integers are exact; all-ones rows count
    the bag; a single weighted row is one fma; mean divides by the length."""
    rng = np.random.default_rng(ty)
    rows, D, nb = 40, 24, 30
    table, stride = H.make_table(rng, ty, rows, D, True, scale_range=(1, 1), bias_range=(0, 0))
    idx, off, lens = H.make_bags(rng, rows, nb, 8, empty_frac=0.2)
    bits = H.BITS[ty]
    q = table.reshape(rows, stride)[:, :H.packed_bytes(ty, D)]
    vals = np.stack([(q >> (bits * k)) & ((1 << bits) - 1) for k in range(8 // bits)], axis=2).reshape(rows, -1)[:, :D]
    ok, out = oracle.spmdm(ty, D, table, idx, off, data_size=rows)
    want = np.stack([vals[idx[off[b]:off[b + 1]]].sum(axis=0) for b in range(nb)]).astype(np.float32)
    assert ok and (out.reshape(nb, D) == want).all()
    ones, _ = H.make_table(rng, ty, rows, D, True, ones=True)
    ok, out = oracle.spmdm(ty, D, ones, idx, off, data_size=rows, normalize=True)
    assert ok and (out.reshape(nb, D) == (lens > 0).astype(np.float32)[:, None]).all()
    # one row, weight w: fma(w*s, q, w*b) with every product rounded to fp32
    table, stride = H.make_table(rng, ty, rows, D, True)
    t2 = table.reshape(rows, stride)
    pb = H.packed_bytes(ty, D)
    if ty == INT8:
        s, b = t2[5, pb:pb + 8].copy().view(np.float32)
    else:
        s, b = t2[5, pb:pb + 4].copy().view(np.float16).astype(np.float32)
    w = np.float32(0.37)
    ok, out = oracle.spmdm(ty, D, table, np.array([5], np.int64), np.array([0, 1], np.int32),
                           weights=np.array([w], np.float32), data_size=rows)
    qrow = np.stack([(t2[5, :pb] >> (bits * k)) & ((1 << bits) - 1) for k in range(8 // bits)], axis=1).reshape(-1)[:D]
    ws, wb = np.float32(w * s), np.float32(w * b)
    want = (np.float64(ws) * qrow.astype(np.float64) + np.float64(wb)).astype(np.float32)  # single rounding
    assert ok and (out == want).all()


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32])
def test_float64_brute_force(oracle, ty):
    """The fp32 result stays within 1e-5 relative of an exact (float64) evaluation on
    well-conditioned inputs (positive terms): a dropped term, a wrong nibble order
    or a transposed scale/bias is orders of magnitude outside."""
    rng = np.random.default_rng(40 + ty)
    for D in (2 if ty != INT2 else 4, 7 if ty != INT2 else 8, 8, 40, 56, 86 if ty != INT2 else 88, 164):
        rows, nb = 30, 10
        table, stride = H.make_table(rng, ty, rows, D, True, bias_range=(0.0, 1.0))
        idx, off, _ = H.make_bags(rng, rows, nb, 6)
        w = rng.uniform(0.1, 1.0, len(idx)).astype(np.float32)
        ok, out = oracle.spmdm(ty, D, table, idx, off, weights=w, data_size=rows)
        t2 = table.reshape(rows, stride)
        pb = H.packed_bytes(ty, D)
        if ty in (INT8, INT4, INT2):
            bits = H.BITS[ty]
            q = np.stack([(t2[:, :pb] >> (bits * k)) & ((1 << bits) - 1) for k in range(8 // bits)], axis=2).reshape(rows, -1)[:, :D]
            sb = t2[:, pb:pb + 8].copy().view(np.float32) if ty == INT8 else t2[:, pb:pb + 4].copy().view(np.float16).astype(np.float32)
            deq = q.astype(np.float64) * sb[:, :1].astype(np.float64) + sb[:, 1:2].astype(np.float64)
        elif ty == FP16:
            deq = np.abs(t2[:, :pb].copy().view(np.float16).astype(np.float64))
            table = table.copy(); t2 = table.reshape(rows, stride)
            t2[:, :pb] = np.abs(t2[:, :pb].copy().view(np.float16)).view(np.uint8)
            ok, out = oracle.spmdm(ty, D, table, idx, off, weights=w, data_size=rows)
        else:
            deq = np.abs(t2[:, :pb].copy().view(np.float32).astype(np.float64))
            table = table.copy(); t2 = table.reshape(rows, stride)
            t2[:, :pb] = np.abs(t2[:, :pb].copy().view(np.float32)).view(np.uint8)
            ok, out = oracle.spmdm(ty, D, table, idx, off, weights=w, data_size=rows)
        want = np.stack([(deq[idx[off[b]:off[b + 1]]] * w[off[b]:off[b + 1], None].astype(np.float64)).sum(axis=0) for b in range(nb)])
        assert ok
        rel = np.abs(out.reshape(nb, D) - want) / np.maximum(np.abs(want), 1e-30)
        assert rel.max() < 1e-5, (ty, D, rel.max())


def test_tbe_exact_count_fixture(oracle):
    """fbgemm_gpu/test/tbe/inference/nbit_forward_test.py:577-659, on the oracle."""
    from test_tbe_gpu import build_weights
    E, Ds = 100, [16, 24, 40]
    Ls = [[0, 2, 5, 0, 3, 4], [1, 0, 4, 2, 0, 6], [3, 3, 0, 1, 5, 0]]
    fully_pruned = [4, 2, 3]
    T, B = 3, 6
    rng = np.random.default_rng(0)
    for ty in (FP16, INT8, INT4, INT2):
        specs = [(E, d, ty) for d in Ds]
        weights, wo, _ = build_weights(rng, specs, 16, ones=True)
        idx, off, running = [], [0], 0
        expected = np.zeros((B, sum(Ds)), np.float32)
        dpre = np.cumsum([0] + Ds)
        for t in range(T):
            for b in range(B):
                kept = 0
                for _ in range(Ls[t][b]):
                    prune = b == fully_pruned[t] or running % 3 == 0
                    idx.append(-1 if prune else running % E)
                    kept += 0 if prune else 1
                    running += 1
                off.append(len(idx))
                expected[b, dpre[t]:dpre[t + 1]] = kept
        rc, out = oracle.tbe_forward(weights, wo, np.full(T, ty, np.uint8), dpre.astype(np.int32), sum(Ds),
                                     np.array(idx, np.int32), np.array(off, np.int32), 0, None, FP32, 16)
        assert rc == 0 and (out == expected).all()
