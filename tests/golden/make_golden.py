"""Writes tests/golden/spmdm_cases.npz: inputs and the outputs of the
reference's own scalar implementation (compiled from its sources into
oracle/_ref by `make -C oracle ref`) for a fixed list of small cases.

Run in the build container, where the reference tree is mounted:
    python tests/golden/make_golden.py
The vectors are data (inputs + expected output bits); the reference itself does
not travel with the repository."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import helpers as H  # noqa: E402
import oracle  # noqa: E402

FP32, FP16, INT8, INT4, INT2, BF16 = 0, 1, 2, 3, 4, 5

# (ty, D, rows, bags, avg_len, scale_bias_last, out_ty, weighted(0/1/2 positional), normalize, idx64, off64, use_offsets, remap, corner)
CASES = []
for ty in (INT8, INT4, INT2, FP16, FP32, BF16):
    for D in (4, 8, 40, 128):
        for k, (sbl, out_ty, weighted, normalize, idx64, off64, use_off) in enumerate([
                (True, FP32, 0, False, True, False, True), (True, FP16, 1, True, False, False, True),
                (False, BF16, 1, False, True, True, True), (False, FP16, 2, True, False, True, False)]):
            CASES.append((ty, D, 60, 7, 6, sbl, out_ty, weighted, normalize, idx64, off64, use_off, False, 0))
for ty in (INT8, INT4, INT2, FP16, FP32):
    CASES.append((ty, 48, 80, 9, 5, True, FP32, 1, True, True, False, True, True, 0))  # row-wise sparse
for corner in (1, 2, 3):  # empty indices, out-of-range index, lengths-sum mismatch
    CASES.append((INT4, 32, 50, 6, 4, True, FP32, 0, False, True, False, True, False, corner))


def build(case, seed):
    ty, D, rows, nb, avg, sbl, out_ty, weighted, normalize, idx64, off64, use_off, sparse, corner = case
    rng = np.random.default_rng(seed)
    logical = rows
    remap = None
    if sparse:
        keep = rng.random(logical) >= 0.7
        remap = np.full(logical, -1, np.int32)
        remap[keep] = np.arange(int(keep.sum()), dtype=np.int32)
        rows = max(1, int(keep.sum()))
    table, stride = H.make_table(rng, ty, rows, D, sbl)
    idx, off, lens = H.make_bags(rng, logical, nb, avg, np.int64 if idx64 else np.int32,
                                 np.int64 if off64 else np.int32, empty_frac=0.2)
    if not sbl and len(idx):
        idx[rng.random(len(idx)) < 0.2] = -1
    index_size = len(idx)
    if corner == 1:
        idx = idx[:0]; index_size = 0
    elif corner == 2:
        idx[len(idx) // 2] = logical
    elif corner == 3:
        index_size = len(idx) - 1
    w = None
    if weighted == 1:
        w = rng.normal(size=max(1, len(idx))).astype(np.float32)
    elif weighted == 2:
        w = rng.normal(size=max(1, int(lens.max()))).astype(np.float32)
    return dict(table=table, idx=idx, off=off, lens=lens, w=w, remap=remap, logical=logical, index_size=index_size)


def main():
    assert oracle.have_ref(), "build oracle/_ref first: make -C oracle ref"
    out = {"cases": np.array(CASES, dtype=np.int64)}
    for i, case in enumerate(CASES):
        ty, D, rows, nb, avg, sbl, out_ty, weighted, normalize, idx64, off64, use_off, sparse, corner = case
        b = build(case, 9000 + i)
        ok, res = oracle.spmdm(ty, D, b["table"], b["idx"], b["off"] if use_off else b["lens"], weights=b["w"],
                               normalize=bool(normalize), out_ty=out_ty, positional=weighted == 2,
                               use_offsets=bool(use_off), scale_bias_last=bool(sbl), remap=b["remap"],
                               data_size=b["logical"], output_size=nb, index_size=b["index_size"], impl="ref")
        out[f"ok_{i}"] = np.array(int(ok))
        out[f"out_{i}"] = res
        for k in ("table", "idx", "off", "lens"):
            out[f"{k}_{i}"] = b[k]
        if b["w"] is not None:
            out[f"w_{i}"] = b["w"]
        if b["remap"] is not None:
            out[f"remap_{i}"] = b["remap"]
        out[f"index_size_{i}"] = np.array(b["index_size"])
        out[f"logical_{i}"] = np.array(b["logical"])
    # conversions: every half pattern widened, a spread of floats narrowed both ways
    h = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(1)
    f = np.concatenate([rng.integers(0, 2**32, size=4096, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e30, 6.1e-5, 5.96e-8, 2.98e-8, 2.9802326e-8,
                                  1e-10, np.inf, -np.inf, 1.0009766, 1.00048828125, 1.0014648], np.float32)])
    out["half_in"] = h
    out["half_to_float"] = oracle.half2float(h, "ref")
    out["float_in"] = f
    out["float_to_half"] = oracle.float2half_rn(f, "ref")
    out["float_to_bf16"] = oracle.float2bf16(f, "ref")
    path = os.path.join(HERE, "spmdm_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(CASES), "cases")


if __name__ == "__main__":
    main()
