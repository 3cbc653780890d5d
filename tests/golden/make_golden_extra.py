"""Writes tests/golden/extra_cases.npz: inputs and the outputs of the reference's
own scalar code (compiled from its sources into oracle/_ref by `make -C oracle ref`)
for the forms added beside the pooled lookup: no_bag rows, pooled 8-bit-float
rows, and the fp32 -> hfp8 encoder.

Run in the build container, where the reference tree is mounted:
    python tests/golden/make_golden_extra.py
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
STORAGE = {FP32: np.float32, FP16: np.uint16, BF16: np.uint16}

# (in_ty, out_ty, scale_bias_last, D, rows, n, weighted, output_stride)
NOBAG = [(INT8, FP32, 1, 40, 30, 25, 1, -1), (INT8, FP16, 0, 128, 50, 64, 1, 133), (INT8, BF16, 1, 7, 9, 12, 0, -1),
         (INT8, INT8, 1, 32, 20, 15, 0, 40), (INT8, INT8, 0, 32, 20, 15, 0, 30), (INT4, INT4, 1, 64, 25, 18, 0, -1),
         (INT4, INT4, 0, 10, 8, 9, 0, -1), (FP32, FP32, 1, 33, 12, 20, 1, -1), (FP32, BF16, 1, 16, 12, 20, 0, 19),
         (FP16, FP32, 1, 48, 14, 22, 1, -1), (FP16, FP16, 1, 8, 5, 6, 0, -1), (BF16, BF16, 1, 24, 10, 11, 1, -1)]
# (D, rows, bags, avg_len, weighted(0/1/2 positional), normalize, use_offsets, out_ty, ebits, bias, pad)
FP8 = [(8, 50, 6, 3, 0, 0, 1, FP32, 4, 7, 0), (33, 40, 9, 5, 1, 1, 1, FP16, 4, 7, 2), (128, 100, 12, 6, 1, 0, 0, BF16, 5, 15, 0),
       (64, 30, 5, 4, 2, 1, 1, FP32, 4, 15, 0), (1, 5, 3, 2, 0, 1, 1, FP32, 3, 3, 0)]
HFP8_FORMATS = [(4, 7), (5, 15), (3, 3), (2, 1), (4, 4)]


def nobag_inputs(case, seed):
    in_ty, out_ty, sbl, D, rows, n, weighted, ostride = case
    rng = np.random.default_rng(seed)
    table_b, stride_b = H.make_table(rng, in_ty, rows, D, bool(sbl))
    table = table_b.view(STORAGE.get(in_ty, np.uint8))
    idx = rng.integers(0, rows, size=n).astype(np.int64)
    w = rng.normal(size=n).astype(np.float32) if weighted else None
    return table, idx, w


def fp8_inputs(case, seed):
    D, rows, nb, avg, weighted, normalize, use_off, out_ty, ebits, bias, pad = case
    rng = np.random.default_rng(seed)
    table = rng.integers(0, 256, size=rows * (D + pad), dtype=np.uint8)
    idx, off, lens = H.make_bags(rng, rows, nb, avg, np.int64, np.int64, empty_frac=0.15)
    w = None
    if weighted == 1:
        w = rng.normal(size=max(1, len(idx))).astype(np.float32)
    elif weighted == 2:
        w = rng.normal(size=max(1, int(lens.max()))).astype(np.float32)
    return table, idx, off, lens.astype(np.int64), w


def hfp8_inputs(ebits, bias):
    rng = np.random.default_rng(ebits * 10 + bias)
    mags = np.array([oracle.float8_to_float(b, ebits, bias) for b in range(128)], dtype=np.float32)
    mid = ((mags[:-1].astype(np.float64) + mags[1:]) / 2).astype(np.float32)
    x = np.concatenate([mags, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
                        rng.normal(size=500).astype(np.float32) * np.float32(mags[-1] / 4),
                        (rng.uniform(-1, 1, size=500) * 2.0 ** rng.integers(-30, 20, size=500)).astype(np.float32),
                        np.array([0.0, 1e-30, 1e-45, 3e38, np.inf], dtype=np.float32)])
    return np.concatenate([x, -x])


def main():
    assert oracle.have_ref(), "build oracle/_ref first: make -C oracle ref"
    out = {"nobag": np.array(NOBAG, dtype=np.int64), "fp8": np.array(FP8, dtype=np.int64),
           "hfp8_formats": np.array(HFP8_FORMATS, dtype=np.int64)}
    for i, case in enumerate(NOBAG):
        in_ty, out_ty, sbl, D, rows, n, weighted, ostride = case
        table, idx, w = nobag_inputs(case, 7000 + i)
        ok, res = oracle.spmdm_nobag(in_ty, D, table, idx, weights=w, out_ty=out_ty, output_stride=ostride,
                                     scale_bias_last=bool(sbl), data_size=rows, impl="ref")
        assert ok
        out[f"nobag_table_{i}"], out[f"nobag_idx_{i}"], out[f"nobag_out_{i}"] = table, idx, res
        if w is not None:
            out[f"nobag_w_{i}"] = w
    for i, case in enumerate(FP8):
        D, rows, nb, avg, weighted, normalize, use_off, out_ty, ebits, bias, pad = case
        table, idx, off, lens, w = fp8_inputs(case, 7100 + i)
        ok, res = oracle.spmdm_fp8(D, table, idx, off if use_off else lens, weights=w, normalize=bool(normalize), out_ty=out_ty,
                                   positional=weighted == 2, use_offsets=bool(use_off), input_stride=D + pad,
                                   exponent_bits=ebits, exponent_bias=bias, data_size=rows, output_size=nb, impl="ref")
        assert ok
        out[f"fp8_table_{i}"], out[f"fp8_idx_{i}"], out[f"fp8_off_{i}"], out[f"fp8_lens_{i}"] = table, idx, off, lens
        out[f"fp8_out_{i}"] = res
        if w is not None:
            out[f"fp8_w_{i}"] = w
    for i, (ebits, bias) in enumerate(HFP8_FORMATS):
        x = hfp8_inputs(ebits, bias)
        out[f"hfp8_in_{i}"] = x
        out[f"hfp8_codes_{i}"] = oracle.float_to_hfp8(x, ebits, bias, impl="ref")
        out[f"hfp8_decoded_{i}"] = np.array([oracle.float8_to_float(b, ebits, bias, impl="ref") for b in range(256)], dtype=np.float32)
    path = os.path.join(HERE, "extra_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
