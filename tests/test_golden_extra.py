"""The oracle against committed vectors produced by the reference's own scalar code
(tests/golden/extra_cases.npz, written by tests/golden/make_golden_extra.py): no_bag
rows, pooled 8-bit-float rows, the hfp8 encoder and decoder. Needs neither the
reference tree nor a GPU."""
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
FP32 = 0


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(HERE, "golden", "extra_cases.npz"))


def bits(a):
    return a.view({4: np.uint32, 2: np.uint16, 1: np.uint8}[a.dtype.itemsize])


def test_no_bag_cases(vec):
    for i, (in_ty, out_ty, sbl, D, rows, n, weighted, ostride) in enumerate(vec["nobag"].tolist()):
        w = vec[f"nobag_w_{i}"] if weighted else None
        ok, got = oracle.spmdm_nobag(in_ty, D, vec[f"nobag_table_{i}"], vec[f"nobag_idx_{i}"], weights=w, out_ty=out_ty,
                                     output_stride=ostride, scale_bias_last=bool(sbl), data_size=rows)
        want = vec[f"nobag_out_{i}"]
        assert ok and got.dtype == want.dtype and (bits(got) == bits(want)).all(), i


def test_pooled_fp8_cases(vec):
    for i, (D, rows, nb, avg, weighted, normalize, use_off, out_ty, ebits, bias, pad) in enumerate(vec["fp8"].tolist()):
        w = vec[f"fp8_w_{i}"] if weighted else None
        ool = vec[f"fp8_off_{i}"] if use_off else vec[f"fp8_lens_{i}"]
        ok, got = oracle.spmdm_fp8(D, vec[f"fp8_table_{i}"], vec[f"fp8_idx_{i}"], ool, weights=w, normalize=bool(normalize),
                                   out_ty=out_ty, positional=weighted == 2, use_offsets=bool(use_off), input_stride=D + pad,
                                   exponent_bits=ebits, exponent_bias=bias, data_size=rows, output_size=nb)
        want = vec[f"fp8_out_{i}"]
        assert ok and (bits(got) == bits(want)).all(), i


def test_hfp8_codes(vec):
    for i, (ebits, bias) in enumerate(vec["hfp8_formats"].tolist()):
        assert (oracle.float_to_hfp8(vec[f"hfp8_in_{i}"], ebits, bias) == vec[f"hfp8_codes_{i}"]).all()
        dec = np.array([oracle.float8_to_float(b, ebits, bias) for b in range(256)], dtype=np.float32)
        assert (dec.view(np.uint32) == vec[f"hfp8_decoded_{i}"].view(np.uint32)).all()
