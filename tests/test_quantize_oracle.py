"""Pins oracle/quantize_oracle.c without the GPU: bit for bit against the
reference's own scalar row-wise quantizers compiled from its sources (the *Ref
routines its test/QuantUtilsTest.cc holds the vector code to), and against
what the arithmetic fixes. Caller-supplied extremes (rowwise_min_max), which only the
reference's AVX2 routines take, are pinned against those routines compiled from its
sources and against the known answers of its test/QuantUtilsTest.cc:547-611."""
import numpy as np
import pytest

import oracle
from oracle import LAYOUT_TBE, LAYOUT_TRAILER, ST_BF16, ST_FP16, ST_FP32

needs_ref = pytest.mark.skipif(not oracle.have_ref_quant(), reason="oracle/_ref/libfbgemm_ref_quant.so not built")


def rows_of(rng, kind, rows, cols, dtype):
    if kind == "normal":
        x = rng.normal(0, 1, size=(rows, cols))
    elif kind == "uniform":
        x = rng.uniform(-5, 5, size=(rows, cols))
    elif kind == "constant":
        x = np.repeat(rng.normal(0, 3, size=(rows, 1)), cols, axis=1)
    elif kind == "tiny":
        x = rng.normal(0, 1e-7, size=(rows, cols))
    elif kind == "large":
        x = rng.normal(0, 3e4, size=(rows, cols)) if dtype == np.float16 else rng.normal(0, 1e30, size=(rows, cols))
    elif kind == "zeros":
        x = np.zeros((rows, cols))
        x[::2, ::3] = -0.0
    else:
        raise ValueError(kind)
    return x.astype(dtype)


KINDS = ["normal", "uniform", "constant", "tiny", "large", "zeros"]


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
def test_quantize_matches_reference(dtype, bit_rate, sb_float):
    rng = np.random.default_rng(21)
    for kind in KINDS:
        for cols in (1, 2, 3, 7, 8, 31, 64, 100, 128, 257):
            x = rows_of(rng, kind, 9, cols, dtype)
            want = oracle.quantize_rowwise(x, bit_rate, sb_float, impl="ref")
            got = oracle.quantize_rowwise(x, bit_rate, sb_float, impl="oracle")
            assert (got == want).all(), (kind, cols)


@needs_ref
@pytest.mark.parametrize("out_ty", [ST_FP32, ST_FP16, ST_BF16])
@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
def test_dequantize_matches_reference(out_ty, bit_rate, sb_float):
    rng = np.random.default_rng(22)
    for cols in (1, 4, 8, 30, 64, 100, 256):
        stride = oracle.quantized_row_bytes(cols, bit_rate, sb_float, LAYOUT_TRAILER)
        q = rng.integers(0, 256, size=(11, stride), dtype=np.uint8)
        # sane scale / bias patterns (random bytes would be NaNs now and then)
        if sb_float:
            q[:, -8:] = np.stack([rng.uniform(1e-3, 1, 11), rng.uniform(-3, 3, 11)], 1).astype(np.float32).view(np.uint8)
        else:
            q[:, -4:] = np.stack([rng.uniform(1e-3, 1, 11), rng.uniform(-3, 3, 11)], 1).astype(np.float16).view(np.uint8)
        want = oracle.dequantize_rowwise(q, cols, bit_rate, sb_float, out_ty=out_ty, impl="ref")
        got = oracle.dequantize_rowwise(q, cols, bit_rate, sb_float, out_ty=out_ty, impl="oracle")
        assert (got.view(np.uint32 if out_ty == ST_FP32 else np.uint16) ==
                want.view(np.uint32 if out_ty == ST_FP32 else np.uint16)).all()


@pytest.mark.parametrize("bit_rate", [2, 4, 8])
def test_closed_forms(bit_rate):
    rng = np.random.default_rng(23)
    cols = 64
    epb = 8 // bit_rate
    maxq = (1 << bit_rate) - 1
    # constant row: all zeros, scale 1, bias = the constant rounded to fp16
    x = np.full((1, cols), 2.5, np.float32)
    q = oracle.quantize_rowwise(x, bit_rate)
    assert (q[0, :cols // epb] == 0).all()
    assert q[0, cols // epb:].view(np.float16).tolist() == [1.0, 2.5]
    # a row on the grid min + k * scale (all exactly representable) round-trips exactly
    scale, mn = 0.25, -3.0
    ks = rng.integers(0, maxq + 1, size=cols)
    ks[0], ks[1] = 0, maxq
    x = (mn + ks * scale).astype(np.float32)[None, :]
    q = oracle.quantize_rowwise(x, bit_rate)
    assert q[0, cols // epb:].view(np.float16).tolist() == [scale, mn]
    unpacked = [(int(q[0, j // epb]) >> ((j % epb) * bit_rate)) & maxq for j in range(cols)]
    assert unpacked == ks.tolist()
    back = oracle.dequantize_rowwise(q, cols, bit_rate)
    assert (back == x).all()
    # error bound on ordinary data: half a step, plus the rounding of the bias to fp16
    x = rng.normal(0, 1, size=(20, cols)).astype(np.float32)
    q = oracle.quantize_rowwise(x, bit_rate)
    back = oracle.dequantize_rowwise(q, cols, bit_rate)
    sb = q[:, cols // epb:].view(np.float16).astype(np.float32)
    bound = sb[:, :1] * 0.5 + np.abs(sb[:, 1:]) * 2.0 ** -10 + 1e-6
    inside = (x >= sb[:, 1:]) & (x <= sb[:, 1:] + sb[:, :1] * maxq)
    assert (np.abs(back - x)[inside] <= np.broadcast_to(bound, x.shape)[inside]).all()


def test_first_extreme_decides_the_sign_of_zero():
    # min_element / max_element return the FIRST of equal elements: +0 before -0 gives
    # a +0 bias, -0 before +0 a -0 bias (fp32 pair of the 8-bit format shows it)
    a = np.array([[0.0, -0.0, 0.0, -0.0]], np.float32)
    b = np.array([[-0.0, 0.0, -0.0, 0.0]], np.float32)
    qa = oracle.quantize_rowwise(a, 8, True)
    qb = oracle.quantize_rowwise(b, 8, True)
    assert qa[0, 4:].view(np.uint32).tolist() == [0x00000000, 0x00000000]
    assert qb[0, 4:].view(np.uint32).tolist()[1] == 0x80000000
    if oracle.have_ref_quant():
        assert (oracle.quantize_rowwise(a, 8, True, impl="ref") == qa).all()
        assert (oracle.quantize_rowwise(b, 8, True, impl="ref") == qb).all()


@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, True)])
def test_tbe_layout_is_the_trailer_layout_rearranged(bit_rate, sb_float):
    """quantize_embs (fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:47-70): elements
    unchanged, the (scale, bias) pair moved to the front as two fp16 (an fp32 pair
    rounded to nearest even, as torch's .to(float16) rounds)."""
    rng = np.random.default_rng(24)
    cols = 40
    x = rng.normal(0, 2, size=(13, cols)).astype(np.float32)
    tr = oracle.quantize_rowwise(x, bit_rate, sb_float, LAYOUT_TRAILER)
    stride = 48
    tbe = oracle.quantize_rowwise(x, bit_rate, sb_float, LAYOUT_TBE, out_stride=stride, fill=0xAB)
    epb = 8 // bit_rate
    nb = cols // epb
    assert (tbe[:, 4:4 + nb] == tr[:, :nb]).all()
    if sb_float:
        want_sb = tr[:, nb:].copy().view(np.float32).astype(np.float16).view(np.uint8)
    else:
        want_sb = tr[:, nb:]
    assert (tbe[:, :4] == want_sb).all()
    assert (tbe[:, 4 + nb:] == 0xAB).all()  # padding untouched
    back = oracle.dequantize_rowwise(tbe, cols, bit_rate, False, LAYOUT_TBE)
    want = oracle.dequantize_rowwise(np.concatenate([tr[:, :nb], want_sb], 1), cols, bit_rate, False, LAYOUT_TRAILER)
    assert (back == want).all()


# ---- caller-supplied extremes (rowwise_min_max) -------------------------------------------

# test/QuantUtilsTest.cc:551-598: two rows of four, their true extremes, and the bytes the
# reference's authors worked out by hand for every format
FIXED_INPUT = np.array([[1, 1, 1, 1], [-64, -2.75, 61.625, 191]], np.float32)
FIXED_MIN_MAX = np.array([[1, 1], [-64, 191]], np.float32)
FIXED_EXPECTED = {
    (8, False): [[0, 0, 0, 0, 0x00, 0x3c, 0x00, 0x3c], [0, 61, 126, 255, 0x00, 0x3c, 0x00, 0xd4]],
    (4, False): [[0x00, 0x00, 0x00, 0x3c, 0x00, 0x3c], [0x40, 0xf7, 0x40, 0x4c, 0x00, 0xd4]],
    (2, False): [[0b00000000, 0x00, 0x3c, 0x00, 0x3c], [0b11010100, 0x50, 0x55, 0x00, 0xd4]],
    (8, True): [[0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0x80, 0x3f], [0, 61, 126, 255, 0, 0, 0x80, 0x3f, 0, 0, 0x80, 0xc2]],
}


@pytest.mark.parametrize("bit_rate,sb_float", list(FIXED_EXPECTED))
def test_min_max_known_answers(bit_rate, sb_float):
    want = np.array(FIXED_EXPECTED[(bit_rate, sb_float)], np.uint8)
    for dtype in (np.float32, np.float16):
        x, mm = FIXED_INPUT.astype(dtype), FIXED_MIN_MAX.astype(dtype)
        assert (oracle.quantize_rowwise(x, bit_rate, sb_float, min_max=mm) == want).all()
        assert (oracle.quantize_rowwise(x, bit_rate, sb_float) == want).all()
    # other extremes give other rows (QuantUtilsTest.cc:880-909)
    wrong = np.array([[10, 15], [-14, 1]], np.float32)
    assert (oracle.quantize_rowwise(FIXED_INPUT, bit_rate, sb_float, min_max=wrong) != want).any()


def bracketing(rng, x, mode):
    lo, hi = x.astype(np.float32).min(1), x.astype(np.float32).max(1)
    if mode == "true":
        pass
    elif mode == "wider":
        lo, hi = lo - rng.uniform(0, 2, lo.shape), hi + rng.uniform(0, 2, hi.shape)
    elif mode == "narrower":  # elements fall outside: clamping / wrapping rules show
        mid, half = (lo + hi) / 2, (hi - lo) / 2
        lo, hi = mid - half * rng.uniform(0.1, 0.9, lo.shape), mid + half * rng.uniform(0.1, 0.9, hi.shape)
    elif mode == "far":  # (x - min) * inverse_scale beyond the 32-bit integers
        lo, hi = lo + 1e-3, lo + 1e-3 + 1e-12
    elif mode == "steep":  # a tiny step under values spread widely: beyond 32 bits, within 64
        lo, hi = np.zeros_like(lo), np.full_like(hi, 1e-6)
    return np.stack([lo, hi], 1).astype(x.dtype)


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
def test_min_max_matches_reference_avx2(dtype, bit_rate, sb_float):
    rng = np.random.default_rng(24)
    for kind in ("normal", "uniform", "constant", "large"):
        for cols in (4, 8, 12, 31, 32, 36, 40, 63, 64, 72, 100, 128, 260):
            if cols % (8 // bit_rate):
                continue
            x = rows_of(rng, kind, 9, cols, dtype)
            for mode in ("true", "wider", "narrower", "far", "steep"):
                if mode == "steep":
                    x = (x * (1e4 if kind != "large" else 1)).astype(dtype)
                if mode in ("far", "steep") and dtype == np.float16:
                    continue
                mm = bracketing(rng, x, mode)
                want = oracle.quantize_rowwise(x, bit_rate, sb_float, impl="ref_avx2", min_max=mm)
                got = oracle.quantize_rowwise(x, bit_rate, sb_float, min_max=mm)
                assert (got == want).all(), (kind, cols, mode)


@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
def test_true_extremes_change_nothing(bit_rate, sb_float):
    rng = np.random.default_rng(25)
    for dtype in (np.float32, np.float16):
        x = rows_of(rng, "normal", 13, 96, dtype)
        mm = np.stack([x.min(1), x.max(1)], 1)
        assert (oracle.quantize_rowwise(x, bit_rate, sb_float, min_max=mm) ==
                oracle.quantize_rowwise(x, bit_rate, sb_float)).all()
