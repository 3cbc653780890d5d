"""The bound of the tolerance-grade mode (fbgemm_amd/tolerance.py) on hand-made cases: the
element-wise reading applies to every element that is not a cancellation (fp32: an eighth of the
block's magnitude and more; 16-bit: 2^-10 of it and more), the fp32 rounding floor only below
that, and what needed it is counted. No GPU."""
import numpy as np

from fbgemm_amd import tolerance as T


def test_fp32_elementwise_bound_and_block_clause():
    want = np.array([[1.0, 2.0, 1e-3, 0.0, 0.25]], np.float32)
    got = want.copy()
    got[0, 0] *= 1 + 5e-6      # within 1e-5 of itself
    got[0, 2] += 2e-6          # 2e-3 of itself, but 1e-6 of the block's 2.0: a cancellation, under the floor of 1.25e-6
    r = T.grade(got, want, 0, np)
    assert r["ok"] and r["cancellations"] == 2 and r["needed_block_clause"] == 1
    assert abs(r["worst"] - 5e-6) < 1e-7 and abs(r["worst_block"] - 1e-6) < 1e-8
    got[0, 1] *= 1 + 2e-5      # a full-sized element off by 2e-5: the floor must not rescue it
    assert not T.grade(got, want, 0, np)["ok"]
    got = want.copy()
    got[0, 2] += 4e-6          # a cancellation beyond the floor (2e-6 of the block)
    assert not T.grade(got, want, 0, np)["ok"]
    got = want.copy()
    got[0, 4] += 0.25 * 3e-5   # an eighth of the block: held to 1e-5 of itself, although 3.75e-6 of the block
    assert not T.grade(got, want, 0, np)["ok"]
    got[0, 4] = want[0, 4] * (1 + 8e-6)
    assert T.grade(got, want, 0, np)["ok"]


def test_sixteen_bit_one_unit_in_the_last_place():
    for out_ty, dt in ((1, np.float16), (5, None)):
        if dt is not None:
            want = np.array([[1.0, 0.5, 1e-4, -3.0]], dt).view(np.uint16)
        else:
            want = (np.array([[1.0, 0.5, 1e-4, -3.0]], np.float32).view(np.uint32) >> 16).astype(np.uint16)
        got = want.copy()
        got[0, 0] += 1
        got[0, 3] += 1          # one unit, negative value
        got[0, 2] += 3          # three units of a cancellation (1e-4 of the block): under the fp32 floor
        r = T.grade(got, want, out_ty, np)
        assert r["ok"] and r["worst"] == 1 and r["needed_block_clause"] == 1
        got[0, 1] += 2
        r = T.grade(got, want, out_ty, np)
        assert not r["ok"] and r["worst"] == 2


def test_signs_zeros_and_non_finite_values():
    want = np.array([[0.0, -0.0, np.inf, np.nan, 4.0]], np.float32)
    got = np.array([[-0.0, 0.0, np.inf, np.nan, 4.0]], np.float32)
    assert T.grade(got, want, 0, np)["ok"]
    h = np.array([[0x0000, 0x8000, 0x3c00]], np.uint16)  # +0, -0, 1.0 in fp16
    g = np.array([[0x8000, 0x0000, 0x3c00]], np.uint16)
    assert T.grade(g, h, 1, np)["ok"]
    assert T.grade(np.zeros((0, 4), np.float32), np.zeros((0, 4), np.float32), 0, np)["ok"]
