"""GPU parity, through the C ABI, of two more forms of the single-table kernels:
no_bag (one output row per index, src/RefImplementations.cc:1235-1288,1352-1376,
1466-1484) and rows of 8-bit floats (EmbeddingSpMDMFP8_ref, :1544-1616), against
the CPU oracle on the same seeded inputs. Every output bit must match, bytes
the reference leaves alone must stay as they were, and the calls must return
false where the reference does."""
import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

SENT8 = 0xA5


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def storage(table_bytes, ty):
    """The flat byte table as the storage type the oracle's strides count in."""
    return table_bytes.view({FP32: np.float32, FP16: np.uint16, BF16: np.uint16}.get(ty, np.uint8))


NOBAG_CASES = [(INT8, FP32, True), (INT8, FP16, True), (INT8, BF16, False), (INT8, FP32, False), (INT8, INT8, True),
               (INT8, INT8, False), (INT4, INT4, True), (INT4, INT4, False), (FP32, FP32, True), (FP32, BF16, True),
               (FP16, FP32, True), (FP16, FP16, True), (BF16, BF16, True), (BF16, FP32, True)]


@pytest.mark.parametrize("ty,out_ty,sbl", NOBAG_CASES)
@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
def test_no_bag_matches_oracle(ops, oracle, ty, out_ty, sbl, idx_dt):
    rng = np.random.default_rng(100 + ty * 16 + out_ty + (1 if sbl else 0))
    for D, rows, n, pad, weighted in [(8, 20, 13, 0, False), (34, 17, 40, 3, True), (128, 500, 1000, 0, True),
                                      (2, 3, 5, 0, False), (64, 9, 0, 0, True), (260, 40, 300, 16, False), (1024, 30, 77, 0, True)]:
        elem = H.BITS[ty] // 8 if H.BITS[ty] >= 8 else 1
        stride_b = H.default_stride_bytes(ty, D, sbl) + pad * elem
        table_b, _ = H.make_table(rng, ty, rows, D, sbl, stride_bytes=stride_b)
        table = storage(table_b, ty)
        in_stride = stride_b // elem
        idx = rng.integers(0, rows, size=n).astype(idx_dt)
        if n:
            idx[0] = rows - 1
        w = rng.normal(size=n).astype(np.float32) if weighted and out_ty not in (INT8, INT4) else None
        copies = out_ty in (INT8, INT4)
        ostrides = [-1, in_stride, in_stride + 3, max(1, in_stride - 2)] if out_ty == INT8 else ([-1] if out_ty == INT4 else [-1, D + 5])
        for ostride in ostrides:
            step = in_stride if out_ty == INT4 else (D if ostride == -1 else ostride)
            np_dt = np.uint8 if copies else (np.float32 if out_ty == FP32 else np.uint16)
            sentinel = np_dt(SENT8) if copies else (np.float32(-12345.5) if out_ty == FP32 else np.uint16(0xBEEF))
            pre = np.full(n * step + 10, sentinel, dtype=np_dt)
            t_out = dev(pre.view(np.int16) if np_dt == np.uint16 else pre)
            if ty in (INT4, INT2):
                kern = ops.generate_embedding_spmdm_nbit_with_strides(4, D, w is not None, False, 16, False, True, ostride,
                                                                      in_stride if pad else -1, sbl, no_bag=True, output_bit_rate=4)
            else:
                kern = ops.generate_embedding_spmdm_with_strides(ty, D, w is not None, False, 16, False, True, ostride,
                                                                 in_stride if pad else -1, sbl, no_bag=True, out_ty=out_ty)
            ok = kern(n, n, rows, dev(table), dev(idx), None, None if w is None else dev(w), t_out)
            got = t_out.cpu().numpy()
            got = got.view(np.uint16) if np_dt == np.uint16 else got
            want = pre.copy()
            ok_o, _ = oracle.spmdm_nobag(ty, D, table, idx, weights=w, out_ty=out_ty, output_stride=ostride,
                                         input_stride=in_stride if pad else -1, scale_bias_last=sbl, data_size=rows, out=want)
            assert ok and ok_o
            # includes the bytes between rows and after the last one, which both leave as they were
            H.assert_same_bits(got, want, f"no_bag ty={ty} out={out_ty} sbl={sbl} D={D} n={n} ostride={ostride}")


@pytest.mark.parametrize("ty,out_ty,sbl", [(INT8, FP32, True), (INT8, INT8, False), (FP16, FP16, True), (INT4, INT4, False), (FP32, FP32, True)])
def test_no_bag_rejects_what_the_reference_rejects(ops, oracle, ty, out_ty, sbl):
    rng = np.random.default_rng(9)
    D, rows = 16, 10
    table_b, stride_b = H.make_table(rng, ty, rows + 1, D, sbl)
    table = storage(table_b, ty)
    def run(idx):
        out = torch.zeros(len(idx) * (8 * D + 2 * stride_b), dtype=torch.uint8, device="cuda")
        if ty == INT4:
            kern = ops.generate_embedding_spmdm_nbit_with_strides(4, D, False, False, scale_bias_last=sbl, no_bag=True, output_bit_rate=4)
        else:
            kern = ops.generate_embedding_spmdm_with_strides(ty, D, False, False, scale_bias_last=sbl, no_bag=True, out_ty=out_ty)
        return kern(len(idx), len(idx), rows, dev(table), dev(idx), None, None, out)
    assert run(np.array([1, 2, 3], dtype=np.int64))
    for bad in (-1, -5, rows + 1, 1 << 40):
        idx = np.array([1, 2, bad, 3], dtype=np.int64)
        assert not run(idx)
        assert not oracle.spmdm_nobag(ty, D, table, idx, out_ty=out_ty, scale_bias_last=sbl, data_size=rows)[0]
    # idx == data_size: out of range here for every row type (the reference's 4-bit copy reads that row: `idx > data_size`)
    assert not run(np.array([1, rows, 3], dtype=np.int64))


def test_no_bag_forms_the_reference_does_not_have(ops):
    kern = ops.generate_embedding_spmdm_nbit_with_strides(2, 16, False, False, no_bag=True, output_bit_rate=4)
    assert kern(0, 0, 0, None, None, None, None, None) is False
    kern = ops.generate_embedding_spmdm_nbit_with_strides(4, 16, False, False, no_bag=True)
    assert kern(0, 0, 0, None, None, None, None, None) is False
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    kern = ops.generate_embedding_spmdm_with_strides(FP16, 16, False, False, no_bag=True, out_ty=INT8)
    with pytest.raises(RuntimeError):
        kern(1, 1, 1, t.view(torch.int16), torch.zeros(1, dtype=torch.int64, device="cuda"), None, None, t)


@pytest.mark.parametrize("out_ty", [FP32, FP16, BF16])
@pytest.mark.parametrize("fmt", [(4, 7), (5, 15), (4, 15), (3, 3)])
def test_fp8_rows_match_oracle(ops, oracle, out_ty, fmt):
    ebits, bias = fmt
    rng = np.random.default_rng(500 + out_ty * 10 + ebits + bias)
    for D, rows, nb, avg, weighted, normalize, use_offsets, positional, pad, idx_dt, off_dt in [
            (8, 50, 6, 3, False, False, True, False, 0, np.int64, np.int32),
            (33, 40, 9, 5, True, True, True, False, 2, np.int32, np.int32),
            (128, 1000, 300, 12, True, False, False, False, 0, np.int64, np.int64),
            (64, 30, 5, 4, True, True, True, True, 0, np.int32, np.int64),
            (1, 5, 3, 2, False, True, True, False, 0, np.int64, np.int32),
            (256, 2000, 64, 40, False, False, True, False, 16, np.int64, np.int32),
            (1000, 100, 20, 8, True, False, True, False, 0, np.int64, np.int32)]:
        stride = D + pad
        table = rng.integers(0, 256, size=rows * stride, dtype=np.uint8)
        idx, off, lens = H.make_bags(rng, rows, nb, avg, idx_dt, off_dt, empty_frac=0.15)
        w = None
        if weighted:
            w = rng.normal(size=max(1, int(lens.max()) if len(lens) else 1) if positional else len(idx)).astype(np.float32)
        ool = off if use_offsets else lens.astype(off_dt)
        ostride = D + 3
        np_dt = np.float32 if out_ty == FP32 else np.uint16
        sentinel = np.float32(-12345.5) if out_ty == FP32 else np.uint16(0xBEEF)
        pre = np.full(nb * ostride + 10, sentinel, dtype=np_dt)
        t_out = dev(pre.view(np.int16) if np_dt == np.uint16 else pre)
        kern = ops.generate_embedding_spmdm_fp8_with_strides(D, normalize, positional, use_offsets, ostride, stride, ebits, bias, out_ty=out_ty)
        ok = kern(nb, len(idx), rows, dev(table), dev(idx), dev(ool), None if w is None else dev(w), t_out)
        ok_o, want = oracle.spmdm_fp8(D, table, idx, ool, weights=w, normalize=normalize, out_ty=out_ty, positional=positional,
                                      use_offsets=use_offsets, output_stride=ostride, input_stride=stride, exponent_bits=ebits,
                                      exponent_bias=bias, data_size=rows, output_size=nb)
        assert ok and ok_o
        got = t_out.cpu().numpy()
        got = got.view(np.uint16) if np_dt == np.uint16 else got
        got = got[:nb * ostride].reshape(nb, ostride)
        H.assert_same_bits(got[:, :D], want.reshape(nb, ostride)[:, :D], f"fp8 D={D} fmt={fmt}")
        assert (got[:, D:] == sentinel).all()


def test_fp8_rows_reject_minus_one_and_out_of_range(ops, oracle):
    D, rows = 16, 10
    table = np.arange(rows * D, dtype=np.uint8)
    off = np.array([0, 2, 4], dtype=np.int32)
    kern = ops.generate_embedding_spmdm_fp8_with_strides(D, False)
    out = torch.zeros(2 * D, dtype=torch.float32, device="cuda")
    assert kern(2, 4, rows, dev(table), dev(np.array([0, 1, 2, 9], dtype=np.int64)), dev(off), None, out)
    for bad in (-1, rows, 1 << 33):
        idx = np.array([0, 1, bad, 3], dtype=np.int64)
        assert not kern(2, 4, rows, dev(table), dev(idx), dev(off), None, out)
        assert not oracle.spmdm_fp8(D, table, idx, off, data_size=rows)[0]
    with pytest.raises(RuntimeError):
        ops.generate_embedding_spmdm_fp8_with_strides(D, False, exponent_bits=0)(2, 4, rows, dev(table), dev(np.zeros(4, dtype=np.int64)), dev(off), None, out)
