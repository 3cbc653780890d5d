"""GPU parity of the single-table pooled lookup, through the C ABI, against the
CPU oracle on the same seeded inputs. Integer/index behaviour and every output
bit must match: the kernels consume rows in index order with one lane per
output column, so fp32 results are bit-identical (tolerance 0; the path's
stated bound is 1e-5 relative for fp32 and 1 ulp for fp16).

Parameter space after test/EmbeddingSpMDMNBitTest.cc:92-418 and
test/EmbeddingSpMDM8BitTest.cc:82-372: bit rates, weighted / positional,
normalize, offsets vs lengths, index and offset widths, output types, odd
dims, corner cases, and ten sentinel values after the output."""
import itertools

import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("lane_shape")]

SENTINELS = 10

SHAPES = [
    (10, 400, 2, 5), (10, 400, 4, 5), (10, 400, 7, 5), (10, 400, 8, 5), (10, 400, 16, 5),
    (10, 400, 32, 5), (10, 400, 40, 5), (10, 400, 48, 5), (10, 400, 56, 5), (10, 400, 64, 5),
    (3, 1000, 86, 20), (20, 1000, 128, 50), (10, 400, 164, 5), (40, 300, 256, 10),
    (7, 200, 384, 12), (5, 100, 1024, 9), (3, 60, 2048, 7), (2, 40, 2600, 5),
    (1, 50, 32, 100), (300, 5000, 128, 20), (0, 20, 32, 5),
]


def dev(a, torch_dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t


def run_gpu(ops, *, ty, D, table, idx, off_or_len, w, normalize, out_ty, positional, use_offsets,
            output_stride, input_stride, sbl, remap, data_size, output_size, index_size=None):
    stride = D if output_stride == -1 else output_stride
    np_dt = np.float32 if out_ty == FP32 else np.uint16
    sentinel = np.float32(-12345.5) if out_ty == FP32 else np.uint16(0xBEEF)
    out_host = np.full(output_size * stride + SENTINELS, sentinel, dtype=np_dt)
    t_out = dev(out_host.view(np.int16) if np_dt == np.uint16 else out_host)
    t_table = dev(table)
    if ty in (FP16, BF16):
        assert t_table.data_ptr() % 2 == 0
    t_idx, t_off = dev(idx), dev(off_or_len)
    t_w = None if w is None else dev(w)
    t_remap = None if remap is None else dev(remap)
    if remap is not None:
        kern = (ops.generate_embedding_spmdm_nbit_rowwise_sparse(
                    4 if ty == INT4 else 2, D, w is not None, normalize, 16, positional, use_offsets)
                if ty in (INT4, INT2) else
                ops.generate_embedding_spmdm_rowwise_sparse(
                    ty, D, w is not None, normalize, 16, positional, use_offsets))
    elif ty in (INT4, INT2):
        kern = ops.generate_embedding_spmdm_nbit_with_strides(
            4 if ty == INT4 else 2, D, w is not None, normalize, 16, positional, use_offsets,
            output_stride, input_stride, sbl, out_ty=out_ty)
    else:
        kern = ops.generate_embedding_spmdm_with_strides(
            ty, D, w is not None, normalize, 16, positional, use_offsets, output_stride,
            input_stride, sbl, out_ty=out_ty)
    ok = kern(output_size, len(idx) if index_size is None else index_size, data_size, t_table,
              t_idx, t_off, t_w, t_out, t_remap) if remap is not None else \
        kern(output_size, len(idx) if index_size is None else index_size, data_size, t_table,
             t_idx, t_off, t_w, t_out)
    res = t_out.cpu().numpy()
    res = res.view(np.uint16) if np_dt == np.uint16 else res
    n = output_size * stride
    assert (res[n:] == sentinel).all(), "wrote past the end of the output"
    return ok, res[:n], sentinel


def check_case(ops, oracle, *, ty, D, table, idx, off_or_len, w=None, normalize=False, out_ty=FP32,
               positional=False, use_offsets=True, output_stride=-1, input_stride=-1, sbl=True,
               remap=None, data_size, output_size, index_size=None, what=""):
    stride = D if output_stride == -1 else output_stride
    np_dt = np.float32 if out_ty == FP32 else np.uint16
    ok_g, out_g, sentinel = run_gpu(
        ops, ty=ty, D=D, table=table, idx=idx, off_or_len=off_or_len, w=w, normalize=normalize,
        out_ty=out_ty, positional=positional, use_offsets=use_offsets, output_stride=output_stride,
        input_stride=input_stride, sbl=sbl, remap=remap, data_size=data_size,
        output_size=output_size, index_size=index_size)
    pre = np.full(output_size * stride, sentinel, dtype=np_dt)
    ok_o, out_o = oracle.spmdm(
        ty, D, table, idx, off_or_len, weights=w, normalize=normalize, out_ty=out_ty,
        positional=positional, use_offsets=use_offsets, output_stride=output_stride,
        input_stride=input_stride, scale_bias_last=sbl, remap=remap, data_size=data_size,
        output_size=output_size, index_size=index_size, out=pre)
    assert ok_g == ok_o, f"{what}: gpu returned {ok_g}, oracle {ok_o}"
    if ok_o:
        H.assert_same_bits(out_g, out_o, what)
    return ok_g


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32, BF16])
@pytest.mark.parametrize("shape", SHAPES)
def test_parity_grid(ops, oracle, ty, shape):
    nb, rows, D, avg = shape
    if ty == INT2 and D % 4 and D > 4:
        D = (D + 3) // 4 * 4
    rng = np.random.default_rng(hash((ty, shape, 1)) % 2**32)
    ran = 0
    combos = list(itertools.product(
        (True, False), (FP32, FP16, BF16), (0, 1, 2), (False, True),
        (np.int32, np.int64), (np.int32, np.int64), (True, False)))
    rng.shuffle(combos)
    for sbl, out_ty, weighted, normalize, idx_dt, off_dt, use_offsets in combos[:6]:
        table, stride = H.make_table(rng, ty, rows, D, sbl)
        idx, off, lens = H.make_bags(rng, rows, nb, avg, idx_dt, off_dt, empty_frac=0.15)
        if not sbl and len(idx):
            idx[rng.random(len(idx)) < 0.2] = -1
        w = None
        if weighted == 1:
            w = rng.normal(size=len(idx)).astype(np.float32)
        elif weighted == 2:
            w = rng.normal(size=max(1, int(lens.max()) if len(lens) else 1)).astype(np.float32)
        what = f"ty={ty} shape={shape} sbl={sbl} out={out_ty} w={weighted} norm={normalize} " \
               f"idx={np.dtype(idx_dt).name} off={np.dtype(off_dt).name} use_offsets={use_offsets}"
        print(what, flush=True)
        ok = check_case(ops, oracle, ty=ty, D=D, table=table, idx=idx,
                        off_or_len=off if use_offsets else lens, w=w, normalize=normalize,
                        out_ty=out_ty, positional=weighted == 2, use_offsets=use_offsets, sbl=sbl,
                        data_size=rows, output_size=nb, what=what)
        assert ok
        ran += 1
    assert ran


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32])
@pytest.mark.parametrize("align", [1, 4, 16])
def test_tbe_row_layout_and_strides(ops, oracle, ty, align):
    rng = np.random.default_rng(100 + ty * 7 + align)
    for D in (8, 24, 64, 128, 200):
        rows, nb = 300, 33
        stride = oracle.padded_row_bytes(D, ty, align)
        if ty == FP32:
            stride = (stride + 3) // 4 * 4
        table, stride = H.make_table(rng, ty, rows, D, False, stride_bytes=stride)
        idx, off, _ = H.make_bags(rng, rows, nb, 9, empty_frac=0.1)
        idx[::4] = -1
        for out_ty, total_D in ((FP16, D + 24), (FP32, D + 3), (BF16, D)):
            what = f"ty={ty} align={align} D={D} out={out_ty} total_D={total_D}"
            print(what, flush=True)
            assert check_case(ops, oracle, ty=ty, D=D, table=table, idx=idx, off_or_len=off,
                              w=rng.uniform(size=len(idx)).astype(np.float32), out_ty=out_ty,
                              output_stride=total_D, input_stride=H.input_stride_elems(ty, stride),
                              sbl=False, data_size=rows, output_size=nb, what=what)


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16])
def test_rejections(ops, oracle, ty):
    rng = np.random.default_rng(11 + ty)
    rows, D, nb = 100, 32, 8
    table, _ = H.make_table(rng, ty, rows, D, True)
    idx, off, _ = H.make_bags(rng, rows, nb, 5)
    kw = dict(ty=ty, D=D, table=table, data_size=rows, output_size=nb)
    assert check_case(ops, oracle, idx=idx, off_or_len=off, what="valid", **kw)
    bad = idx.copy(); bad[len(bad) // 2] = rows
    assert not check_case(ops, oracle, idx=bad, off_or_len=off, what="idx == rows", **kw)
    bad = idx.copy(); bad[1] = -1
    assert not check_case(ops, oracle, idx=bad, off_or_len=off, what="-1 in trailer layout", **kw)
    bad = idx.copy(); bad[-1] = -7
    assert not check_case(ops, oracle, idx=bad, off_or_len=off, what="negative", **kw)
    assert not check_case(ops, oracle, idx=idx, off_or_len=off, index_size=len(idx) - 1, what="short", **kw)
    longer = np.concatenate([idx, idx[:1]])
    assert not check_case(ops, oracle, idx=longer, off_or_len=off, index_size=len(idx) + 1, what="long", **kw)
    zero_off = np.zeros_like(off)
    assert check_case(ops, oracle, idx=idx[:0], off_or_len=zero_off, what="all bags empty", **kw)
    one = np.zeros(1, idx.dtype)
    assert not check_case(ops, oracle, idx=one, off_or_len=zero_off, index_size=1, what="unused index", **kw)


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32])
def test_rowwise_sparse(ops, oracle, ty):
    rng = np.random.default_rng(23 + ty)
    logical, nb = 500, 37
    for D in (16, 48, 64, 128):
        keep = rng.random(logical) >= 0.7
        mapping = np.full(logical, -1, np.int32)
        mapping[keep] = np.arange(int(keep.sum()), dtype=np.int32)
        rows = max(1, int(keep.sum()))
        table, _ = H.make_table(rng, ty, rows, D, True)
        for weighted, normalize, idx_dt, use_offsets in itertools.product(
                (0, 1, 2), (False, True), (np.int32, np.int64), (True, False)):
            idx, off, lens = H.make_bags(rng, logical, nb, 8, idx_dt, np.int32)
            w = None
            if weighted == 1:
                w = rng.normal(size=len(idx)).astype(np.float32)
            elif weighted == 2:
                w = rng.normal(size=int(lens.max())).astype(np.float32)
            what = f"sparse ty={ty} D={D} w={weighted} norm={normalize} use_offsets={use_offsets}"
            assert check_case(ops, oracle, ty=ty, D=D, table=table, idx=idx,
                              off_or_len=off if use_offsets else lens, w=w, normalize=normalize,
                              positional=weighted == 2, use_offsets=use_offsets, remap=mapping,
                              data_size=logical, output_size=nb, what=what)
        bad = idx.copy(); bad[0] = logical
        assert not check_case(ops, oracle, ty=ty, D=D, table=table, idx=bad, off_or_len=off,
                              remap=mapping, data_size=logical, output_size=nb, what="logical OOB")


def test_closed_forms(ops, oracle):
    """scale=1, bias=0 rows sum to exact integers ("should be exact",
    test/EmbeddingSpMDMNBitTest.cc:490-507); rows of ones count the bag."""
    rng = np.random.default_rng(1)
    rows, D, nb = 64, 64, 50
    for ty in (INT8, INT4, INT2):
        table, stride = H.make_table(rng, ty, rows, D, True, scale_range=(1, 1), bias_range=(0, 0))
        idx, off, lens = H.make_bags(rng, rows, nb, 10)
        ok, out, _ = run_gpu(ops, ty=ty, D=D, table=table, idx=idx, off_or_len=off, w=None,
                             normalize=False, out_ty=FP32, positional=False, use_offsets=True,
                             output_stride=-1, input_stride=-1, sbl=True, remap=None,
                             data_size=rows, output_size=nb)
        assert ok
        bits = H.BITS[ty]
        pb = H.packed_bytes(ty, D)
        q = table.reshape(rows, stride)[:, :pb]
        epb = 8 // bits
        vals = np.stack([(q >> (bits * k)) & ((1 << bits) - 1) for k in range(epb)], axis=2).reshape(rows, -1)[:, :D]
        want = np.stack([vals[idx[off[b]:off[b + 1]]].sum(axis=0) for b in range(nb)]).astype(np.float32)
        assert (out.reshape(nb, D) == want).all()
        ones, _ = H.make_table(rng, ty, rows, D, True, ones=True)
        ok, out, _ = run_gpu(ops, ty=ty, D=D, table=ones, idx=idx, off_or_len=off, w=None,
                             normalize=False, out_ty=FP16, positional=False, use_offsets=True,
                             output_stride=-1, input_stride=-1, sbl=True, remap=None,
                             data_size=rows, output_size=nb)
        assert ok
        got = out.view(np.float16).reshape(nb, D).astype(np.float32)
        assert (got == lens.astype(np.float32)[:, None]).all()


def test_large_call_takes_the_ordered_path(ops, oracle):
    """More than two million lookups in one single-table call: the library
    orders the bags by length first (it skips that for smaller calls)."""
    rng = np.random.default_rng(77)
    rows, D, nb = 5000, 32, 90_000
    table, _ = H.make_table(rng, INT4, rows, D, True)
    lens = rng.integers(0, 60, size=nb)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = rng.integers(0, rows, size=int(off[-1])).astype(np.int32)
    assert len(idx) > (1 << 21)
    kw = dict(ty=INT4, D=D, table=table, normalize=True, out_ty=FP16, data_size=rows, output_size=nb)
    assert check_case(ops, oracle, idx=idx, off_or_len=off, what="2.6 M lookups, ordered bags", **kw)
    # what the reference rejects is rejected on this path too
    assert not check_case(ops, oracle, idx=idx, off_or_len=off, index_size=len(idx) - 1, what="ordered, short", **kw)
    longer = np.concatenate([idx, idx[:1]])
    assert not check_case(ops, oracle, idx=longer, off_or_len=off, index_size=len(idx) + 1, what="ordered, long", **kw)
    bad = idx.copy(); bad[len(bad) // 3] = rows
    assert not check_case(ops, oracle, idx=bad, off_or_len=off, what="ordered, idx == rows", **kw)
    # offsets that step back once: a bag of negative length, which the scheduler's entry cannot hold
    # (the reference's result for it is unspecified; the library always rejects it)
    back = off.copy(); back[nb // 2] = back[nb // 2 - 1] - 3
    ok, _, _ = run_gpu(ops, idx=idx, off_or_len=back, w=None, positional=False, use_offsets=True, output_stride=-1,
                       input_stride=-1, sbl=True, remap=None, **kw)
    assert not ok


def same_bits_or_both_nan(got, want, what):
    """Bit equality, except that any NaN matches any NaN (the sign and payload of a NaN an
    invalid operation makes differ between the CPU and the GPU)."""
    if got.dtype == np.float32:
        gn, wn = np.isnan(got), np.isnan(want)
        gb, wb = got.view(np.uint32), want.view(np.uint32)
    else:  # fp16 / bf16 patterns
        f = lambda a: (a & 0x7C00) == 0x7C00 if what.endswith("fp16") else (a & 0x7F80) == 0x7F80
        gn = f(got) & ((got & (0x03FF if what.endswith("fp16") else 0x007F)) != 0)
        wn = f(want) & ((want & (0x03FF if what.endswith("fp16") else 0x007F)) != 0)
        gb, wb = got, want
    assert (gn == wn).all(), f"{what}: NaNs in different places"
    assert (gb[~wn] == wb[~wn]).all(), f"{what}: {np.argwhere(gb[~wn] != wb[~wn])[:4]}"


@pytest.mark.parametrize("ty,sbl", [(INT8, True), (INT8, False), (INT4, True), (INT4, False), (INT2, False), (FP16, True), (FP32, True)])
def test_special_values(ops, oracle, ty, sbl):
    """Scales at and beyond 2^100 (where the 4- and 8-bit kernels leave their pre-scaled arithmetic and a
    wave redoes its work the plain way), infinities, NaNs, denormals and signed zeros in scales, biases,
    per-sample weights and float rows: every finite result bit for bit, NaN where the reference has NaN."""
    rng = np.random.default_rng(31 + ty)
    rows, D, nb = 40, 64, 30
    table, stride = H.make_table(rng, ty, rows, D, sbl)
    t2 = table.reshape(rows, stride)
    specials32 = np.array([1e35, -3e33, np.inf, -np.inf, np.nan, 1e-40, -1e-42, 0.0, -0.0, 2.0 ** 100, np.nextafter(np.float32(2.0 ** 100), np.float32(0))], np.float32)
    np.seterr(over="ignore")  # the casts of 1e35 to half give inf on purpose
    if ty in (INT8, INT4, INT2):
        pb = H.packed_bytes(ty, D)
        for r in range(len(specials32)):
            if ty == INT8 and sbl:  # fp32 pair behind the data
                t2[r, pb:pb + 4] = specials32[r:r + 1].view(np.uint8)
                t2[r + 12, pb + 4:pb + 8] = specials32[r:r + 1].view(np.uint8)
            else:  # fp16 pair: behind (sbl) or in front of the data
                o = pb if sbl else 0
                t2[r, o:o + 2] = specials32[r:r + 1].astype(np.float16).view(np.uint8)
                t2[r + 12, o + 2:o + 4] = specials32[r:r + 1].astype(np.float16).view(np.uint8)
    elif ty == FP16:
        t2.view(np.uint16)[:len(specials32), 3] = specials32.astype(np.float16).view(np.uint16)
        t2.view(np.uint16)[5, 7] = 0x0001  # the smallest half denormal
    else:
        t2.view(np.float32)[:len(specials32), 3] = specials32
    idx, off, lens = H.make_bags(rng, rows, nb, 6)
    wts = rng.normal(size=len(idx)).astype(np.float32)
    wts[::7] = 1e30   # times an fp16 scale of ~0.05: beyond 2^100
    wts[3::11] = np.float32(1e-40)
    wts[5::13] = np.inf
    wts[6::17] = np.nan
    wts[8::19] = -0.0
    table = np.ascontiguousarray(t2).reshape(-1)
    for w in (None, wts):
        for out_ty, name in ((FP32, "fp32"), (FP16, "fp16"), (BF16, "bf16")):
            for normalize in (False, True):
                ok_g, out_g, sentinel = run_gpu(
                    ops, ty=ty, D=D, table=table, idx=idx, off_or_len=off, w=w, normalize=normalize, out_ty=out_ty,
                    positional=False, use_offsets=True, output_stride=-1, input_stride=-1, sbl=sbl, remap=None,
                    data_size=rows, output_size=nb)
                ok_o, out_o = oracle.spmdm(ty, D, table, idx, off, weights=w, normalize=normalize, out_ty=out_ty,
                                           scale_bias_last=sbl, data_size=rows, output_size=nb)
                assert ok_g and ok_o
                same_bits_or_both_nan(out_g, out_o, f"special values ty={ty} sbl={sbl} weighted={w is not None} {name}")
