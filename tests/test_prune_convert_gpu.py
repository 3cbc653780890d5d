"""GPU parity of embedding_bag_rowwise_prune (C ABI, Python mirror, torch operator)
against the oracle, and of the inference converter built on it: what the
converter leaves in the module equals the oracle's prune -> quantize of the same
tables byte for byte, and lookups through the converted module equal the oracle's
forward over those bytes."""
import os

import numpy as np
import pytest

import helpers as H
from helpers import FP16

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("idx_dt", [torch.int32, torch.int64])
def test_prune_matches_oracle(ops, oracle, idx_dt):
    rng = np.random.default_rng(77)
    np_dt = np.int32 if idx_dt == torch.int32 else np.int64
    for rows, cols, min_rows, use_abs, thr in [
            (50, 8, 0, True, 0.7), (1000, 3, 0, False, 0.2), (200, 16, 150, True, 1.0), (64, 1, 64, True, 0.5),
            (64, 4, 100, True, 0.5), (1, 5, 0, True, 0.1), (300, 2, 299, False, 0.9), (4096, 4, 0, True, 0.7),
            (4097, 5, 4000, True, 1.5), (100000, 16, 0, True, 0.67), (300001, 33, 250000, False, 0.3),
            (5000, 128, 0, True, 100.0), (5000, 7, 0, True, 0.0)]:
        w = rng.normal(size=(rows, cols)).astype(np.float32)
        ind = rng.normal(size=rows).astype(np.float32)
        want_w, want_r = oracle.rowwise_prune(w, ind, thr, np_dt, use_abs, min_rows)
        got_w, got_r = ops.embedding_bag_rowwise_prune(cu(w), cu(ind), thr, idx_dt, use_abs, min_rows, None)
        assert got_r.dtype == idx_dt and (got_r.cpu().numpy() == want_r).all(), (rows, cols, min_rows)
        assert tuple(got_w.shape) == want_w.shape
        H.assert_same_bits(got_w.cpu().numpy(), want_w, f"pruned rows {rows}x{cols}")
    # half-precision rows move as bytes
    w16 = rng.normal(size=(999, 10)).astype(np.float16)
    ind = rng.normal(size=999).astype(np.float32)
    _, want_r = oracle.rowwise_prune(w16.astype(np.float32), ind, 0.5, np_dt, True, 0)
    got_w, got_r = ops.embedding_bag_rowwise_prune(cu(w16), cu(ind), 0.5, idx_dt, True, 0, None)
    assert (got_r.cpu().numpy() == want_r).all()
    assert (got_w.cpu().numpy().view(np.uint16) == w16[want_r >= 0].view(np.uint16)).all()


def test_prune_argument_checks_and_save_ratio(ops):
    w = torch.zeros(10, 4, device="cuda")
    ind = torch.ones(10, device="cuda")
    with pytest.raises(ValueError, match="Threshold"):
        ops.embedding_bag_rowwise_prune(w, ind, -1.0, torch.int32)
    with pytest.raises(ValueError, match="indicator"):
        ops.embedding_bag_rowwise_prune(w, ind[:5], 0.5, torch.int32)
    with pytest.raises(ValueError, match="Int/Long"):
        ops.embedding_bag_rowwise_prune(w, ind, 0.5, torch.int16)
    # one column: the map costs as much as the rows, nothing is saved, the weights come back whole
    w1 = torch.zeros(10, 1, device="cuda")
    out, remap = ops.embedding_bag_rowwise_prune(w1, ind, 0.5, torch.int32)
    assert out is w1 and remap.tolist() == [0]


def test_prune_torch_operator(oracle):
    lib = os.path.join(ROOT, "fbgemm_amd", "lib", "libfbgemm_amd_torch.so")
    assert os.path.exists(lib), "build it with `python -m fbgemm_amd.build`"
    torch.ops.load_library(lib)
    rng = np.random.default_rng(78)
    w = rng.normal(size=(777, 12)).astype(np.float32)
    ind = rng.normal(size=777).astype(np.float32)
    want_w, want_r = oracle.rowwise_prune(w, ind, 0.4, np.int64, True, 500)
    got_w, got_r = torch.ops.fbgemm.embedding_bag_rowwise_prune(cu(w), cu(ind), 0.4, torch.int64, True, 500, None)
    assert (got_r.cpu().numpy() == want_r).all() and (got_w.cpu().numpy().view(np.uint32) == want_w.view(np.uint32)).all()
    want_w, want_r = oracle.rowwise_prune(w, ind, 0.4, np.int32, True, 0)
    got_w, got_r = torch.ops.fbgemm.embedding_bag_rowwise_prune(cu(w), cu(ind), 0.4, torch.int32)
    assert (got_r.cpu().numpy() == want_r).all() and (got_w.cpu().numpy().view(np.uint32) == want_w.view(np.uint32)).all()
    out, remap = torch.ops.fbgemm.embedding_bag_rowwise_prune(cu(w[:, :1]), cu(ind), 0.4, torch.int32)
    assert tuple(out.shape) == (777, 1) and remap.tolist() == [0]
    with pytest.raises(RuntimeError, match="Threshold"):
        torch.ops.fbgemm.embedding_bag_rowwise_prune(cu(w), cu(ind), -0.1, torch.int32)


@pytest.mark.parametrize("ty_name,ratio,use_array", [("INT4", 0.5, True), ("INT8", 0.25, False), ("INT2", 0.9, True),
                                                     ("FP16", 0.5, True), ("FP8", 0.3, True), ("INT4", None, True)])
def test_converter_matches_oracle_pipeline(ops, oracle, ty_name, ratio, use_array):
    from fbgemm_amd import converter, module as M
    ty = getattr(M.SparseType, ty_name)
    rng = np.random.default_rng(900 + len(ty_name) + int((ratio or 0) * 100))
    shapes = [(300, 64), (1000, 32), (57, 128)]
    tables = [(rng.normal(size=s) * rng.uniform(0.2, 2.0, size=(s[0], 1))).astype(np.float32) for s in shapes]
    cfg = converter.FP8QuantizationConfig(4, 7) if ty_name == "FP8" else None
    conv = converter.SplitEmbInferenceConverter(ty, ratio, use_array_for_index_remapping=use_array, quantization_config=cfg)
    m = conv.convert_tables([cu(t) for t in tables], M.PoolingMode.SUM, bounds_check_mode=M.BoundsCheckMode.NONE,
                            output_dtype=M.SparseType.FP16)
    # the oracle's pipeline on the same tables, with the norms the converter used
    views = m.split_embedding_weights_with_scale_bias(0)
    remaps = []
    for t, (whole, _, _), (_, n, d, got_ty, _) in zip(tables, views, m.embedding_specs):
        assert got_ty == ty
        if ratio is None:
            kept, remap = t, None
        else:
            new_rows = int(np.ceil(len(t) * (1.0 - ratio)))
            ind, thr = conv._prune_by_weights_l2_norm(new_rows, cu(t))
            kept, remap = oracle.rowwise_prune(t, ind.cpu().numpy(), thr, np.int32, True, 0)
            assert len(kept) == new_rows  # random norms: no ties
        remaps.append(remap)
        assert n == len(kept)
        got = whole.cpu().numpy()
        if ty_name in ("INT4", "INT8", "INT2"):
            bits = ty.bit_rate()
            if bits == 8:  # quantize_embs: the fp32 (scale, bias) of the 8-bit rows is rounded to fp16 and moved to the front
                q = oracle.quantize_rowwise(kept, 8, True)
                sb = q[:, -8:].copy().view(np.float32).astype(np.float16).view(np.uint8)
                want = np.concatenate([sb, q[:, :-8]], axis=1)
            else:
                want = oracle.quantize_rowwise(kept, bits, False, oracle.LAYOUT_TBE)
            assert (got[:, :want.shape[1]] == want).all()
        elif ty_name == "FP16":
            assert (got[:, :2 * d] == kept.astype(np.float16).view(np.uint8).reshape(len(kept), -1)).all()
        else:
            assert (got[:, :d] == oracle.float_to_hfp8(kept, 4, 7, 240.0)).all()
    # lookups by original row id: pruned rows add nothing
    B = 11
    lens = rng.integers(0, 9, size=len(shapes) * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    idx = np.concatenate([rng.integers(0, shapes[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(len(shapes))]).astype(np.int32)
    got = m(cu(idx), cu(off))
    dense = idx.copy()
    pos = 0
    for t in range(len(shapes)):
        cnt = int(lens[t * B:(t + 1) * B].sum())
        if remaps[t] is not None:
            dense[pos:pos + cnt] = remaps[t][idx[pos:pos + cnt]]
        pos += cnt
    got = got.cpu().view(torch.int16).numpy().view(np.uint16)
    if ty_name == "FP8":
        # the table-batched oracle has no 8-bit float rows: per table, the pooled FP8 oracle with the operator's -1 skip
        weights = m.weights_dev.cpu().numpy()
        wo, Do = m.weights_offsets.cpu().numpy(), m.D_offsets.cpu().numpy()
        for t, (_, n, d, _, _) in enumerate(m.embedding_specs):
            s0, e0 = int(off[t * B]), int(off[(t + 1) * B])
            rb = (d + m.row_alignment - 1) // m.row_alignment * m.row_alignment
            ok, want = oracle.spmdm_fp8(d, weights[wo[t]:wo[t] + n * rb], dense[s0:e0], off[t * B:(t + 1) * B + 1] - s0,
                                        out_ty=FP16, input_stride=rb, exponent_bits=4, exponent_bias=7, skip_minus_one=True,
                                        data_size=n, output_size=B)
            assert ok
            H.assert_same_bits(np.ascontiguousarray(got[:, Do[t]:Do[t + 1]]), want.reshape(B, d), f"converted FP8 table {t}")
        return
    rc, want = oracle.tbe_forward(m.weights_dev.cpu().numpy(), m.weights_offsets.cpu().numpy(), m.weights_tys.cpu().numpy(),
                                  m.D_offsets.cpu().numpy(), m.total_D, dense, off, 0, None, FP16, m.row_alignment)
    assert rc == 0
    H.assert_same_bits(got, want, f"converted {ty_name} ratio={ratio}")


class FloatTables(torch.nn.Module):
    """Test stand-in for the float module the reference's converter reads its tables from
    (split_embedding_weights(), pooling_mode; forward = plain pooled sums in fp32)."""

    def __init__(self, tables):
        super().__init__()
        self.tables = [t.cuda() for t in tables]
        self.pooling_mode = 0

    def split_embedding_weights(self):
        return self.tables

    def forward(self, indices, offsets):
        T = len(self.tables)
        B = (offsets.numel() - 1) // T
        off = offsets.cpu().tolist()
        out = torch.zeros(B, sum(t.size(1) for t in self.tables), device="cuda")
        col = 0
        for t, tbl in enumerate(self.tables):
            for b in range(B):
                s, e = off[t * B + b], off[t * B + b + 1]
                if e > s:
                    out[b, col:col + tbl.size(1)] = tbl[indices[s:e].long()].sum(0)
            col += tbl.size(1)
        return out


class Arch(torch.nn.Module):
    def __init__(self, tables):
        super().__init__()
        self.emb_module = FloatTables(tables)

    def forward(self, indices, offsets):
        return self.emb_module(indices, offsets)


@pytest.mark.parametrize("use_array", [True, False])
@pytest.mark.parametrize("ty_name", ["FP32", "FP16", "INT8", "INT4", "INT2"])
def test_l2_norm_pruning_workflow_fixture(ty_name, use_array):
    """The reference's fully specified pruning fixture
    (fbgemm_gpu/test/tbe/inference/inference_converter_test.py:263-343): two tables of five constant rows,
    pruning ratios 0.9 / 0.5 / 0.1; lookups through the converted module by original row id must equal the
    float lookups over the indices the reference lists as surviving, to the reference's tolerance, and the
    surviving rows must be the ones of largest norm."""
    from fbgemm_amd import converter, module as M
    D, E = 128, 5
    indices = torch.tensor([3, 0, 2, 2, 3, 4, 2], dtype=torch.int32)
    offsets = torch.tensor([0, 1, 4, 6, 7], dtype=torch.int32)
    scales = [[0.4, 0.1, -0.2, 0.2, 0.3], [-0.8, 0.2, 0.5, -0.1, 0.9]]
    weights = [torch.tensor(s).view(E, 1) * torch.ones(E, D) for s in scales]
    cases = [(0.9, [0, 4], [0, 0, 1, 2, 2], [[0], [4]]),
             (0.5, [3, 0, 2, 2, 4, 2], [0, 1, 4, 5, 6], [[0, 2, 3, 4], [0, 2, 4]]),
             (0.1, indices.tolist(), offsets.tolist(), [[0, 1, 2, 3, 4], [0, 1, 2, 3, 4]])]
    # ratio 0.5 keeps ceil(2.5) = 3 rows, and every row that ties with the third: |-0.2| == |0.2| keeps four in table 0
    for ratio, rem_idx, rem_off, kept_rows in cases:
        arch = Arch(weights)
        want = arch(torch.tensor(rem_idx, dtype=torch.int32).cuda(), torch.tensor(rem_off, dtype=torch.int32).cuda())
        conv = converter.SplitEmbInferenceConverter(getattr(M.SparseType, ty_name), ratio, use_array_for_index_remapping=use_array)
        conv.convert_model(arch)
        assert type(arch.emb_module) is M.IntNBitTableBatchedEmbeddingBagsCodegen
        assert [e[1] for e in arch.emb_module.embedding_specs] == [len(k) for k in kept_rows]
        got = arch(indices.cuda(), offsets.cuda())
        torch.testing.assert_close(want.float().cpu(), got.float().cpu(), atol=1.0e-1, rtol=1.0e-1)
