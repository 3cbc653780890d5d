"""The inference module on the GPU against the oracle: weights produced on the
GPU by the row-wise quantizer, pruning through the array and through the hash
map, the three bounds-check modes, shared tables (feature_table_map), and the
reference's exact-count fixture
(fbgemm_gpu/test/tbe/inference/nbit_forward_test.py:577-659)."""
import numpy as np
import pytest

import helpers as H
from helpers import FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("lane_shape")]


@pytest.fixture(scope="module")
def M():
    assert torch.cuda.is_available()
    from fbgemm_amd import module
    return module


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_inputs(rng, rows_per_feature, B, max_L, dt):
    T = len(rows_per_feature)
    lens = rng.integers(0, max_L, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, rows_per_feature[t], size=int(lens[t * B:(t + 1) * B].sum()))
                          for t in range(T)] + [np.zeros(0, np.int64)]).astype(dt)
    return idx, off


def oracle_forward(oracle, m, idx, off, pooling, psw, out_ty):
    return oracle.tbe_forward(m.weights_dev.cpu().numpy(), m.weights_offsets.cpu().numpy(), m.weights_tys.cpu().numpy(),
                              m.D_offsets.cpu().numpy(), m.total_D, idx, off, pooling, psw, out_ty, m.row_alignment)


def bits_of(t, out_ty):
    t = t.cpu()
    return t.numpy() if out_ty == FP32 else t.view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("pooling", [0, 1])
def test_module_forward_matches_oracle(M, oracle, pooling):
    rng = np.random.default_rng(300 + pooling)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    specs = [("a", 211, 64, S.INT4, L), ("b", 97, 128, S.INT8, L), ("c", 53, 32, S.FP16, L), ("d", 300, 32, S.INT2, L),
             ("e", 40, 16, S.FP32, L)]
    ftm = [0, 1, 2, 1, 3, 4, 0]  # tables 0 and 1 serve two features each
    m = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, feature_table_map=ftm, pooling_mode=M.PoolingMode(pooling),
                                                  bounds_check_mode=M.BoundsCheckMode.NONE, output_dtype=S.FP16)
    tables = [rng.normal(0, 1, size=(n, d)).astype(np.float32) for _, n, d, _, _ in specs]
    m.quantize_and_assign([torch.from_numpy(t) for t in tables])
    # what the GPU quantizer wrote is what the oracle's quantizer writes
    for (whole, _, _), t, (_, n, d, ty, _) in zip(m.split_embedding_weights_with_scale_bias(0), tables, specs):
        if not ty.is_float():
            want = oracle.quantize_rowwise(t, ty.bit_rate(), False, oracle.LAYOUT_TBE, out_stride=whole.shape[1])
            assert (whole.cpu().numpy() == want).all()
    idx, off = make_inputs(rng, [specs[t][1] for t in ftm], 17, 12, np.int32)
    psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
    for w in (None, psw):
        got = m(cu(idx), cu(off), None if w is None else cu(w))
        rc, want = oracle_forward(oracle, m, idx, off, pooling, w, FP16)
        assert rc == 0 and tuple(got.shape) == (17, m.total_D)
        H.assert_same_bits(bits_of(got, FP16), want, f"module pooling={pooling} weighted={w is not None}")
    # split views: elements and (scale, bias) of table 0 round-trip through assign
    before = m.weights_dev.clone()
    m.assign_embedding_weights([(w.clone(), None if sb is None else sb.clone()) for w, sb in m.split_embedding_weights()])
    assert torch.equal(before, m.weights_dev)


@pytest.mark.parametrize("use_array", [True, False])
@pytest.mark.parametrize("mode", ["NONE", "WARNING", "IGNORE", "FATAL"])
def test_module_pruned_tables(M, oracle, use_array, mode):
    rng = np.random.default_rng(400)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    logical = [500, 300, 200]
    remaps, phys = [], []
    for t, n in enumerate(logical):
        if t == 1:
            remaps.append(None)  # not pruned
            phys.append(n)
            continue
        keep = rng.random(n) < 0.5
        r = np.full(n, -1, np.int32)
        r[keep] = np.arange(int(keep.sum()))
        remaps.append(torch.from_numpy(r))
        phys.append(int(keep.sum()))
    specs = [(f"t{t}", phys[t], 64, S.INT4, L) for t in range(3)]
    m = M.IntNBitTableBatchedEmbeddingBagsCodegen(
        specs, index_remapping=remaps, pooling_mode=M.PoolingMode.MEAN, bounds_check_mode=M.BoundsCheckMode[mode],
        output_dtype=S.FP32, use_array_for_index_remapping=use_array, indices_dtype=torch.int64)
    m.quantize_and_assign([torch.from_numpy(rng.normal(0, 1, size=(n, 64)).astype(np.float32)) for n in phys])
    idx, off = make_inputs(rng, logical, 23, 15, np.int64)
    got = m(cu(idx), cu(off))
    dense = idx.copy()
    B = 23
    for t in range(3):
        s, e = int(off[t * B]), int(off[(t + 1) * B])
        if remaps[t] is not None:
            dense[s:e] = remaps[t].numpy()[idx[s:e]]
    rc, want = oracle_forward(oracle, m, dense, off, 1, None, FP32)
    assert rc == 0
    H.assert_same_bits(bits_of(got, FP32), want, f"pruned array={use_array} mode={mode}")
    assert int(m.bounds_check_warning.item()) == 0
    if mode in ("WARNING", "IGNORE"):
        # an index beyond the logical rows is repaired to row 0 (and counted), as the reference does
        bad = idx.copy()
        bad[3] = 10 ** 6
        got = m(cu(bad), cu(off))
        fixed = idx.copy()
        fixed[3] = 0
        dense = fixed.copy()
        for t in range(3):
            s, e = int(off[t * B]), int(off[(t + 1) * B])
            if remaps[t] is not None:
                dense[s:e] = remaps[t].numpy()[fixed[s:e]]
        rc, want = oracle_forward(oracle, m, dense, off, 1, None, FP32)
        H.assert_same_bits(bits_of(got, FP32), want, "repaired index")
        # the counter restarts with every WARNING-mode check (embedding_bounds_check_host_cpu.cpp:108-110),
        # and the second check, after the remap, finds nothing left to repair
        assert int(m.bounds_check_warning.item()) == 0
    if mode == "FATAL":
        bad = idx.copy()
        bad[3] = 10 ** 6
        with pytest.raises(RuntimeError):
            m(cu(bad), cu(off))


def test_module_exact_count_fixture(M):
    """All rows dequantize to ones, every third logical id is pruned: a bag's sum
    is the number of kept ids in it (nbit_forward_test.py:577-659)."""
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    E, Ds, B = 100, [16, 24, 40], 6
    T = len(Ds)
    remap, n_kept, running = [], 0, 0
    for i in range(E):
        if running % 3 == 0:
            remap.append(-1)
        else:
            remap.append(n_kept)
            n_kept += 1
        running += 1
    m = M.IntNBitTableBatchedEmbeddingBagsCodegen(
        [(f"t{t}", n_kept, Ds[t], S.INT4, L) for t in range(T)],
        index_remapping=[torch.tensor(remap, dtype=torch.int32) for _ in range(T)],
        pooling_mode=M.PoolingMode.SUM, output_dtype=S.FP32, indices_dtype=torch.int32)
    m.initialize_weights()
    for w, s, b in m.split_embedding_weights_with_scale_bias(2):
        w.fill_(0x11)  # every nibble is 1
        s.fill_(1.0)
        b.fill_(0.0)
    rng = np.random.default_rng(5)
    lens = rng.integers(0, 9, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    idx = rng.integers(0, E, size=int(off[-1])).astype(np.int32)
    got = m(cu(idx), cu(off)).cpu().numpy()
    for t in range(T):
        for b in range(B):
            s, e = off[t * B + b], off[t * B + b + 1]
            kept = sum(1 for i in idx[s:e] if remap[i] != -1)
            assert (got[b, sum(Ds[:t]):sum(Ds[:t + 1])] == kept).all()


def test_module_sequence_output(M, oracle):
    rng = np.random.default_rng(6)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    specs = [("a", 80, 32, S.INT4, L), ("b", 60, 32, S.INT8, L)]
    m = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, pooling_mode=M.PoolingMode.NONE, output_dtype=S.FP16,
                                                  bounds_check_mode=M.BoundsCheckMode.WARNING)
    m.quantize_and_assign([torch.from_numpy(rng.normal(0, 1, size=(n, 32)).astype(np.float32)) for _, n, _, _, _ in specs])
    idx, off = make_inputs(rng, [80, 60], 9, 7, np.int32)
    got = m(cu(idx), cu(off))
    ok, want = oracle.tbe_forward_nobag(m.weights_dev.cpu().numpy(), m.weights_offsets.cpu().numpy(),
                                        m.weights_tys.cpu().numpy(), [80, 60], 32, idx, off, FP16, 16)
    assert ok and tuple(got.shape) == (len(idx), 32)
    H.assert_same_bits(bits_of(got, FP16), want, "module, no pooling")


def test_module_fused_pooled_embedding_quantization(M, oracle):
    """The reference's check of the 8-bit pooled output
    (fbgemm_gpu/test/tbe/inference/nbit_forward_test.py:293-340): per table, the dequantized 8-bit block
    equals the fp32 module's block quantized and dequantized by the row-wise 8-bit operators, to 1e-2."""
    from fbgemm_amd import ops
    rng = np.random.default_rng(77)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    specs = [("a", 150, 64, S.INT4, L), ("b", 90, 32, S.INT8, L), ("c", 70, 16, S.FP16, L)]
    tables = [torch.from_numpy(rng.normal(size=(n, d)).astype(np.float32)) for _, n, d, _, _ in specs]
    mods = {}
    for out in (S.INT8, S.FP32):
        m = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, bounds_check_mode=M.BoundsCheckMode.NONE, output_dtype=out)
        m.quantize_and_assign(tables)
        mods[out] = m
    idx, off = make_inputs(rng, [s[1] for s in specs], 9, 10, np.int32)
    low = mods[S.INT8](cu(idx), cu(off))
    ref = mods[S.FP32](cu(idx), cu(off))
    Ds = [s[2] for s in specs]
    assert low.dtype == torch.uint8 and tuple(low.shape) == (9, sum(Ds) + 8 * len(Ds))
    for blk, want in zip(torch.split(low, [d + 8 for d in Ds], dim=1), torch.split(ref, Ds, dim=1)):
        deq = ops.dequantize_rowwise(blk.contiguous(), want.size(1), 8, True)
        requant = ops.dequantize_rowwise(ops.quantize_rowwise(want.contiguous(), 8, True), want.size(1), 8, True)
        torch.testing.assert_close(deq, requant, rtol=1e-2, atol=1e-2)
        assert torch.equal(deq, requant)  # here the two are the same arithmetic


def test_module_with_managed_tables(M, oracle):
    """EmbeddingLocation.MANAGED tables live in the operator's second weights buffer (in HBM here): the same
    lookups as an all-DEVICE module holding the same rows."""
    rng = np.random.default_rng(88)
    S, L = M.SparseType, M.EmbeddingLocation
    shapes = [("a", 120, 64, S.INT4), ("b", 80, 32, S.INT8), ("c", 60, 16, S.FP16), ("d", 90, 128, S.INT4)]
    tables = [torch.from_numpy(rng.normal(size=(n, d)).astype(np.float32)) for _, n, d, _ in shapes]
    mods = []
    for locs in ([L.DEVICE] * 4, [L.MANAGED, L.DEVICE, L.MANAGED, L.DEVICE], [L.MANAGED] * 4):
        m = M.IntNBitTableBatchedEmbeddingBagsCodegen([s + (loc,) for s, loc in zip(shapes, locs)],
                                                      bounds_check_mode=M.BoundsCheckMode.NONE, output_dtype=S.FP32)
        m.quantize_and_assign(tables)
        mods.append(m)
    assert mods[1].weights_uvm.numel() > 0 and mods[1].weights_placements.tolist() == [1, 0, 1, 0]
    idx, off = make_inputs(rng, [s[1] for s in shapes], 11, 9, np.int64)
    want = mods[0](cu(idx), cu(off))
    for m in mods[1:]:
        assert torch.equal(m(cu(idx), cu(off)), want)
    with pytest.raises(NotImplementedError):
        M.IntNBitTableBatchedEmbeddingBagsCodegen([shapes[0] + (L.MANAGED_CACHING,)])


@pytest.mark.parametrize("mode", ["NONE", "WARNING"])
def test_module_pruned_tables_shared_by_features(M, oracle, mode):
    """Features that share a pruned table: every feature's lookups go through its table's mapping
    (fused into the forward without bounds check, as a separate pruned_array_lookup with one)."""
    rng = np.random.default_rng(401)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    logical = [400, 250, 320]
    ftm = [0, 1, 0, 2, 2, 1]
    remaps, phys = [], []
    for t, n in enumerate(logical):
        if t == 1:
            remaps.append(None)
            phys.append(n)
            continue
        keep = rng.random(n) < 0.6
        r = np.full(n, -1, np.int32)
        r[keep] = np.arange(int(keep.sum()))
        remaps.append(torch.from_numpy(r))
        phys.append(int(keep.sum()))
    specs = [(f"t{t}", phys[t], [64, 128, 32][t], S.INT4, L) for t in range(3)]
    m = M.IntNBitTableBatchedEmbeddingBagsCodegen(
        specs, feature_table_map=ftm, index_remapping=remaps, pooling_mode=M.PoolingMode.SUM,
        bounds_check_mode=M.BoundsCheckMode[mode], output_dtype=S.FP16, indices_dtype=torch.int64)
    m.quantize_and_assign([torch.from_numpy(rng.normal(0, 1, size=(n, d)).astype(np.float32))
                           for n, (_, _, d, _, _) in zip(phys, specs)])
    B = 17
    idx, off = make_inputs(rng, [logical[t] for t in ftm], B, 12, np.int64)
    got = m(cu(idx), cu(off))
    dense = idx.copy()
    for f, t in enumerate(ftm):
        s, e = int(off[f * B]), int(off[(f + 1) * B])
        if remaps[t] is not None:
            dense[s:e] = remaps[t].numpy()[idx[s:e]]
    rc, want = oracle_forward(oracle, m, dense, off, 0, None, FP16)
    assert rc == 0
    H.assert_same_bits(bits_of(got, FP16), want, f"shared pruned tables, mode={mode}")
