"""GPU parity of the in-place row update (emb_inplace_update,
fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update.cu:28-101) and of
pruned_array_lookup_from_row_idx (:359-465) through the C ABI against the
oracle, byte for byte over both weights buffers, on the shapes of the
reference's tests (embedding_inplace_update_test.cpp;
fbgemm_gpu/test/tbe/utils/split_embeddings_test.py:271-415 for the module)."""
import random

import numpy as np
import pytest

from test_update_oracle import known_row_bytes, make_case

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def M():
    from fbgemm_amd import module
    return module


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gpu_update(ops, c, **kw):
    bufs = [cu(b.copy()) for b in c["bufs"]]
    ops.emb_inplace_update(bufs[0], bufs[1], cu(c["places"]), cu(c["offs"]), cu(c["tys"]), cu(c["D_offsets"]), cu(c["uw"]),
                           cu(c["ut"]), cu(c["ur"]), cu(c["uo"]), c["align"], **kw)
    return [b.cpu().numpy() for b in bufs]


def oracle_update(oracle, c):
    bufs = [b.copy() for b in c["bufs"]]
    oracle.emb_inplace_update(bufs[0], bufs[1], c["places"], c["offs"], c["tys"], c["D_offsets"], c["uw"], c["ut"], c["ur"],
                              c["uo"], c["align"])
    return bufs


@pytest.mark.parametrize("align", [16, 1, 4])
@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
def test_matches_oracle(ops, oracle, align, idx_dt):
    rng = np.random.default_rng(40 + align)
    for _ in range(25):
        c = make_case(rng, align=align, idx_dt=idx_dt)
        got, want = gpu_update(ops, c), oracle_update(oracle, c)
        assert (got[0] == want[0]).all() and (got[1] == want[1]).all(), (c["T"], c["tys"], c["Ds"])


def test_wide_rows_and_many_updates(ops, oracle):
    """Rows of several 256-byte steps and more updates than one pass of the grid holds: every updated row
    reads back as its source, every other byte is untouched."""
    rng = np.random.default_rng(8)
    specs = [(0, 1024, 3000), (1, 640, 50000), (3, 256, 400000), (2, 100, 7)]  # (type, D, rows): 4096 / 1280 / 144 / 112 bytes
    tys = np.array([s[0] for s in specs], np.uint8)
    rbs = [known_row_bytes(D, ty, 16) for ty, D, _ in specs]
    assert rbs == [4096, 1280, 144, 112]
    sizes = [rb * n for rb, (_, _, n) in zip(rbs, specs)]
    offs = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int64)
    dev = torch.randint(0, 255, (int(sum(sizes)),), dtype=torch.uint8, device="cuda")
    before = dev.clone()
    per_table = [2000, 30000, 300000, 7]
    ut = np.concatenate([np.full(k, t, np.int32) for t, k in enumerate(per_table)])
    ur = np.concatenate([rng.choice(specs[t][2], size=k, replace=False) for t, k in enumerate(per_table)]).astype(np.int64)
    order = rng.permutation(len(ut))
    ut, ur = ut[order], ur[order]
    uo = np.concatenate([[0], np.cumsum([rbs[t] for t in ut])]).astype(np.int64)
    uw = torch.randint(0, 255, (int(uo[-1]),), dtype=torch.uint8, device="cuda")
    ops.emb_inplace_update(dev, torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(4, np.int32)), cu(offs), cu(tys),
                           cu(np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)), uw, cu(ut), cu(ur),
                           cu(uo), 16)
    touched = torch.zeros_like(dev, dtype=torch.bool)
    for t, rb in enumerate(rbs):
        sel = np.nonzero(ut == t)[0]
        view = dev[int(offs[t]):int(offs[t]) + sizes[t]].view(-1, rb)
        src = torch.stack([uw[int(uo[i]):int(uo[i]) + rb] for i in sel[:200]])  # a sample row by row …
        assert torch.equal(view[cu(ur[sel[:200]])], src)
        # … and all of them through one gather of the source bytes
        pos = cu(uo[sel])[:, None] + torch.arange(rb, device="cuda")[None, :]
        assert torch.equal(view[cu(ur[sel])], uw[pos])
        touched[int(offs[t]):int(offs[t]) + sizes[t]].view(-1, rb)[cu(ur[sel])] = True
    assert torch.equal(dev[~touched], before[~touched])


def test_rejected_and_skipped_updates(ops, oracle):
    rng = np.random.default_rng(2)
    c = make_case(rng, T=3)
    good = oracle_update(oracle, c)
    # a pruned row (-1) is skipped silently
    c2 = dict(c, ur=np.concatenate([c["ur"], [-1]]).astype(np.int64), ut=np.concatenate([c["ut"], [0]]).astype(np.int32),
              uo=np.concatenate([c["uo"], [0]]).astype(np.int64))
    got = gpu_update(ops, c2)
    assert (got[0] == good[0]).all() and (got[1] == good[1]).all()
    # a row past its table, a table that does not exist, an update that reads past update_weights: skipped, reported
    for bad_t, bad_r, bad_o, msg in [(0, c["rows"][0], 0, "does not exist"), (0, -2, 0, "does not exist"),
                                     (3, 0, 0, "does not exist"), (-1, 0, 0, "does not exist"),
                                     (1, 0, len(c["uw"]) - 1, "past the end")]:
        c3 = dict(c, ur=np.concatenate([c["ur"], [bad_r]]).astype(np.int64),
                  ut=np.concatenate([c["ut"], [bad_t]]).astype(np.int32), uo=np.concatenate([c["uo"][:-1], [bad_o]]).astype(np.int64))
        with pytest.raises(RuntimeError, match=msg):
            gpu_update(ops, c3)
        st = ops.Status()
        got = gpu_update(ops, c3, status=st)
        bits, pos = st.read()
        assert bits == (2 if "past" in msg else 1) and (pos == len(c["ur"]) or "past" in msg)
        assert (got[0] == good[0]).all() and (got[1] == good[1]).all()
    # nothing to do
    c4 = dict(c, ur=c["ur"][:0], ut=c["ut"][:0], uo=c["uo"][:1], uw=c["uw"][:0])
    got = gpu_update(ops, c4)
    assert (got[0] == c["bufs"][0]).all() and (got[1] == c["bufs"][1]).all()
    with pytest.raises(ValueError, match="no CPU path"):
        ops.emb_inplace_update(torch.zeros(4, dtype=torch.uint8), torch.zeros(0, dtype=torch.uint8), None, None, None, None,
                               torch.zeros(4, dtype=torch.uint8), torch.zeros(1, dtype=torch.int32),
                               torch.zeros(1, dtype=torch.int64), torch.zeros(2, dtype=torch.int64))


@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
@pytest.mark.parametrize("remap_dt", [np.int32, np.int64])
def test_from_row_idx_matches_oracle(ops, oracle, idx_dt, remap_dt):
    rng = np.random.default_rng(21)
    for n in (0, 1, 63, 1000, 300000):
        T = int(rng.integers(1, 9))
        caps = [int(rng.integers(5, 5000)) if rng.uniform() < 0.7 else 0 for _ in range(T)]
        ro = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
        remap = np.concatenate([np.where(rng.uniform(size=c) < 0.5, -1, rng.integers(0, 1000, size=c)) for c in caps]
                               + [np.zeros(0)]).astype(remap_dt)
        tables = rng.integers(0, T, size=n).astype(np.int32)
        hi = np.array([caps[t] if caps[t] else 1000 for t in tables], dtype=np.int64).reshape(n)
        rows = (rng.integers(0, 1 << 30, size=n) % np.maximum(hi, 1)).astype(idx_dt)
        want = oracle.pruned_array_lookup_from_row_idx(rows, tables, remap, ro)
        got = ops.pruned_array_lookup_from_row_idx(cu(rows), cu(tables), cu(remap), cu(ro))
        assert got.dtype == cu(rows).dtype and (got.cpu().numpy() == want).all()
    # outside the mapping / outside the tables: -1 instead of the reference's out-of-bounds read
    got = ops.pruned_array_lookup_from_row_idx(cu(np.array([5, -3, 2, 2], idx_dt)), cu(np.array([0, 0, 7, -1], np.int32)),
                                               cu(np.arange(5).astype(remap_dt)), cu(np.array([0, 5], np.int64)))
    assert got.tolist() == [-1, -1, -1, -1]


def test_torch_operators(ops, oracle):
    import os
    lib = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fbgemm_amd", "lib", "libfbgemm_amd_torch.so")
    assert os.path.exists(lib), "build it with `python -m fbgemm_amd.build`"
    torch.ops.load_library(lib)
    rng = np.random.default_rng(77)
    c = make_case(rng, T=4)
    want = oracle_update(oracle, c)
    bufs = [cu(b.copy()) for b in c["bufs"]]
    torch.ops.fbgemm.emb_inplace_update(bufs[0], bufs[1], cu(c["places"]), cu(c["offs"]), cu(c["tys"]), cu(c["D_offsets"]),
                                        cu(c["uw"]), cu(c["ut"]), cu(c["ur"]), cu(c["uo"]), 16)
    assert (bufs[0].cpu().numpy() == want[0]).all() and (bufs[1].cpu().numpy() == want[1]).all()
    assert torch.ops.fbgemm_amd.lookup_status(bufs[0]) == 0
    rows, tables = np.array([3, 0, 4], np.int64), np.array([0, 1, 0], np.int32)
    remap, ro = np.array([0, -1, 1, 2, -1], np.int32), np.array([0, 5, 5], np.int64)
    got = torch.ops.fbgemm.pruned_array_lookup_from_row_idx(cu(rows), cu(tables), cu(remap), cu(ro))
    assert got.tolist() == [2, 0, -1] == oracle.pruned_array_lookup_from_row_idx(rows, tables, remap, ro).tolist()


@pytest.mark.parametrize("weights_ty", ["FP32", "FP16", "INT8", "INT4", "INT2"])
@pytest.mark.parametrize("internal", [False, True])
def test_module_inplace_update(M, weights_ty, internal):
    """split_embeddings_test.py:271-415: rows of one module copied into another, by scatter_ (the open
    source path) and by the operator; the updated rows of both then agree, and so do their forwards."""
    seed = sum(map(ord, weights_ty)) + int(internal)
    rng = np.random.default_rng(seed)
    random.seed(seed)
    S, L = M.SparseType, M.EmbeddingLocation
    ty = getattr(S, weights_ty)
    T = int(rng.integers(1, 6))
    Ds = [int(-(-rng.integers(8, 128) // 8) * 8) for _ in range(T)]
    Es = [int(rng.integers(50, 2000)) for _ in range(T)]
    locs = [L.DEVICE if rng.uniform() < 0.7 else L.MANAGED for _ in range(T)]
    specs = [("", E, D, ty, loc) for E, D, loc in zip(Es, Ds, locs)]
    op = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, output_dtype=S.FP16, bounds_check_mode=M.BoundsCheckMode.NONE)
    op.fill_random_weights()
    op_ref = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, output_dtype=S.FP16, bounds_check_mode=M.BoundsCheckMode.NONE)
    op_ref.fill_random_weights()
    before = [w.clone() for w, _ in op.split_embedding_weights(split_scale_shifts=False)]
    ref_rows = [w for w, _ in op_ref.split_embedding_weights(split_scale_shifts=False)]
    tables, rows, weights, tables2, rows2, flat = [], [], [], [], [], []
    for t in range(T):
        n = int(rng.integers(0, 40))
        if n == 0:
            continue
        r = random.sample(range(Es[t]), n)
        tables.append(t), rows.append(r), weights.append(ref_rows[t][cu(np.array(r))])
        tables2 += [t] * n
        rows2 += r
        flat.append(weights[-1].reshape(-1))
    if internal:
        op.embedding_inplace_update_internal(tables2, rows2, torch.cat(flat) if flat else torch.zeros(0, dtype=torch.uint8, device="cuda"))
    else:
        op.embedding_inplace_update(tables, rows, weights)
    after = [w for w, _ in op.split_embedding_weights(split_scale_shifts=False)]
    for t in range(T):
        assert after[t].shape == ref_rows[t].shape
        mask = torch.zeros(Es[t], dtype=torch.bool, device="cuda")
        if t in tables:
            r = cu(np.array(rows[tables.index(t)]))
            assert torch.equal(after[t][r], ref_rows[t][r])
            mask[r] = True
        assert torch.equal(after[t][~mask], before[t][~mask])
    # lookups of updated rows only: both modules pool the same bytes
    if tables2:
        B = 4
        idx, off = [], [0]
        for t in range(T):
            pool = rows[tables.index(t)] if t in tables else []
            for _ in range(B):
                k = int(rng.integers(0, 6)) if pool else 0
                idx += [pool[i] for i in rng.integers(0, len(pool), size=k)] if k else []
                off.append(len(idx))
        idx_t, off_t = cu(np.array(idx, np.int32)), cu(np.array(off, np.int32))
        a, b = op(idx_t, off_t), op_ref(idx_t, off_t)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_module_inplace_update_through_pruning_arrays(M):
    """Logical rows go through the module's remap arrays; updates of pruned rows are dropped."""
    rng = np.random.default_rng(91)
    S, L = M.SparseType, M.EmbeddingLocation.DEVICE
    logical = [300, 200, 150]
    maps = []
    for n in logical[:2]:
        keep = rng.uniform(size=n) < 0.6
        m = np.full(n, -1, np.int32)
        m[keep] = np.arange(int(keep.sum()), dtype=np.int32)
        maps.append(m)
    specs = [("", int((maps[0] >= 0).sum()), 32, S.INT4, L), ("", int((maps[1] >= 0).sum()), 64, S.INT8, L), ("", logical[2], 16, S.FP16, L)]
    op = M.IntNBitTableBatchedEmbeddingBagsCodegen(specs, output_dtype=S.FP32, bounds_check_mode=M.BoundsCheckMode.NONE,
                                                  index_remapping=[torch.from_numpy(maps[0]), torch.from_numpy(maps[1]), None])
    op.fill_random_weights()
    before = [w.clone() for w, _ in op.split_embedding_weights(split_scale_shifts=False)]
    tables, rows = [], []
    for t in range(3):
        r = rng.choice(logical[t], size=40, replace=False)
        tables += [t] * 40
        rows += [int(x) for x in r]
    rbs = [before[t].shape[1] for t in tables]
    uw = torch.randint(0, 255, (sum(rbs),), dtype=torch.uint8, device="cuda")
    op.embedding_inplace_update_internal(tables, rows, uw)
    after = [w for w, _ in op.split_embedding_weights(split_scale_shifts=False)]
    want = [b.clone() for b in before]
    o = 0
    for t, r, rb in zip(tables, rows, rbs):
        phys = int(maps[t][r]) if t < 2 else r
        if phys >= 0:
            want[t][phys] = uw[o:o + rb]
        o += rb
    for t in range(3):
        assert torch.equal(after[t], want[t])
