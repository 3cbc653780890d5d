"""GPU parity of the compacting pruned-row remap (fbgemm::compressed_indices_remap,
src/RefImplementations.cc:2308-2333) through the C ABI, against the oracle: indices,
offsets and weights bit for bit, after test/EmbeddingSpMDMTest.cc:1040-1192 (half
of the rows pruned)."""
import numpy as np
import pytest

import helpers as H

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_mapping(rng, rows, sparsity):
    keep = rng.uniform(size=rows) >= sparsity
    mapping = np.full(rows, -1, dtype=np.int32)
    mapping[keep] = np.arange(int(keep.sum()), dtype=np.int32)
    return mapping


@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
@pytest.mark.parametrize("weighted", [False, True])
def test_matches_oracle(ops, oracle, idx_dt, weighted):
    rng = np.random.default_rng(12 + int(weighted))
    for bags, rows, max_len, sparsity, first in [(10, 400, 10, 0.5, 0), (1, 50, 100, 0.5, 0), (500, 5000, 40, 0.5, 0),
                                                 (4096, 100000, 90, 0.3, 0), (64, 100, 5, 1.0, 0), (64, 100, 5, 0.0, 0),
                                                 (33, 1000, 20, 0.5, 7), (5, 10, 1, 0.5, 0), (3000, 2000, 200, 0.9, 0)]:
        mapping = make_mapping(rng, rows, sparsity)
        lens = rng.integers(0, max_len + 1, size=bags)
        off = (first + np.concatenate([[0], np.cumsum(lens)])).astype(idx_dt)
        idx = rng.integers(0, rows, size=int(off[-1])).astype(idx_dt)  # the entries before offsets[0] are never visited
        w = rng.normal(size=len(idx)).astype(np.float32) if weighted else None
        want_i, want_o, want_w = oracle.compressed_indices_remap(idx, mapping, off, w)
        got_i, got_o, got_w = ops.compressed_indices_remap(cu(idx), cu(mapping), cu(off), None if w is None else cu(w))
        n = int(want_o[-1])
        assert got_o.dtype == torch.from_numpy(off).dtype and (got_o.cpu().numpy() == want_o).all(), (bags, rows)
        assert (got_i.cpu().numpy()[:n] == want_i).all()
        if weighted:
            H.assert_same_bits(got_w.cpu().numpy()[:n], want_w, "remapped weights")
        else:
            assert got_w is None


def test_empty_and_rejected_inputs(ops):
    mapping = cu(np.array([0, -1, 1], dtype=np.int32))
    i, o, w = ops.compressed_indices_remap(cu(np.zeros(0, np.int64)), mapping, cu(np.zeros(4, np.int64)))
    assert o.tolist() == [0, 0, 0, 0] and i.numel() == 0 and w is None
    i, o, _ = ops.compressed_indices_remap(cu(np.array([2, 1, 0, 2], np.int32)), mapping, cu(np.array([0, 2, 2, 4], np.int32)))
    assert o.tolist() == [0, 1, 1, 3] and i.tolist()[:3] == [1, 0, 1]
    with pytest.raises(IndexError, match="position 1"):
        ops.compressed_indices_remap(cu(np.array([2, 3, 0], np.int32)), mapping, cu(np.array([0, 3], np.int32)))
    with pytest.raises(IndexError):
        ops.compressed_indices_remap(cu(np.array([-1], np.int64)), mapping, cu(np.array([0, 1], np.int64)))
    with pytest.raises(TypeError):
        ops.compressed_indices_remap(cu(np.array([0], np.int64)), mapping, cu(np.array([0, 1], np.int32)))
