"""Pins the oracle's embedding_bag_rowwise_prune without the GPU: the compaction
against torch._rowwise_prune (the ATen routine the reference's operator ends in),
the keep rule against the closed form it has (a prefix count plus a forced
suffix), and both against brute force on short inputs."""
import itertools

import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")


def closed_form_mask(ind, threshold, use_abs, min_rows):
    n = len(ind)
    v = np.abs(ind) if use_abs else ind
    nat = v.astype(np.float64) > threshold
    before = np.concatenate([[0], np.cumsum(nat)[:-1]]) if n else np.zeros(0, dtype=np.int64)
    forced = before + (n - np.arange(n)) <= min_rows
    return nat | forced


@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
def test_matches_aten_rowwise_prune(idx_dt):
    rng = np.random.default_rng(1)
    for rows, cols, min_rows, use_abs in [(50, 8, 0, True), (1000, 3, 0, False), (200, 16, 150, True), (64, 1, 64, True),
                                          (64, 4, 100, True), (1, 5, 0, True), (300, 2, 299, False)]:
        w = rng.normal(size=(rows, cols)).astype(np.float32)
        ind = rng.normal(size=rows).astype(np.float32)
        thr = 0.7
        kept, remap = oracle.rowwise_prune(w, ind, thr, idx_dt, use_abs, min_rows)
        mask = closed_form_mask(ind, thr, use_abs, min_rows)
        tw, tr = torch._rowwise_prune(torch.from_numpy(w), torch.from_numpy(mask), torch.int32 if idx_dt == np.int32 else torch.int64)
        assert remap.dtype == idx_dt and (remap == tr.numpy()).all()
        assert kept.shape == tuple(tw.shape) and (kept.view(np.uint32) == tw.numpy().view(np.uint32)).all()
        assert len(kept) >= min(min_rows, rows)


def test_keep_rule_by_brute_force():
    # every pattern of 8 indicators above / below the threshold, every minimum
    for bits in itertools.product([0.0, 1.0], repeat=8):
        ind = np.array(bits, dtype=np.float32)
        for min_rows in range(0, 11):
            _, remap = oracle.rowwise_prune(np.zeros((8, 1), np.float32), ind, 0.5, np.int32, True, min_rows)
            # the reference's loop, in Python
            kept, want = 0, []
            for i in range(8):
                keep = ind[i] > 0.5
                if kept < min_rows and kept + (8 - i) <= min_rows:
                    keep = True
                want.append(kept if keep else -1)
                kept += bool(keep)
            assert remap.tolist() == want
            assert ((remap >= 0) == closed_form_mask(ind, 0.5, True, min_rows)).all()


def test_threshold_is_compared_in_double_and_abs_is_optional():
    ind = np.array([0.1, -0.9, np.float32(0.7), 0.70000005], dtype=np.float32)
    # float32(0.7) = 0.699999988... is not above the double 0.7
    _, remap = oracle.rowwise_prune(np.zeros((4, 1), np.float32), ind, 0.7, np.int64, True, 0)
    assert remap.tolist() == [-1, 0, -1, 1]
    _, remap = oracle.rowwise_prune(np.zeros((4, 1), np.float32), ind, 0.7, np.int64, False, 0)
    assert remap.tolist() == [-1, -1, -1, 0]
