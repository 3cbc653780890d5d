"""Pins the oracle's in-place row update (emb_inplace_update,
fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update_cpu.cpp:25-70) and
pruned_array_lookup_from_row_idx (:199-251) against formulations that share no
code with it: numpy fancy assignment on per-table row views, the row sizes the
reference tabulates (embedding_common.h:189-225), and the checks of the
reference's own test (embedding_inplace_update_test.cpp: every updated row
equals its source bytes), on that test's shapes (2-4 tables of random type,
D = 2..32, 10-59 rows, either weights buffer)."""
import numpy as np
import pytest

TYS = [0, 1, 2, 3, 4]  # FP32, FP16, INT8, INT4, INT2


def known_row_bytes(D, ty, align):
    data = {0: 4 * D, 1: 2 * D, 2: D + 4, 3: D // 2 + 4, 4: D // 4 + 4}[ty]
    return (data + align - 1) // align * align


def make_case(rng, T=None, align=16, idx_dt=np.int64, duplicates=False):
    T = T or int(rng.integers(2, 5))
    tys, Ds, rows, places, offs = [], [], [], [], []
    size = [0, 0]
    for _ in range(T):
        ty = int(rng.choice(TYS))
        D = 1 << int(rng.integers(2 if ty == 4 else 1, 6))
        n = int(rng.integers(10, 60))
        p = int(rng.integers(0, 2))
        tys.append(ty), Ds.append(D), rows.append(n), places.append(p), offs.append(size[p])
        size[p] += known_row_bytes(D, ty, align) * n
    bufs = [rng.integers(0, 255, size=size[0], dtype=np.uint8), rng.integers(0, 255, size=size[1], dtype=np.uint8)]
    ut, ur = [], []
    for t in range(T):
        k = int(rng.integers(5, 15))
        r = rng.integers(0, rows[t], size=k) if duplicates else rng.choice(rows[t], size=min(k, rows[t]), replace=False)
        ut += [t] * len(r)
        ur += list(r)
    order = rng.permutation(len(ut))
    ut, ur = np.array(ut, np.int32)[order], np.array(ur, idx_dt)[order]
    sizes = [known_row_bytes(Ds[t], tys[t], align) for t in ut]
    uo = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    uw = rng.integers(0, 255, size=int(uo[-1]), dtype=np.uint8)
    return dict(T=T, tys=np.array(tys, np.uint8), D_offsets=np.concatenate([[0], np.cumsum(Ds)]).astype(np.int32), rows=rows,
                places=np.array(places, np.int32), offs=np.array(offs, np.int64), bufs=bufs, ut=ut, ur=ur, uo=uo, uw=uw,
                align=align, Ds=Ds)


def numpy_update(c):
    """Row views + fancy assignment, update by update."""
    bufs = [b.copy() for b in c["bufs"]]
    for i in range(len(c["ut"])):
        t = int(c["ut"][i])
        rb = known_row_bytes(c["Ds"][t], int(c["tys"][t]), c["align"])
        view = bufs[c["places"][t]][c["offs"][t]:c["offs"][t] + rb * c["rows"][t]].reshape(c["rows"][t], rb)
        view[int(c["ur"][i])] = c["uw"][c["uo"][i]:c["uo"][i] + rb]
    return bufs


def run_oracle(oracle, c):
    bufs = [b.copy() for b in c["bufs"]]
    oracle.emb_inplace_update(bufs[0], bufs[1], c["places"], c["offs"], c["tys"], c["D_offsets"], c["uw"], c["ut"], c["ur"],
                              c["uo"], c["align"])
    return bufs


def test_row_sizes_are_the_reference_table(oracle):
    # embedding_common.h:189-225 and the constants of embedding_inplace_update_test.cpp (alignment 16)
    assert oracle.padded_row_bytes(2, 0, 16) == 16 and oracle.padded_row_bytes(32, 3, 16) == 32
    assert oracle.padded_row_bytes(8, 4, 1) == 6 and oracle.padded_row_bytes(16, 2, 16) == 32
    for ty in TYS:
        for D in (4, 8, 16, 32, 128):
            for a in (1, 16):
                assert oracle.padded_row_bytes(D, ty, a) == known_row_bytes(D, ty, a)


@pytest.mark.parametrize("align", [16, 1])
@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
def test_update_matches_row_view_assignment(oracle, align, idx_dt):
    rng = np.random.default_rng(5 + align)
    for _ in range(40):
        c = make_case(rng, align=align, idx_dt=idx_dt)
        got, want = run_oracle(oracle, c), numpy_update(c)
        assert (got[0] == want[0]).all() and (got[1] == want[1]).all()
        # the reference test's check: every updated row holds its source bytes; everything else is untouched
        touched = [np.zeros(len(b), bool) for b in got]
        for i in range(len(c["ut"])):
            t = int(c["ut"][i])
            rb = known_row_bytes(c["Ds"][t], int(c["tys"][t]), align)
            lo = int(c["offs"][t]) + rb * int(c["ur"][i])
            assert (got[c["places"][t]][lo:lo + rb] == c["uw"][c["uo"][i]:c["uo"][i] + rb]).all()
            touched[c["places"][t]][lo:lo + rb] = True
        for p in range(2):
            assert (got[p][~touched[p]] == c["bufs"][p][~touched[p]]).all()


def test_duplicate_rows_last_update_wins(oracle):
    rng = np.random.default_rng(3)
    for _ in range(20):
        c = make_case(rng, duplicates=True)
        got, want = run_oracle(oracle, c), numpy_update(c)
        assert (got[0] == want[0]).all() and (got[1] == want[1]).all()
    # two updates of one row, by hand
    c = make_case(rng, T=2)
    c["ut"] = np.array([0, 0], np.int32)
    c["ur"] = np.array([3, 3], np.int64)
    rb = known_row_bytes(c["Ds"][0], int(c["tys"][0]), 16)
    c["uo"] = np.array([0, rb, 2 * rb], np.int64)
    c["uw"] = np.concatenate([np.full(rb, 7, np.uint8), np.full(rb, 9, np.uint8)])
    got = run_oracle(oracle, c)
    lo = int(c["offs"][0]) + 3 * rb
    assert (got[c["places"][0]][lo:lo + rb] == 9).all()


def test_no_updates_changes_nothing(oracle):
    c = make_case(np.random.default_rng(1))
    c["ut"], c["ur"], c["uo"], c["uw"] = c["ut"][:0], c["ur"][:0], c["uo"][:1], c["uw"][:0]
    got = run_oracle(oracle, c)
    assert (got[0] == c["bufs"][0]).all() and (got[1] == c["bufs"][1]).all()


@pytest.mark.parametrize("idx_dt", [np.int32, np.int64])
@pytest.mark.parametrize("remap_dt", [np.int32, np.int64])
def test_from_row_idx_matches_numpy(oracle, idx_dt, remap_dt):
    rng = np.random.default_rng(11)
    for _ in range(20):
        T = int(rng.integers(1, 6))
        caps = [int(rng.integers(5, 50)) if rng.uniform() < 0.7 else 0 for _ in range(T)]
        ro = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
        remap = np.concatenate([np.where(rng.uniform(size=c) < 0.5, -1, rng.integers(0, 1000, size=c)) for c in caps] + [np.zeros(0)]).astype(remap_dt)
        n = int(rng.integers(0, 200))
        tables = rng.integers(0, T, size=n).astype(np.int32)
        rows = np.array([rng.integers(0, caps[t]) if caps[t] else rng.integers(0, 1000) for t in tables], dtype=idx_dt).reshape(n)
        want = np.array([remap[ro[t] + r] if caps[t] else r for t, r in zip(tables, rows)], dtype=idx_dt).reshape(n)
        got = oracle.pruned_array_lookup_from_row_idx(rows, tables, remap, ro)
        assert got.dtype == idx_dt and (got == want).all()
