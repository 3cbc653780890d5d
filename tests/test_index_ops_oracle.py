"""Pins oracle/index_ops_oracle.c (bounds_check_indices, pruned hash map) without
the GPU: the properties the reference's own test asserts
(fbgemm_gpu/test/tbe/utils/split_embeddings_utils_test.py:237-465, :476-560),
the closed form of the repaired offsets, MurmurHash3's published finalizer
values, and a Python dict as the model of the map."""
import numpy as np
import pytest

import oracle

FATAL, WARNING, IGNORE = oracle.BOUNDS_FATAL, oracle.BOUNDS_WARNING, oracle.BOUNDS_IGNORE


def make_problem(rng, T, B, max_L, dt):
    rows = rng.integers(1, 1000, size=T).astype(np.int64)
    Ls = rng.integers(0, max_L, size=T * B)
    off = np.concatenate([[0], np.cumsum(Ls)]).astype(dt)
    idx = np.concatenate([rng.integers(0, rows[t], size=int(Ls[t * B:(t + 1) * B].sum())) for t in range(T)]
                         + [np.zeros(0, np.int64)]).astype(dt)
    return rows, idx, off


@pytest.mark.parametrize("mode", [FATAL, WARNING, IGNORE])
@pytest.mark.parametrize("dt", [np.int32, np.int64])
def test_reference_test_properties(mode, dt):
    rng = np.random.default_rng(11)
    for _ in range(20):
        T, B, max_L = int(rng.integers(1, 20)), int(rng.integers(1, 20)), int(rng.integers(1, 30))
        rows, idx, off = make_problem(rng, T, B, max_L, dt)
        warning = np.zeros(1, np.int64)
        # in bounds: nothing is modified
        i2, o2 = idx.copy(), off.copy()
        assert oracle.bounds_check_indices(rows, i2, o2, mode, warning) == 0
        assert (i2 == idx).all() and (o2 == off).all() and warning[0] == 0
        # every index out of range: zeroed and counted one by one
        i2[:] = np.iinfo(dt).max
        rc = oracle.bounds_check_indices(rows, i2, o2, mode, warning)
        if mode == FATAL:
            assert (rc != 0) == (idx.size > 0)
        else:
            assert rc == 0 and (i2 == 0).all()
            if mode == WARNING:
                assert warning[0] == idx.size
        # offsets[0] = -100, offsets[-1] += 100
        i2, o2 = idx.copy(), off.copy()
        o2[0] = -100
        o2[-1] += 100
        rc = oracle.bounds_check_indices(rows, i2, o2, mode, warning)
        if mode == FATAL:
            assert rc != 0
        else:
            assert o2[0] == 0 and o2[-1] == idx.size
            if mode == WARNING:
                assert warning[0] >= min(2, o2.size - 1)


@pytest.mark.parametrize("mode", [WARNING, IGNORE])
def test_repaired_offsets_are_the_running_maximum_of_the_clamped_offsets(mode):
    rng = np.random.default_rng(12)
    for trial in range(200):
        T, B = int(rng.integers(1, 5)), int(rng.integers(1, 8))
        n = int(rng.integers(0, 40))
        off = rng.integers(-10, n + 10, size=T * B + 1).astype(np.int64)
        if trial % 3 == 0:
            off = np.sort(off)
        idx = rng.integers(-3, 60, size=n).astype(np.int64)
        rows = rng.integers(1, 50, size=T).astype(np.int64)
        want_off = off.copy()
        want_off[-1] = n
        want_off = np.maximum.accumulate(np.clip(want_off, 0, n))
        i2, o2, warning = idx.copy(), off.copy(), np.zeros(1, np.int64)
        assert oracle.bounds_check_indices(rows, i2, o2, mode, warning) == 0
        assert (o2 == want_off).all(), (off, o2, want_off)
        # indices: inside the repaired bags, anything but -1 outside [0, rows) becomes 0
        want_idx, bad_idx = idx.copy(), 0
        for bag in range(T * B):
            t = bag // B
            for i in range(want_off[bag], want_off[bag + 1]):
                if idx[i] != -1 and (idx[i] < 0 or idx[i] >= rows[t]):
                    want_idx[i] = 0
                    bad_idx += 1
        assert (i2 == want_idx).all()
        if mode == WARNING:
            # bad bags, judged on what the loop has repaired so far
            bad_bags = int(off[-1] != n)
            cur = off.copy()
            cur[-1] = n
            for bag in range(T * B):
                s, e = cur[bag], cur[bag + 1]
                if s < 0 or s > e or e > n:
                    bad_bags += 1
                    s = max(0, min(s, n))
                    e = max(s, min(e, n))
                    cur[bag], cur[bag + 1] = s, e
            assert warning[0] == bad_bags + bad_idx


def test_variable_batch_sizes():
    rng = np.random.default_rng(13)
    Bs = [3, 1, 5]
    B_offsets = np.concatenate([[0], np.cumsum(Bs)]).astype(np.int32)
    rows = np.array([10, 20, 5], np.int64)
    Ls = rng.integers(0, 6, size=sum(Bs))
    off = np.concatenate([[0], np.cumsum(Ls)]).astype(np.int64)
    idx = np.full(int(off[-1]), 7, np.int64)  # valid for tables 0 and 1 only
    warning = np.zeros(1, np.int64)
    assert oracle.bounds_check_indices(rows, idx, off, WARNING, warning, B_offsets) == 0
    n_t2 = int(off[B_offsets[3]] - off[B_offsets[2]])
    assert warning[0] == n_t2 and (idx[off[B_offsets[2]]:] == 0).all() and (idx[:off[B_offsets[2]]] == 7).all()


def test_murmur3_finalizers_known_answers():
    # fmix32 / fmix64 of MurmurHash3 (public domain, Austin Appleby): values
    # computed from the published definition in exact integer arithmetic
    def fmix32(h):
        h ^= h >> 16; h = (h * 0x85EBCA6B) & 0xFFFFFFFF
        h ^= h >> 13; h = (h * 0xC2B2AE35) & 0xFFFFFFFF
        return h ^ (h >> 16)

    def fmix64(k):
        k ^= k >> 33; k = (k * 0xFF51AFD7ED558CCD) & (2**64 - 1)
        k ^= k >> 33; k = (k * 0xC4CEB9FE1A85EC53) & (2**64 - 1)
        return k ^ (k >> 33)

    assert oracle.pruned_hash(0, 32) == 0 and oracle.pruned_hash(0, 64) == 0
    assert oracle.pruned_hash(1, 32) == 0x514E28B7  # fmix32(1), a widely quoted value
    assert oracle.pruned_hash(1, 64) == 0xB456BCFC34C2CB2C  # fmix64(1)
    rng = np.random.default_rng(14)
    for x in rng.integers(0, 2**32, size=200):
        assert oracle.pruned_hash(int(x), 32) == fmix32(int(x))
    for x in rng.integers(0, 2**63, size=200):
        assert oracle.pruned_hash(int(x), 64) == fmix64(int(x))


@pytest.mark.parametrize("dt,hdt", [(np.int32, np.int32), (np.int32, np.int64), (np.int64, np.int64), (np.int64, np.int32)])
def test_hashmap_against_a_dict(dt, hdt):
    rng = np.random.default_rng(15)
    T, B, L = 4, 6, 5
    original_E = 2000
    caps = [int(B * L / 0.8) + 1, 0, B * L, int(B * L / 0.5)]  # table 1 has no map, table 2 is exactly full
    hto = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    table = np.full((int(hto[-1]), 2), -1, hdt)
    idx = np.concatenate([rng.choice(original_E, size=B * L, replace=False) for _ in range(T)]).astype(dt)
    dense = rng.integers(0, 1000, size=T * B * L).astype(dt)
    dense[rng.random(dense.size) < 0.3] = -1  # pruned: not inserted
    off = (np.arange(T * B + 1) * L).astype(dt)
    oracle.pruned_hashmap_insert(idx, dense, off, table, hto)
    model = [dict() for _ in range(T)]
    for t in range(T):
        for i in range(t * B * L, (t + 1) * B * L):
            if dense[i] != -1:
                model[t][int(idx[i])] = int(dense[i])
    # every slot that is used holds a pair of the model; nothing else was written
    for t in range(T):
        if caps[t] == 0:
            continue
        seg = table[hto[t]:hto[t + 1]]
        used = seg[seg[:, 0] != -1]
        assert len(used) == len(model[t]) and all(model[t][int(k)] == int(v) for k, v in used)
    # look up present and absent keys
    q = np.concatenate([rng.integers(0, original_E, size=B * L) for _ in range(T)]).astype(dt)
    q[::2] = idx[::2]
    got = oracle.pruned_hashmap_lookup(q, off, table, hto)
    for t in range(T):
        for i in range(t * B * L, (t + 1) * B * L):
            want = int(q[i]) if caps[t] == 0 else model[t].get(int(q[i]), -1)
            assert got[i] == want


def test_hashmap_probe_wraps_and_handles_collisions():
    # capacity 3: many keys share a first slot and the probe wraps round the end
    for bits, dt in ((32, np.int32), (64, np.int64)):
        cap = 3
        keys = []
        k = 0
        while len(keys) < 3:
            if oracle.pruned_hash(k, bits) % cap == 2:
                keys.append(k)
            k += 1
        table = np.full((cap, 2), -1, dt)
        idx = np.array(keys, dt)
        dense = np.array([10, 20, 30], dt)
        off = np.array([0, 3], dt)
        oracle.pruned_hashmap_insert(idx, dense, off, table, np.array([0, cap], np.int64))
        assert (table[2] == [keys[0], 10]).all() and (table[0] == [keys[1], 20]).all() and (table[1] == [keys[2], 30]).all()
        got = oracle.pruned_hashmap_lookup(np.array(keys + [k + 1], dt), np.array([0, 4], dt), table, np.array([0, cap], np.int64))
        assert list(got) == [10, 20, 30, -1]  # the absent key ends after one trip round the full table


@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("hdt", [np.int32, np.int64])
def test_library_host_insert_builds_the_oracles_table(idt, hdt):
    """fbgemm_amd_pruned_hashmap_insert_host is host code (the reference builds the
    map on the CPU as well): its table equals the oracle's, slot for slot."""
    import ctypes as C

    from fbgemm_amd import _lib
    rng = np.random.default_rng(31)
    T = 4
    ns = [0, 57, 300, 1]
    caps = [0 if n == 0 else int(n / 0.5) + 3 for n in ns]
    hto = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    keys = np.concatenate([rng.choice(10 ** 6, size=n, replace=False) for n in ns]).astype(idt)
    dense = np.concatenate([np.arange(n) for n in ns]).astype(idt)
    dense[rng.random(len(dense)) < 0.2] = -1  # pruned rows are not inserted
    off = np.concatenate([[0], np.cumsum(ns)]).astype(idt)
    want = np.full((int(hto[-1]), 2), -1, hdt)
    oracle.pruned_hashmap_insert(keys, dense, off, want, hto)
    got = np.full((int(hto[-1]), 2), -1, hdt)
    p = lambda a: C.c_void_p(a.ctypes.data)
    rc = _lib.lib().fbgemm_amd_pruned_hashmap_insert_host(
        p(keys), p(dense), p(off), 8 * keys.itemsize, len(off), p(got), 8 * got.itemsize, p(hto), T)
    assert rc == 0 and (got == want).all()
    # a full table is refused instead of probing for ever
    tiny = np.full((2, 2), -1, hdt)
    k3, o3, h3 = np.arange(3, dtype=idt), np.asarray([0, 3], idt), np.asarray([0, 2], np.int64)
    rc = _lib.lib().fbgemm_amd_pruned_hashmap_insert_host(
        p(k3), p(k3), p(o3), 8 * k3.itemsize, 2, p(tiny), 8 * tiny.itemsize, p(h3), 1)
    assert rc < 0


@pytest.mark.parametrize("idx_dtype,remap_dtype", [(np.int32, np.int32), (np.int64, np.int32), (np.int64, np.int64), (np.int32, np.int64)])
def test_pruned_array_lookup_is_numpy_indexing(oracle, idx_dtype, remap_dtype):
    """oracle.pruned_array_lookup against its definition in numpy (embedding_forward_quantized_cpu_template.cpp:605-659):
    dense[i] = remap[remap_offsets[t] + indices[i]] for the positions of a table that owns a mapping, a copy
    for a table whose slice of the mapping array is empty (capacity 0: the table is not pruned)."""
    rng = np.random.default_rng(31)
    T, B = 5, 7
    caps = [40, 0, 25, 0, 60]  # tables 1 and 3 are not pruned
    remap_offsets = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    remap = np.concatenate([np.where(rng.random(c) < 0.4, -1, rng.integers(0, 1000, size=c)) for c in caps]).astype(remap_dtype)
    lens = rng.integers(0, 9, size=T * B)
    offsets = np.concatenate([[0], np.cumsum(lens)]).astype(idx_dtype)
    indices = np.concatenate([rng.integers(0, caps[t] if caps[t] else 500, size=int(lens[t * B:(t + 1) * B].sum()))
                              for t in range(T)]).astype(idx_dtype)
    got = oracle.pruned_array_lookup(indices, offsets, remap, remap_offsets)
    want = indices.copy()
    for t in range(T):
        s, e = int(offsets[t * B]), int(offsets[(t + 1) * B])
        if caps[t]:
            want[s:e] = remap[remap_offsets[t] + indices[s:e]].astype(idx_dtype)
    assert got.dtype == indices.dtype and (got == want).all()
    # every table unpruned: the identity
    none = oracle.pruned_array_lookup(indices, offsets, np.zeros(0, remap_dtype), np.zeros(T + 1, np.int64))
    assert (none == indices).all()
