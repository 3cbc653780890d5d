"""GPU parity of the table-batched forward and of pruned_array_lookup, through
the C ABI, against the CPU oracle. Bit-exact (tolerance 0) for fp32, fp16 and
bf16 outputs; the path's stated bound is 1e-5 relative / 1 ulp.

Cases after fbgemm_gpu/test/tbe/inference/nbit_forward_test.py: the exact-count
fixture (:577-659), an out-of-range index in one table (:661-688), mixed
types / dims / pooling / index widths (:746-815)."""
import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("lane_shape")]


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def build_weights(rng, specs, row_alignment, ones=False):
    """specs: (rows, D, ty). Returns (flat uint8 weights, weights_offsets, row_bytes)."""
    import oracle
    blobs, offs, rbs, cur = [], [], [], 0
    for rows, D, ty in specs:
        rb = oracle.padded_row_bytes(D, ty, row_alignment)
        tbl, _ = H.make_table(rng, ty, rows, D, False, stride_bytes=rb, ones=ones)
        offs.append(cur)
        rbs.append(rb)
        size = (tbl.size + 127) // 128 * 128
        blobs.append(tbl)
        blobs.append(rng.integers(0, 256, size=size - tbl.size, dtype=np.uint8))
        cur += size
    return np.concatenate(blobs), np.array(offs, np.int64), rbs


def run_both(ops, oracle, weights, wo, specs, indices, offsets, pooling, psw, out_ty, row_alignment):
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"),
        cu(np.zeros(len(specs), np.int32)), cu(wo), cu(tys), cu(D_offsets), total_D,
        maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(indices), cu(offsets),
        pooling, None if psw is None else cu(psw), out_ty, row_alignment=row_alignment)
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, indices, offsets, pooling,
                                  psw, out_ty, row_alignment)
    assert rc == 0
    g = got.cpu()
    g = g.numpy() if out_ty == FP32 else g.view(torch.int16).numpy().view(np.uint16)
    return g, want


def test_exact_count_fixture(ops, oracle):
    """Rows of ones: every output column equals the number of kept indices of
    its (table, bag); empty and fully pruned bags give exact zeros."""
    E, Ds = 100, [16, 24, 40]
    Ls = [[0, 2, 5, 0, 3, 4], [1, 0, 4, 2, 0, 6], [3, 3, 0, 1, 5, 0]]
    fully_pruned = [4, 2, 3]
    T, B = len(Ds), len(Ls[0])
    rng = np.random.default_rng(0)
    for ty in (FP16, INT8, INT4, INT2, FP32):
        specs = [(E, d, ty) for d in Ds]
        for align in (16, 1):
            weights, wo, _ = build_weights(rng, specs, align, ones=True)
            idx, off, running = [], [0], 0
            expected = np.zeros((B, sum(Ds)), np.float32)
            dpre = np.cumsum([0] + Ds)
            for t in range(T):
                for b in range(B):
                    kept = 0
                    for _ in range(Ls[t][b]):
                        prune = b == fully_pruned[t] or running % 3 == 0
                        idx.append(-1 if prune else running % E)
                        kept += 0 if prune else 1
                        running += 1
                    off.append(len(idx))
                    expected[b, dpre[t]:dpre[t + 1]] = kept
            for out_ty in (FP32, FP16, BF16):
                for dt in (np.int32, np.int64):
                    got, want = run_both(ops, oracle, weights, wo, specs, np.array(idx, dt),
                                         np.array(off, dt), 0, None, out_ty, align)
                    H.assert_same_bits(got, want, f"ty={ty} out={out_ty}")
                    if out_ty == FP32:
                        val = got
                    elif out_ty == FP16:
                        val = got.view(np.float16).astype(np.float32)
                    else:
                        val = (got.astype(np.uint32) << 16).view(np.float32)
                    assert (val == expected).all()


@pytest.mark.parametrize("seed", range(12))
def test_mixed_tables_random(ops, oracle, seed):
    rng = np.random.default_rng(500 + seed)
    T = int(rng.integers(1, 11))
    B = int(rng.integers(1, 41))
    dims = {INT8: [4, 8, 16, 32, 64, 100, 128, 256, 1024], INT4: [8, 16, 24, 32, 40, 64, 128, 160, 256, 1024],
            INT2: [16, 32, 64, 128, 256], FP16: [4, 8, 16, 64, 128, 256, 2048], FP32: [4, 8, 32, 128]}
    specs = []
    for _ in range(T):
        ty = int(rng.choice([INT8, INT4, INT2, FP16, FP32]))
        specs.append((int(rng.integers(1, 300)), int(rng.choice(dims[ty])), ty))
    align = int(rng.choice([1, 16]))
    weights, wo, _ = build_weights(rng, specs, align)
    lens = rng.integers(0, 25, size=T * B)
    lens[rng.random(T * B) < 0.1] = 0
    dt = rng.choice([np.int32, np.int64])
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum()))
                          for t in range(T)] + [np.zeros(0, np.int64)]).astype(dt)
    idx[rng.random(len(idx)) < 0.15] = -1
    for pooling in (0, 1):
        for weighted in (False, True):
            psw = rng.uniform(0, 1, size=len(idx)).astype(np.float32) if weighted else None
            for out_ty in (FP32, FP16, BF16):
                what = f"seed={seed} T={T} B={B} specs={specs} align={align} pool={pooling} w={weighted} out={out_ty}"
                print(what, flush=True)
                got, want = run_both(ops, oracle, weights, wo, specs, idx, off, pooling, psw, out_ty, align)
                H.assert_same_bits(got, want, what)


def test_out_of_range_index_raises(ops, oracle):
    rng = np.random.default_rng(9)
    E = 100
    specs = [(E, 16, INT8), (E, 32, INT8)]
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([INT8, INT8], np.uint8)
    D_offsets = np.array([0, 16, 48], np.int32)
    args = lambda idx, off: (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"),
                            cu(np.zeros(2, np.int32)), cu(wo), cu(tys), cu(D_offsets), 48, 0, 0, 32, 0, 0,
                            cu(idx), cu(off), 0, None, FP16)
    idx = np.array([0, E + 500000, 3], np.int32)
    off = np.array([0, 1, 1, 2, 3], np.int32)
    with pytest.raises(RuntimeError, match="out of bounds"):
        ops.int_nbit_split_embedding_codegen_lookup_function(*args(idx, off), row_alignment=16)
    rc, _ = oracle.tbe_forward(weights, wo, tys, D_offsets, 48, idx, off, 0, None, FP16, 16)
    assert rc == 2  # the oracle blames the second table too
    # asynchronous form: the caller reads the status block
    st = ops.Status()
    out = ops.int_nbit_split_embedding_codegen_lookup_function(*args(idx, off), row_alignment=16, status=st)
    bits, pos = st.read()
    assert bits == ops.ERR_INDEX_OUT_OF_RANGE and pos == 1
    assert torch.isfinite(out.float()).all()
    # the inferred row bound includes the table's 128-byte padding, as in the reference
    rb = oracle.padded_row_bytes(32, INT8, 16)
    bound = (len(weights) - int(wo[1])) // rb
    idx = np.array([0, bound - 1, 3], np.int32)
    ops.int_nbit_split_embedding_codegen_lookup_function(*args(idx, off), row_alignment=16)
    idx = np.array([0, bound, 3], np.int32)
    with pytest.raises(RuntimeError):
        ops.int_nbit_split_embedding_codegen_lookup_function(*args(idx, off), row_alignment=16)


@pytest.mark.parametrize("dt,rdt", [(np.int32, np.int32), (np.int64, np.int32), (np.int64, np.int64), (np.int32, np.int64)])
def test_pruned_array_lookup(ops, oracle, dt, rdt):
    rng = np.random.default_rng(3)
    T, B = 5, 17
    caps = [200, 0, 1000, 50, 0]
    remap_off = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    remap = np.full(int(remap_off[-1]), -1, rdt)
    for t in range(T):
        s, e = remap_off[t], remap_off[t + 1]
        keep = rng.random(e - s) < 0.5
        remap[s:e][keep] = np.arange(int(keep.sum()), dtype=rdt)
    lens = rng.integers(0, 12, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, caps[t] if caps[t] else 10**6, size=int(lens[t * B:(t + 1) * B].sum()))
                          for t in range(T)]).astype(dt)
    got = ops.pruned_array_lookup(cu(idx), cu(off), cu(remap), cu(remap_off)).cpu().numpy()
    want = oracle.pruned_array_lookup(idx, off, remap, remap_off)
    assert got.dtype == want.dtype and (got == want).all()


def test_config3_scaled(ops, oracle):
    """The headline workload at 1/50 scale, checked in full against the oracle."""
    from fbgemm_amd import bench_configs as bc
    p = bc.config3("cuda", scale=0.02)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        p.dev_weights, torch.zeros(0, dtype=torch.uint8, device="cuda"),
        cu(np.zeros(p.T, np.int32)), cu(p.weights_offsets), cu(p.tys), cu(p.D_offsets), p.total_D,
        0, 256, 256, 256, 0, p.indices, p.offsets, p.pooling_mode, p.indice_weights, p.output_dtype,
        row_alignment=p.row_alignment)
    rc, want = oracle.tbe_forward(p.dev_weights.cpu().numpy(), p.weights_offsets, p.tys, p.D_offsets,
                                  p.total_D, p.host_indices, p.host_offsets, p.pooling_mode,
                                  p.host_weights, p.output_dtype, p.row_alignment)
    assert rc == 0
    H.assert_same_bits(got.cpu().view(torch.int16).numpy().view(np.uint16), want, "config3 @ 0.02")


@pytest.mark.parametrize("seed", range(6))
def test_forward_with_fused_remap(ops, oracle, seed):
    """Logical ids + per-table mappings in one call == pruned_array_lookup (oracle)
    followed by the forward (oracle), bit for bit; tables with an empty mapping
    take their ids as they are; MEAN divides by the full bag length."""
    rng = np.random.default_rng(900 + seed)
    T = int(rng.integers(1, 8))
    B = int(rng.integers(1, 50))
    specs, caps = [], []
    for _ in range(T):
        ty = int(rng.choice([INT8, INT4, INT2, FP16, FP32]))
        D = int(rng.choice({INT8: [8, 64, 128], INT4: [8, 64, 128, 256], INT2: [16, 64], FP16: [8, 64, 256], FP32: [4, 32]}[ty]))
        specs.append((int(rng.integers(1, 200)), D, ty))
        caps.append(0 if rng.random() < 0.3 else int(rng.integers(1, 600)))
    align = int(rng.choice([1, 4, 16]))
    weights, wo, _ = build_weights(rng, specs, align)
    rdt = rng.choice([np.int32, np.int64])
    dt = rng.choice([np.int32, np.int64])
    remap_off = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    remap = np.full(int(remap_off[-1]), -1, rdt)
    for t in range(T):
        s, e = int(remap_off[t]), int(remap_off[t + 1])
        keep = rng.random(e - s) < 0.5
        remap[s:e][keep] = rng.integers(0, specs[t][0], size=int(keep.sum()))
    lens = rng.integers(0, 30, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, caps[t] if caps[t] else specs[t][0], size=int(lens[t * B:(t + 1) * B].sum()))
                          for t in range(T)] + [np.zeros(0, np.int64)]).astype(dt)
    dense = oracle.pruned_array_lookup(idx, off, remap, remap_off)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    for pooling in (0, 1):
        for weighted in (False, True):
            psw = rng.uniform(0, 1, size=len(idx)).astype(np.float32) if weighted else None
            for out_ty in (FP32, FP16):
                what = f"seed={seed} T={T} B={B} specs={specs} caps={caps} align={align} pool={pooling} w={weighted} out={out_ty}"
                print(what, flush=True)
                got = ops.int_nbit_split_embedding_codegen_lookup_function(
                    cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)),
                    cu(wo), cu(tys), cu(D_offsets), total_D, 0, 0, 0, 0, 0, cu(idx), cu(off), pooling,
                    None if psw is None else cu(psw), out_ty, row_alignment=align,
                    index_remappings=cu(remap), index_remappings_offsets=cu(remap_off)).cpu()
                rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, dense, off, pooling, psw, out_ty, align)
                assert rc == 0
                g = got.numpy() if out_ty == FP32 else got.view(torch.int16).numpy().view(np.uint16)
                H.assert_same_bits(g, want, what)


def test_fused_remap_rejects_ids_outside_the_mapping(ops):
    rng = np.random.default_rng(5)
    specs = [(50, 16, INT4)]
    weights, wo, _ = build_weights(rng, specs, 16)
    remap = np.arange(20, dtype=np.int32)
    args = lambda idx: (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(1, np.int32)),
                        cu(wo), cu(np.array([INT4], np.uint8)), cu(np.array([0, 16], np.int32)), 16, 0, 16, 0, 0, 0,
                        cu(idx), cu(np.array([0, len(idx)], np.int32)), 0, None, FP32)
    kw = dict(row_alignment=16, index_remappings=cu(remap), index_remappings_offsets=cu(np.array([0, 20], np.int64)))
    ops.int_nbit_split_embedding_codegen_lookup_function(*args(np.array([0, 19], np.int32)), **kw)
    with pytest.raises(RuntimeError, match="out of bounds"):
        ops.int_nbit_split_embedding_codegen_lookup_function(*args(np.array([0, 20], np.int32)), **kw)


def test_config4_batched_scaled(ops, oracle):
    """Config 4 as one table-batched call with the remap fused in, at 1/50 scale, in full."""
    from fbgemm_amd import bench_configs as bc
    p = bc.config4_batched("cuda", scale=0.02)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        p.dev_weights, torch.zeros(0, dtype=torch.uint8, device="cuda"),
        cu(np.zeros(p.T, np.int32)), cu(p.weights_offsets), cu(p.tys), cu(p.D_offsets), p.total_D,
        0, 64, 0, 0, 0, p.indices, p.offsets, p.pooling_mode, None, p.output_dtype,
        row_alignment=p.row_alignment, index_remappings=p.extra["remap"],
        index_remappings_offsets=p.extra["remap_offsets"])
    dense = oracle.pruned_array_lookup(p.host_indices, p.host_offsets, p.extra["host_remap"], p.extra["host_remap_offsets"])
    assert (dense == p.extra["host_dense"]).all()
    rc, want = oracle.tbe_forward(p.dev_weights.cpu().numpy(), p.weights_offsets, p.tys, p.D_offsets,
                                  p.total_D, dense, p.host_offsets, p.pooling_mode, None, p.output_dtype, p.row_alignment)
    assert rc == 0
    H.assert_same_bits(got.cpu().numpy(), want, "config4 batched @ 0.02")


@pytest.mark.parametrize("dt", [np.int32, np.int64])
@pytest.mark.parametrize("D", [4, 32, 56, 128, 260])
def test_no_pooling_matches_oracle(ops, oracle, dt, D):
    """PoolingMode.NONE (sequence output): every index is a bag of one
    (embedding_forward_quantized_cpu_template.cpp:390-420); after
    nbit_forward_test.py:1060-1160 (nobag equals bags of length one)."""
    rng = np.random.default_rng(900 + D)
    tys = [INT4, INT8, FP16, INT2, FP32, INT4]
    specs = [(int(rng.integers(20, 300)), D, ty) for ty in tys]
    T, B = len(specs), 13
    for row_alignment in (16, 1):
        weights, wo, _ = build_weights(rng, specs, row_alignment)
        lens = rng.integers(0, 7, size=T * B)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(dt)
        idx[rng.random(len(idx)) < 0.1] = -1
        wt = np.array(tys, np.uint8)
        D_offsets = (np.arange(T + 1) * D).astype(np.int32)
        maxd = lambda ty: D if ty in tys else 0
        for out_ty, tdt in ((FP32, torch.float32), (FP16, torch.float16), (BF16, torch.bfloat16)):
            got = ops.int_nbit_split_embedding_codegen_lookup_function(
                cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt),
                cu(D_offsets), T * D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
                ops.POOL_NONE, None, out_ty, row_alignment=row_alignment)
            assert got.dtype == tdt and tuple(got.shape) == (len(idx), D)
            ok, want = oracle.tbe_forward_nobag(weights, wo, wt, [s[0] for s in specs], D, idx, off, out_ty, row_alignment)
            assert ok
            g = got.cpu()
            g = g.numpy() if out_ty == FP32 else g.view(torch.int16).numpy().view(np.uint16)
            H.assert_same_bits(g, want, f"no pooling D={D} out={out_ty} align={row_alignment}")
        # an index past the table is reported
        if len(idx):
            bad = idx.copy()
            bad[len(bad) // 2] = 10 ** 6
            with pytest.raises(RuntimeError, match="out of bounds"):
                ops.int_nbit_split_embedding_codegen_lookup_function(
                    cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt),
                    cu(D_offsets), T * D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(bad), cu(off),
                    ops.POOL_NONE, None, FP16, row_alignment=row_alignment)


def _no_pooling_case(ops, oracle, rng, specs, B, max_len, dt, row_alignment, out_ty, tag):
    T, D = len(specs), specs[0][1]
    tys = [s[2] for s in specs]
    weights, wo, _ = build_weights(rng, specs, row_alignment)
    lens = rng.integers(0, max_len + 1, size=T * B)
    for t in range(T):
        if rng.random() < 0.15:
            lens[t * B:(t + 1) * B] = 0  # a table nobody asks for
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]
                         + [np.zeros(0, np.int64)]).astype(dt)
    idx[rng.random(len(idx)) < 0.05] = -1
    wt = np.array(tys, np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    maxd = lambda ty: D if ty in tys else 0
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt),
        cu(D_offsets), T * D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
        ops.POOL_NONE, None, out_ty, row_alignment=row_alignment)
    assert tuple(got.shape) == (len(idx), D)
    ok, want = oracle.tbe_forward_nobag(weights, wo, wt, [s[0] for s in specs], D, idx, off, out_ty, row_alignment)
    assert ok
    g = got.cpu()
    g = g.numpy() if out_ty == FP32 else g.view(torch.int16).numpy().view(np.uint16)
    H.assert_same_bits(g, want, tag)


@pytest.mark.parametrize("seed", range(12))
def test_no_pooling_random_shapes(ops, oracle, seed):
    """Random table counts, row types, widths (narrower and wider than what the lanes of a row cover in one
    pass), alignments and bag lengths: the positions a wave takes together then begin and end anywhere inside
    tables, cross table boundaries and run past the end of the index array."""
    rng = np.random.default_rng(7000 + seed)
    for _ in range(6):
        T = int(rng.integers(1, 7))
        D = int(rng.choice([8, 16, 40, 64, 100, 128, 256, 520, 1024]))
        tys = [int(rng.choice([INT4, INT8, FP16, INT2, FP32])) for _ in range(T)]
        if any(ty == INT2 for ty in tys) and D % 4:
            D += 4 - D % 4
        specs = [(int(rng.integers(1, 400)), D, ty) for ty in tys]
        B = int(rng.integers(1, 40))
        max_len = int(rng.choice([1, 3, 9, 40]))
        if T * B * max_len * D > 6_000_000:
            max_len = 3
        dt = rng.choice([np.int32, np.int64])
        align = int(rng.choice([16, 4, 1]))
        out_ty = int(rng.choice([FP32, FP16, BF16]))
        _no_pooling_case(ops, oracle, rng, specs, B, max_len, dt, align, out_ty,
                         f"seed {seed}: T={T} D={D} tys={tys} B={B} L<={max_len} align={align} out={out_ty}")


def test_no_pooling_more_positions_than_one_pass_of_the_grid(ops, oracle):
    """Rows of 512 columns take a whole wave; 300 K positions are more than the largest grid covers at once, so
    every wave walks several groups and uses the indices it fetched one group ahead."""
    rng = np.random.default_rng(31)
    specs = [(500, 512, INT4), (300, 512, INT8), (200, 512, INT4)]
    _no_pooling_case(ops, oracle, rng, specs, 2500, 80, np.int64, 16, FP16, "300 K positions of 512 columns")


def test_no_pooling_with_more_tables_than_the_kernel_keeps_in_lds(ops, oracle):
    """1100 small tables (some without any index): the table boundaries no longer fit the
    workgroup's LDS and the bisection reads them from memory."""
    rng = np.random.default_rng(990)
    D, T, B = 32, 1100, 2
    tys = [INT4, INT8, FP16]
    specs = [(int(rng.integers(3, 12)), D, tys[t % 3]) for t in range(T)]
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.integers(0, 4, size=T * B)
    lens[5 * B:9 * B] = 0
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    wt = np.array([s[2] for s in specs], np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt),
        cu(D_offsets), T * D, 0, D, D, D, 0, cu(idx), cu(off), ops.POOL_NONE, None, FP32, row_alignment=16)
    ok, want = oracle.tbe_forward_nobag(weights, wo, wt, [s[0] for s in specs], D, idx, off, FP32, 16)
    assert ok
    H.assert_same_bits(got.cpu().numpy(), want, "no pooling, 1100 tables")


@pytest.mark.parametrize("ty", [INT8, INT4])
def test_no_pooling_quantized_output_copies_rows(ops, oracle, ty):
    rng = np.random.default_rng(950 + ty)
    D, T, B = 64, 3, 9
    specs = [(int(rng.integers(20, 100)), D, ty) for _ in range(T)]
    weights, wo, rbs = build_weights(rng, specs, 16)
    lens = rng.integers(0, 6, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    wt = np.full(T, ty, np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt),
        cu(D_offsets), T * D, 0, D if ty == INT4 else 0, D if ty == INT8 else 0, 0, 0, cu(idx), cu(off),
        ops.POOL_NONE, None, ty, row_alignment=16).cpu().numpy()
    ok, want = oracle.tbe_forward_nobag(weights, wo, wt, [s[0] for s in specs], D, idx, off, ty, 16)
    assert ok and got.shape == want.shape and (got == want).all()
    # the copied rows are the stored rows: header first, then the packed elements
    t0_rows = weights[wo[0]:wo[0] + specs[0][0] * rbs[0]].reshape(-1, rbs[0])
    n0 = int(off[B])
    assert (got[:n0] == t0_rows[idx[:n0], :got.shape[1]]).all()
    # a table of another type is refused
    wt2 = wt.copy()
    wt2[1] = FP16
    with pytest.raises(RuntimeError, match="same type"):
        ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(wt2),
            cu(D_offsets), T * D, 0, D, D, D, 0, cu(idx), cu(off), ops.POOL_NONE, None, ty, row_alignment=16)


@pytest.mark.parametrize("out_ty", [FP32, FP16, BF16])
def test_long_bags_of_nine_chunk_rows(ops, oracle, out_ty):
    """Rows of 9 or 17 sixteen-byte chunks (int4 / int8, D = 256) with long bags:
    the plan lays 7 bags of 9 lanes end to end in a wave, so bags straddle the
    quarters of the wave and one lane idles."""
    rng = np.random.default_rng(1200 + out_ty)
    # 9, 9 (17 chunks, two per lane), 5, 9, 10 and 12 lanes per bag
    specs = [(400, 256, INT4), (300, 256, INT8), (350, 128, INT4), (200, 256, INT4), (100, 288, INT4), (100, 352, INT4)]
    T, B = len(specs), 45  # 45 bags: 6 full waves of 7 and a ragged one
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.integers(20, 60, size=T * B)
    lens[3] = 0
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    idx[rng.random(len(idx)) < 0.05] = -1
    psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
    for pooling, w in ((0, psw), (1, None), (0, None)):
        got, want = run_both(ops, oracle, weights, wo, specs, idx, off, pooling, w, out_ty, 16)
        H.assert_same_bits(got, want, f"nine-chunk rows pooling={pooling} weighted={w is not None} out={out_ty}")


def test_many_batch_sizes_reuse_and_recycle_work_lists(ops, oracle):
    """One plan, 40 different batch sizes (the plan keeps a work list per batch
    size and recycles them past 16), then the first size again."""
    rng = np.random.default_rng(1300)
    specs = [(120, 64, INT4), (80, 32, FP16), (60, 128, INT8)]
    T = len(specs)
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    d = [cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets)]
    for B in list(range(1, 41)) + [1, 7]:
        lens = rng.integers(0, 9, size=T * B)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]
                             + [np.zeros(0, np.int64)]).astype(np.int64)
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            *d, total_D, 0, 64, 128, 32, 0, cu(idx), cu(off), 0, None, FP32, row_alignment=16).cpu().numpy()
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP32, 16)
        assert rc == 0
        H.assert_same_bits(got, want, f"B={B}")


@pytest.mark.parametrize("pooling", [0, 1])
@pytest.mark.parametrize("dt", [np.int32, np.int64])
def test_pooled_int8_output_is_the_rowwise_quantized_fp32_output(ops, oracle, pooling, dt):
    """output_dtype INT8 of the pooled modes (the reference GPU operator's fused pooled-embedding
    quantization; expected value after fbgemm_gpu/test/tbe/inference/nbit_forward_test.py:293-340):
    every table's block is FloatToFused8BitRowwiseQuantized of that table's pooled fp32 vector,
    D_t bytes + fp32 scale + fp32 bias. Byte for byte against the pooled oracle followed by the
    quantizer oracle."""
    rng = np.random.default_rng(1300 + pooling)
    specs = [(200, 64, INT4), (150, 128, INT8), (90, 32, FP16), (300, 40, INT2), (60, 8, FP32), (120, 256, INT4), (50, 4, INT8)]
    T, B = len(specs), 37
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.integers(0, 12, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(dt)
    idx[rng.random(len(idx)) < 0.05] = -1
    psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    for w in (None, psw):
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
            pooling, None if w is None else cu(w), INT8, row_alignment=16)
        assert got.dtype == torch.uint8 and tuple(got.shape) == (B, total_D + 8 * T)
        got = got.cpu().numpy()
        rc, pooled = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, w, FP32, 16)
        assert rc == 0
        for t in range(T):
            D = specs[t][1]
            want = oracle.quantize_rowwise(np.ascontiguousarray(pooled[:, D_offsets[t]:D_offsets[t + 1]]), 8, True)
            block = got[:, D_offsets[t] + 8 * t:D_offsets[t] + 8 * t + D + 8]
            assert (block == want).all(), (t, np.argwhere(block != want)[:4])
        # and the float forward on the same plan is not disturbed by the scratch the 8-bit one uses
        f = ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
            pooling, None if w is None else cu(w), FP32, row_alignment=16)
        H.assert_same_bits(f.cpu().numpy(), pooled, "fp32 forward after the 8-bit one")


@pytest.mark.parametrize("mixed", [False, True])
def test_pooled_int8_output_at_a_size_the_lean_kernel_takes(ops, oracle, mixed):
    """A forward large enough for 16-byte lanes: the lean kernel quantizes its tables' pooled
    vectors in its own output stage (no float round trip); with `mixed`, tables of other shapes
    sit between them and go through the float scratch and the quantizer, which must leave the
    lean tables' blocks alone. Empty bags (an all-zero block: both extremes are zeros), bags
    whose weights are all -0.0 or 0.0 (zeros of both signs: the FIRST zero decides the sign of
    the stored bias and scale) and mean pooling are in. Byte for byte against pooled oracle +
    quantizer oracle."""
    rng = np.random.default_rng(1350 + mixed)
    specs = [(500, 64, INT4), (300, 128, INT8), (200, 64, FP16), (400, 256, INT4), (250, 32, INT8), (100, 96, INT4)]
    if mixed:
        specs = [specs[0], (300, 40, INT2), specs[1], (60, 8, FP32), specs[2], specs[3], (50, 4, INT8), specs[4], specs[5]]
    T, B = len(specs), 1500
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.integers(0, 12, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    idx[rng.random(len(idx)) < 0.05] = -1
    psw = rng.uniform(-1, 1, len(idx)).astype(np.float32)
    for b in range(0, T * B, 7):  # every seventh bag: weights that are zeros of one sign or of both
        lo, hi = int(off[b]), int(off[b + 1])
        psw[lo:hi] = [0.0, -0.0, 0.0][b % 3]
        if b % 3 == 2 and hi - lo > 1:
            psw[lo] = -0.0
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    for pooling, w in ((0, None), (0, psw), (1, None)):
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
            pooling, None if w is None else cu(w), INT8, row_alignment=16)
        assert got.dtype == torch.uint8 and tuple(got.shape) == (B, total_D + 8 * T)
        got = got.cpu().numpy()
        rc, pooled = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, w, FP32, 16)
        assert rc == 0
        for t in range(T):
            D = specs[t][1]
            want = oracle.quantize_rowwise(np.ascontiguousarray(pooled[:, D_offsets[t]:D_offsets[t + 1]]), 8, True)
            block = got[:, D_offsets[t] + 8 * t:D_offsets[t] + 8 * t + D + 8]
            assert (block == want).all(), (mixed, pooling, w is not None, t, np.argwhere(block != want)[:4])


@pytest.mark.parametrize("accumulate", ["exact", "fast"])
def test_plan_of_wide_4bit_tables_with_scales_beyond_the_prescaled_range(ops, oracle, accumulate, request):
    """A forward that orders its bags over tables that all have 4-bit rows in bags of 8 lanes and
    more (D = 256 and 1024 at 16-byte row alignment, bags of about 15 rows): the lean kernel's
    four-waves-per-SIMD instance. That instance does not carry the plain arithmetic: a wave that
    meets weight x scale beyond 2^100 queues its bags for the kernel behind it. Some bags here have
    per-sample weights of 2^110, one of them in the last wave of a table; the fp32 output matches
    the oracle bit for bit in the exact mode and to the bound in the tolerance-grade mode, twice in a row (the queue's counters are set
    back by every forward)."""
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    rng = np.random.default_rng(1370)
    specs = [(4000, 256, INT4), (1500, 1024, INT4), (2500, 256, INT4)]
    T, B = len(specs), 48_000
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.poisson(15, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    assert int(off[-1]) >= 1 << 21
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lib.fbgemm_amd_set_wide4(2)  # that instance, not whichever the first forwards find faster
    request.addfinalizer(lambda: lib.fbgemm_amd_set_wide4(-1))
    for rep in range(2):
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(off[(t + 1) * B] - off[t * B])) for t in range(T)]).astype(np.int64)
        psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
        huge = list(rng.integers(0, T * B, size=12)) + [B - 1, 2 * B - 1]
        for b in huge:
            psw[int(off[b]):int(off[b + 1])] = np.float32(2.0 ** 110)
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, 0, 1024, 0, 0, 0, cu(idx), cu(off), 0, cu(psw), FP32, row_alignment=16,
            accumulate=ops.ACC_FAST if accumulate == "fast" else ops.ACC_EXACT).cpu().numpy()
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, psw, FP32, 16)
        assert rc == 0
        if accumulate == "exact":
            H.assert_same_bits(got, want, f"wide 4-bit plan, pass {rep}")
        else:
            from fbgemm_amd import tolerance
            for t in range(T):
                blk = slice(int(D_offsets[t]), int(D_offsets[t + 1]))
                r = tolerance.grade(np.ascontiguousarray(got[:, blk]), np.ascontiguousarray(want[:, blk]), FP32, np)
                assert r["ok"], (t, r)


def test_wide_4bit_plan_settles_on_one_of_its_two_lean_kernels(ops, oracle):
    """By default the first forwards of such a plan (per batch size) run the general-purpose lean
    kernel and the four-waves-per-SIMD instance in turn, timed by events, and then stay with the
    faster one. Both compute the same bits: twenty forwards of the same inputs, each equal to the
    oracle's result, whatever kernel it took."""
    rng = np.random.default_rng(1371)
    specs = [(4000, 256, INT4), (2500, 256, INT4)]
    T, B = len(specs), 72_000
    weights, wo, _ = build_weights(rng, specs, 16)
    lens = rng.poisson(15, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    assert (1 << 21) <= int(off[-1]) < 20 * T * B
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(off[(t + 1) * B] - off[t * B])) for t in range(T)]).astype(np.int64)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    args = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, 0, 256, 0, 0, 0, cu(idx), cu(off), 0, None, FP16)
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP16, 16)
    assert rc == 0
    for k in range(20):
        got = ops.int_nbit_split_embedding_codegen_lookup_function(*args, row_alignment=16)
        H.assert_same_bits(got.cpu().view(torch.int16).numpy().view(np.uint16), want, f"forward {k}")


def test_int8_output_forwards_of_one_plan_on_two_streams(ops, oracle):
    """Forwards of one plan that go through the plan's float scratch (8-bit output of tables the
    lean kernel does not take) may be issued on different streams without ordering them: the
    library makes the later one wait for the earlier one's use of the scratch. Through the C ABI,
    without a synchronization between the calls: two streams, two sets of indices, alternating,
    every result against the same forward run alone."""
    import ctypes as C
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    rng = np.random.default_rng(1360)
    specs = [(500, 64, INT4), (300, 40, INT2), (60, 8, FP32), (200, 64, FP16), (100, 72, INT8)]
    T, B = len(specs), 1200
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    d_weights = cu(weights)
    plan = ops.TbePlan(torch.from_numpy(wo), torch.from_numpy(tys), torch.from_numpy(D_offsets),
                       torch.zeros(T, dtype=torch.int32), d_weights.numel(), 0, 16)
    inputs = []
    for _ in range(2):
        lens = rng.integers(0, 12, size=T * B)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
        inputs.append((cu(idx), cu(off), torch.zeros((B, total_D + 8 * T), dtype=torch.uint8, device="cuda"), ops.Status("cuda")))
    p = lambda t: C.c_void_p(t.data_ptr())

    def enqueue(k):
        idx, off, out, st = inputs[k]
        rc = lib.fbgemm_amd_tbe_forward(plan.handle, p(d_weights), None, p(idx), p(off), 64, idx.numel(), off.numel(), 0, None,
                                        INT8, p(out), p(st.buf), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.fbgemm_amd_last_error().decode()

    alone = []
    for k in (0, 1):
        enqueue(k)
        torch.cuda.synchronize()
        alone.append(inputs[k][2].clone())
    assert not torch.equal(alone[0], alone[1])
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(20):
        for k in (0, 1):
            inputs[k][2].zero_()
        torch.cuda.synchronize()
        for k in (0, 1, 0, 1):
            with torch.cuda.stream(streams[k]):
                enqueue(k)
        torch.cuda.synchronize()
        for k in (0, 1):
            assert torch.equal(inputs[k][2], alone[k]), f"round {rep}: the forward on stream {k} differs from the same forward run alone"
            assert inputs[k][3].read()[0] == 0


@pytest.mark.parametrize("pooling", [0, 2])
def test_tables_in_both_weights_buffers(ops, oracle, pooling):
    """weights_placements: tables 1 and 3 live in the second buffer (uvm_weights), whose offsets
    count from its own start; the row bound of a table comes from the next table of the SAME buffer."""
    rng = np.random.default_rng(1400 + pooling)
    D = 64
    specs = [(120, D, INT4), (80, D, INT8), (60, D, FP16), (200, D, INT4), (30, D, INT2)]
    T, B = len(specs), 21
    weights, wo, rbs = build_weights(rng, specs, 16)
    # the same table bytes dealt to two buffers
    bufs, offs = [[], []], [0, 0]
    place = np.array([0, 1, 0, 1, 0], np.int32)
    wo2 = np.zeros(T, np.int64)
    for t, (rows, _, _) in enumerate(specs):
        blob = weights[wo[t]:wo[t] + rows * rbs[t]]
        pad = (-len(blob)) % 128
        wo2[t] = offs[place[t]]
        bufs[place[t]] += [blob, np.zeros(pad, np.uint8)]
        offs[place[t]] += len(blob) + pad
    dev, uvm = np.concatenate(bufs[0]), np.concatenate(bufs[1])
    lens = rng.integers(0, 9, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    idx[0] = specs[0][0] - 1
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    maxd = lambda ty: D if ty in tys else 0
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(dev), cu(uvm), cu(place), cu(wo2), cu(tys), cu(D_offsets), T * D, maxd(INT2), maxd(INT4), maxd(INT8),
        maxd(FP16), 0, cu(idx), cu(off), pooling, None, FP32, row_alignment=16).cpu().numpy()
    if pooling == 2:
        ok, want = oracle.tbe_forward_nobag(weights, wo, tys, [s[0] for s in specs], D, idx, off, FP32, 16)
        assert ok
    else:
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, T * D, idx, off, pooling, None, FP32, 16)
        assert rc == 0
    H.assert_same_bits(got, want, f"two buffers, pooling {pooling}")
    # the last row of the last table of each buffer is in range, the one after it is not
    for t in (3, 4):
        s = int(off[t * B])
        if int(off[(t + 1) * B]) > s:
            bad = idx.copy()
            bad[s] = specs[t][0] + (128 // rbs[t]) + 1  # past the rows and past the buffer's padding
            with pytest.raises(RuntimeError, match="out of bounds"):
                ops.int_nbit_split_embedding_codegen_lookup_function(
                    cu(dev), cu(uvm), cu(place), cu(wo2), cu(tys), cu(D_offsets), T * D, maxd(INT2), maxd(INT4), maxd(INT8),
                    maxd(FP16), 0, cu(bad), cu(off), pooling, None, FP32, row_alignment=16)


@pytest.mark.parametrize("long_bags", [False, True])
def test_special_values_in_the_table_batched_forward(ops, oracle, long_bags):
    """Per-sample weights that push weight * scale beyond 2^100 (the 4- and 8-bit lanes then redo their
    work without the pre-scaled arithmetic), infinite / NaN / denormal / signed-zero weights and fp16
    scale-bias pairs: finite results bit for bit, NaN where the oracle has NaN. Long bags take the
    end-to-end lane layout of the 9-chunk rows."""
    from test_spmdm_gpu import same_bits_or_both_nan
    np.seterr(over="ignore")
    rng = np.random.default_rng(1500 + int(long_bags))
    specs = [(60, 256, INT4), (50, 128, INT8), (40, 64, INT4), (30, 32, FP16), (45, 256, INT8), (25, 16, INT2)]
    T, B = len(specs), 19
    weights, wo, rbs = build_weights(rng, specs, 16)
    specials = np.array([np.inf, -np.inf, np.nan, 6e-8, -6e-8, 0.0, -0.0, 65504.0], np.float32).astype(np.float16)
    for t, (rows, D, ty) in enumerate(specs):
        if ty == FP16:
            continue
        tbl = weights[wo[t]:wo[t] + rows * rbs[t]].reshape(rows, rbs[t])
        for r in range(len(specials)):
            tbl[r, 0:2] = specials[r:r + 1].view(np.uint8)
            tbl[r + 10, 2:4] = specials[r:r + 1].view(np.uint8)
    lens = rng.integers(20, 40, size=T * B) if long_bags else rng.integers(0, 9, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    psw = rng.normal(size=len(idx)).astype(np.float32)
    psw[::9] = 1e30
    psw[4::11] = np.float32(1e-40)
    psw[5::23] = np.inf
    psw[6::29] = np.nan
    psw[7::31] = -0.0
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    for w in (None, psw):
        for pooling in (0, 1):
            for out_ty, name in ((FP32, "fp32"), (FP16, "fp16"), (BF16, "bf16")):
                got = ops.int_nbit_split_embedding_codegen_lookup_function(
                    cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
                    cu(D_offsets), total_D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), 0, cu(idx), cu(off), pooling,
                    None if w is None else cu(w), out_ty, row_alignment=16).cpu()
                got = got.numpy() if out_ty == FP32 else got.view(torch.int16).numpy().view(np.uint16)
                rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, w, out_ty, 16)
                assert rc == 0
                same_bits_or_both_nan(got, want, f"special values weighted={w is not None} pooling={pooling} {name}")


def _monotone_mapping(rng, logical, keep_frac, dt):
    keep = rng.random(logical) < keep_frac
    m = np.full(logical, -1, dt)
    m[keep] = np.arange(int(keep.sum()), dtype=dt)
    return m, int(keep.sum())


@pytest.mark.parametrize("rdt", [np.int32, np.int64])
def test_rank_records_replace_order_preserving_mappings(ops, oracle, rdt):
    """The compact form of the pruned-row mappings (a kept-row bitmap with running counts): taken
    for the tables whose mapping numbers the kept rows in logical order, not for a table whose
    mapping does anything else, and never a different result than the array gives (integers)."""
    rng = np.random.default_rng(77)
    logical = [1000, 37, 5000, 64, 2049, 300]
    maps, specs = [], []
    for t, n in enumerate(logical):
        if t == 3:
            maps.append(np.zeros(0, rdt))  # this table is not pruned
            specs.append((n, 64, INT4))
            continue
        m, kept = _monotone_mapping(rng, n, [0.5, 1.0, 0.3, 0, 0.0, 0.7][t], rdt)
        if t == 5:  # two kept rows swapped: a valid mapping, but not order-preserving
            k = np.nonzero(m >= 0)[0]
            m[k[3]], m[k[9]] = m[k[9]], m[k[3]]
        maps.append(m)
        specs.append((max(kept, 1), [64, 128, 256, 64, 32, 128][t], [INT4, INT8, INT4, INT4, FP16, INT4][t]))
    T, B = len(specs), 33
    weights, wo, _ = build_weights(rng, specs, 16)
    remap = np.concatenate(maps)
    remap_off = np.concatenate([[0], np.cumsum([len(m) for m in maps])]).astype(np.int64)
    lens = rng.integers(0, 25, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, logical[t], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    dense = oracle.pruned_array_lookup(idx, off, remap, remap_off)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    plan = ops.TbePlan(torch.from_numpy(wo), torch.from_numpy(tys), torch.from_numpy(D_offsets), torch.zeros(T, dtype=torch.int32),
                       len(weights), 0, 16)
    d_remap, d_remap_off = cu(remap), cu(remap_off)
    assert plan.set_index_remappings(d_remap, d_remap_off) == 4  # tables 0, 1, 2, 4; not 3 (none) and 5 (swapped)
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 0, 256, 128, 32, 0, cu(idx), cu(off), 1, None, FP32, row_alignment=16, plan=plan,
        index_remappings=d_remap, index_remappings_offsets=d_remap_off).cpu().numpy()
    with_records = call()
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, dense, off, 1, None, FP32, 16)
    assert rc == 0
    H.assert_same_bits(with_records, want, "rank records")
    # a forward that uses the records slices the mappings with the offsets the records were built
    # for, not with whatever offsets it is handed (here: zeros, which would switch the remap off)
    stale = torch.zeros_like(d_remap_off)
    plan._rank_key = ops.TbePlan.rank_key(d_remap, stale)  # keep the wrapper from rebuilding the records
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 0, 256, 128, 32, 0, cu(idx), cu(off), 1, None, FP32, row_alignment=16, plan=plan,
        index_remappings=d_remap, index_remappings_offsets=stale).cpu().numpy()
    H.assert_same_bits(got, want, "rank records, other offsets handed to the forward")
    plan.set_index_remappings(None, None)
    plan._rank_key = ops.TbePlan.rank_key(d_remap, d_remap_off)  # keep the wrapper from rebuilding them
    assert plan.rank_tables() == 0
    H.assert_same_bits(call(), want, "mapping arrays")


def test_remap_offsets_must_cover_every_feature(ops):
    rng = np.random.default_rng(78)
    specs = [(50, 64, INT4), (60, 64, INT4), (70, 64, INT4)]
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = (np.arange(4) * 64).astype(np.int32)
    off = (np.arange(3 * 4 + 1) * 2).astype(np.int64)
    idx = rng.integers(0, 50, size=24).astype(np.int64)
    remap = np.arange(100, dtype=np.int32)
    with pytest.raises(ValueError, match="features need 4"):
        ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(3, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), 192, 0, 64, 0, 0, 0, cu(idx), cu(off), 0, None, FP32, row_alignment=16,
            index_remappings=cu(remap), index_remappings_offsets=cu(np.array([0, 50, 100], np.int64)))
    # and the C entry point itself refuses it (callers that bind the library directly)
    import ctypes as C
    from fbgemm_amd import _lib
    plan = ops.TbePlan(torch.from_numpy(wo), torch.from_numpy(tys), torch.from_numpy(D_offsets), torch.zeros(3, dtype=torch.int32),
                       len(weights), 0, 16)
    d = [cu(weights), cu(idx), cu(off), cu(remap), cu(np.array([0, 50, 100], np.int64)), torch.empty(4, 192, device="cuda")]
    st = ops.Status()
    p = lambda t: C.c_void_p(t.data_ptr())
    rc = _lib.lib().fbgemm_amd_tbe_forward_pruned(plan.handle, p(d[0]), None, p(d[1]), p(d[2]), 64, 24, 13, 0, None, 0, p(d[5]),
                                                  p(d[3]), 32, p(d[4]), 3, p(st.buf), None)
    assert rc == -1 and b"need 4" in _lib.lib().fbgemm_amd_last_error()
