"""GPU parity of the operators either side of the lookup, through the C ABI:
bounds_check_indices, pruned_hashmap_lookup, the row-wise quantizers and their
inverses. Integer and byte results are compared bit for bit with the oracle on
the same seeded inputs; the cases follow the reference's own tests
(fbgemm_gpu/test/tbe/utils/split_embeddings_utils_test.py:237-465,
fbgemm_gpu/test/quantize/fused_nbit_rowwise_test.py:58-476)."""
import numpy as np
import pytest

import oracle
from oracle import LAYOUT_TBE, LAYOUT_TRAILER, ST_BF16, ST_FP16, ST_FP32

pytestmark = pytest.mark.gpu

FATAL, WARNING, IGNORE = 0, 1, 2


@pytest.fixture(scope="module")
def env():
    import torch

    from fbgemm_amd import ops

    assert torch.cuda.is_available()
    return torch, ops


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_problem(rng, T, B, max_L, dt):
    rows = rng.integers(1, 1000, size=T).astype(np.int64)
    Ls = rng.integers(0, max_L, size=T * B)
    off = np.concatenate([[0], np.cumsum(Ls)]).astype(dt)
    idx = np.concatenate([rng.integers(0, rows[t], size=int(Ls[t * B:(t + 1) * B].sum())) for t in range(T)]
                         + [np.zeros(0, np.int64)]).astype(dt)
    return rows, idx, off


def run_bounds(torch, ops, rows, idx, off, mode, B_offsets=None):
    """Both sides on copies. Returns ((idx, off, warning, error bits), same for the oracle)."""
    d_idx, d_off = dev(torch, idx), dev(torch, off)
    d_warn = torch.full((1,), 77, dtype=torch.int64, device="cuda")
    st = ops.Status()
    bo = None if B_offsets is None else dev(torch, np.asarray(B_offsets, np.int32))
    from fbgemm_amd import _lib
    rpt = dev(torch, rows)
    _lib.check(_lib.lib().fbgemm_amd_bounds_check_indices(
        ops._ptr(rpt), len(rows), ops._ptr(d_idx), ops._ptr(d_off), ops._bits(d_idx), d_idx.numel(), d_off.numel(),
        mode, ops._ptr(d_warn), ops._ptr(bo), ops._ptr(st.buf), ops._stream()))
    bits, pos = st.read()
    o_idx, o_off, o_warn = idx.copy(), off.copy(), np.full(1, 77, np.int64)
    rc = oracle.bounds_check_indices(rows, o_idx, o_off, mode, o_warn, B_offsets)
    return (d_idx.cpu().numpy(), d_off.cpu().numpy(), int(d_warn.item()), bits, pos), (o_idx, o_off, int(o_warn[0]), rc)


@pytest.mark.parametrize("mode", [FATAL, WARNING, IGNORE])
@pytest.mark.parametrize("dt", [np.int32, np.int64])
def test_bounds_check_matches_oracle(env, mode, dt):
    torch, ops = env
    rng = np.random.default_rng(101)
    for trial in range(24):
        T, B, max_L = int(rng.integers(1, 20)), int(rng.integers(1, 40)), int(rng.integers(1, 30))
        rows, idx, off = make_problem(rng, T, B, max_L, dt)
        kind = trial % 6
        if kind == 1 and idx.size:  # some indices out of range, some pruned
            sel = rng.random(idx.size) < 0.2
            idx[sel] = rng.choice([-1, -2, 1000, np.iinfo(dt).max], size=int(sel.sum())).astype(dt)
        elif kind == 2:  # the reference test's offsets damage
            off[0] = -100
            off[-1] += 100
        elif kind == 3:  # arbitrary offsets: negative, decreasing, beyond the end
            off = rng.integers(-10, idx.size + 10, size=off.size).astype(dt)
        elif kind == 4 and off.size > 2:  # one decreasing pair in the middle
            k = int(rng.integers(1, off.size - 1))
            off[k] = off[k - 1] - 1 if off[k - 1] > 0 else off[k] + 5
        elif kind == 5:
            off[-1] = max(0, int(off[-1]) - 3)
        got, want = run_bounds(torch, ops, rows, idx, off, mode)
        if mode == FATAL:
            # nothing modified; the status says whether the reference would raise
            assert (got[0] == idx).all() and (got[1] == off).all(), (trial, kind)
            assert (got[3] != 0) == (want[3] != 0), (trial, kind, got[3], want[3])
            assert got[2] == 77
        else:
            assert (got[0] == want[0]).all(), (trial, kind)
            assert (got[1] == want[1]).all(), (trial, kind, off, got[1], want[1])
            assert got[3] == 0
            if mode == WARNING:
                assert got[2] == want[2], (trial, kind)
            else:
                assert got[2] == 77  # IGNORE never touches the counter


def test_bounds_check_fatal_reports_first_bad_index(env):
    torch, ops = env
    rng = np.random.default_rng(102)
    rows, idx, off = make_problem(rng, 7, 33, 20, np.int64)
    bad = sorted(rng.choice(idx.size, size=5, replace=False).tolist())
    t_of = np.searchsorted(off[::33], bad, side="right") - 1
    for p, t in zip(bad, t_of):
        idx[p] = rows[t]  # one past the last row
    got, want = run_bounds(torch, ops, rows, idx, off, FATAL)
    assert got[3] == ops.ERR_INDEX_OUT_OF_RANGE and got[4] == bad[0]
    assert want[3] != 0
    with pytest.raises(RuntimeError, match=f"Index {bad[0]} is out of bounds"):
        ops.bounds_check_indices(dev(torch, rows), dev(torch, idx), dev(torch, off), FATAL,
                                 torch.zeros(1, dtype=torch.int64, device="cuda"))


@pytest.mark.parametrize("mode", [WARNING, IGNORE])
def test_bounds_check_variable_batch_sizes(env, mode):
    torch, ops = env
    rng = np.random.default_rng(103)
    for _ in range(8):
        T = int(rng.integers(1, 12))
        Bs = rng.integers(0, 30, size=T)
        B_offsets = np.concatenate([[0], np.cumsum(Bs)]).astype(np.int32)
        total_B = int(B_offsets[-1])
        rows = rng.integers(1, 500, size=T).astype(np.int64)
        Ls = rng.integers(0, 12, size=total_B)
        off = np.concatenate([[0], np.cumsum(Ls)]).astype(np.int64)
        idx = rng.integers(-2, 600, size=int(off[-1])).astype(np.int64)
        got, want = run_bounds(torch, ops, rows, idx, off, mode, B_offsets)
        assert (got[0] == want[0]).all() and (got[1] == want[1]).all()
        if mode == WARNING:
            assert got[2] == want[2]


def test_bounds_check_large_offsets_scan(env):
    """More offsets than one scan block holds, damaged so that the repaired value
    has to be carried across blocks."""
    torch, ops = env
    rng = np.random.default_rng(104)
    T, B = 13, 1499
    rows, idx, off = make_problem(rng, T, B, 6, np.int32)
    off[5000] = off[-1] + 9  # everything after it is raised to num_indices
    off[3] = -4
    got, want = run_bounds(torch, ops, rows, idx, off, WARNING)
    assert (got[1] == want[1]).all() and (got[0] == want[0]).all() and got[2] == want[2]
    assert got[1][5000] == idx.size and (np.diff(got[1]) >= 0).all()


def test_bounds_check_more_scan_blocks_than_a_workgroup_has_threads(env):
    """4.5 M bags: the running maximum then goes through the separate carry pass (with fewer blocks every
    block takes the maximum of the earlier blocks itself)."""
    torch, ops = env
    rng = np.random.default_rng(105)
    T, B = 3, 1_500_000
    rows, idx, off = make_problem(rng, T, B, 2, np.int32)
    off[2_000_000] = off[-1] + 1  # everything after it is raised to num_indices
    off[7] = -1
    idx[::1000] = 10 ** 6
    got, want = run_bounds(torch, ops, rows, idx, off, WARNING)
    assert (got[1] == want[1]).all() and (got[0] == want[0]).all() and got[2] == want[2]


@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("hdt", [np.int32, np.int64])
def test_pruned_hashmap_lookup_matches_oracle(env, idt, hdt):
    torch, ops = env
    rng = np.random.default_rng(105)
    T, B = 6, 17
    caps, tables, ins_idx, ins_dense, ins_off = [], [], [], [], [0]
    for t in range(T):
        n = 0 if t == 2 else int(rng.integers(1, 400))  # table 2 has no map: indices pass through
        keys = rng.choice(5000, size=n, replace=False)
        cap = 0 if n == 0 else int(n / 0.6) + 1
        caps.append(cap)
        ins_idx.append(keys)
        ins_dense.append(np.arange(n))
        ins_off.append(ins_off[-1] + n)
    hto = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    hash_table = np.full((int(hto[-1]), 2), -1, hdt)
    # the oracle's insert takes (table, bag) offsets: one bag per table here
    oracle.pruned_hashmap_insert(np.concatenate(ins_idx).astype(idt), np.concatenate(ins_dense).astype(idt),
                                 np.asarray(ins_off, idt), hash_table, hto)
    Ls = rng.integers(0, 9, size=T * B)
    off = np.concatenate([[0], np.cumsum(Ls)]).astype(idt)
    idx = rng.integers(0, 5000, size=int(off[-1])).astype(idt)
    want = oracle.pruned_hashmap_lookup(idx, off, hash_table, hto)
    got = ops.pruned_hashmap_lookup(dev(torch, idx), dev(torch, off), dev(torch, hash_table), dev(torch, hto))
    assert (got.cpu().numpy() == want).all()
    # the model: a dict per table
    for t in range(T):
        d = dict(zip(ins_idx[t].tolist(), ins_dense[t].tolist()))
        for i in range(int(off[t * B]), int(off[(t + 1) * B])):
            assert want[i] == (idx[i] if caps[t] == 0 else d.get(int(idx[i]), -1))


def rows_of(rng, kind, rows, cols, dtype):
    if kind == "normal":
        x = rng.normal(0, 1, size=(rows, cols))
    elif kind == "uniform":
        x = rng.uniform(-5, 5, size=(rows, cols))
    elif kind == "constant":
        x = np.repeat(rng.normal(0, 3, size=(rows, 1)), cols, axis=1)
    elif kind == "tiny":
        x = rng.normal(0, 1e-7, size=(rows, cols))
    elif kind == "large":
        x = rng.normal(0, 1e4, size=(rows, cols)) if dtype == np.float16 else rng.normal(0, 1e30, size=(rows, cols))
    else:
        x = np.zeros((rows, cols))
        x[::2, ::3] = -0.0
    return x.astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
@pytest.mark.parametrize("layout", [LAYOUT_TRAILER, LAYOUT_TBE])
def test_quantize_matches_oracle(env, dtype, bit_rate, sb_float, layout):
    torch, ops = env
    rng = np.random.default_rng(106)
    for kind in ("normal", "uniform", "constant", "tiny", "large", "zeros"):
        for cols in (1, 2, 3, 7, 8, 31, 64, 100, 128, 257, 1024):
            x = rows_of(rng, kind, 9, cols, dtype)
            want = oracle.quantize_rowwise(x, bit_rate, sb_float, layout)
            got = ops.quantize_rowwise(dev(torch, x), bit_rate, sb_float, layout)
            assert (got.cpu().numpy() == want).all(), (kind, cols)


def caller_extremes(rng, x, mode):
    lo, hi = x.astype(np.float32).min(1), x.astype(np.float32).max(1)
    if mode == "wider":
        lo, hi = lo - rng.uniform(0, 2, lo.shape), hi + rng.uniform(0, 2, hi.shape)
    elif mode == "narrower":  # elements outside the extremes: the clamping / wrapping rules show
        mid, half = (lo + hi) / 2, (hi - lo) / 2
        lo, hi = mid - half * rng.uniform(0.1, 0.9, lo.shape), mid + half * rng.uniform(0.1, 0.9, hi.shape)
    elif mode == "far":  # no range at all under spread-out values: beyond the 32-bit integers
        lo, hi = lo + 1e-3, lo + 1e-3
    elif mode == "steep":  # a tiny step: beyond 32 bits, and for the "large" rows beyond 64
        lo, hi = np.zeros_like(lo), np.full_like(hi, 1e-6)
    return np.stack([lo, hi], 1).astype(x.dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bit_rate,sb_float", [(2, False), (4, False), (8, False), (8, True)])
@pytest.mark.parametrize("layout", [LAYOUT_TRAILER, LAYOUT_TBE])
def test_quantize_with_caller_extremes_matches_oracle(env, dtype, bit_rate, sb_float, layout):
    # rowwise_min_max of the reference's quantizers (include/fbgemm/QuantUtils.h:277-283, :311-317)
    torch, ops = env
    rng = np.random.default_rng(108)
    for kind in ("normal", "uniform", "constant", "large"):
        for cols in (1, 4, 8, 12, 31, 32, 36, 40, 63, 64, 72, 100, 128, 260, 1024):
            x = rows_of(rng, kind, 9, cols, dtype)
            for mode in ("true", "wider", "narrower", "far", "steep"):
                if mode in ("far", "steep") and dtype == np.float16:
                    continue
                if mode == "steep" and kind != "large":
                    x = (x * 1e4).astype(dtype)
                mm = caller_extremes(rng, x, mode)
                want = oracle.quantize_rowwise(x, bit_rate, sb_float, layout, min_max=mm)
                got = ops.quantize_rowwise(dev(torch, x), bit_rate, sb_float, layout, rowwise_min_max=dev(torch, mm))
                assert (got.cpu().numpy() == want).all(), (kind, cols, mode)
    with pytest.raises(ValueError):
        ops.quantize_rowwise(dev(torch, x), bit_rate, sb_float, layout, rowwise_min_max=dev(torch, mm[:-1]))


def test_quantize_into_padded_rows_leaves_padding_alone(env):
    torch, ops = env
    rng = np.random.default_rng(107)
    x = rng.normal(0, 1, size=(50, 100)).astype(np.float32)
    stride = 64  # 4 + 50 = 54 bytes of row in 64-byte slots
    want = oracle.quantize_rowwise(x, 4, False, LAYOUT_TBE, out_stride=stride, fill=0xAB)
    out = torch.full((50, stride), 0xAB, dtype=torch.uint8, device="cuda")
    ops.quantize_rowwise(dev(torch, x), 4, False, LAYOUT_TBE, out=out)
    assert (out.cpu().numpy() == want).all()
    assert (out.cpu().numpy()[:, 54:] == 0xAB).all()


@pytest.mark.parametrize("out_ty", [ST_FP32, ST_FP16, ST_BF16])
@pytest.mark.parametrize("bit_rate,sb_float,layout", [(2, False, LAYOUT_TRAILER), (4, False, LAYOUT_TRAILER),
                                                       (8, False, LAYOUT_TRAILER), (8, True, LAYOUT_TRAILER),
                                                       (4, False, LAYOUT_TBE), (8, False, LAYOUT_TBE)])
def test_dequantize_matches_oracle(env, out_ty, bit_rate, sb_float, layout):
    torch, ops = env
    rng = np.random.default_rng(108)
    tdt = {ST_FP32: torch.float32, ST_FP16: torch.float16, ST_BF16: torch.bfloat16}[out_ty]
    for cols in (1, 4, 8, 30, 64, 100, 256, 1000):
        stride = oracle.quantized_row_bytes(cols, bit_rate, sb_float, layout) + int(rng.integers(0, 3)) * 4
        q = rng.integers(0, 256, size=(11, stride), dtype=np.uint8)
        nb = (cols + 8 // bit_rate - 1) // (8 // bit_rate)
        sb_at = 0 if layout == LAYOUT_TBE else nb
        if sb_float:
            q[:, sb_at:sb_at + 8] = np.stack([rng.uniform(1e-3, 1, 11), rng.uniform(-3, 3, 11)], 1).astype(np.float32).view(np.uint8)
        else:
            q[:, sb_at:sb_at + 4] = np.stack([rng.uniform(1e-3, 1, 11), rng.uniform(-3, 3, 11)], 1).astype(np.float16).view(np.uint8)
        want = oracle.dequantize_rowwise(q, cols, bit_rate, sb_float, layout, out_ty)
        got = ops.dequantize_rowwise(dev(torch, q), cols, bit_rate, sb_float, layout, tdt)
        g = got.cpu().view(torch.int32 if out_ty == ST_FP32 else torch.int16).numpy()
        w = want.view(np.int32 if out_ty == ST_FP32 else np.int16)
        assert (g == w).all(), cols


def test_quantized_tables_feed_the_lookup(env):
    """fp32 rows -> 4-bit TBE rows on the GPU -> table-batched lookup: equals the
    oracle's lookup over the oracle's quantized rows (the producer and the
    consumer agree on the format)."""
    torch, ops = env
    rng = np.random.default_rng(109)
    E, D, B = 300, 64, 16
    x = rng.normal(0, 1, size=(E, D)).astype(np.float32)
    stride = ops.padded_row_size_in_bytes(D, ops.INT4, 16)
    rows_gpu = torch.zeros((E, stride), dtype=torch.uint8, device="cuda")
    ops.quantize_rowwise(dev(torch, x), 4, False, LAYOUT_TBE, out=rows_gpu)
    rows_cpu = oracle.quantize_rowwise(x, 4, False, LAYOUT_TBE, out_stride=stride, fill=0)
    assert (rows_gpu.cpu().numpy() == rows_cpu).all()
    Ls = rng.integers(0, 9, size=B)
    off = np.concatenate([[0], np.cumsum(Ls)]).astype(np.int64)
    idx = rng.integers(0, E, size=int(off[-1])).astype(np.int64)
    wo, tys, Do = np.zeros(1, np.int64), np.full(1, ops.INT4, np.uint8), np.asarray([0, D], np.int32)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        rows_gpu.reshape(-1), torch.empty(0, dtype=torch.uint8, device="cuda"), dev(torch, np.zeros(1, np.int32)),
        dev(torch, wo), dev(torch, tys), dev(torch, Do), D, 0, D, 0, 0, 0, dev(torch, idx), dev(torch, off),
        ops.POOL_SUM, None, ops.FP32, row_alignment=16)
    rc, want = oracle.tbe_forward(rows_cpu.reshape(-1), wo, tys, Do, D, idx, off, ops.POOL_SUM, None, ST_FP32, 16)
    assert rc == 0
    assert (got.cpu().numpy().view(np.uint32) == want.view(np.uint32)).all()
