"""The tolerance-grade accumulate mode (FBGEMM_AMD_ACC_FAST) against the oracle.

In this mode the biases of a bag are summed apart from the scaled elements and
bags of a launch too small to fill the device are cut into segments whose
partial sums are added afterwards, so the fp32 roundings are not the
reference's. The stated bound of the path, element by element: fp32 output
within 1e-5 relative, fp16 / bf16 output within one unit in the last place.
Every element that is not a cancellation (|expected| at least 2^-10 of the
largest magnitude in the bag's block of the output) is held to exactly that;
an element below it may instead be within 1e-5 of the block's magnitude
(fbgemm_amd/tolerance.py). Each test prints the worst error it met and how
many elements needed the second clause. The default mode stays bit-exact and
is what every other test file checks."""
import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    import fbgemm_amd.ops as o
    return o


@pytest.fixture(autouse=True, params=["wide", "default"])
def lanes(request):
    """Test-sized launches would take 4-byte lanes (the general kernel, which is exact in either
    mode): "wide" gives them the 16-byte lanes and the lean kernel that large launches get."""
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    if request.param == "wide":
        lib.fbgemm_amd_set_narrow_below_waves(0)
    yield request.param
    lib.fbgemm_amd_set_narrow_below_waves(-1)


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


NEEDED_BLOCK_CLAUSE = {"elements": 0, "cancellations": 0, "needed": 0}


def check_grade(got, want, out_ty, rows, what):
    """got / want: fp32 arrays or uint16 bit patterns, reshaped to [rows, -1] (one table's block per
    row). Asserts the bound of fbgemm_amd/tolerance.py and returns the worst element-wise error:
    relative (fp32) or units in the last place."""
    from fbgemm_amd import tolerance
    r = tolerance.grade(got.reshape(rows, -1), want.reshape(rows, -1), out_ty, np)
    NEEDED_BLOCK_CLAUSE["elements"] += r["elements"]
    NEEDED_BLOCK_CLAUSE["cancellations"] += r["cancellations"]
    NEEDED_BLOCK_CLAUSE["needed"] += r["needed_block_clause"]
    unit = "relative" if out_ty == FP32 else "units in the last place"
    assert r["ok"], (f"{what}: worst element-wise error {r['worst']:.3g} {unit}; {r['needed_block_clause']} of "
                     f"{r['cancellations']} cancellations needed the block clause, worst {r['worst_block']:.3g} of the block")
    return r["worst"]


@pytest.fixture(scope="module", autouse=True)
def report_block_clause():
    yield
    print(f"\ntolerance grade: {NEEDED_BLOCK_CLAUSE['needed']} of {NEEDED_BLOCK_CLAUSE['elements']} elements "
          f"({NEEDED_BLOCK_CLAUSE['cancellations']} cancellations) needed the block-relative clause")


def bits_of(t, out_ty):
    t = t.cpu()
    return t.numpy() if out_ty == FP32 else t.view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("ty", [INT4, INT8])
@pytest.mark.parametrize("shape", [(300, 5000, 128, 20), (40, 300, 256, 10), (64, 2000, 64, 33), (3, 1000, 128, 300),
                                   (10, 4000, 256, 100), (1, 500, 64, 400), (20, 1000, 48, 50)])
def test_single_table_fast_mode(ops, oracle, ty, shape):
    """Regular shapes (the lean kernel, biases summed apart), few long bags (split into
    segments) and a width the lean kernel does not take (D = 48: the general kernel, exact)."""
    nb, rows, D, avg = shape
    rng = np.random.default_rng(hash((ty, shape)) % 2**32)
    worst = {}
    for sbl in (True, False):
        for out_ty in (FP32, FP16, BF16):
            for weighted in (False, True):
                for normalize in (False, True):
                    table, _ = H.make_table(rng, ty, rows, D, sbl)
                    idx, off, _ = H.make_bags(rng, rows, nb, avg, np.int64, np.int32, empty_frac=0.1)
                    if not sbl and len(idx) > 3:
                        idx[3] = -1  # a pruned row
                    w = rng.uniform(0, 1, len(idx)).astype(np.float32) if weighted else None  # as the configurations draw them
                    kern = (ops.generate_embedding_spmdm_nbit_with_strides(4, D, weighted, normalize, 16, False, True, -1, -1, sbl, out_ty=out_ty)
                            if ty == INT4 else
                            ops.generate_embedding_spmdm_with_strides(INT8, D, weighted, normalize, 16, False, True, -1, -1, sbl, out_ty=out_ty))
                    out = torch.full((nb * D,), 7.0, dtype={FP32: torch.float32, FP16: torch.float16, BF16: torch.bfloat16}[out_ty], device="cuda")
                    ok = kern(nb, len(idx), rows, cu(table), cu(idx), cu(off), None if w is None else cu(w), out,
                              accumulate=ops.ACC_FAST)
                    ok_o, want = oracle.spmdm(ty, D, table, idx, off, weights=w, normalize=normalize, out_ty=out_ty,
                                              scale_bias_last=sbl, data_size=rows)
                    assert ok and ok_o
                    e = check_grade(bits_of(out, out_ty), want, out_ty, nb, f"ty={ty} {shape} sbl={sbl} out={out_ty} w={weighted} norm={normalize}")
                    worst[out_ty] = max(worst.get(out_ty, 0), e)
    print(f"worst error, ty={ty} shape={shape}: fp32 relative {worst[FP32]:.3g}, fp16 {worst[FP16]} ulp, bf16 {worst[BF16]} ulp")


def test_cancellation_heavy_bags(ops, oracle):
    """Bags whose terms cancel: the same rows with weights +w and -w, and biases that sum to
    nearly nothing. The error stays within 1e-5 of the magnitude of what was summed."""
    rng = np.random.default_rng(5)
    rows, D, nb, L = 400, 128, 50, 24
    for ty in (INT4, INT8):
        table, _ = H.make_table(rng, ty, rows, D, False, scale_range=(0.5, 2.0), bias_range=(-100.0, 100.0))
        half = rng.integers(0, rows, size=(nb, L // 2))
        idx = np.concatenate([half, half], axis=1).reshape(-1).astype(np.int64)
        w = rng.uniform(0.5, 1.5, size=(nb, L // 2)).astype(np.float32)
        w = np.concatenate([w, -w], axis=1).reshape(-1)
        off = (np.arange(nb + 1) * L).astype(np.int32)
        kern = (ops.generate_embedding_spmdm_nbit_with_strides(4, D, True, False, 16, False, True, -1, -1, False) if ty == INT4 else
                ops.generate_embedding_spmdm_with_strides(INT8, D, True, False, 16, False, True, -1, -1, False))
        out = torch.empty(nb * D, dtype=torch.float32, device="cuda")
        assert kern(nb, len(idx), rows, cu(table), cu(idx), cu(off), cu(w), out, accumulate=ops.ACC_FAST)
        ok, want = oracle.spmdm(ty, D, table, idx, off, weights=w, scale_bias_last=False, data_size=rows)
        assert ok
        got = out.cpu().numpy().astype(np.float64).reshape(nb, D)
        # what was summed per bag: |w| * (|scale| * 15 or 255 + |bias|) is of the order of 100
        err = np.abs(got - want.reshape(nb, D).astype(np.float64)).max()
        assert err <= 1e-5 * 100.0 * L, f"ty={ty}: absolute error {err}"
        print(f"cancelling bags, ty={ty}: largest absolute error {err:.3g} against terms of magnitude ~100")


def tbe_problem(rng, specs, B, max_L, row_alignment, weighted):
    from test_tbe_gpu import build_weights
    weights, wo, _ = build_weights(rng, specs, row_alignment)
    T = len(specs)
    lens = rng.integers(0, max_L, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)] + [np.zeros(0, np.int64)]).astype(np.int64)
    idx[rng.random(len(idx)) < 0.05] = -1
    psw = rng.uniform(0, 1, len(idx)).astype(np.float32) if weighted else None
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    return weights, wo, tys, D_offsets, idx, off, psw


@pytest.mark.parametrize("B,max_L", [(257, 40), (3, 900), (1, 2000)])
def test_table_batched_fast_mode(ops, oracle, B, max_L):
    """Mixed tables (lean and general shapes together) in the tolerance-grade mode; with few, long
    bags the forward cuts them into segments."""
    rng = np.random.default_rng(1000 + B)
    specs = [(500, 64, INT4), (300, 128, INT8), (200, 256, FP16), (100, 32, INT2), (400, 256, INT4), (64, 48, INT4),
             (150, 16, FP32), (700, 128, INT4), (90, 256, INT8)]
    for row_alignment in (16, 4):
        for weighted in (False, True):
            weights, wo, tys, D_offsets, idx, off, psw = tbe_problem(rng, specs, B, max_L, row_alignment, weighted)
            T, total_D = len(specs), int(D_offsets[-1])
            for pooling in (0, 1):
                for out_ty in (FP32, FP16, BF16):
                    got = ops.int_nbit_split_embedding_codegen_lookup_function(
                        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
                        cu(D_offsets), total_D, 32, 256, 256, 256, 16, cu(idx), cu(off), pooling, None if psw is None else cu(psw),
                        out_ty, row_alignment=row_alignment, accumulate=ops.ACC_FAST)
                    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, psw, out_ty, row_alignment)
                    assert rc == 0
                    # per table, so that a table of small values is not held to another table's magnitudes
                    g = bits_of(got, out_ty).reshape(B, total_D)
                    for t in range(T):
                        c0, c1 = int(D_offsets[t]), int(D_offsets[t + 1])
                        check_grade(np.ascontiguousarray(g[:, c0:c1]), np.ascontiguousarray(want.reshape(B, total_D)[:, c0:c1]), out_ty, B,
                                    f"B={B} L<{max_L} align={row_alignment} w={weighted} pool={pooling} out={out_ty} table={t}")


@pytest.mark.parametrize("ty", [FP16, FP32, INT2])
def test_rows_without_fast_arithmetic_stay_exact_with_long_bags(ops, oracle, ty):
    """fp16 / fp32 / 2-bit rows are summed the reference's way in either mode. A call of few, long
    bags over them is not cut into segments either (4- and 8-bit rows of such a call are): the
    results stay bit-identical, for a single table and for a plan that holds one such table."""
    rng = np.random.default_rng(77 + ty)
    nb, rows, D, L = 3, 900, 128, 400
    table, _ = H.make_table(rng, ty, rows, D, False)
    idx, off, _ = H.make_bags(rng, rows, nb, L, np.int64, np.int32, fixed_len=L)
    kern = (ops.generate_embedding_spmdm_nbit_with_strides(2, D, False, False, 16, False, True, -1, -1, False) if ty == INT2 else
            ops.generate_embedding_spmdm_with_strides(ty, D, False, False, 16, False, True, -1, -1, False))
    out = torch.empty(nb * D, dtype=torch.float32, device="cuda")
    assert kern(nb, len(idx), rows, cu(table), cu(idx), cu(off), None, out, accumulate=ops.ACC_FAST)
    ok, want = oracle.spmdm(ty, D, table, idx, off, scale_bias_last=False, data_size=rows)
    assert ok
    H.assert_same_bits(out.cpu().numpy(), want, f"single table ty={ty}, fast mode, long bags")
    # the same kind of table beside 4-bit ones in a plan: no table of the plan is cut into segments
    specs = [(500, 128, INT4), (300, D, ty), (400, 256, INT4)]
    weights, wo, tys, D_offsets, idx, off, _ = tbe_problem(rng, specs, 2, 900, 16, False)
    T, total_D = len(specs), int(D_offsets[-1])
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
        cu(D_offsets), total_D, 128, 256, 0, 128, 128, cu(idx), cu(off), 0, None, FP32, row_alignment=16, accumulate=ops.ACC_FAST)
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP32, 16)
    assert rc == 0
    c0, c1 = int(D_offsets[1]), int(D_offsets[2])
    H.assert_same_bits(np.ascontiguousarray(got.cpu().numpy()[:, c0:c1]), np.ascontiguousarray(want.reshape(2, total_D)[:, c0:c1]),
                       f"table of ty={ty} in a fast-mode plan, long bags")


def test_int8_pooled_output_of_split_bags(ops, oracle):
    """The 8-bit pooled output of a tolerance-grade forward whose few, long bags are cut into
    segments: partial sums, the ordered combine into the plan's float scratch, then the quantizer
    over every (bag, table) block. The pooled floats are within the mode's bound of the oracle's, so
    every dequantized element is within half a quantization step (plus that bound) of the oracle's
    pooled value, and scale and bias are those of a vector within the bound."""
    rng = np.random.default_rng(4242)
    specs = [(500, 128, INT4), (300, 64, INT8), (700, 256, INT4)]
    T, B, L = len(specs), 5, 400
    weights, wo, tys, D_offsets, idx, off, _ = tbe_problem(rng, specs, B, L, 16, False)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
        cu(D_offsets), total_D, 0, maxd(INT4), maxd(INT8), 0, 0, cu(idx), cu(off), 0, None, INT8, row_alignment=16,
        accumulate=ops.ACC_FAST).cpu().numpy()
    assert got.shape == (B, total_D + 8 * T)
    rc, pooled = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP32, 16)
    assert rc == 0
    for t in range(T):
        D = specs[t][1]
        block = got[:, D_offsets[t] + 8 * t:D_offsets[t] + 8 * t + D + 8]
        want = pooled[:, D_offsets[t]:D_offsets[t + 1]].astype(np.float64)
        scale = np.ascontiguousarray(block[:, D:D + 4]).view(np.float32).astype(np.float64)
        bias = np.ascontiguousarray(block[:, D + 4:D + 8]).view(np.float32).astype(np.float64)
        mag = np.abs(want).max(axis=1, keepdims=True)
        rng_w = want.max(axis=1, keepdims=True) - want.min(axis=1, keepdims=True)
        assert np.all(np.abs(bias - want.min(axis=1, keepdims=True)) <= 1e-5 * mag), t
        assert np.all(np.abs(scale * 255.0 - rng_w) <= 4e-5 * mag), t
        deq = block[:, :D].astype(np.float64) * scale + bias
        assert np.all(np.abs(deq - want) <= 0.5 * scale + 4e-5 * mag), (t, np.abs(deq - want).max(), scale.max())


def test_rebuilding_rank_records_leaves_the_split_bag_scratch_alone(ops, oracle):
    """A plan that has cut long bags into segments (plan-owned scratch) and is then given its
    pruned-row mappings twice: building the compact mappings again replaces only what was made
    from the mappings, and the next forward of long bags gives the same bits as the first."""
    rng = np.random.default_rng(4242)
    logical = [900, 700]
    specs, maps = [], []
    for n in logical:
        keep = rng.random(n) < 0.6
        m = np.full(n, -1, np.int32)
        m[keep] = np.arange(int(keep.sum()), dtype=np.int32)
        maps.append(m)
        specs.append((int(keep.sum()), 128, INT4))
    T, B = len(specs), 2
    from test_tbe_gpu import build_weights
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.integers(600, 900, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, logical[t], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    remap = np.concatenate(maps)
    remap_off = np.concatenate([[0], np.cumsum([len(m) for m in maps])]).astype(np.int64)
    plan = ops.TbePlan(torch.from_numpy(wo), torch.from_numpy(tys), torch.from_numpy(D_offsets), torch.zeros(T, dtype=torch.int32),
                       len(weights), 0, 16)
    plan.set_accumulate(ops.ACC_FAST)
    d_remap, d_remap_off = cu(remap), cu(remap_off)
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 0, 128, 0, 0, 0, cu(idx), cu(off), 0, None, FP32, row_alignment=16, plan=plan,
        index_remappings=d_remap, index_remappings_offsets=d_remap_off).cpu().numpy()
    assert plan.set_index_remappings(d_remap, d_remap_off) == 2
    first = call()
    dense = oracle.pruned_array_lookup(idx, off, remap, remap_off)
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, dense, off, 0, None, FP32, 16)
    assert rc == 0
    check_grade(first, want, FP32, B, "long bags, first forward")
    assert plan.set_index_remappings(d_remap, d_remap_off) == 2  # the records are made again
    again = call()
    assert (again.view(np.uint32) == first.view(np.uint32)).all()
    del plan  # and the plan frees its scratch once


def test_configs_scaled_fast_mode(ops, oracle):
    """Configs 3, 4 (batched, pruned) and 5 at reduced size, in full, in the tolerance-grade mode."""
    from fbgemm_amd import bench_configs as bc
    for name, p in (("config3", bc.config3("cuda", scale=0.05)), ("config4", bc.config4_batched("cuda", scale=0.05)),
                    ("config5", bc.config5("cuda", scale=0.01, tables_int4=6, tables_int2=3))):
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            p.dev_weights, torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(p.T, np.int32)), cu(p.weights_offsets),
            cu(p.tys), cu(p.D_offsets), p.total_D, 32, 256, 256, 256, 0, p.indices, p.offsets, p.pooling_mode, p.indice_weights,
            p.output_dtype, row_alignment=p.row_alignment, index_remappings=p.extra.get("remap"),
            index_remappings_offsets=p.extra.get("remap_offsets"), accumulate=ops.ACC_FAST)
        rc, want = oracle.tbe_forward(p.dev_weights.cpu().numpy(), p.weights_offsets, p.tys, p.D_offsets, p.total_D,
                                      p.physical_indices, p.host_offsets, p.pooling_mode, p.host_weights, p.output_dtype,
                                      p.row_alignment)
        assert rc == 0
        g = bits_of(got, p.output_dtype).reshape(p.B, p.total_D)
        worst = 0
        for t in range(p.T):
            c0, c1 = int(p.D_offsets[t]), int(p.D_offsets[t + 1])
            worst = max(worst, check_grade(np.ascontiguousarray(g[:, c0:c1]), np.ascontiguousarray(want.reshape(p.B, p.total_D)[:, c0:c1]),
                                           p.output_dtype, p.B, f"{name} table {t}"))
        print(f"{name} (scaled) in the tolerance-grade mode: worst error {worst}")
