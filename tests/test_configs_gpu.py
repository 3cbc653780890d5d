"""The five benchmark configurations on the GPU. Configs 1, 2 and 4 (a table
subset) are checked in full against the oracle; config 3 at its real size on
sampled tables plus size-independent properties (determinism, independence of
a bag from the rest of the batch, exact zeros for empty bags); config 5 at
1/100 scale in full (its real size is exercised by bench.py --config 5 --check)."""
import numpy as np
import pytest

import helpers as H

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    import fbgemm_amd.ops as o
    return o


def bits_of(t, out_ty):
    t = t.cpu()
    return t.numpy() if out_ty == 0 else t.view(torch.int16).numpy().view(np.uint16)


def run_spmdm_problem(ops, p):
    out = torch.empty(p.num_bags * p.D, dtype={0: torch.float32, 1: torch.float16, 5: torch.bfloat16}[p.out_ty], device="cuda")
    if p.remap is not None:
        kern = ops.generate_embedding_spmdm_nbit_rowwise_sparse(4, p.D, False, p.normalize)
        ok = kern(p.num_bags, p.lookups, p.data_size, p.table, p.indices, p.offsets, None, out, p.remap)
    elif p.ty == 2:
        kern = ops.generate_embedding_spmdm(ops.INT8, p.D, False, p.normalize, out_ty=p.out_ty)
        ok = kern(p.num_bags, p.lookups, p.data_size, p.table, p.indices, p.offsets, None, out)
    else:
        kern = ops.generate_embedding_spmdm_nbit(4, p.D, False, p.normalize, out_ty=p.out_ty)
        ok = kern(p.num_bags, p.lookups, p.data_size, p.table, p.indices, p.offsets, None, out)
    return ok, out


def check_spmdm_problem(ops, oracle, p):
    ok, out = run_spmdm_problem(ops, p)
    ok_o, want = oracle.spmdm(p.ty, p.D, p.table.cpu().numpy(), p.host_indices, p.host_offsets,
                              normalize=p.normalize, out_ty=p.out_ty, remap=p.host_remap, data_size=p.data_size)
    assert ok and ok_o
    H.assert_same_bits(bits_of(out, p.out_ty), want, p.name)


def test_config1_full(ops, oracle):
    from fbgemm_amd import bench_configs as bc
    check_spmdm_problem(ops, oracle, bc.config1("cuda"))


def test_config2_full(ops, oracle):
    from fbgemm_amd import bench_configs as bc
    check_spmdm_problem(ops, oracle, bc.config2("cuda"))


def test_config4_two_tables_full(ops, oracle):
    from fbgemm_amd import bench_configs as bc
    for p in bc.config4("cuda", tables=2):
        check_spmdm_problem(ops, oracle, p)
        kept = int((p.host_remap[p.host_indices] != -1).sum())
        assert 0.3 < kept / p.lookups < 0.7  # pruned rows are hit at the base rate


def tbe_forward(ops, p, indices=None, offsets=None, weights="same"):
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    w = p.indice_weights if weights == "same" else weights
    return ops.int_nbit_split_embedding_codegen_lookup_function(
        p.dev_weights, torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(p.T, np.int32)),
        cu(p.weights_offsets), cu(p.tys), cu(p.D_offsets), p.total_D, 32, 256, 256, 256, 0,
        p.indices if indices is None else indices, p.offsets if offsets is None else offsets, p.pooling_mode, w,
        p.output_dtype, row_alignment=p.row_alignment)


def oracle_table(oracle, p, t):
    s, e = int(p.host_offsets[t * p.B]), int(p.host_offsets[(t + 1) * p.B])
    ty = int(p.tys[t])
    elem = 4 if ty == 0 else 2 if ty == 1 else 1
    ok, want = oracle.spmdm(ty, int(p.Ds[t]), p.table_host_bytes(t), p.host_indices[s:e],
                            p.host_offsets[t * p.B:(t + 1) * p.B + 1] - p.host_offsets[t * p.B],
                            weights=None if p.host_weights is None else p.host_weights[s:e],
                            normalize=p.pooling_mode == 1, out_ty=p.output_dtype,
                            input_stride=int(p.row_bytes[t]) // elem, scale_bias_last=False,
                            data_size=int(p.rows[t]), output_size=p.B)
    assert ok
    return want.reshape(p.B, int(p.Ds[t]))


def test_config3_full_size(ops, oracle):
    from fbgemm_amd import bench_configs as bc
    p = bc.config3("cuda")
    out = tbe_forward(ops, p)
    got = bits_of(out, p.output_dtype)
    # one table of every (type, D) combination present, against the oracle
    seen = {}
    for t in range(p.T):
        seen.setdefault((int(p.tys[t]), int(p.Ds[t])), t)
    for t in sorted(seen.values()):
        c0, c1 = int(p.D_offsets[t]), int(p.D_offsets[t + 1])
        H.assert_same_bits(np.ascontiguousarray(got[:, c0:c1]), oracle_table(oracle, p, t), f"config3 table {t}")
    # determinism: the bag order inside the scheduler may differ between runs, the bits may not
    assert torch.equal(out, tbe_forward(ops, p))
    # a bag's result does not depend on the rest of the batch: reverse the bag order of every table
    B, T = p.B, p.T
    lens = p.lengths.reshape(T, B)
    rev_lens = lens[:, ::-1].reshape(-1)
    rev_off = np.concatenate([[0], np.cumsum(rev_lens)]).astype(np.int64)
    starts = p.host_offsets[:-1].reshape(T, B)[:, ::-1].reshape(-1)
    gather = np.concatenate([np.arange(s, s + l) for s, l in zip(starts, rev_lens)])
    rev_idx = p.host_indices[gather]
    rev_w = p.host_weights[gather]
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out_rev = tbe_forward(ops, p, cu(rev_idx), cu(rev_off), cu(rev_w))
    assert torch.equal(out_rev.flip(0), out)
    # empty bags are exact zeros
    empty = np.nonzero(lens == 0)
    for t, b in zip(*empty):
        assert (got[b, int(p.D_offsets[t]):int(p.D_offsets[t + 1])] == 0).all()


def test_config5_scaled(ops, oracle):
    from fbgemm_amd import bench_configs as bc
    p = bc.config5("cuda", scale=0.01, tables_int4=6, tables_int2=3)
    out = tbe_forward(ops, p)
    rc, want = oracle.tbe_forward(p.dev_weights.cpu().numpy(), p.weights_offsets, p.tys, p.D_offsets, p.total_D,
                                  p.host_indices, p.host_offsets, p.pooling_mode, None, p.output_dtype, p.row_alignment)
    assert rc == 0
    H.assert_same_bits(bits_of(out, p.output_dtype), want, "config5 @ 0.01")
