"""The two compiled host faces of the library on the GPU: the C++ factory
templates (include/fbgemm_amd_embedding.hpp, driven by tests/cpp/test_factories.cpp
against the C oracle) and the torch operator library that registers the
reference's schema."""
import os
import subprocess

import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_factories_against_oracle():
    exe = os.path.join(ROOT, "tests", "cpp", "_build", "test_factories")
    assert os.path.exists(exe), "build it with `python tests/cpp/build_cpp_tests.py`"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(proc.stdout[-3000:])
    assert proc.returncode == 0 and "PASSED" in proc.stdout


@pytest.fixture(scope="module")
def torch_ops():
    assert torch.cuda.is_available()
    lib = os.path.join(ROOT, "fbgemm_amd", "lib", "libfbgemm_amd_torch.so")
    assert os.path.exists(lib), "build it with `python -m fbgemm_amd.build`"
    torch.ops.load_library(lib)
    return torch.ops.fbgemm


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_registered_schema_is_the_references(torch_ops):
    schema = str(torch_ops.int_nbit_split_embedding_codegen_lookup_function.default._schema)
    assert schema == (
        "fbgemm::int_nbit_split_embedding_codegen_lookup_function(Tensor dev_weights, Tensor uvm_weights, "
        "Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys, Tensor D_offsets, SymInt total_D, "
        "int max_int2_D, int max_int4_D, int max_int8_D, int max_float16_D, int max_float32_D, Tensor indices, "
        "Tensor offsets, int pooling_mode, Tensor? indice_weights, int output_dtype=1, "
        "Tensor? lxu_cache_weights=None, Tensor? lxu_cache_locations=None, int? row_alignment=None, "
        "int? max_float8_D=0, int? fp8_exponent_bits=-1, int? fp8_exponent_bias=-1) -> Tensor")
    assert str(torch_ops.pruned_array_lookup.default._schema) == (
        "fbgemm::pruned_array_lookup(Tensor indices, Tensor offsets, Tensor index_remappings, "
        "Tensor index_remappings_offsets) -> Tensor")


def test_torch_operator_matches_oracle(torch_ops, oracle):
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(77)
    specs = [(300, 64, INT4), (200, 128, INT8), (100, 32, FP16), (150, 256, INT4), (80, 32, INT2), (60, 16, FP32)]
    T, B = len(specs), 29
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.integers(0, 30, size=T * B)
    for dt in (np.int32, np.int64):
        off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(dt)
        idx[rng.random(len(idx)) < 0.1] = -1
        psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
        for pooling, w, out_ty, tdt in ((0, psw, FP16, torch.float16), (1, None, FP32, torch.float32), (0, None, BF16, torch.bfloat16)):
            got = torch_ops.int_nbit_split_embedding_codegen_lookup_function(
                cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
                cu(D_offsets), total_D, 32, 256, 128, 32, 16, cu(idx), cu(off), pooling,
                None if w is None else cu(w), out_ty, None, None, 16)
            assert got.dtype == tdt and tuple(got.shape) == (B, total_D)
            rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, w, out_ty, 16)
            assert rc == 0
            g = got.cpu()
            g = g.numpy() if out_ty == FP32 else g.view(torch.int16).numpy().view(np.uint16)
            H.assert_same_bits(g, want, f"torch op dt={dt} pool={pooling} out={out_ty}")
    assert torch.ops.fbgemm_amd.lookup_status(cu(weights)) == 0
    # an out-of-range index is recorded, not fatal (the GPU operator of the reference does not check at all)
    bad = idx.copy(); bad[5] = 10**6
    out = torch_ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
        cu(D_offsets), total_D, 32, 256, 128, 32, 16, cu(bad), cu(off), 0, None, FP16, None, None, 16)
    assert torch.isfinite(out.float()).all()
    assert torch.ops.fbgemm_amd.lookup_status(cu(weights)) == 1
    assert torch.ops.fbgemm_amd.lookup_status(cu(weights)) == 0


def test_torch_pruned_array_lookup(torch_ops, oracle):
    rng = np.random.default_rng(5)
    T, B = 3, 9
    caps = [50, 0, 400]
    ro = np.concatenate([[0], np.cumsum(caps)]).astype(np.int64)
    remap = np.where(rng.random(int(ro[-1])) < 0.5, -1, rng.integers(0, 1000, int(ro[-1]))).astype(np.int32)
    lens = rng.integers(0, 8, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, caps[t] or 99, size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    got = torch_ops.pruned_array_lookup(cu(idx), cu(off), cu(remap), cu(ro)).cpu().numpy()
    assert (got == oracle.pruned_array_lookup(idx, off, remap, ro)).all()


def test_torch_bounds_check_and_hashmap(torch_ops, oracle):
    rng = np.random.default_rng(6)
    T, B = 5, 21
    rows = rng.integers(1, 500, size=T).astype(np.int64)
    lens = rng.integers(0, 9, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = rng.integers(-2, 600, size=int(off[-1])).astype(np.int64)
    off[7] = off[6] - 1 if off[6] > 0 else off[7]
    off[-1] += 3
    for mode in (1, 2):
        d_idx, d_off = cu(idx), cu(off)
        warning = torch.full((1,), 5, dtype=torch.int64, device="cuda")
        torch_ops.bounds_check_indices(cu(rows), d_idx, d_off, mode, warning)
        o_idx, o_off, o_warn = idx.copy(), off.copy(), np.full(1, 5, np.int64)
        assert oracle.bounds_check_indices(rows, o_idx, o_off, mode, o_warn) == 0
        assert (d_idx.cpu().numpy() == o_idx).all() and (d_off.cpu().numpy() == o_off).all()
        assert int(warning.item()) == int(o_warn[0])
    with pytest.raises(RuntimeError):
        torch_ops.bounds_check_indices(cu(rows), cu(idx), cu(off), 0, torch.zeros(1, dtype=torch.int64, device="cuda"))
    # hash map
    keys = rng.choice(3000, size=200, replace=False).astype(np.int64)
    hto = np.asarray([0, 401], np.int64)
    table = np.full((401, 2), -1, np.int64)
    oracle.pruned_hashmap_insert(keys, np.arange(200, dtype=np.int64), np.asarray([0, 200], np.int64), table, hto)
    q = rng.integers(0, 3000, size=300).astype(np.int64)
    qoff = np.asarray([0, 100, 300], np.int64)
    got = torch_ops.pruned_hashmap_lookup(cu(q), cu(qoff), cu(table), cu(hto)).cpu().numpy()
    assert (got == oracle.pruned_hashmap_lookup(q, qoff, table, hto)).all()


def test_torch_rowwise_quantize_ops(torch_ops, oracle):
    rng = np.random.default_rng(7)
    x = rng.normal(0, 1, size=(37, 128)).astype(np.float32)
    # 8-bit, fp32 scale/bias trailer
    q8 = torch_ops.FloatToFused8BitRowwiseQuantized(cu(x))
    want8 = oracle.quantize_rowwise(x, 8, True)
    assert tuple(q8.shape) == (37, 136) and (q8.cpu().numpy() == want8).all()
    qh = torch_ops.FloatOrHalfToFused8BitRowwiseQuantized(cu(x.astype(np.float16)))
    assert (qh.cpu().numpy() == oracle.quantize_rowwise(x.astype(np.float16), 8, True)).all()
    back = torch_ops.Fused8BitRowwiseQuantizedToFloat(q8)
    assert (back.cpu().numpy().view(np.uint32) == oracle.dequantize_rowwise(want8, 128, 8, True).view(np.uint32)).all()
    back16 = torch_ops.Fused8BitRowwiseQuantizedToHalf(q8)
    assert (back16.cpu().view(torch.int16).numpy().view(np.uint16) ==
            oracle.dequantize_rowwise(want8, 128, 8, True, out_ty=oracle.ST_FP16)).all()
    # 4- and 2-bit, fp16 scale/bias
    for bit_rate in (4, 2):
        qn = torch_ops.FloatToFusedNBitRowwiseQuantizedSBHalf(cu(x), bit_rate)
        wantn = oracle.quantize_rowwise(x, bit_rate)
        assert (qn.cpu().numpy() == wantn).all()
        for out_ty, tdt in ((oracle.ST_FP32, torch.float32), (oracle.ST_FP16, torch.float16), (oracle.ST_BF16, torch.bfloat16)):
            got = torch_ops.FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf(qn, bit_rate, out_ty)
            assert got.dtype == tdt
            want = oracle.dequantize_rowwise(wantn, 128, bit_rate, out_ty=out_ty)
            g = got.cpu().view(torch.int32 if out_ty == oracle.ST_FP32 else torch.int16).numpy()
            assert (g == want.view(g.dtype)).all()
    with pytest.raises(RuntimeError):
        torch_ops.FloatToFusedNBitRowwiseQuantizedSBHalf(cu(x[:, :3]), 4)


def test_torch_operator_without_pooling(torch_ops, oracle):
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(78)
    D = 64
    specs = [(120, D, INT4), (90, D, INT8), (70, D, FP16)]
    T, B = len(specs), 11
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    lens = rng.integers(0, 6, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    got = torch_ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
        cu(D_offsets), T * D, 0, D, D, D, 0, cu(idx), cu(off), 2, None, FP16, None, None, 16)
    ok, want = oracle.tbe_forward_nobag(weights, wo, tys, [s[0] for s in specs], D, idx, off, FP16, 16)
    assert ok and tuple(got.shape) == (len(idx), D)
    H.assert_same_bits(got.cpu().view(torch.int16).numpy().view(np.uint16), want, "torch op, no pooling")
