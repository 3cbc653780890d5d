"""GPU parity of 8-bit float (hfp8) tables in the table-batched operator,
against the oracle's restatement of EmbeddingSpMDMFP8_ref, table by table the
way the reference's CPU operator runs them
(embedding_forward_quantized_cpu_template.cpp:476-479). Tolerance 0."""
import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("lane_shape")]
FP8 = 6


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    import fbgemm_amd.ops as o
    return o


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def build(rng, specs, oracle, align=16):
    blobs, offs, cur = [], [], 0
    for rows, D, ty in specs:
        rb = (D + align - 1) // align * align if ty == FP8 else oracle.padded_row_bytes(D, ty, align)
        if ty == FP8:
            tbl = rng.integers(0, 256, size=(rows, rb), dtype=np.uint8).reshape(-1)
        else:
            tbl, _ = H.make_table(rng, ty, rows, D, False, stride_bytes=rb)
        offs.append(cur)
        size = (tbl.size + 127) // 128 * 128
        blobs += [tbl, rng.integers(0, 256, size=size - tbl.size, dtype=np.uint8)]
        cur += size
    return np.concatenate(blobs), np.array(offs, np.int64)


@pytest.mark.parametrize("ebits,bias", [(4, 7), (5, 15)])
@pytest.mark.parametrize("out_ty", [FP32, FP16, BF16])
def test_fp8_tables_match_oracle(ops, oracle, ebits, bias, out_ty):
    rng = np.random.default_rng(7000 + ebits + out_ty)
    specs = [(300, 64, FP8), (200, 128, INT4), (150, 256, FP8), (90, 32, FP8), (70, 20, FP8), (60, 64, INT8)]
    T, B = len(specs), 19
    weights, wo = build(rng, specs, oracle)
    tys = np.array([s[2] for s in specs], np.uint8)
    Ds = [s[1] for s in specs]
    D_offsets = np.concatenate([[0], np.cumsum(Ds)]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.integers(0, 40, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int64)
    idx[rng.random(len(idx)) < 0.05] = -1
    psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    for pooling, w in ((0, psw), (1, None)):
        got = ops.int_nbit_split_embedding_codegen_lookup_function(
            cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), total_D, 0, maxd(INT4), maxd(INT8), 0, 0, cu(idx), cu(off), pooling,
            None if w is None else cu(w), out_ty, row_alignment=16, max_float8_D=maxd(FP8), fp8_exponent_bits=ebits,
            fp8_exponent_bias=bias).cpu()
        got = got.numpy() if out_ty == FP32 else got.view(torch.int16).numpy().view(np.uint16)
        for t, (rows, D, ty) in enumerate(specs):
            s, e = int(off[t * B]), int(off[(t + 1) * B])
            local_off = off[t * B:(t + 1) * B + 1] - off[t * B]
            if ty == FP8:
                rb = (D + 15) // 16 * 16
                ok, want = oracle.spmdm_fp8(D, weights[wo[t]:wo[t] + rows * rb], idx[s:e], local_off,
                                            weights=None if w is None else w[s:e], normalize=pooling == 1, out_ty=out_ty,
                                            input_stride=rb, exponent_bits=ebits, exponent_bias=bias,
                                            skip_minus_one=True, data_size=rows, output_size=B)
            else:
                rb = oracle.padded_row_bytes(D, ty, 16)
                ok, want = oracle.spmdm(ty, D, weights[wo[t]:wo[t] + rows * rb], idx[s:e], local_off,
                                        weights=None if w is None else w[s:e], normalize=pooling == 1, out_ty=out_ty,
                                        input_stride=rb, scale_bias_last=False, data_size=rows, output_size=B)
            assert ok
            H.assert_same_bits(np.ascontiguousarray(got[:, D_offsets[t]:D_offsets[t + 1]]).reshape(-1), want,
                               f"table {t} ty={ty} D={D} pooling={pooling} out={out_ty}")


def test_fp8_without_pooling_and_parameter_check(ops, oracle):
    rng = np.random.default_rng(7100)
    D = 48
    specs = [(100, D, FP8), (80, D, FP8)]
    T, B = 2, 7
    weights, wo = build(rng, specs, oracle)
    tys = np.full(T, FP8, np.uint8)
    D_offsets = (np.arange(T + 1) * D).astype(np.int32)
    lens = rng.integers(0, 6, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]).astype(np.int32)
    args = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
            cu(D_offsets), T * D, 0, 0, 0, 0, 0, cu(idx), cu(off))
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        *args, ops.POOL_NONE, None, FP32, row_alignment=16, max_float8_D=D, fp8_exponent_bits=4, fp8_exponent_bias=7)
    assert tuple(got.shape) == (len(idx), D)
    got = got.cpu().numpy()
    rb = 48
    for i, r in enumerate(idx.tolist()):
        t = 0 if i < int(off[B]) else 1
        row = weights[wo[t] + r * rb: wo[t] + r * rb + D]
        # a bag of one: fma(1, value, +0), so a negative zero comes out positive
        want = np.array([oracle.float8_to_float(b, 4, 7) for b in row], np.float32) + np.float32(0.0)
        assert (got[i].view(np.uint32) == want.view(np.uint32)).all()
    with pytest.raises(RuntimeError, match="fp8_exponent"):
        ops.int_nbit_split_embedding_codegen_lookup_function(*args, ops.POOL_SUM, None, FP32, row_alignment=16, max_float8_D=D)
