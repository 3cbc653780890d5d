"""Third opinion on the oracle: the reference's production AVX2/AVX-512 kernels
(generated at run time by fbgemm::GenerateEmbeddingSpMDM*WithStrides, reached
through the copy of the library inside libtorch_cpu.so). The reference's own
unit tests require these kernels to equal its scalar code bit for bit
(test/EmbeddingSpMDMNBitTest.cc:396, test/EmbeddingSpMDM8BitTest.cc), so the
oracle must equal them too."""
import numpy as np
import pytest

import helpers as H
from helpers import BF16, FP16, FP32, INT2, INT4, INT8


@pytest.fixture(scope="module")
def jit():
    try:
        from oracle import jit_baseline
        jit_baseline.lib()
    except Exception as e:  # libtorch without the fbgemm symbols, or no compiler
        pytest.skip(f"JIT bridge unavailable: {e}")
    return jit_baseline


@pytest.mark.parametrize("ty", [INT8, INT4, INT2, FP16, FP32])
@pytest.mark.parametrize("D", [4, 8, 32, 40, 64, 128, 164, 256])
def test_matches_jit_kernels(oracle, jit, ty, D):
    rng = np.random.default_rng(ty * 1000 + D)
    rows, nb = 500, 24
    for sbl in (True, False):
        for out_ty in (FP32, FP16, BF16):
            for weighted, normalize in ((False, False), (True, False), (False, True), (True, True)):
                if sbl:
                    table, stride = H.make_table(rng, ty, rows, D, True)
                else:
                    table, stride = H.make_table(rng, ty, rows, D, False,
                                                 stride_bytes=oracle.padded_row_bytes(D, ty, 16))
                idx, off, _ = H.make_bags(rng, rows, nb, 12, np.int64, np.int64, empty_frac=0.1)
                if not sbl:
                    idx[::5] = -1
                w = rng.uniform(0, 1, len(idx)).astype(np.float32) if weighted else None
                kw = dict(weights=w, normalize=normalize, out_ty=out_ty, output_stride=D + 8,
                          input_stride=H.input_stride_elems(ty, stride), scale_bias_last=sbl, data_size=rows)
                ok_o, out_o = oracle.spmdm(ty, D, table, idx, off, **kw)
                ok_j, out_j = jit.spmdm(ty, D, table, idx, off, **kw)
                assert ok_o and ok_j
                H.assert_same_bits(out_o, out_j, f"ty={ty} D={D} sbl={sbl} out={out_ty} w={weighted} n={normalize}")


def test_jit_rejections(oracle, jit):
    rng = np.random.default_rng(1)
    rows, D = 100, 32
    table, _ = H.make_table(rng, INT4, rows, D, True)
    idx, off, _ = H.make_bags(rng, rows, 8, 5, np.int64, np.int64)
    bad = idx.copy(); bad[3] = rows
    assert not jit.spmdm(INT4, D, table, bad, off, data_size=rows)[0]
    assert not oracle.spmdm(INT4, D, table, bad, off, data_size=rows)[0]
