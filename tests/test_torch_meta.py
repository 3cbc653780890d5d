"""The torch operator library without a GPU: it loads, the schemas are the
reference's, and the shape functions (DispatchKey::Meta) give what the
reference's do (fbgemm_gpu/fbgemm_gpu/sparse_ops.py:503-581)."""
import os

import pytest

torch = pytest.importorskip("torch")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "fbgemm_amd", "lib", "libfbgemm_amd_torch.so")


@pytest.fixture(scope="module")
def fb():
    if not os.path.exists(LIB):
        from fbgemm_amd import build
        build.build_library()
        build.build_torch_op()
    torch.ops.load_library(LIB)
    return torch.ops.fbgemm


def meta(shape, dtype):
    return torch.empty(shape, dtype=dtype, device="meta")


def lookup(fb, pooling, out_ty, T=3, B=5, L=40, total_D=96, max_D=(0, 32, 64, 0, 0)):
    return fb.int_nbit_split_embedding_codegen_lookup_function(
        meta([1000], torch.uint8), meta([0], torch.uint8), meta([T], torch.int32), meta([T], torch.int64),
        meta([T], torch.uint8), meta([T + 1], torch.int32), total_D, *max_D, meta([L], torch.int32),
        meta([T * B + 1], torch.int32), pooling, None, out_ty)


def test_lookup_shapes(fb):
    for out_ty, dt in [(0, torch.float32), (1, torch.float16), (5, torch.bfloat16)]:
        out = lookup(fb, 0, out_ty)
        assert out.device.type == "meta" and tuple(out.shape) == (5, 96) and out.dtype == dt
        assert tuple(lookup(fb, 1, out_ty).shape) == (5, 96)
        seq = lookup(fb, 2, out_ty)
        assert tuple(seq.shape) == (40, 64) and seq.dtype == dt
    # rows copied as stored: 8-bit rows carry their 4 bytes of scale / bias
    assert tuple(lookup(fb, 2, 2).shape) == (40, 68) and lookup(fb, 2, 2).dtype == torch.uint8
    # pooled 8-bit output: every table's block carries 8 bytes of scale and bias
    q = lookup(fb, 0, 2)
    assert tuple(q.shape) == (5, 96 + 8 * 3) and q.dtype == torch.uint8
    with pytest.raises(RuntimeError):
        lookup(fb, 0, 3)


def test_remap_shapes_and_schemas(fb):
    idx, off = meta([17], torch.int64), meta([4], torch.int64)
    out = fb.pruned_array_lookup(idx, off, meta([100], torch.int32), meta([4], torch.int64))
    assert tuple(out.shape) == (17,) and out.dtype == torch.int64 and out.device.type == "meta"
    out = fb.pruned_hashmap_lookup(idx, off, meta([64, 2], torch.int64), meta([4], torch.int64))
    assert tuple(out.shape) == (17,) and out.dtype == torch.int64
    names = ["FloatToHFP8Quantized", "HFP8QuantizedToFloat", "embedding_bag_rowwise_prune", "bounds_check_indices",
             "FloatToFusedNBitRowwiseQuantizedSBHalf", "Fused8BitRowwiseQuantizedToFloat"]
    for n in names:
        assert getattr(fb, n).default._schema.name == f"fbgemm::{n}"
    assert str(fb.embedding_bag_rowwise_prune.default._schema) == (
        "fbgemm::embedding_bag_rowwise_prune(Tensor weight, Tensor indicator, float threshold, ScalarType "
        "compressed_indices_dtype, bool abs=True, SymInt min_num_rows=0, float? min_save_ratio=1.) -> (Tensor, Tensor)")
