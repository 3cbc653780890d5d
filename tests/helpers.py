"""Shared input builders for the tests: tables in the two row layouts of the
path, bags, and the three-way comparison (HIP library, oracle, reference)."""
import numpy as np

FP32, FP16, INT8, INT4, INT2, BF16 = 0, 1, 2, 3, 4, 5
QUANT = (INT8, INT4, INT2)
BITS = {FP32: 32, FP16: 16, BF16: 16, INT8: 8, INT4: 4, INT2: 2}


def packed_bytes(ty, D):
    return (D * BITS[ty] + 7) // 8


def default_stride_bytes(ty, D, scale_bias_last):
    if ty in QUANT:
        sb = 8 if (ty == INT8 and scale_bias_last) else 4
        return packed_bytes(ty, D) + sb
    return packed_bytes(ty, D)


def make_table(rng, ty, rows, D, scale_bias_last=True, stride_bytes=None,
               scale_range=(0.01, 0.1), bias_range=(-1.0, 1.0), ones=False):
    """Random table as a flat uint8 array of rows * stride_bytes bytes.

    Quantised rows get random packed bytes plus a sane (scale, bias); padding
    bytes are random too, so that a kernel reading them shows up."""
    stride = stride_bytes or default_stride_bytes(ty, D, scale_bias_last)
    tbl = rng.integers(0, 256, size=(rows, stride), dtype=np.uint8)
    pb = packed_bytes(ty, D)
    if ty in QUANT:
        scale = rng.uniform(*scale_range, size=rows).astype(np.float32)
        bias = rng.uniform(*bias_range, size=rows).astype(np.float32)
        if ones:  # every element dequantises to exactly 1.0: q = 1, scale = 1, bias = 0
            scale[:] = 1.0
            bias[:] = 0.0
            unit = {INT8: 0x01, INT4: 0x11, INT2: 0x55}[ty]
            data = np.full((rows, pb), unit, dtype=np.uint8)
        else:
            data = tbl[:, :pb].copy()
        if ty == INT8 and scale_bias_last:
            sb = np.stack([scale, bias], axis=1).view(np.uint8)  # two floats
        else:
            sb = np.stack([scale, bias], axis=1).astype(np.float16).view(np.uint8)
        if scale_bias_last:
            tbl[:, :pb] = data
            tbl[:, pb:pb + sb.shape[1]] = sb
        else:
            tbl[:, :sb.shape[1]] = sb
            tbl[:, sb.shape[1]:sb.shape[1] + pb] = data
    elif ty == FP32:
        vals = np.ones((rows, D), np.float32) if ones else rng.uniform(-1, 1, size=(rows, D)).astype(np.float32)
        tbl[:, :pb] = vals.view(np.uint8)
    elif ty == FP16:
        vals = np.ones((rows, D), np.float16) if ones else rng.uniform(-1, 1, size=(rows, D)).astype(np.float16)
        tbl[:, :pb] = vals.view(np.uint8)
    else:  # BF16: top halves of floats
        vals = np.ones((rows, D), np.float32) if ones else rng.uniform(-1, 1, size=(rows, D)).astype(np.float32)
        tbl[:, :pb] = (vals.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    return np.ascontiguousarray(tbl).reshape(-1), stride


def make_bags(rng, rows, num_bags, avg_len, idx_dtype=np.int64, off_dtype=np.int32,
              fixed_len=None, empty_frac=0.0):
    """lengths U[1, min(2*avg+1, rows)] like test/EmbeddingSpMDMTestUtils.cc:18-87,
    first index = rows - 1 to touch the bound."""
    if fixed_len is not None:
        lengths = np.full(num_bags, fixed_len, dtype=np.int64)
    else:
        hi = max(1, min(2 * avg_len + 1, rows))
        lengths = rng.integers(1, hi + 1, size=num_bags)
    if empty_frac > 0:
        lengths[rng.random(num_bags) < empty_frac] = 0
    total = int(lengths.sum())
    indices = rng.integers(0, rows, size=total).astype(idx_dtype)
    if total:
        indices[0] = rows - 1
    offsets = np.zeros(num_bags + 1, dtype=off_dtype)
    offsets[1:] = np.cumsum(lengths)
    return indices, offsets, lengths.astype(off_dtype)


def input_stride_elems(ty, stride_bytes):
    """Bytes -> the storage-element count the reference's input_stride uses."""
    if ty in (FP16, BF16):
        assert stride_bytes % 2 == 0
        return stride_bytes // 2
    if ty == FP32:
        assert stride_bytes % 4 == 0
        return stride_bytes // 4
    return stride_bytes


def assert_same_bits(a, b, what=""):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype, (a.shape, b.shape, a.dtype, b.dtype)
    av = a.view(np.uint32 if a.dtype == np.float32 else a.dtype)
    bv = b.view(np.uint32 if b.dtype == np.float32 else b.dtype)
    bad = np.nonzero(av != bv)[0] if av.ndim == 1 else np.argwhere(av != bv)
    assert len(bad) == 0, f"{what}: {len(bad)} of {av.size} elements differ, first at {bad[0]}: {a.flat[0] if a.size else None}"
