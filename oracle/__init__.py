"""TEST INFRASTRUCTURE ONLY: ctypes front-end of the CPU checkers.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this
package; the shipped library never does.

Two back-ends expose the same call:
  * ``impl="oracle"``: our C restatement (oracle/embedding_oracle.c).
  * ``impl="ref"``: the reference's own scalar code, compiled from its
    sources by ``make -C oracle ref`` into oracle/_ref/ (present only where it
    was built).
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "_build", "libembedding_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libfbgemm_ref.so")
REF_QUANT_SO = os.path.join(HERE, "_ref", "libfbgemm_ref_quant.so")
JIT_SO = os.path.join(HERE, "_build", "libfbgemm_jit_bridge.so")

ST_FP32, ST_FP16, ST_INT8, ST_INT4, ST_INT2, ST_BF16 = 0, 1, 2, 3, 4, 5
POOL_SUM, POOL_MEAN = 0, 1

_c = ctypes
_SPMDM_ARGS = [
    _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p,
    _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int,
    _c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p,
]
_REMAP_ARGS = [
    _c.c_int32, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p,
    _c.c_void_p, _c.c_void_p, _c.c_void_p,
]


def build(targets=("oracle",)):
    """Compile the requested checker libraries (gcc/g++ only)."""
    subprocess.check_call(["make", "-s", "-C", HERE, *targets])


_libs = {}


def _lib(impl):
    if impl in _libs:
        return _libs[impl]
    if impl == "oracle":
        if not os.path.exists(ORACLE_SO):
            build(("oracle",))
        lib = _c.CDLL(ORACLE_SO)
        lib.oracle_embedding_spmdm.argtypes = _SPMDM_ARGS
        lib.oracle_embedding_spmdm.restype = _c.c_int
        lib.oracle_compressed_indices_remap.argtypes = _REMAP_ARGS
        lib.oracle_compressed_indices_remap.restype = None
        lib.oracle_pruned_array_lookup.argtypes = [
            _c.c_int32, _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p,
            _c.c_int, _c.c_void_p, _c.c_void_p]
        lib.oracle_pruned_array_lookup.restype = None
        lib.oracle_tbe_forward.argtypes = [
            _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32,
            _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int,
            _c.c_void_p, _c.c_int, _c.c_int64, _c.c_void_p]
        lib.oracle_tbe_forward.restype = _c.c_int
        lib.oracle_padded_row_bytes.argtypes = [_c.c_int32, _c.c_int, _c.c_int32, _c.c_int32]
        lib.oracle_padded_row_bytes.restype = _c.c_int32
        lib.oracle_bounds_check_indices.argtypes = [
            _c.c_void_p, _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64,
            _c.c_int, _c.c_void_p, _c.c_void_p]
        lib.oracle_bounds_check_indices.restype = _c.c_int
        lib.oracle_pruned_hash32.argtypes = [_c.c_uint32]
        lib.oracle_pruned_hash32.restype = _c.c_uint32
        lib.oracle_pruned_hash64.argtypes = [_c.c_uint64]
        lib.oracle_pruned_hash64.restype = _c.c_uint64
        lib.oracle_pruned_hashmap_insert.argtypes = [
            _c.c_int32, _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p,
            _c.c_int, _c.c_void_p]
        lib.oracle_pruned_hashmap_insert.restype = _c.c_int
        lib.oracle_pruned_hashmap_lookup.argtypes = [
            _c.c_int32, _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int,
            _c.c_void_p, _c.c_void_p]
        lib.oracle_pruned_hashmap_lookup.restype = None
        lib.oracle_quantize_rowwise.argtypes = [
            _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_void_p]
        lib.oracle_quantize_rowwise.restype = None
        lib.oracle_quantize_rowwise_min_max.argtypes = lib.oracle_quantize_rowwise.argtypes + [_c.c_void_p]
        lib.oracle_quantize_rowwise_min_max.restype = None
        lib.oracle_dequantize_rowwise.argtypes = [
            _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_void_p]
        lib.oracle_dequantize_rowwise.restype = None
    elif impl == "ref":
        if not os.path.exists(REF_SO):
            raise FileNotFoundError(REF_SO)
        lib = _c.CDLL(REF_SO)
        lib.ref_embedding_spmdm.argtypes = _SPMDM_ARGS
        lib.ref_embedding_spmdm.restype = _c.c_int
        lib.ref_compressed_indices_remap.argtypes = _REMAP_ARGS
        lib.ref_compressed_indices_remap.restype = None
    elif impl == "refquant":
        if not os.path.exists(REF_QUANT_SO):
            raise FileNotFoundError(REF_QUANT_SO)
        # lazy binding: of the reference's vector translation units only the AVX2 quantizers
        # are part of this build, and nothing that is called here reaches the others
        lib = _c.CDLL(REF_QUANT_SO, mode=os.RTLD_LAZY)
        lib.ref_quantize_nbit.argtypes = [_c.c_int, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int, _c.c_void_p]
        lib.ref_quantize_8bit.argtypes = [_c.c_void_p, _c.c_int, _c.c_int64, _c.c_int, _c.c_void_p]
        lib.ref_dequantize_nbit.argtypes = [_c.c_int, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_int, _c.c_void_p]
        lib.ref_dequantize_8bit.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int, _c.c_int, _c.c_void_p]
        lib.ref_quantize_nbit_avx2.argtypes = lib.ref_quantize_nbit.argtypes + [_c.c_void_p]
        lib.ref_quantize_8bit_avx2.argtypes = lib.ref_quantize_8bit.argtypes + [_c.c_void_p]
        for f in (lib.ref_quantize_nbit, lib.ref_quantize_8bit, lib.ref_dequantize_nbit, lib.ref_dequantize_8bit,
                  lib.ref_quantize_nbit_avx2, lib.ref_quantize_8bit_avx2):
            f.restype = None
    else:
        raise ValueError(impl)
    _libs[impl] = lib
    return lib


def have_ref_quant():
    return os.path.exists(REF_QUANT_SO)


def have_ref():
    return os.path.exists(REF_SO)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_c.c_void_p)


def _is64(a):
    if a.dtype == np.int64:
        return 1
    if a.dtype == np.int32:
        return 0
    raise TypeError(f"index arrays must be int32 or int64, got {a.dtype}")


def out_dtype(out_ty):
    return np.float32 if out_ty == ST_FP32 else np.uint16


def spmdm(in_ty, block_size, table, indices, offsets_or_lengths, *, weights=None,
          normalize=False, out_ty=ST_FP32, positional=False, use_offsets=True,
          output_stride=-1, input_stride=-1, scale_bias_last=True, remap=None,
          data_size, output_size=None, index_size=None, impl="oracle", out=None):
    """Pooled lookup on the CPU. Returns (ok, out); fp16/bf16 outputs are the
    raw 16-bit patterns (uint16). ``out`` may be passed in to observe which
    positions the call leaves untouched."""
    table = np.ascontiguousarray(table)
    indices = np.ascontiguousarray(indices)
    offsets_or_lengths = np.ascontiguousarray(offsets_or_lengths)
    if output_size is None:
        output_size = len(offsets_or_lengths) - (1 if use_offsets else 0)
    if index_size is None:
        index_size = len(indices)
    stride = block_size if output_stride == -1 else output_stride
    if out is None:
        out = np.zeros(max(output_size, 0) * stride, dtype=out_dtype(out_ty))
    if weights is not None:
        weights = np.ascontiguousarray(weights, dtype=np.float32)
    if remap is not None:
        remap = np.ascontiguousarray(remap, dtype=np.int32)
    lib = _lib(impl)
    fn = lib.oracle_embedding_spmdm if impl == "oracle" else lib.ref_embedding_spmdm
    ok = fn(in_ty, block_size, output_size, index_size, data_size, _ptr(table),
            _ptr(indices), _is64(indices), _ptr(offsets_or_lengths),
            _is64(offsets_or_lengths), _ptr(weights), int(normalize), _ptr(out), out_ty,
            int(positional), int(use_offsets), output_stride, input_stride,
            int(scale_bias_last), _ptr(remap))
    return bool(ok), out


def float8_to_float(b, exponent_bits, exponent_bias, impl="oracle"):
    lib = _lib(impl)
    fn = lib.oracle_float8_to_float if impl == "oracle" else lib.ref_float8_to_float
    fn.restype = _c.c_float
    fn.argtypes = [_c.c_uint8, _c.c_int, _c.c_int]
    return fn(int(b), exponent_bits, exponent_bias)


def hfp8_max_pos(exponent_bits, exponent_bias):
    fn = _lib("oracle").oracle_hfp8_max_pos
    fn.restype = _c.c_float
    fn.argtypes = [_c.c_int, _c.c_int]
    return fn(exponent_bits, exponent_bias)


def float_to_hfp8(x, exponent_bits, exponent_bias, max_pos=None, impl="oracle"):
    """fp32 array -> hfp8 codes (uint8). ``impl="ref"`` is the reference's FloatToFloat8_ref,
    which computes max_pos itself."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib = _lib(impl)
    if impl == "oracle":
        if max_pos is None:
            max_pos = hfp8_max_pos(exponent_bits, exponent_bias)
        fn = lib.oracle_float_to_hfp8_array
        fn.restype = None
        fn.argtypes = [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_int, _c.c_float]
        fn(_ptr(x), _ptr(out), x.size, exponent_bits, exponent_bias, max_pos)
    else:
        assert max_pos is None
        fn = lib.ref_float_to_float8_array
        fn.restype = None
        fn.argtypes = [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_int]
        fn(_ptr(x), _ptr(out), x.size, exponent_bits, exponent_bias)
    return out


def spmdm_fp8(block_size, table, indices, offsets_or_lengths, *, weights=None, normalize=False, out_ty=ST_FP32,
              positional=False, use_offsets=True, output_stride=-1, input_stride=-1, exponent_bits=4,
              exponent_bias=7, skip_minus_one=False, data_size, output_size=None, impl="oracle"):
    """Pooled lookup over 8-bit float rows (EmbeddingSpMDMFP8_ref). ``impl="ref"`` takes int64 indices / offsets."""
    table = np.ascontiguousarray(table, dtype=np.uint8)
    indices = np.ascontiguousarray(indices)
    offsets_or_lengths = np.ascontiguousarray(offsets_or_lengths)
    if output_size is None:
        output_size = len(offsets_or_lengths) - (1 if use_offsets else 0)
    stride = block_size if output_stride == -1 else output_stride
    out = np.zeros(max(output_size, 0) * stride, dtype=out_dtype(out_ty))
    if weights is not None:
        weights = np.ascontiguousarray(weights, dtype=np.float32)
    lib = _lib(impl)
    if impl == "oracle":
        fn = lib.oracle_embedding_spmdm_fp8
        fn.restype = _c.c_int
        fn.argtypes = [_c.c_int64] * 4 + [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p,
                                          _c.c_int, _c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_int64, _c.c_int64,
                                          _c.c_int, _c.c_int, _c.c_int]
        ok = fn(block_size, output_size, len(indices), data_size, _ptr(table), _ptr(indices), _is64(indices),
                _ptr(offsets_or_lengths), _is64(offsets_or_lengths), _ptr(weights), int(normalize), _ptr(out), out_ty,
                int(positional), int(use_offsets), output_stride, input_stride, exponent_bits, exponent_bias,
                int(skip_minus_one))
    else:
        assert indices.dtype == np.int64 and offsets_or_lengths.dtype == np.int64 and not skip_minus_one
        fn = lib.ref_embedding_spmdm_fp8
        fn.restype = _c.c_int
        fn.argtypes = [_c.c_int64] * 4 + [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p,
                                          _c.c_int, _c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int]
        ok = fn(block_size, output_size, len(indices), data_size, _ptr(table), _ptr(indices), _ptr(offsets_or_lengths),
                _ptr(weights), int(normalize), _ptr(out), out_ty, int(positional), int(use_offsets), output_stride,
                input_stride, exponent_bits, exponent_bias)
    return bool(ok), out


def spmdm_nobag(in_ty, block_size, table, indices, *, weights=None, out_ty=ST_FP32, output_stride=-1, input_stride=-1,
                scale_bias_last=True, data_size, impl="oracle", out=None):
    """One output row per index (the no_bag mode of EmbeddingSpMDM_ref / EmbeddingSpMDMNBit_ref).
    out_ty ST_INT8 (8-bit rows) / ST_INT4 (4-bit rows) copy row bytes; the result is then uint8.
    Returns (ok, out) with out flat, output rows output_stride (INT4: input_stride) elements apart."""
    table = np.ascontiguousarray(table)
    indices = np.ascontiguousarray(indices)
    n = len(indices)
    if in_ty in (ST_INT4, ST_INT2):
        stride = (block_size + 1) // 2 + 4 if input_stride == -1 else input_stride
    else:
        stride = block_size if output_stride == -1 else output_stride
    if out is None:
        out = np.zeros(n * stride, dtype=np.uint8 if out_ty in (ST_INT8, ST_INT4) else out_dtype(out_ty))
    if weights is not None:
        weights = np.ascontiguousarray(weights, dtype=np.float32)
    lib = _lib(impl)
    if impl == "oracle":
        fn = lib.oracle_embedding_spmdm_nobag
        fn.restype = _c.c_int
        fn.argtypes = [_c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p,
                       _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int]
        ok = fn(in_ty, block_size, n, data_size, _ptr(table), _ptr(indices), _is64(indices), _ptr(weights), _ptr(out),
                out_ty, output_stride, input_stride, int(scale_bias_last))
    else:
        assert indices.dtype == np.int64
        fn = lib.ref_embedding_spmdm_nobag
        fn.restype = _c.c_int
        fn.argtypes = [_c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
                       _c.c_int, _c.c_int64, _c.c_int64, _c.c_int]
        ok = fn(in_ty, block_size, n, data_size, _ptr(table), _ptr(indices), _ptr(weights), _ptr(out), out_ty,
                output_stride, input_stride, int(scale_bias_last))
    return bool(ok), out


def compressed_indices_remap(indices, mapping, offsets, weights=None, impl="oracle"):
    """Compacting remap. Returns (out_indices[:n], out_offsets, out_weights[:n])."""
    indices = np.ascontiguousarray(indices)
    offsets = np.ascontiguousarray(offsets, dtype=indices.dtype)
    mapping = np.ascontiguousarray(mapping, dtype=np.int32)
    out_idx = np.zeros_like(indices)
    out_off = np.zeros_like(offsets)
    out_w = None
    if weights is not None:
        weights = np.ascontiguousarray(weights, dtype=np.float32)
        out_w = np.zeros_like(weights)
    lib = _lib(impl)
    fn = (lib.oracle_compressed_indices_remap if impl == "oracle"
          else lib.ref_compressed_indices_remap)
    fn(len(offsets), _ptr(indices), _is64(indices), _ptr(mapping), _ptr(offsets),
       _ptr(weights), _ptr(out_idx), _ptr(out_off), _ptr(out_w))
    n = int(out_off[-1])
    return out_idx[:n], out_off, (None if out_w is None else out_w[:n])


def pruned_array_lookup(indices, offsets, remap, remap_offsets):
    indices = np.ascontiguousarray(indices)
    offsets = np.ascontiguousarray(offsets, dtype=indices.dtype)
    remap = np.ascontiguousarray(remap)
    remap_offsets = np.ascontiguousarray(remap_offsets, dtype=np.int64)
    T = len(remap_offsets) - 1
    B = (len(offsets) - 1) // T
    dense = np.empty_like(indices)
    _lib("oracle").oracle_pruned_array_lookup(
        T, B, _ptr(indices), _ptr(offsets), _is64(indices), _ptr(remap), _is64(remap),
        _ptr(remap_offsets), _ptr(dense))
    return dense


def pruned_array_lookup_from_row_idx(update_row_indices, update_table_indices, remap, remap_offsets):
    rows = np.ascontiguousarray(update_row_indices)
    tables = np.ascontiguousarray(update_table_indices, dtype=np.int32)
    remap = np.ascontiguousarray(remap)
    remap_offsets = np.ascontiguousarray(remap_offsets, dtype=np.int64)
    dense = np.empty_like(rows)
    fn = _lib("oracle").oracle_pruned_array_lookup_from_row_idx
    fn.restype = None
    fn.argtypes = [_c.c_int64, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p]
    fn(len(rows), _ptr(rows), _is64(rows), _ptr(tables), _ptr(remap), _is64(remap), _ptr(remap_offsets), _ptr(dense))
    return dense


def emb_inplace_update(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys, D_offsets,
                       update_weights, update_table_indices, update_row_indices, update_offsets, row_alignment):
    """In place on ``dev_weights`` / ``uvm_weights`` (contiguous uint8 arrays), updates applied in order."""
    assert dev_weights.flags.c_contiguous and uvm_weights.flags.c_contiguous
    assert dev_weights.dtype == np.uint8 and uvm_weights.dtype == np.uint8
    wp = np.ascontiguousarray(weights_placements, dtype=np.int32)
    wo = np.ascontiguousarray(weights_offsets, dtype=np.int64)
    wt = np.ascontiguousarray(weights_tys, dtype=np.uint8)
    do = np.ascontiguousarray(D_offsets, dtype=np.int32)
    uw = np.ascontiguousarray(update_weights, dtype=np.uint8)
    ut = np.ascontiguousarray(update_table_indices, dtype=np.int32)
    ur = np.ascontiguousarray(update_row_indices)
    uo = np.ascontiguousarray(update_offsets, dtype=np.int64)
    fn = _lib("oracle").oracle_emb_inplace_update
    fn.restype = None
    fn.argtypes = [_c.c_void_p] * 9 + [_c.c_int, _c.c_void_p, _c.c_int64, _c.c_int64]
    fn(_ptr(dev_weights), _ptr(uvm_weights), _ptr(wp), _ptr(wo), _ptr(wt), _ptr(do), _ptr(uw), _ptr(ut), _ptr(ur),
       _is64(ur), _ptr(uo), len(ur), int(row_alignment))


BOUNDS_FATAL, BOUNDS_WARNING, BOUNDS_IGNORE = 0, 1, 2


def bounds_check_indices(rows_per_table, indices, offsets, mode, warning, B_offsets=None):
    """In place on ``indices`` / ``offsets`` / ``warning`` (numpy arrays, index
    arrays of one dtype). Returns 0, or the condition a FATAL run stops at."""
    rows_per_table = np.ascontiguousarray(rows_per_table, dtype=np.int64)
    assert indices.flags.c_contiguous and offsets.flags.c_contiguous and offsets.dtype == indices.dtype
    assert warning.dtype == np.int64
    bo = None if B_offsets is None else np.ascontiguousarray(B_offsets, dtype=np.int32)
    return _lib("oracle").oracle_bounds_check_indices(
        _ptr(rows_per_table), len(rows_per_table), _ptr(indices), _ptr(offsets), _is64(indices),
        indices.size, offsets.size, int(mode), _ptr(warning), _ptr(bo))


def rowwise_prune(weights, indicator, threshold, index_dtype=np.int32, use_abs=True, min_non_pruned_rows=0):
    """embedding_bag_rowwise_prune without its min_save_ratio early exit: returns (kept rows, remap)."""
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    indicator = np.ascontiguousarray(indicator, dtype=np.float32)
    rows, cols = weights.shape
    remap = np.empty(rows, dtype=index_dtype)
    out = np.empty((rows, cols), dtype=np.float32)
    fn = _lib("oracle").oracle_rowwise_prune
    fn.restype = _c.c_int64
    fn.argtypes = [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_double, _c.c_int, _c.c_int64, _c.c_int,
                   _c.c_void_p, _c.c_void_p]
    kept = fn(_ptr(weights), _ptr(indicator), rows, cols, float(threshold), int(use_abs), int(min_non_pruned_rows),
              _is64(remap), _ptr(remap), _ptr(out))
    return out[:kept].copy(), remap


def pruned_hash(x, bits):
    lib = _lib("oracle")
    return lib.oracle_pruned_hash64(x) if bits == 64 else lib.oracle_pruned_hash32(x)


def pruned_hashmap_insert(indices, dense_indices, offsets, hash_table, hash_table_offsets):
    """In place on ``hash_table`` ([slots, 2] int32 or int64, -1 = empty)."""
    indices = np.ascontiguousarray(indices)
    dense_indices = np.ascontiguousarray(dense_indices, dtype=indices.dtype)
    offsets = np.ascontiguousarray(offsets, dtype=indices.dtype)
    hto = np.ascontiguousarray(hash_table_offsets, dtype=np.int64)
    assert hash_table.flags.c_contiguous and hash_table.ndim == 2 and hash_table.shape[1] == 2
    T = len(hto) - 1
    B = (len(offsets) - 1) // T
    rc = _lib("oracle").oracle_pruned_hashmap_insert(
        T, B, _ptr(indices), _ptr(dense_indices), _ptr(offsets), _is64(indices), _ptr(hash_table),
        _is64(hash_table), _ptr(hto))
    if rc:
        raise RuntimeError("hash table full")


def pruned_hashmap_lookup(indices, offsets, hash_table, hash_table_offsets):
    indices = np.ascontiguousarray(indices)
    offsets = np.ascontiguousarray(offsets, dtype=indices.dtype)
    hto = np.ascontiguousarray(hash_table_offsets, dtype=np.int64)
    hash_table = np.ascontiguousarray(hash_table)
    T = len(hto) - 1
    B = (len(offsets) - 1) // T
    dense = np.empty_like(indices)
    _lib("oracle").oracle_pruned_hashmap_lookup(
        T, B, _ptr(indices), _ptr(offsets), _is64(indices), _ptr(hash_table), _is64(hash_table),
        _ptr(hto), _ptr(dense))
    return dense


LAYOUT_TRAILER, LAYOUT_TBE = 0, 1


def quantized_row_bytes(cols, bit_rate, sb_float, layout):
    epb = 8 // bit_rate
    return (cols + epb - 1) // epb + (8 if (sb_float and layout == LAYOUT_TRAILER) else 4)


def quantize_rowwise(x, bit_rate, sb_float=False, layout=LAYOUT_TRAILER, out_stride=None, impl="oracle", fill=0,
                     min_max=None):
    """x: [rows, cols] float32 or float16 (numpy). Returns uint8 [rows, out_stride].
    impl: "oracle", "ref" (the reference's scalar routine, trailer layout only) or "ref_avx2"
    (the reference's AVX2 routine, trailer layout only). min_max: [rows, 2] of x's dtype, the
    extremes to use in place of each row's own ("oracle" and "ref_avx2" only)."""
    x = np.ascontiguousarray(x)
    assert x.ndim == 2 and x.dtype in (np.float32, np.float16)
    rows, cols = x.shape
    if min_max is not None:
        min_max = np.ascontiguousarray(min_max)
        assert min_max.dtype == x.dtype and min_max.shape == (rows, 2)
    need = quantized_row_bytes(cols, bit_rate, sb_float, layout)
    out_stride = need if out_stride is None else out_stride
    out = np.full((rows, out_stride), fill, np.uint8)
    half = int(x.dtype == np.float16)
    if impl == "oracle":
        _lib("oracle").oracle_quantize_rowwise_min_max(_ptr(x), half, rows, cols, bit_rate, int(sb_float), layout,
                                                       out_stride, _ptr(out),
                                                       None if min_max is None else _ptr(min_max))
    elif impl == "ref_avx2":
        assert layout == LAYOUT_TRAILER and out_stride == need
        mm = None if min_max is None else _ptr(min_max)
        if sb_float:
            _lib("refquant").ref_quantize_8bit_avx2(_ptr(x), half, rows, cols, _ptr(out), mm)
        else:
            _lib("refquant").ref_quantize_nbit_avx2(bit_rate, _ptr(x), half, rows, cols, _ptr(out), mm)
    else:
        assert layout == LAYOUT_TRAILER and out_stride == need and min_max is None
        if sb_float:
            _lib("refquant").ref_quantize_8bit(_ptr(x), half, rows, cols, _ptr(out))
        else:
            _lib("refquant").ref_quantize_nbit(bit_rate, _ptr(x), half, rows, cols, _ptr(out))
    return out


def dequantize_rowwise(q, cols, bit_rate, sb_float=False, layout=LAYOUT_TRAILER, out_ty=ST_FP32, impl="oracle"):
    """q: uint8 [rows, stride]. Returns [rows, cols] float32, or uint16 patterns (fp16 / bf16)."""
    q = np.ascontiguousarray(q)
    rows, stride = q.shape
    out = np.zeros((rows, cols), out_dtype(out_ty))
    if impl == "oracle":
        _lib("oracle").oracle_dequantize_rowwise(_ptr(q), rows, stride, cols, bit_rate, int(sb_float), layout,
                                                 out_ty, _ptr(out))
    else:
        assert layout == LAYOUT_TRAILER and stride == quantized_row_bytes(cols, bit_rate, sb_float, layout)
        # the reference derives the column count from the row's bytes: every
        # element slot of the last byte is written (src/QuantUtils.cc:758-760)
        ref_cols = (stride - (8 if sb_float else 4)) * (8 // bit_rate)
        full = np.zeros((rows, ref_cols), out_dtype(out_ty))
        if sb_float:
            _lib("refquant").ref_dequantize_8bit(_ptr(q), rows, stride, out_ty, _ptr(full))
        else:
            _lib("refquant").ref_dequantize_nbit(bit_rate, _ptr(q), rows, stride, out_ty, _ptr(full))
        out = np.ascontiguousarray(full[:, :cols])
    return out


def tbe_forward(dev_weights, weights_offsets, weights_tys, D_offsets, total_D, indices,
                offsets, pooling_mode, indice_weights, out_ty, row_alignment):
    """Table-batched forward on the CPU. Returns (rc, out[B, total_D]); rc is 0
    or 1 + the first failing table."""
    dev_weights = np.ascontiguousarray(dev_weights, dtype=np.uint8)
    weights_offsets = np.ascontiguousarray(weights_offsets, dtype=np.int64)
    weights_tys = np.ascontiguousarray(weights_tys, dtype=np.uint8)
    D_offsets = np.ascontiguousarray(D_offsets, dtype=np.int32)
    indices = np.ascontiguousarray(indices)
    offsets = np.ascontiguousarray(offsets, dtype=indices.dtype)
    if indice_weights is not None:
        indice_weights = np.ascontiguousarray(indice_weights, dtype=np.float32)
    T = len(D_offsets) - 1
    B = (len(offsets) - 1) // T
    out = np.zeros((B, total_D), dtype=out_dtype(out_ty))
    rc = _lib("oracle").oracle_tbe_forward(
        _ptr(dev_weights), dev_weights.size, _ptr(weights_offsets), _ptr(weights_tys),
        _ptr(D_offsets), T, total_D, _ptr(indices), _ptr(offsets), _is64(indices),
        len(offsets), pooling_mode, _ptr(indice_weights), out_ty, row_alignment,
        _ptr(out))
    return rc, out


def tbe_forward_nobag(dev_weights, weights_offsets, weights_tys, rows_per_table, D, indices, offsets,
                      out_ty, row_alignment):
    """PoolingMode.NONE on the CPU, the way the reference's operator runs it
    (embedding_forward_quantized_cpu_template.cpp:390-420): per table, the pooled
    kernel over virtual bags of length one. int8 / int4 output types copy the
    stored rows (src/RefImplementations.cc:1235-1253,1466-1484). Returns
    (ok, out[total_L, D]) resp. uint8 [total_L, row bytes]."""
    dev_weights = np.ascontiguousarray(dev_weights, dtype=np.uint8)
    indices = np.ascontiguousarray(indices)
    T = len(weights_tys)
    B = (len(offsets) - 1) // T
    total_L = len(indices)
    copy_rows = out_ty in (ST_INT8, ST_INT4)
    width = (D + 4 if out_ty == ST_INT8 else (D + 9) // 2) if copy_rows else D
    out = np.zeros((total_L, width), np.uint8 if copy_rows else out_dtype(out_ty))
    ok_all = True
    for t in range(T):
        s, e = int(offsets[t * B]), int(offsets[(t + 1) * B])
        ty = int(weights_tys[t])
        rb = padded_row_bytes(D, ty, row_alignment)
        tbl = dev_weights[int(weights_offsets[t]):int(weights_offsets[t]) + int(rows_per_table[t]) * rb]
        idx = indices[s:e]
        if copy_rows:
            rows2d = tbl.reshape(-1, rb)
            for i, r in enumerate(idx.tolist()):
                if r == -1:
                    continue  # our operator leaves zeros for a pruned row
                if r < 0 or r >= rows_per_table[t]:
                    ok_all = False
                    continue
                n = min(width, unpadded_row_bytes(D, ty))
                out[s + i, :n] = rows2d[r, :n]
            continue
        elem = 4 if ty == ST_FP32 else 2 if ty in (ST_FP16, ST_BF16) else 1
        ok, o = spmdm(ty, D, tbl, idx, np.arange(e - s + 1, dtype=indices.dtype), out_ty=out_ty,
                      input_stride=rb // elem, scale_bias_last=False, data_size=int(rows_per_table[t]),
                      output_size=e - s)
        ok_all = ok_all and ok
        out[s:e] = o.reshape(e - s, D)
    return ok_all, out


def unpadded_row_bytes(dim, ty, scale_bias_bytes=4):
    bits = {ST_FP32: 32, ST_FP16: 16, ST_BF16: 16, ST_INT8: 8, ST_INT4: 4, ST_INT2: 2}[ty]
    return (dim * bits + 7) // 8 + (scale_bias_bytes if bits <= 8 else 0)


def _conv(name, arr, in_dt, out_dt, impl):
    arr = np.ascontiguousarray(arr, dtype=in_dt)
    out = np.empty(arr.shape, dtype=out_dt)
    fn = getattr(_lib(impl), ("oracle_" if impl == "oracle" else "ref_") + name + "_array")
    fn.argtypes = [_c.c_void_p, _c.c_void_p, _c.c_int64]
    fn.restype = None
    fn(_ptr(arr), _ptr(out), arr.size)
    return out


def half2float(h, impl="oracle"):
    """uint16 half patterns -> float32."""
    return _conv("half2float", h, np.uint16, np.float32, impl)


def float2half_rn(f, impl="oracle"):
    """float32 -> uint16 half patterns, round to nearest even."""
    return _conv("float2half_rn", f, np.float32, np.uint16, impl)


def float2bf16(f, impl="oracle"):
    """float32 -> uint16 bf16 patterns, the reference's add-0x8000-and-truncate rule."""
    return _conv("float2bf16", f, np.float32, np.uint16, impl)


def padded_row_bytes(dim, ty, row_alignment, scale_bias_bytes=4):
    return _lib("oracle").oracle_padded_row_bytes(dim, ty, row_alignment, scale_bias_bytes)
