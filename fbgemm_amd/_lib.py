"""Loader of the HIP library behind the C ABI (include/fbgemm_amd.h), and of the
benchmark-only library (include/fbgemm_amd_bench.h).

The library is built in-tree by ``fbgemm_amd.build`` (hipcc, gfx950). There is
no CPU fallback: if the shared object is missing or a symbol cannot be bound,
importing the ops fails loudly.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libfbgemm_amd.so")
BENCH_LIB_PATH = os.path.join(HERE, "lib", "libfbgemm_amd_bench.so")

# every symbol include/fbgemm_amd.h declares: name -> (restype, argtypes)
_P, _I32, _I64 = C.c_void_p, C.c_int32, C.c_int64


class SpmdmConfig(C.Structure):
    """struct fbgemm_amd_spmdm_config."""
    _fields_ = [
        ("weight_ty", _I32), ("output_ty", _I32), ("index_bits", _I32), ("offset_bits", _I32),
        ("block_size", _I64), ("output_stride", _I64), ("input_stride", _I64),
        ("normalize_by_lengths", _I32), ("is_weight_positional", _I32),
        ("use_offsets", _I32), ("scale_bias_last", _I32),
        ("no_bag", _I32), ("fp8_exponent_bits", _I32), ("fp8_exponent_bias", _I32), ("accumulate", _I32),
    ]


SYMBOLS = {
    "fbgemm_amd_last_error": (C.c_char_p, []),
    "fbgemm_amd_version": (C.c_char_p, []),
    "fbgemm_amd_status_clear": (C.c_int, [_P, _P]),
    "fbgemm_amd_stream_synchronize": (C.c_int, [_P]),
    "fbgemm_amd_status_read": (C.c_int, [_P, _P, C.POINTER(_I32), C.POINTER(_I64)]),
    "fbgemm_amd_spmdm_launch": (C.c_int, [C.POINTER(SpmdmConfig), _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _P]),
    "fbgemm_amd_spmdm_launch_noalloc": (C.c_int, [C.POINTER(SpmdmConfig), _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _P]),
    "fbgemm_amd_noalloc_max_bags": (_I64, []),
    "fbgemm_amd_spmdm_run": (C.c_int, [C.POINTER(SpmdmConfig), _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "fbgemm_amd_tbe_plan_create": (C.c_int, [C.POINTER(_P), _I32, _P, _P, _P, _P, _I64, _I64, _I64]),
    "fbgemm_amd_tbe_plan_destroy": (None, [_P]),
    "fbgemm_amd_tbe_forward": (C.c_int, [_P, _P, _P, _P, _P, _I32, _I64, _I64, _I32, _P, _I32, _P, _P, _P]),
    "fbgemm_amd_tbe_forward_pruned": (C.c_int, [_P, _P, _P, _P, _P, _I32, _I64, _I64, _I32, _P, _I32, _P, _P, _I32, _P, _I64, _P, _P]),
    "fbgemm_amd_tbe_plan_set_index_remappings": (C.c_int, [_P, _P, _I32, _P, _I64, _P]),
    "fbgemm_amd_tbe_plan_rank_tables": (_I32, [_P]),
    "fbgemm_amd_tbe_plan_set_fp8": (C.c_int, [_P, _I32, _I32]),
    "fbgemm_amd_tbe_plan_set_accumulate": (C.c_int, [_P, _I32]),
    "fbgemm_amd_tbe_plan_trim": (C.c_int, [_P]),
    "fbgemm_amd_tbe_plan_cached_work": (_I64, [_P]),
    "fbgemm_amd_tbe_plan_pinned_work": (C.c_int64, [_P]),
    "fbgemm_amd_tbe_forward_nobag": (C.c_int, [_P, _P, _P, _P, _P, _I32, _I64, _I64, _I32, _I32, _P, _P, _P]),
    "fbgemm_amd_bounds_check_indices": (C.c_int, [_P, _I32, _P, _P, _I32, _I64, _I64, _I32, _P, _P, _P, _P]),
    "fbgemm_amd_pruned_hashmap_lookup": (C.c_int, [_P, _P, _I32, _I64, _P, _I32, _P, _I32, _P, _P]),
    "fbgemm_amd_pruned_hashmap_insert_host": (C.c_int, [_P, _P, _P, _I32, _I64, _P, _I32, _P, _I32]),
    "fbgemm_amd_quantize_rowwise": (C.c_int, [_P, _I32, _I64, _I32, _I32, _I32, _I32, _I64, _P, _P]),
    "fbgemm_amd_quantize_rowwise_min_max": (C.c_int, [_P, _I32, _I64, _I32, _I32, _I32, _I32, _I64, _P, _P, _P]),
    "fbgemm_amd_dequantize_rowwise": (C.c_int, [_P, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _P, _P]),
    "fbgemm_amd_float_to_hfp8": (C.c_int, [_P, _I64, _I32, _I32, C.c_float, _P, _P]),
    "fbgemm_amd_hfp8_to_float": (C.c_int, [_P, _I64, _I32, _I32, _P, _P]),
    "fbgemm_amd_compressed_indices_remap": (C.c_int, [_I32, _P, _I32, _P, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "fbgemm_amd_rowwise_prune_map": (C.c_int, [_P, _I64, C.c_double, _I32, _I64, _I32, _P, C.POINTER(_I64), _P]),
    "fbgemm_amd_rowwise_prune_gather": (C.c_int, [_P, _I64, _I64, _P, _I32, _P, _I64, _P]),
    "fbgemm_amd_tbe_plan_num_rows": (_I64, [_P, _I32]),
    "fbgemm_amd_tbe_plan_row_bytes": (_I64, [_P, _I32]),
    "fbgemm_amd_pruned_array_lookup": (C.c_int, [_P, _P, _I32, _I64, _P, _I32, _P, _I32, _P, _P]),
    "fbgemm_amd_tbe_inplace_update": (C.c_int, [_P, _P, _P, _P, _I64, _P, _P, _I32, _P, _I64, _P, _P]),
    "fbgemm_amd_pruned_array_lookup_from_row_idx": (C.c_int, [_P, _I32, _P, _I64, _P, _I32, _P, _I32, _P, _P]),
    "fbgemm_amd_unpadded_row_size_in_bytes": (_I32, [_I32, _I32, _I32]),
    "fbgemm_amd_padded_row_size_in_bytes": (_I32, [_I32, _I32, _I32, _I32]),
}

# what include/fbgemm_amd_bench.h declares: the switches inside libfbgemm_amd.so ...
BENCH_SWITCHES = {
    "fbgemm_amd_set_lean": (C.c_int, [_I32]),
    "fbgemm_amd_set_narrow_below_waves": (C.c_int, [_I32]),
    "fbgemm_amd_set_wide4": (C.c_int, [_I32]),
    "fbgemm_amd_tbe_plan_reuse_order": (C.c_int, [_P, _I32]),
}
# ... and the yardsticks of libfbgemm_amd_bench.so
BENCH_SYMBOLS = {
    "fbgemm_amd_bench_last_error": (C.c_char_p, []),
    "fbgemm_amd_bench_calibration_copy": (C.c_int, [_P, _P, _I64, _P]),
    "fbgemm_amd_bench_stream_read": (C.c_int, [_P, _I64, _P, _I64, _P]),
    "fbgemm_amd_bench_gather": (C.c_int, [_P, _I64, _I64, _I32, _I32, _P, _I64, _P, _I64, _I32, _I32, _P]),
}

_lib = None
_bench_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m fbgemm_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in list(SYMBOLS.items()) + list(BENCH_SWITCHES.items()):
            fn = getattr(handle, name)  # AttributeError if the symbol is absent
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def bench_lib():
    """The benchmark-only library (yardstick kernels); raises if it has not been built."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise RuntimeError(f"{BENCH_LIB_PATH} is missing: build it with `python -m fbgemm_amd.build`")
        handle = C.CDLL(BENCH_LIB_PATH)
        for name, (res, args) in BENCH_SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _bench_lib = handle
    return _bench_lib


def bench_check(rc):
    if rc < 0:
        raise RuntimeError(f"fbgemm_amd bench error {rc}: {bench_lib().fbgemm_amd_bench_last_error().decode()}")
    return rc


def check(rc):
    if rc < 0:
        raise RuntimeError(f"fbgemm_amd error {rc}: {lib().fbgemm_amd_last_error().decode()}")
    return rc
