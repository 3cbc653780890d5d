"""TEST / BASELINE INFRASTRUCTURE ONLY: ctypes front-end of oracle/jit_bridge.cc,
the reference's AVX2/AVX-512 kernels as exported by libtorch_cpu.so."""
import ctypes as C
import os

import numpy as np

from . import HERE, JIT_SO, build

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(JIT_SO):
            build(("jit",))
        import torch  # noqa: F401  (loads libtorch_cpu.so / libc10.so into the process first)
        h = C.CDLL(JIT_SO)
        h.jit_embedding_spmdm.argtypes = [
            C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int]
        h.jit_embedding_spmdm.restype = C.c_int
        h.jit_tbe_tables.argtypes = [
            C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        h.jit_tbe_tables.restype = C.c_int
        h.jit_max_threads.restype = C.c_int
        _lib = h
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def spmdm(in_ty, D, table, indices, offsets, *, weights=None, normalize=False, out_ty=0,
          output_stride=-1, input_stride=-1, scale_bias_last=True, data_size, output_size=None, out=None):
    """One pooled lookup through the JIT kernels. Returns (ok, out)."""
    table = np.ascontiguousarray(table)
    indices = np.ascontiguousarray(indices, dtype=np.int64)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    if weights is not None:
        weights = np.ascontiguousarray(weights, dtype=np.float32)
    if output_size is None:
        output_size = len(offsets) - 1
    stride = D if output_stride == -1 else output_stride
    if out is None:
        out = np.zeros(output_size * stride, dtype=np.float32 if out_ty == 0 else np.uint16)
    ok = lib().jit_embedding_spmdm(in_ty, D, output_size, len(indices), data_size, _p(table), _p(indices),
                                   _p(offsets), _p(weights), int(normalize), _p(out), out_ty, output_stride,
                                   input_stride, int(scale_bias_last))
    return bool(ok), out


def tbe_tables(t0, t1, weights, weights_offsets, weights_tys, D_offsets, row_bytes, num_rows, total_D,
               indices, offsets, B, pooling_mode, indice_weights, out_ty, output, threads=1):
    """The CPU operator's table loop over tables [t0, t1). `weights_offsets`
    index into `weights`. Returns 0 or 1 + the first failing table."""
    return lib().jit_tbe_tables(
        t0, t1, _p(weights), _p(np.ascontiguousarray(weights_offsets, dtype=np.int64)),
        _p(np.ascontiguousarray(weights_tys, dtype=np.uint8)), _p(np.ascontiguousarray(D_offsets, dtype=np.int32)),
        _p(np.ascontiguousarray(row_bytes, dtype=np.int64)), _p(np.ascontiguousarray(num_rows, dtype=np.int64)),
        total_D, _p(indices), _p(offsets), B, pooling_mode, _p(indice_weights), out_ty, _p(output), threads)


def max_threads():
    return lib().jit_max_threads()
