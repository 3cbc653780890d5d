"""CPU-side checks of the boundary: the shared library loads without a GPU and
exports every entry point include/fbgemm_amd.h declares (the benchmark-only
header include/fbgemm_amd_bench.h likewise, in its two libraries); the host-only
helpers agree with the oracle; the Python face refuses CPU tensors instead of
falling back."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header="fbgemm_amd.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fbgemm_amd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import fbgemm_amd
    if not os.path.exists(fbgemm_amd.LIB_PATH):
        from fbgemm_amd import build
        build.build_library()
    handle = ctypes.CDLL(fbgemm_amd.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(handle, n), f"{n} is declared in include/fbgemm_amd.h but not exported"
    # and the Python binding table covers the same set
    assert sorted(fbgemm_amd.SYMBOLS) == names
    fbgemm_amd.lib()


def test_bench_header_matches_its_two_libraries():
    """include/fbgemm_amd_bench.h: fbgemm_amd_bench_* come from libfbgemm_amd_bench.so, the
    switches from the product library; nothing of it is declared in the drop-in header, and the
    product library exports no yardstick."""
    from fbgemm_amd import _lib
    if not os.path.exists(_lib.BENCH_LIB_PATH):
        from fbgemm_amd import build
        build.build_bench_library()
    names = declared_functions("fbgemm_amd_bench.h")
    yard = [n for n in names if n.startswith("fbgemm_amd_bench_")]
    switches = [n for n in names if not n.startswith("fbgemm_amd_bench_")]
    assert sorted(_lib.BENCH_SYMBOLS) == yard and sorted(_lib.BENCH_SWITCHES) == switches
    bench = ctypes.CDLL(_lib.BENCH_LIB_PATH)
    main = ctypes.CDLL(_lib.LIB_PATH)
    for n in yard:
        assert hasattr(bench, n) and not hasattr(main, n), n
    for n in switches:
        assert hasattr(main, n), n
    assert not set(names) & set(declared_functions())
    _lib.bench_lib()


def test_row_size_helpers_match_oracle(oracle):
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    for ty in range(6):
        for D in (4, 8, 24, 32, 40, 64, 100, 128, 256, 1024):
            for align in (1, 4, 16, 32):
                want = oracle.padded_row_bytes(D, ty, align) if ty != 5 else (2 * D + align - 1) // align * align
                assert lib.fbgemm_amd_padded_row_size_in_bytes(D, ty, align, 4) == want
    # the reference's table (embedding_common.h:189-215)
    assert lib.fbgemm_amd_unpadded_row_size_in_bytes(128, 3, 4) == 68
    assert lib.fbgemm_amd_unpadded_row_size_in_bytes(128, 2, 8) == 136
    assert lib.fbgemm_amd_unpadded_row_size_in_bytes(32, 4, 4) == 12
    assert lib.fbgemm_amd_padded_row_size_in_bytes(256, 3, 16, 4) == 144


def test_argument_checks_need_no_gpu():
    import fbgemm_amd
    from fbgemm_amd._lib import SpmdmConfig
    lib = fbgemm_amd.lib()
    cfg = SpmdmConfig(weight_ty=9, output_ty=0, index_bits=64, offset_bits=32, block_size=8, output_stride=-1,
                      input_stride=-1, normalize_by_lengths=0, is_weight_positional=0, use_offsets=1, scale_bias_last=1)
    rc = lib.fbgemm_amd_spmdm_launch(ctypes.byref(cfg), 1, 1, 1, None, None, None, None, None, None, None, None)
    assert rc == -1 and b"weight_ty" in lib.fbgemm_amd_last_error()
    cfg.weight_ty = 3
    cfg.index_bits = 16
    assert lib.fbgemm_amd_spmdm_launch(ctypes.byref(cfg), 1, 1, 1, None, None, None, None, None, None, None, None) == -1
    assert lib.fbgemm_amd_status_clear(None, None) == -1
    assert lib.fbgemm_amd_tbe_forward(None, None, None, None, None, 64, 0, 1, 0, None, 1, None, None, None) == -1
    assert lib.fbgemm_amd_version() == b"0.1"


def test_ops_refuse_cpu_tensors():
    torch = pytest.importorskip("torch")
    from fbgemm_amd import ops
    kern = ops.generate_embedding_spmdm_nbit(4, 32, False, False)
    t = torch.zeros(10 * 20, dtype=torch.uint8)
    idx = torch.zeros(4, dtype=torch.int64)
    off = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(ValueError, match="no CPU path"):
        kern(1, 4, 10, t, idx, off, None, torch.zeros(32))
    with pytest.raises(ValueError, match="input_bit_rate"):
        ops.generate_embedding_spmdm_nbit_with_strides(3, 32, False, False)
    # no_bag of 4-bit rows exists for a 4-bit output only; the others return false, as the reference does
    assert ops.generate_embedding_spmdm_nbit_with_strides(4, 32, False, False, no_bag=True)(0, 0, 0, t, idx, None, None, t) is False
    with pytest.raises(ValueError, match="no CPU path"):
        ops.generate_embedding_spmdm_nbit_with_strides(4, 32, False, False, no_bag=True, output_bit_rate=4)(
            4, 4, 10, t, idx, None, None, torch.zeros(80, dtype=torch.uint8))


def test_workload_generators_are_seeded():
    torch = pytest.importorskip("torch")
    from fbgemm_amd import bench_configs as bc
    a, b = bc.config3("cpu", 0.01), bc.config3("cpu", 0.01)
    assert (a.host_indices == b.host_indices).all() and (a.host_offsets == b.host_offsets).all()
    assert torch.equal(a.dev_weights, b.dev_weights)
    assert a.T == 64 and set(np.unique(a.tys)) <= {1, 2, 3} and set(np.unique(a.Ds)) <= {64, 128, 256}
    assert a.useful_row_bytes() > 0 and a.lookups == int(a.lengths.sum())
    p1 = bc.config1("cpu", 0.01)
    assert p1.row_bytes() == 136 and (np.diff(p1.host_offsets) == 20).all()
    p2 = bc.config2("cpu", 0.001)
    assert p2.row_bytes() == 68 and np.diff(p2.host_offsets).min() >= 1 and np.diff(p2.host_offsets).max() <= 40
    p4 = bc.config4("cpu", 0.001, tables=2)
    assert p4[0].row_bytes() == 36 and abs((p4[0].host_remap == -1).mean() - 0.5) < 0.1

