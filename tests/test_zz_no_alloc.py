"""The entry point that allocates nothing, fbgemm_amd_spmdm_launch_noalloc,
against fbgemm_amd_spmdm_launch on the same inputs, through the C ABI: two
calls in a row, the second with a smaller input, every output bit equal. The
cases use both pieces of scratch the entry point keeps in its static device
array: the prefix sum of Caffe2-style lengths, and (from 2^21 lookups on) the
bag order of the scheduler."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
from helpers import FP16, FP32, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _call(lib, fn, cfg, nb, n_idx, rows, table, idx, lens_or_off, w, out, st):
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
    lib.fbgemm_amd_status_clear(p(st), stream)
    rc = fn(C.byref(cfg), nb, n_idx, rows, p(table), p(idx), p(lens_or_off), p(w), p(out), None, p(st), stream)
    assert rc == 0, lib.fbgemm_amd_last_error().decode()
    bits = C.c_int32(-1)
    assert lib.fbgemm_amd_status_read(p(st), stream, C.byref(bits), None) == 0
    return bits.value


def _case(lib, rng, ty, D, rows, nb, avg, use_offsets, weighted, out_ty):
    from fbgemm_amd._lib import SpmdmConfig
    table, _ = H.make_table(rng, ty, rows, D, True)
    lens = rng.integers(max(0, avg - 5), avg + 6, size=nb).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n_idx = int(off[-1])
    idx = rng.integers(0, rows, size=n_idx).astype(np.int64)
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    t_table, t_idx = cu(table), cu(idx)
    t_lo = cu(off if use_offsets else lens)
    t_w = cu(rng.uniform(0, 1, size=n_idx).astype(np.float32)) if weighted else None
    st = torch.zeros(16, dtype=torch.uint8, device="cuda")
    dt = torch.float32 if out_ty == FP32 else torch.float16
    cfg = SpmdmConfig(weight_ty=ty, output_ty=out_ty, index_bits=64, offset_bits=32, block_size=D, output_stride=-1,
                      input_stride=-1, normalize_by_lengths=0, is_weight_positional=0, use_offsets=int(use_offsets),
                      scale_bias_last=1)
    outs = []
    for fn in (lib.fbgemm_amd_spmdm_launch, lib.fbgemm_amd_spmdm_launch_noalloc):
        out = torch.full((nb * D,), -7.0, dtype=dt, device="cuda")
        assert _call(lib, fn, cfg, nb, n_idx, rows, t_table, t_idx, t_lo, t_w, out, st) == 0
        outs.append(out)
    assert torch.equal(outs[0].view(torch.int32 if out_ty == FP32 else torch.int16),
                       outs[1].view(torch.int32 if out_ty == FP32 else torch.int16)), \
        f"noalloc differs: ty={ty} D={D} nb={nb} avg={avg} use_offsets={use_offsets}"
    return outs[1]


def test_noalloc_matches_launch_two_calls_in_a_row():
    import fbgemm_amd
    lib = fbgemm_amd.lib()
    assert lib.fbgemm_amd_noalloc_max_bags() == 65536
    rng = np.random.default_rng(77)
    # 1: lengths (prefix sum in the static array) AND >= 2^21 lookups (bag order in the static array)
    _case(lib, rng, INT4, 128, 200_000, 50_000, 48, False, True, FP16)
    # 2: smaller, right after it, same scratch: stale offsets / order entries of call 1 lie behind what it writes
    _case(lib, rng, INT4, 128, 200_000, 3_000, 9, False, False, FP16)
    # 3: another row type and output, offsets given, large enough for the scheduler; 4: small again, lengths
    _case(lib, rng, INT8, 64, 100_000, 65_536, 34, True, False, FP32)
    _case(lib, rng, INT8, 64, 100_000, 17, 3, False, True, FP32)


def test_noalloc_rejects_more_bags_than_its_array_holds():
    import fbgemm_amd
    from fbgemm_amd._lib import SpmdmConfig
    lib = fbgemm_amd.lib()
    cfg = SpmdmConfig(weight_ty=INT8, output_ty=FP32, index_bits=64, offset_bits=32, block_size=8, output_stride=-1,
                      input_stride=-1, normalize_by_lengths=0, is_weight_positional=0, use_offsets=0, scale_bias_last=1)
    dummy = torch.zeros(64, dtype=torch.uint8, device="cuda")
    p = C.c_void_p(dummy.data_ptr())
    rc = lib.fbgemm_amd_spmdm_launch_noalloc(C.byref(cfg), 65537, 0, 1, p, p, p, None, p, None, p, None)
    assert rc == -1 and b"at most 65536 bags" in lib.fbgemm_amd_last_error()


def test_noalloc_allocates_nothing_and_replays_from_a_graph():
    """What the entry point exists for: after its first call on the device (which asks the runtime
    for the address of the static array) further calls leave the device's free memory as it is, and
    a call that uses both pieces of scratch (lengths, and 2^21 lookups for the bag order) can be
    captured in a HIP graph; every replay gives the bits of the allocating entry point."""
    import fbgemm_amd
    from fbgemm_amd._lib import SpmdmConfig
    lib = fbgemm_amd.lib()
    rng = np.random.default_rng(9)
    ty, D, rows, nb, avg = INT4, 128, 150_000, 48_000, 46
    table, _ = H.make_table(rng, ty, rows, D, True)
    lens = rng.integers(avg - 4, avg + 5, size=nb).astype(np.int32)
    n_idx = int(lens.sum())
    assert n_idx >= 1 << 21
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    t_table, t_lens = cu(table), cu(lens)
    t_idx = cu(rng.integers(0, rows, size=n_idx).astype(np.int64))
    st = torch.zeros(16, dtype=torch.uint8, device="cuda")
    cfg = SpmdmConfig(weight_ty=ty, output_ty=FP16, index_bits=64, offset_bits=32, block_size=D, output_stride=-1,
                      input_stride=-1, normalize_by_lengths=0, is_weight_positional=0, use_offsets=0, scale_bias_last=1)
    out = torch.full((nb * D,), -7.0, dtype=torch.float16, device="cuda")
    ref = torch.full((nb * D,), -7.0, dtype=torch.float16, device="cuda")
    # outside any capture: the first call, which takes the array's device address
    assert _call(lib, lib.fbgemm_amd_spmdm_launch_noalloc, cfg, nb, n_idx, rows, t_table, t_idx, t_lens, None, out, st) == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        assert _call(lib, lib.fbgemm_amd_spmdm_launch_noalloc, cfg, nb, n_idx, rows, t_table, t_idx, t_lens, None, out, st) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the entry point that allocates nothing changed the device's free memory"

    p = lambda t: C.c_void_p(t.data_ptr())
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = lib.fbgemm_amd_spmdm_launch_noalloc(C.byref(cfg), nb, n_idx, rows, p(t_table), p(t_idx), p(t_lens), None, p(out),
                                                     None, p(st), stream)
            assert rc == 0, lib.fbgemm_amd_last_error().decode()
    torch.cuda.synchronize()
    for replay in range(3):
        t_idx.copy_(cu(rng.integers(0, rows, size=n_idx).astype(np.int64)))
        out.fill_(-7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert _call(lib, lib.fbgemm_amd_spmdm_launch, cfg, nb, n_idx, rows, t_table, t_idx, t_lens, None, ref, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay {replay} differs from the allocating entry point"
