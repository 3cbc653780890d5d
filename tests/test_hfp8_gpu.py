"""GPU parity of the fp32 <-> 8-bit float (hfp8) converters, through the C ABI and
the torch operators, against the CPU oracle: every code bit for bit."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

FORMATS = [(4, 7), (5, 15), (3, 3), (2, 1), (4, 4)]


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


def inputs(rng, oracle, ebits, bias, n):
    mags = np.array([oracle.float8_to_float(b, ebits, bias) for b in range(128)], dtype=np.float32)
    mid = ((mags[:-1].astype(np.float64) + mags[1:]) / 2).astype(np.float32)
    x = np.concatenate([
        mags, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
        np.array([0.0, 1e-30, 1e-45, 3e38, np.inf, np.nan], dtype=np.float32),
        rng.normal(size=n).astype(np.float32) * np.float32(mags[-1] / 4),
        (rng.uniform(-1, 1, size=n) * 2.0 ** rng.integers(-30, 20, size=n)).astype(np.float32)])
    x = np.concatenate([x, -x])
    rng.shuffle(x)
    return x


@pytest.mark.parametrize("ebits,bias", FORMATS)
def test_encode_matches_oracle(ops, oracle, ebits, bias):
    rng = np.random.default_rng(ebits * 31 + bias)
    x = inputs(rng, oracle, ebits, bias, 20000)
    max_pos = oracle.hfp8_max_pos(ebits, bias)
    for cols in (1, 3, 4, 64, 127):
        rows = len(x) // cols
        xs = x[:rows * cols].reshape(rows, cols)
        got = ops.float_to_hfp8_quantized(torch.from_numpy(xs).cuda(), ebits, bias, max_pos).cpu().numpy()
        want = oracle.float_to_hfp8(xs, ebits, bias, max_pos)
        assert got.shape == want.shape and (got == want).all(), np.argwhere(got != want)[:5]
    # a caller's own clamp
    got = ops.float_to_hfp8_quantized(torch.from_numpy(x[:4096].reshape(64, 64)).cuda(), ebits, bias, 1.5).cpu().numpy()
    assert (got == oracle.float_to_hfp8(x[:4096].reshape(64, 64), ebits, bias, 1.5)).all()


@pytest.mark.parametrize("ebits,bias", FORMATS + [(4, 15), (5, 30)])
def test_decode_matches_oracle(ops, oracle, ebits, bias):
    rng = np.random.default_rng(ebits * 37 + bias)
    codes = np.concatenate([np.arange(256, dtype=np.uint8), rng.integers(0, 256, size=10001, dtype=np.uint8)])
    table = np.array([oracle.float8_to_float(b, ebits, bias) for b in range(256)], dtype=np.float32)
    for cols in (1, 7, 9):
        rows = len(codes) // cols
        c = codes[:rows * cols].reshape(rows, cols)
        got = ops.hfp8_quantized_to_float(torch.from_numpy(c).cuda(), ebits, bias).cpu().numpy()
        assert (got.view(np.uint32) == table[c].view(np.uint32)).all()


def test_unaligned_buffers_and_empty_input_through_the_c_abi(ops, oracle):
    from fbgemm_amd import _lib
    lib = _lib.lib()
    rng = np.random.default_rng(5)
    x = rng.normal(size=1003).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    out = torch.full((1100,), 0xEE, dtype=torch.uint8, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for in_off, out_off, n in [(1, 0, 1000), (0, 1, 1001), (3, 3, 999), (0, 0, 0), (0, 2, 5)]:
        out.fill_(0xEE)
        _lib.check(lib.fbgemm_amd_float_to_hfp8(C.c_void_p(dx.data_ptr() + 4 * in_off), n, 4, 7, 240.0,
                                                C.c_void_p(out.data_ptr() + out_off), stream))
        got = out.cpu().numpy()
        want = oracle.float_to_hfp8(x[in_off:in_off + n], 4, 7, 240.0)
        assert (got[out_off:out_off + n] == want).all()
        assert (got[:out_off] == 0xEE).all() and (got[out_off + n:] == 0xEE).all()
    back = torch.full((1100,), -7.0, dtype=torch.float32, device="cuda")
    codes = torch.from_numpy(oracle.float_to_hfp8(x, 4, 7, 240.0)).cuda()
    for in_off, out_off, n in [(1, 0, 1000), (0, 1, 1001), (2, 3, 999)]:
        back.fill_(-7.0)
        _lib.check(lib.fbgemm_amd_hfp8_to_float(C.c_void_p(codes.data_ptr() + in_off), n, 4, 7,
                                                C.c_void_p(back.data_ptr() + 4 * out_off), stream))
        got = back.cpu().numpy()
        want = np.array([oracle.float8_to_float(int(b), 4, 7) for b in codes.cpu().numpy()[in_off:in_off + n]], dtype=np.float32)
        assert (got[out_off:out_off + n].view(np.uint32) == want.view(np.uint32)).all()
        assert (got[:out_off] == -7.0).all() and (got[out_off + n:] == -7.0).all()
    assert lib.fbgemm_amd_float_to_hfp8(None, 4, 4, 7, 240.0, None, stream) < 0
    assert lib.fbgemm_amd_float_to_hfp8(C.c_void_p(dx.data_ptr()), 4, 9, 7, 240.0, C.c_void_p(out.data_ptr()), stream) < 0


def test_torch_operators(ops, oracle):
    import os
    lib = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fbgemm_amd", "lib", "libfbgemm_amd_torch.so")
    assert os.path.exists(lib), "build it with `python -m fbgemm_amd.build`"
    torch.ops.load_library(lib)
    rng = np.random.default_rng(6)
    x = rng.normal(size=(50, 33)).astype(np.float32)
    q = torch.ops.fbgemm.FloatToHFP8Quantized(torch.from_numpy(x).cuda(), 4, 7, 240.0)
    assert q.dtype == torch.uint8 and (q.cpu().numpy() == oracle.float_to_hfp8(x, 4, 7, 240.0)).all()
    f = torch.ops.fbgemm.HFP8QuantizedToFloat(q, 4, 7)
    # decode(encode(x)) is within half a step of x (3 mantissa bits: 2^-4 relative) or the smallest step 2^-9 absolute
    err = np.abs(f.cpu().numpy() - x)
    assert (err <= np.maximum(np.abs(x) * 2.0 ** -4, 2.0 ** -10)).all()
    # idempotent: a decoded value encodes to its own code
    assert torch.equal(torch.ops.fbgemm.FloatToHFP8Quantized(f, 4, 7, 240.0), q)
