"""A bounded randomized parity sweep with fixed seeds: random shapes, row layouts, strides, index
and offset widths, weights, pooling and output types, through the C ABI against the CPU oracle,
bit for bit. Every case is rebuilt from its seed alone, so a failure names the seed to replay;
a chunk stops at its first mismatch.

The parameter space is the one the reference's tests draw from at random
(test/EmbeddingSpMDMNBitTest.cc:92-418, test/EmbeddingSpMDM8BitTest.cc:82-372 for the single-table
kernels; fbgemm_gpu/test/tbe/inference/nbit_forward_test.py:746-815 for the table-batched forward)."""
import numpy as np
import pytest

import helpers as H
import test_spmdm_gpu as S
import test_tbe_gpu as TB
from helpers import BF16, FP16, FP32, INT2, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

CHUNK = 500
DIMS_SINGLE = [1, 2, 3, 4, 6, 8, 12, 16, 20, 24, 32, 36, 40, 48, 56, 64, 72, 96, 100, 128, 136, 160, 192, 256, 260,
               320, 384, 512, 640, 1000, 1024]
DIMS_BATCHED = [4, 8, 16, 24, 32, 40, 64, 96, 128, 160, 256, 288, 352, 512]


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import fbgemm_amd.ops as o
    return o


@pytest.fixture
def routes():
    """lets a case pick its route: 16-byte or 4-byte lanes, the lean kernel on or off"""
    import fbgemm_amd
    lib = fbgemm_amd.lib()

    def choose(rng):
        lib.fbgemm_amd_set_narrow_below_waves(1024 if rng.random() < 0.4 else 0)
        lib.fbgemm_amd_set_lean(0 if rng.random() < 0.3 else 1)
    yield choose
    lib.fbgemm_amd_set_narrow_below_waves(-1)
    lib.fbgemm_amd_set_lean(-1)


def single_table_case(ops, oracle, seed):
    rng = np.random.default_rng(seed)
    ty = int(rng.choice([INT8, INT4, INT2, FP16, FP32, BF16]))
    D = int(rng.choice(DIMS_SINGLE))
    if ty == INT2:
        D = max(4, (D + 3) // 4 * 4)
    if ty == INT4:
        D = max(2, (D + 1) // 2 * 2)
    rows, nb, avg = int(rng.integers(1, 400)), int(rng.integers(0, 200)), int(rng.integers(1, 40))
    sbl = bool(rng.integers(0, 2))  # scale / bias behind the data, or in front as the operator lays rows out
    out_ty = int(rng.choice([FP32, FP16, BF16]))
    weighted = int(rng.integers(0, 3))  # none, per lookup, per position in the bag
    normalize, use_offsets = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    idt, odt = rng.choice([np.int32, np.int64]), rng.choice([np.int32, np.int64])
    pad = int(rng.choice([0, 0, 1, 3, 4, 16]))
    elem = H.BITS[ty] // 8 if H.BITS[ty] >= 8 else 1
    stride_b = H.default_stride_bytes(ty, D, sbl) + pad * elem
    table, _ = H.make_table(rng, ty, rows, D, sbl, stride_bytes=stride_b)
    idx, off, lens = H.make_bags(rng, rows, nb, avg, idt, odt, empty_frac=0.2)
    if not sbl and len(idx):
        idx[rng.random(len(idx)) < 0.1] = -1  # pruned-row holes, operator layout only
    w = None
    if weighted == 1:
        w = rng.normal(size=max(1, len(idx))).astype(np.float32)
    elif weighted == 2:
        w = rng.normal(size=max(1, int(lens.max()) if len(lens) else 1)).astype(np.float32)
    ostride = -1 if rng.random() < 0.5 else D + int(rng.integers(0, 9))
    what = f"single-table seed {seed}: ty={ty} D={D} rows={rows} bags={nb} trailer={sbl} out={out_ty} " \
           f"weights={weighted} mean={normalize} offsets={use_offsets} pad={pad} out_stride={ostride}"
    S.check_case(ops, oracle, ty=ty, D=D, table=table, idx=idx, off_or_len=off if use_offsets else lens.astype(odt),
                 w=w, normalize=normalize, out_ty=out_ty, positional=weighted == 2, use_offsets=use_offsets,
                 output_stride=ostride, input_stride=stride_b // elem if pad else -1, sbl=sbl, data_size=rows,
                 output_size=nb, what=what)


def table_batched_case(ops, oracle, seed):
    rng = np.random.default_rng(seed)
    T, B = int(rng.integers(1, 9)), int(rng.integers(1, 70))
    specs = []
    for _ in range(T):
        ty = int(rng.choice([INT8, INT4, INT2, FP16, FP32]))
        D = int(rng.choice(DIMS_BATCHED))
        if ty == INT2:
            D = (D + 3) // 4 * 4
        specs.append((int(rng.integers(1, 300)), D, ty))
    align = int(rng.choice([16, 16, 1, 4]))
    weights, wo, _ = TB.build_weights(rng, specs, align)
    max_len = int(rng.choice([3, 10, 45]))
    lens = rng.integers(0, max_len, size=T * B)
    dt = rng.choice([np.int32, np.int64])
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]
                         + [np.zeros(0, np.int64)]).astype(dt)
    if len(idx):
        idx[rng.random(len(idx)) < 0.1] = -1
    pooling, out_ty = int(rng.integers(0, 2)), int(rng.choice([FP32, FP16, BF16]))
    psw = rng.normal(size=len(idx)).astype(np.float32) if rng.random() < 0.5 else None
    what = f"table-batched seed {seed}: specs={specs} B={B} align={align} max_len={max_len} pooling={pooling} " \
           f"out={out_ty} weighted={psw is not None}"
    got, want = TB.run_both(ops, oracle, weights, wo, specs, idx, off, pooling, psw, out_ty, align)
    H.assert_same_bits(got, want, what)


@pytest.mark.parametrize("chunk", range(8))
def test_single_table_sweep(ops, oracle, routes, chunk):
    for seed in range(10_000 + chunk * CHUNK, 10_000 + (chunk + 1) * CHUNK):
        routes(np.random.default_rng(seed + 1_000_000))
        single_table_case(ops, oracle, seed)


@pytest.mark.parametrize("chunk", range(8))
def test_table_batched_sweep(ops, oracle, routes, chunk):
    for seed in range(20_000 + chunk * CHUNK, 20_000 + (chunk + 1) * CHUNK):
        routes(np.random.default_rng(seed + 1_000_000))
        table_batched_case(ops, oracle, seed)


def int8_output_case(ops, oracle, seed):
    """The 8-bit pooled output of a random table-batched forward: every (bag, table) block byte for
    byte against the pooled oracle followed by the quantizer oracle (the lean kernel's own output
    stage, the float route through the quantizer, and plans that mix the two)."""
    rng = np.random.default_rng(seed)
    T, B = int(rng.integers(1, 9)), int(rng.integers(1, 70))
    specs = []
    for _ in range(T):
        ty = int(rng.choice([INT8, INT4, INT4, INT2, FP16, FP32]))
        D = int(rng.choice(DIMS_BATCHED))
        if ty in (INT8, INT4, FP16) and rng.random() < 0.25:
            D = int(rng.choice([2, 6, 10, 14, 18, 26, 30, 38, 50, 70]))  # widths that are not a multiple of 4
        specs.append((int(rng.integers(1, 300)), D, ty))
    align = int(rng.choice([16, 16, 1, 4]))
    weights, wo, _ = TB.build_weights(rng, specs, align)
    max_len = int(rng.choice([3, 10, 45]))
    lens = rng.integers(0, max_len, size=T * B)
    dt = rng.choice([np.int32, np.int64])
    off = np.concatenate([[0], np.cumsum(lens)]).astype(dt)
    idx = np.concatenate([rng.integers(0, specs[t][0], size=int(lens[t * B:(t + 1) * B].sum())) for t in range(T)]
                         + [np.zeros(0, np.int64)]).astype(dt)
    if len(idx):
        idx[rng.random(len(idx)) < 0.1] = -1
    pooling = int(rng.integers(0, 2))
    psw = rng.normal(size=len(idx)).astype(np.float32) if rng.random() < 0.5 else None
    if psw is not None and len(psw):
        psw[rng.random(len(psw)) < 0.05] = -0.0  # zeros of both signs among a block's terms
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    cu = TB.cu
    got = ops.int_nbit_split_embedding_codegen_lookup_function(
        cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys),
        cu(D_offsets), total_D, maxd(INT2), maxd(INT4), maxd(INT8), maxd(FP16), maxd(FP32), cu(idx), cu(off),
        pooling, None if psw is None else cu(psw), INT8, row_alignment=align).cpu().numpy()
    assert got.shape == (B, total_D + 8 * T)
    rc, pooled = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, pooling, psw, FP32, align)
    assert rc == 0
    for t in range(T):
        D = specs[t][1]
        want = oracle.quantize_rowwise(np.ascontiguousarray(pooled[:, D_offsets[t]:D_offsets[t + 1]]), 8, True)
        block = got[:, D_offsets[t] + 8 * t:D_offsets[t] + 8 * t + D + 8]
        assert (block == want).all(), (f"8-bit output seed {seed}: specs={specs} B={B} align={align} pooling={pooling} "
                                       f"weighted={psw is not None} table={t}", np.argwhere(block != want)[:4])


@pytest.mark.parametrize("chunk", range(4))
def test_table_batched_int8_output_sweep(ops, oracle, routes, chunk):
    for seed in range(30_000 + chunk * 150, 30_000 + (chunk + 1) * 150):
        routes(np.random.default_rng(seed + 1_000_000))
        int8_output_case(ops, oracle, seed)
