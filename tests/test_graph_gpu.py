"""The table-batched forward inside a HIP graph (torch.cuda.CUDAGraph): once a plan has
seen a batch size, a forward is kernel launches only (no allocation, no copy, no
synchronization), so a serving loop can capture it. Every replay is checked against
the oracle, with eager work and synchronizations between the replays."""
import numpy as np
import pytest

import helpers as H
from helpers import FP16, FP32, INT4, INT8

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_forward_replays_from_a_graph(oracle):
    assert torch.cuda.is_available()
    from fbgemm_amd import ops
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(2024)
    specs = [(300, 64, INT4), (200, 128, INT8), (100, 32, FP16), (400, 256, INT4)]
    T, B, L = len(specs), 16, 6
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    # fixed-shape inputs: every bag holds L entries, so that the buffers the graph reads keep their size
    off = (np.arange(T * B + 1) * L).astype(np.int32)

    def draw():
        idx = np.concatenate([rng.integers(0, specs[t][0], size=B * L) for t in range(T)]).astype(np.int32)
        return idx, rng.uniform(0, 1, len(idx)).astype(np.float32)

    idx, psw = draw()
    d_idx, d_off, d_psw = cu(idx), cu(off), cu(psw)
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    st = ops.Status()
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 0, maxd(INT4), maxd(INT8), maxd(FP16), 0, d_idx, d_off, 0, d_psw, FP16, row_alignment=16, status=st)
    eager = call()  # makes the plan and its work list for this batch size
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = call()
    torch.cuda.synchronize()
    for replay in range(4):
        idx, psw = draw()
        d_idx.copy_(cu(idx))
        d_psw.copy_(cu(psw))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, psw, FP16, 16)
        assert rc == 0
        H.assert_same_bits(captured.cpu().view(torch.int16).numpy().view(np.uint16), want, f"replay {replay}")
        # eager work of the same plan between the replays
        again = call()
        torch.cuda.synchronize()
        assert torch.equal(again, captured)
    assert st.read() == (0, -1)

    # What the graph holds survives the caches' evictions. The plan of the captured forward has seen
    # one batch size; 24 more batch sizes push its work-list cache past its 16 entries, and 70 other
    # sets of metadata push the cache of plans past its 64: the captured entries and the plan must
    # stay, because the graph replays raw addresses.
    plan = ops._plan_for(meta[0], meta[1], meta[2], meta[3], meta[4], meta[5], 16)
    assert plan.pinned_work() >= 1
    for B2 in range(17, 41):
        off2 = (np.arange(T * B2 + 1) * 2).astype(np.int32)
        idx2 = np.concatenate([rng.integers(0, specs[t][0], size=B2 * 2) for t in range(T)]).astype(np.int32)
        ops.int_nbit_split_embedding_codegen_lookup_function(
            *meta, total_D, 0, maxd(INT4), maxd(INT8), maxd(FP16), 0, cu(idx2), cu(off2), 0, None, FP16, row_alignment=16)
    assert plan.cached_work() <= 18 and plan.pinned_work() >= 1
    others = []
    for k in range(70):
        m2 = (meta[0], meta[1], meta[2].clone(), meta[3].clone(), meta[4].clone(), meta[5].clone())
        others.append(m2)
        ops.int_nbit_split_embedding_codegen_lookup_function(
            *m2, total_D, 0, maxd(INT4), maxd(INT8), maxd(FP16), 0, d_idx, d_off, 0, d_psw, FP16, row_alignment=16)
    torch.cuda.synchronize()
    assert len(ops._plans) <= ops.MAX_CACHED_PLANS + 1
    assert ops._plan_for(meta[0], meta[1], meta[2], meta[3], meta[4], meta[5], 16) is plan
    idx, psw = draw()
    d_idx.copy_(cu(idx))
    d_psw.copy_(cu(psw))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, psw, FP16, 16)
    assert rc == 0
    H.assert_same_bits(captured.cpu().view(torch.int16).numpy().view(np.uint16), want, "replay after evictions")
    # an explicit trim drops everything, pinned entries included (graphs must then be captured again)
    del graph
    plan.trim()
    assert plan.cached_work() == 0 and plan.pinned_work() == 0
    again = call()
    torch.cuda.synchronize()
    H.assert_same_bits(again.cpu().view(torch.int16).numpy().view(np.uint16), want, "eager after trim")


def test_forward_with_both_kernels_replays_from_a_graph(oracle):
    """A forward large enough to order its bags, over tables for both lookup kernels (4-bit rows of a
    lean shape, and 2-bit / odd-width rows): the general kernel runs on the plan's side stream beside
    the lean one (event fork and join). Captured, that is a graph with two branches; every replay is
    checked against the oracle, with eager forwards of the same plan in between."""
    assert torch.cuda.is_available()
    from fbgemm_amd import ops
    from helpers import INT2
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(77)
    specs = [(3000, 128, INT4), (500, 32, INT2), (2000, 64, INT4), (700, 40, INT4)]
    T, B, L = len(specs), 4096, 130  # 2.13 M lookups: the scheduler runs, and with it the side stream
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.integers(L - 30, L + 31, size=T * B)
    lens[-1] += T * B * L - int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    n = int(off[-1])
    assert n >= 1 << 21

    def draw():
        return np.concatenate([rng.integers(0, specs[t][0], size=int(off[(t + 1) * B] - off[t * B])) for t in range(T)]).astype(np.int64)

    idx = draw()
    d_idx, d_off = cu(idx), cu(off)
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    st = ops.Status()
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 32, 128, 0, 0, 0, d_idx, d_off, 0, None, FP16, row_alignment=16, status=st)

    def expect(idx):
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP16, 16)
        assert rc == 0
        return want

    eager = call()
    torch.cuda.synchronize()
    H.assert_same_bits(eager.cpu().view(torch.int16).numpy().view(np.uint16), expect(idx), "eager")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = call()
    torch.cuda.synchronize()
    for replay in range(3):
        idx = draw()
        d_idx.copy_(cu(idx))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        H.assert_same_bits(captured.cpu().view(torch.int16).numpy().view(np.uint16), expect(idx), f"replay {replay}")
        again = call()
        torch.cuda.synchronize()
        assert torch.equal(again, captured)
    assert st.read() == (0, -1)


@pytest.mark.parametrize("mixed", [False, True])
def test_int8_output_forward_replays_from_a_graph(oracle, mixed):
    """The 8-bit pooled output under capture: the lean kernel's instances that quantize in their
    output stage, and (mixed) the float route through the plan's scratch and the quantizer beside
    them, with the side stream's fork and join. Every replay byte for byte against the pooled
    oracle + quantizer oracle, eager forwards of the same plan in between."""
    assert torch.cuda.is_available()
    from fbgemm_amd import ops
    from helpers import INT2, INT8
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(79 + mixed)
    specs = [(3000, 128, INT4), (2000, 64, INT4), (900, 64, INT8)] + ([(500, 32, INT2), (700, 40, INT4)] if mixed else [])
    T, B, L = len(specs), 4096, 180 if not mixed else 110
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.integers(L - 30, L + 31, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    assert int(off[-1]) >= 1 << 21  # the scheduler runs (and, mixed, the side stream)

    def draw():
        return np.concatenate([rng.integers(0, specs[t][0], size=int(off[(t + 1) * B] - off[t * B])) for t in range(T)]).astype(np.int64)

    idx = draw()
    d_idx, d_off = cu(idx), cu(off)
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    st = ops.Status()
    maxd = lambda ty: max([s[1] for s in specs if s[2] == ty], default=0)
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, maxd(INT2), maxd(INT4), maxd(INT8), 0, 0, d_idx, d_off, 0, None, INT8, row_alignment=16, status=st)

    def check(got, idx, what):
        rc, pooled = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, None, FP32, 16)
        assert rc == 0
        got = got.cpu().numpy()
        for t in range(T):
            D = specs[t][1]
            want = oracle.quantize_rowwise(np.ascontiguousarray(pooled[:, D_offsets[t]:D_offsets[t + 1]]), 8, True)
            block = got[:, D_offsets[t] + 8 * t:D_offsets[t] + 8 * t + D + 8]
            assert (block == want).all(), (what, t, np.argwhere(block != want)[:4])

    eager = call()  # outside the capture: work lists, side stream, float scratch
    torch.cuda.synchronize()
    check(eager, idx, "eager")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = call()
    torch.cuda.synchronize()
    for replay in range(3):
        idx = draw()
        d_idx.copy_(cu(idx))
        captured.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check(captured, idx, f"replay {replay}")
        again = call()
        torch.cuda.synchronize()
        assert torch.equal(again, captured)
    assert st.read() == (0, -1)


def test_wide_4bit_plan_with_its_redo_queue_replays_from_a_graph(oracle, request):
    """A plan whose tables all have 4-bit rows in bags of 8 lanes: the lean kernel's four-waves-per-SIMD
    instance and the kernel behind it that pools what that instance queues (bags with weight x scale
    beyond the pre-scaled range). The queue's counters are set back by the second kernel itself, so a
    captured forward replays: every replay draws new indices and moves the huge weights to other bags,
    and is checked bit for bit against the oracle."""
    assert torch.cuda.is_available()
    import fbgemm_amd
    from fbgemm_amd import ops
    from test_tbe_gpu import build_weights
    lib = fbgemm_amd.lib()
    lib.fbgemm_amd_set_wide4(2)  # that instance, not whichever the first forwards find faster
    request.addfinalizer(lambda: lib.fbgemm_amd_set_wide4(-1))
    rng = np.random.default_rng(81)
    specs = [(3000, 256, INT4), (2000, 256, INT4)]
    T, B = len(specs), 72_000
    weights, wo, _ = build_weights(rng, specs, 16)
    tys = np.array([s[2] for s in specs], np.uint8)
    D_offsets = np.concatenate([[0], np.cumsum([s[1] for s in specs])]).astype(np.int32)
    total_D = int(D_offsets[-1])
    lens = rng.poisson(15, size=T * B)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    n = int(off[-1])
    assert (1 << 21) <= n < 20 * T * B  # the bags are ordered; short enough to keep 8 lanes per bag

    def draw():
        idx = np.concatenate([rng.integers(0, specs[t][0], size=int(off[(t + 1) * B] - off[t * B])) for t in range(T)]).astype(np.int64)
        w = rng.uniform(0, 1, n).astype(np.float32)
        for b in rng.integers(0, T * B, size=9):
            w[int(off[b]):int(off[b + 1])] = np.float32(2.0 ** 108)
        return idx, w

    idx, w = draw()
    d_idx, d_off, d_w = cu(idx), cu(off), cu(w)
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(T, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    st = ops.Status()
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, total_D, 0, 256, 0, 0, 0, d_idx, d_off, 0, d_w, FP32, row_alignment=16, status=st)

    def expect(idx, w):
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, total_D, idx, off, 0, w, FP32, 16)
        assert rc == 0
        return want

    eager = call()
    torch.cuda.synchronize()
    H.assert_same_bits(eager.cpu().numpy(), expect(idx, w), "eager")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = call()
    torch.cuda.synchronize()
    for replay in range(3):
        idx, w = draw()
        d_idx.copy_(cu(idx))
        d_w.copy_(cu(w))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        H.assert_same_bits(captured.cpu().numpy(), expect(idx, w), f"replay {replay}")
        again = call()
        torch.cuda.synchronize()
        assert torch.equal(again, captured)
    assert st.read() == (0, -1)


def test_mappings_changed_before_a_capture_are_refused(oracle):
    """Pruned-row mappings edited in place keep their address: a forward under stream capture cannot
    rebuild the plan's compact form of them (that allocates and synchronizes) and must not take the
    old one into the graph. It raises; after one forward outside the capture the capture works."""
    assert torch.cuda.is_available()
    from fbgemm_amd import ops
    from test_tbe_gpu import build_weights
    rng = np.random.default_rng(5)
    logical, kept = 400, 250
    m = np.full(logical, -1, np.int32)
    m[np.sort(rng.choice(logical, kept, replace=False))] = np.arange(kept, dtype=np.int32)
    specs = [(kept, 64, INT4)]
    weights, wo, _ = build_weights(rng, specs, 16)
    tys, D_offsets = np.array([INT4], np.uint8), np.array([0, 64], np.int32)
    B, L = 8, 5
    off = (np.arange(B + 1) * L).astype(np.int64)
    idx = rng.integers(0, logical, size=B * L).astype(np.int64)
    d_remap, d_remap_off = cu(m), cu(np.array([0, logical], np.int64))
    meta = (cu(weights), torch.zeros(0, dtype=torch.uint8, device="cuda"), cu(np.zeros(1, np.int32)), cu(wo), cu(tys), cu(D_offsets))
    d_idx, d_off = cu(idx), cu(off)
    st = ops.Status()  # read by the test, not by the forward: a forward under capture cannot synchronize
    call = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(
        *meta, 64, 0, 64, 0, 0, 0, d_idx, d_off, 0, None, FP16, row_alignment=16,
        index_remappings=d_remap, index_remappings_offsets=d_remap_off, status=st)

    def expect(mapping):
        dense = oracle.pruned_array_lookup(idx, off, mapping, np.array([0, logical], np.int64))
        rc, want = oracle.tbe_forward(weights, wo, tys, D_offsets, 64, dense, off, 0, None, FP16, 16)
        assert rc == 0
        return want

    H.assert_same_bits(call().cpu().view(torch.int16).numpy().view(np.uint16), expect(m), "first forward")
    # prune one more row, in place: kept rows behind it move up by one
    victim = int(np.nonzero(m >= 0)[0][3])
    m2 = m.copy()
    m2[victim] = -1
    m2[m2 > m[victim]] -= 1
    d_remap.copy_(cu(m2))
    side = torch.cuda.Stream()
    refused = None
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            d_off.add_(0)  # something to capture: the refused forward launches nothing
            try:
                call()
            except RuntimeError as e:  # caught inside, so that the capture ends in order
                refused = str(e)
    torch.cuda.synchronize()
    assert refused is not None and "outside the stream capture" in refused, refused
    del graph
    H.assert_same_bits(call().cpu().view(torch.int16).numpy().view(np.uint16), expect(m2), "forward after the change")
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = call()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    H.assert_same_bits(captured.cpu().view(torch.int16).numpy().view(np.uint16), expect(m2), "replay")
    assert st.read() == (0, -1)
