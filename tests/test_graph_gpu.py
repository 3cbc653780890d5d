"""The table-batched forward inside a HIP graph (torch.cuda.CUDAGraph): once a plan has
seen a batch size, a forward is kernel launches only (no allocation, no copy, no
synchronization), so a serving loop can capture it. Every replay is checked against
the oracle, with eager work and synchronizations between the replays."""
import numpy as np
import pytest

import helpers as H
from helpers import FP16, INT4, INT8

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
