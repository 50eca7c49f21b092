"""Host-side ring plan, chunk views and algorithm selection (no GPU needed).

The plan is checked by running it symbolically: every rank's chunk slot holds
the expression tree of what has been folded into it.  After the reduce-scatter
half the owner's tree must be the left fold the oracle's closed form uses
(start at orc_ring_first_rank(c), then the following ranks in order; the oracle
itself is pinned against a step-by-step simulation in test_oracle_ring.py), and
after the all-gather half every rank must hold that same tree in every slot.
Formulas: csrc/backend/ProcessGroupMCCL.cpp:1764-1785 (chunked), :2016-2035
(basic)."""
import pytest
import torch
import torch.distributed  # noqa: F401

import oracle


@pytest.fixture(scope="module")
def C():
    from mccl_amd import _C
    return _C


def _run_symbolic(C, ws, chunked):
    m = 2 * ws if chunked else ws
    plans = [C._ring_plan(r, ws, chunked) for r in range(ws)]
    state = [[("x", r) for _ in range(m)] for r in range(ws)]
    nsteps = len(plans[0])
    assert nsteps == (4 if chunked else 2) * (ws - 1)
    after_rs = None
    for s in range(nsteps):
        snap = [list(row) for row in state]  # every send of a step reads pre-step data
        for q in range(ws):
            p = (q - 1) % ws
            send_idx, recv_idx, send_tid, recv_tid, kind = plans[q][s]
            assert plans[p][s][0] == recv_idx and plans[p][s][2] == recv_tid
            assert send_idx != recv_idx
            assert send_tid == (s << 16 | send_idx) and recv_tid == (s << 16 | recv_idx)
            assert kind == ("reduce" if s < nsteps // 2 else "copy")
            if kind == "reduce":
                state[q][recv_idx] = ("op", snap[q][recv_idx], snap[p][recv_idx])  # local op incoming
            else:
                state[q][recv_idx] = snap[p][recv_idx]
        if s == nsteps // 2 - 1:
            after_rs = [list(row) for row in state]
    return state, after_rs, m


def _closed_form(c, ws, schedule):
    s = oracle.lib.orc_ring_first_rank(c, ws, schedule)
    acc = ("x", s)
    for j in range(1, ws):
        acc = ("op", ("x", (s + j) % ws), acc)
    return acc


@pytest.mark.parametrize("ws", [2, 3, 4, 5, 8, 13])
@pytest.mark.parametrize("chunked", [False, True])
def test_plan_folds_in_the_oracles_order_and_gathers_everything(C, ws, chunked):
    state, after_rs, m = _run_symbolic(C, ws, chunked)
    schedule = oracle.RING_CHUNKED if chunked else oracle.RING_BASIC
    assert oracle.lib.orc_ring_chunks(ws, schedule) == m
    for c in range(m):
        want = _closed_form(c, ws, schedule)
        owners = [r for r in range(ws) if after_rs[r][c] == want]
        assert len(owners) == 1          # exactly one rank holds the finished chunk after reduce-scatter
        for r in range(ws):
            assert state[r][c] == want   # and everyone after all-gather


def test_plan_known_answers(C):
    # ws=3 basic, rank 1: reduce-scatter sends 1,0 and receives 0,2; all-gather sends 2,1 and receives 1,0
    assert [(a, b, k) for a, b, _, _, k in C._ring_plan(1, 3, False)] == [
        (1, 0, "reduce"), (0, 2, "reduce"), (2, 1, "copy"), (1, 0, "copy")]
    # ws=2 chunked, rank 0: (2r-step, 2r-step-2) mod 4, then (2r+2-step, 2r-step) mod 4
    assert [(a, b) for a, b, _, _, _ in C._ring_plan(0, 2, True)] == [(0, 2), (3, 1), (2, 0), (1, 3)]
    assert C._ring_plan(0, 1, True) == []
    with pytest.raises(RuntimeError, match="rank out of range"):
        C._ring_plan(3, 3, True)


@pytest.mark.parametrize("n,ws,chunked", [(70_001, 3, False), (70_001, 3, True), (5, 8, True), (0, 4, False),
                                          (16, 8, True), (6_553_600, 8, False)])
def test_chunk_views_match_the_oracles_chunking(C, n, ws, chunked):
    t = torch.arange(n, dtype=torch.int32)
    views = C._ring_chunk_views(t, ws, chunked)
    schedule = oracle.RING_CHUNKED if chunked else oracle.RING_BASIC
    per = oracle.lib.orc_ring_chunk_elems(n, ws, schedule)
    assert len(views) == (2 * ws if chunked else ws)
    assert sum(v.numel() for v in views) == n
    for i, v in enumerate(views):
        lo = min(i * per, n)
        assert v.numel() == min(per, n - lo)
        if v.numel():
            assert v.data_ptr() == t.data_ptr() + 4 * lo and int(v[0]) == lo
    with pytest.raises(RuntimeError, match="contiguous"):
        C._ring_chunk_views(torch.zeros(4, 4).t(), ws, chunked)


def test_ring_algo_env(C, monkeypatch):
    monkeypatch.delenv("MCCL_RING_ALGO", raising=False)
    assert C._ring_algo_from_env() == "chunked"
    for v in ("basic", "ring", "plain"):
        monkeypatch.setenv("MCCL_RING_ALGO", v)
        assert C._ring_algo_from_env() == "basic"
    monkeypatch.setenv("MCCL_RING_ALGO", "chunked")
    assert C._ring_algo_from_env() == "chunked"
    monkeypatch.setenv("MCCL_RING_ALGO", "anything")
    assert C._ring_algo_from_env() == "chunked"


def test_group_construction_and_compressors(C):
    g = C.LoopbackGroup(4)
    assert g.size() == 4 and g.compressor(0) is None and g.stats()["collectives"] == 0
    o = C.MCCLOptions()
    o.compression = C.CompressionMode.TOPK
    o.topk_ratio = 0.1
    g = C.LoopbackGroup(3, o)
    assert isinstance(g.compressor(2), C.TopKCompressor) and g.compressor(2).max_compressed_size(4000) == 4 + 8 * 101
    o.compression = C.CompressionMode.FP16
    assert C.LoopbackGroup(2, o).compressor(1).name() == "fp16"
    with pytest.raises(RuntimeError, match="world size"):
        C.LoopbackGroup(0)
    with pytest.raises(RuntimeError, match="rank out of range"):
        g.compressor(3)
