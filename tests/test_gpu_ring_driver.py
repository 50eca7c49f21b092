"""The step-wise ring driver (W ranks as W tensors on one GPU, one stream per
rank, fences between dependent steps) against the oracle's ring-order fold, the
reference's own known answers (tests/test_process_group_local.py:478-578,
:635-647; tests/test_correctness_vs_reference.py:36-78), and the two-rank / hub
paths with and without compression (csrc/backend/ProcessGroupMCCL.cpp:1632-1709,
:2257-2313)."""
import numpy as np
import pytest
import torch
import torch.distributed  # noqa: F401

import oracle
from oracle import F32, F16, BF16, OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX, RING_BASIC, RING_CHUNKED
from tests._gpu_util import DEV, to_dev, to_np, bits, rand_vals, TORCH_DT

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def C():
    from mccl_amd import _C
    return _C


def _check_all_ranks(dts, dt, want):
    for r, t in enumerate(dts):
        assert np.array_equal(bits(to_np(t, dt)), bits(want)), f"rank {r}"


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("ws", [2, 3, 4, 8])
@pytest.mark.parametrize("streams", [True, False])
def test_fp32_ring_equals_oracle(C, chunked, ws, streams):
    g = C.LoopbackGroup(ws, None, streams)
    rng = np.random.default_rng(ws * 11 + int(chunked))
    schedule = RING_CHUNKED if chunked else RING_BASIC
    for n in (1, 5, 2 * ws - 1, 2 * ws + 1, 4097, 70_001, 1_000_003):
        ins = [rand_vals(rng, n, F32, sigma=1e-3, specials=False) for _ in range(ws)]
        for op in (OP_SUM, OP_AVG, OP_MIN, OP_MAX, OP_PRODUCT):
            inv = float(np.float32(1.0 / ws))
            want = oracle.ring_fold(ins, F32, op, schedule, scale_by=inv if op == OP_AVG else None)
            dts = [to_dev(x, F32, pad_front=r % 3) for r, x in enumerate(ins)]
            g.allreduce_ring(dts, op, chunked)
            torch.cuda.synchronize()
            _check_all_ranks(dts, F32, want)
    s = g.stats()
    assert s["last_algo"] == ("ring_chunked" if chunked else "ring")
    assert (s["stream_waits"] > 0) == streams and (s["fences_signalled"] > 0) == streams


@pytest.mark.parametrize("dt", [F16, BF16])
@pytest.mark.parametrize("chunked", [False, True])
def test_half_ring_rounds_every_step_like_the_wire(C, dt, chunked):
    ws = 4
    g = C.LoopbackGroup(ws)
    rng = np.random.default_rng(dt)
    schedule = RING_CHUNKED if chunked else RING_BASIC
    for n in (9, 70_001, 262_147):
        ins = [rand_vals(rng, n, dt, sigma=1.0, specials=False) for _ in range(ws)]
        for op in (OP_SUM, OP_AVG, OP_MAX, OP_MIN):
            want = oracle.ring_fold(ins, dt, op, schedule, scale_by=0.25 if op == OP_AVG else None, stepwise=True)
            dts = [to_dev(x, dt, pad_front=r) for r, x in enumerate(ins)]
            g.allreduce_ring(dts, op, chunked)
            torch.cuda.synchronize()
            _check_all_ranks(dts, dt, want)


@pytest.mark.parametrize("dt", [F16, BF16])
def test_half_ring_three_ranks_scale_in_fp32(C, dt):
    # 1/3 is not exact in any format: the AVG tail multiplies by float(1/3) in fp32 and rounds once
    ws = 3
    g = C.LoopbackGroup(ws)
    rng = np.random.default_rng(31 + dt)
    inv = float(np.float32(1.0 / 3.0))
    for n, chunked in ((70_001, True), (4099, False)):
        ins = [rand_vals(rng, n, dt, sigma=1.0, specials=False) for _ in range(ws)]
        want = oracle.ring_fold(ins, dt, OP_AVG, RING_CHUNKED if chunked else RING_BASIC, scale_by=inv, stepwise=True)
        dts = [to_dev(x, dt) for x in ins]
        g.allreduce_ring(dts, OP_AVG, chunked)
        torch.cuda.synchronize()
        _check_all_ranks(dts, dt, want)


@pytest.mark.parametrize("n", [70_000, 70_001])
@pytest.mark.parametrize("chunked", [False, True])
def test_reference_three_rank_constants(C, n, chunked):
    # rank r holds r+1: SUM 6, AVG exactly 2.0, MIN 1, MAX 3 at zero tolerance
    g = C.LoopbackGroup(3)
    for op, want in ((OP_SUM, 6.0), (OP_AVG, 2.0), (OP_MIN, 1.0), (OP_MAX, 3.0), (OP_PRODUCT, 6.0)):
        ts = [torch.full((n,), float(r + 1), device=DEV) for r in range(3)]
        g.allreduce_ring(ts, op, chunked)
        for t in ts:
            assert float((t - want).abs().max()) == 0.0


@pytest.mark.parametrize("n", [1, 3, 1023, 4097, 70_001, 262_147])
def test_reference_pattern_vs_exact_sum(C, n):
    # arange(n) % 13 - 6 + rank + 1: small integers, every order gives the same bits
    ws = 4
    g = C.LoopbackGroup(ws)
    base = (torch.arange(n, device=DEV) % 13 - 6).float()
    for op, fn in ((OP_SUM, lambda xs: sum(xs)), (OP_AVG, lambda xs: sum(xs) / ws),
                   (OP_MAX, lambda xs: torch.stack(xs).max(0).values)):
        ts = [base + (r + 1) for r in range(ws)]
        want = fn([t.clone() for t in ts])
        g.allreduce(ts, op)          # dispatch: hub below 256 KiB, ring above
        for t in ts:
            assert torch.equal(t, want)
    assert g.stats()["last_algo"] == ("small" if n * 4 <= 262144 else "ring_chunked")


def test_int_rings_and_avg_scale(C):
    ws = 3
    g = C.LoopbackGroup(ws)
    for dtype in (torch.int32, torch.int64):
        for n in (7, 70_001):
            ts = [((torch.arange(n, device=DEV) % 11) + r).to(dtype) for r in range(ws)]
            want = sum(t.clone() for t in ts)
            g.allreduce_ring(ts, OP_SUM, True)
            for t in ts:
                assert torch.equal(t, want)
    # AVG on int64 truncates the scaled sum (csrc/metal/shaders.metal:650)
    ts = [torch.full((100,), 3 * r + 1, device=DEV, dtype=torch.int64) for r in range(ws)]   # 1, 4, 7 -> 12 -> 4
    g.allreduce_ring(ts, OP_AVG, False)
    for t in ts:
        assert int(t.min()) == int(t.max()) == int(np.float32(12) * np.float32(1.0 / 3))


def test_env_selects_the_basic_ring(C, monkeypatch):
    monkeypatch.setenv("MCCL_RING_ALGO", "basic")
    g = C.LoopbackGroup(3)
    ts = [torch.ones(100_000, device=DEV) * (r + 1) for r in range(3)]
    g.allreduce(ts, OP_SUM)
    assert g.stats()["last_algo"] == "ring" and float(ts[2][-1]) == 6.0


def test_full_size_ring_equals_fused_fold(C):
    # 96,510,024 elements, 8 ranks: the step-wise driver and the fused W-way kernel agree bit for bit
    from mccl_amd import hip_ops
    ws, n = 8, 96_510_024
    gens = [torch.Generator(device=DEV).manual_seed(50 + r) for r in range(ws)]
    ins = [torch.randn(n, device=DEV, generator=gens[r]).mul_(1e-3) for r in range(ws)]
    fused = torch.empty(n, device=DEV)
    hip_ops.ring_fold(fused, ins, hip_ops.AVG, hip_ops.RING_CHUNKED, scale_by=0.125)
    g = C.LoopbackGroup(ws)
    g.allreduce_ring(ins, OP_AVG, True)
    torch.cuda.synchronize()
    for r in (0, 3, 7):
        assert torch.equal(ins[r].view(torch.int32), fused.view(torch.int32))
    s = g.stats()
    assert s["reduce_launches"] == 8 * 14 and s["copy_launches"] == 8 * 14


def test_many_ranks_fall_back_to_one_stream(C):
    ws = 24   # 24 * 92 tickets would not fit the fence ring
    g = C.LoopbackGroup(ws)
    ts = [torch.full((1000,), float(r), device=DEV) for r in range(ws)]
    g.allreduce_ring(ts, OP_SUM, True)
    assert g.stats()["fences_signalled"] == 0
    for t in ts:
        assert float(t.min()) == float(t.max()) == sum(range(ws))


def test_two_rank_paths(C):
    g = C.LoopbackGroup(2)
    rng = np.random.default_rng(2)
    for n in (1, 1000, 70_001):
        a, b = (rand_vals(rng, n, F32, specials=False) for _ in range(2))
        for op in (OP_SUM, OP_AVG, OP_MIN, OP_MAX):
            ts = [to_dev(a, F32), to_dev(b, F32)]
            g.allreduce(ts, op)
            want = a.copy()
            if op == OP_AVG:
                oracle.fold2_scale(want, b, F32, 0.5)
            else:
                oracle.fold2(want, b, F32, op)
            _check_all_ranks(ts, F32, want)
    assert g.stats()["last_algo"] == "two_rank"


def test_two_rank_fp16_compression_is_lossless_on_representable_values(C):
    o = C.MCCLOptions(); o.compression = C.CompressionMode.FP16
    g = C.LoopbackGroup(2, o)
    for n in (1024, 70_001):
        ts = [torch.full((n,), (r + 1) * 0.5, device=DEV) for r in range(2)]
        g.allreduce(ts, OP_SUM)
        for t in ts:
            assert int((t != 1.5).sum()) == 0
    assert g.stats()["wire_bytes"] == 2 * (4 + 2 * 1024) + 2 * (4 + 2 * 70_001)
    with pytest.raises(RuntimeError, match="BFloat16 tensors are not supported with compression enabled"):
        g.allreduce([torch.ones(8, device=DEV, dtype=torch.bfloat16) for _ in range(2)], OP_SUM)


def test_hub_with_topk_follows_the_reference_sequence(C):
    # rank 0 folds decompress(compress_p(x_p)) for p = 1..ws-1, scales, then sends
    # compress_0(result) to each peer in turn -- each send applies rank 0's error
    # feedback again (csrc/backend/ProcessGroupMCCL.cpp:2283-2306).
    ws, n, ratio = 4, 20_000, 0.05
    o = C.MCCLOptions(); o.compression = C.CompressionMode.TOPK; o.topk_ratio = ratio
    g = C.LoopbackGroup(ws, o)
    rng = np.random.default_rng(9)
    res = [np.zeros(n, np.float32) for _ in range(ws)]
    ts = [torch.empty(n, device=DEV) for _ in range(ws)]      # stable storage: residuals keyed by address
    for step in range(3):
        xs = [rand_vals(rng, n, F32, specials=False) for _ in range(ws)]
        for r in range(ws):
            ts[r].copy_(torch.from_numpy(xs[r]))
        g.allreduce(ts, OP_AVG)
        acc = xs[0].copy()
        for p in range(1, ws):
            wire, _ = oracle.topk_compress(xs[p], res[p], ratio)
            dense, rc = oracle.topk_decompress(wire, n)
            assert rc == 0
            oracle.fold2(acc, dense, F32, OP_SUM)
        oracle.scale(acc, F32, float(np.float32(1.0 / ws)))
        assert np.array_equal(bits(to_np(ts[0], F32)), bits(acc)), step
        for p in range(1, ws):
            wire, _ = oracle.topk_compress(acc, res[0], ratio)
            dense, _ = oracle.topk_decompress(wire, n)
            assert np.array_equal(bits(to_np(ts[p], F32)), bits(dense)), (step, p)
    assert g.stats()["last_algo"] == "small"
    k = oracle.topk_k(n, ratio)
    assert g.stats()["wire_bytes"] == 3 * 2 * (ws - 1) * (4 + 4 + 8 * k)


def test_framing_checks(C):
    c = C.make_compressor(C.CompressionMode.TOPK, 0.1)
    x = torch.randn(1000, device=DEV)
    size, payload = C._compressed_pack(c, x)
    assert size == payload.numel() == 4 + 8 * 100 and c.max_compressed_size(4000) == 812
    out = torch.empty(1000, device=DEV)
    C._compressed_unpack(c, size, payload, out)
    assert int((out != 0).sum()) == 100
    with pytest.raises(RuntimeError, match=r"Compressed payload size 0 out of range \(max 812\)"):
        C._compressed_unpack(c, 0, payload[:0], out)
    with pytest.raises(RuntimeError, match=r"Compressed payload size 820 out of range \(max 812\)"):
        C._compressed_unpack(c, 820, torch.zeros(820, dtype=torch.uint8, device=DEV), out)
    with pytest.raises(RuntimeError, match="TopK decompress: size mismatch"):
        C._compressed_unpack(c, 796, payload[:796].contiguous(), out)


def test_coalesced_flattens_and_scatters(C):
    ws = 3
    o = C.MCCLOptions(); o.small_msg_threshold = 1024
    g = C.LoopbackGroup(ws, o)
    shapes = [(5, 7), (0,), (1000,), (3, 3, 3)]
    lists = [[torch.full(s, float(r + 1 + i), device=DEV) for i, s in enumerate(shapes)] for r in range(ws)]
    g.allreduce_coalesced(lists, OP_SUM)
    for r in range(ws):
        for i, s in enumerate(shapes):
            assert lists[r][i].shape == torch.Size(s)
            if lists[r][i].numel():
                assert float(lists[r][i].min()) == float(lists[r][i].max()) == 6.0 + 3 * i
    assert g.stats()["last_algo"] == "ring_chunked"
    with pytest.raises(RuntimeError, match="allreduce_coalesced: empty tensor list"):
        g.allreduce_coalesced([[], [], []], OP_SUM)


@pytest.mark.parametrize("ws", [1, 2, 3, 5])
def test_reduce_scatter_order_and_no_avg_scale(C, ws):
    # own contribution first, the others in ascending rank order; AVG adds without scaling
    g = C.LoopbackGroup(ws)
    rng = np.random.default_rng(40 + ws)
    n = 70_001
    for op in (OP_SUM, OP_AVG, OP_MAX):
        host = [[rand_vals(rng, n, F32, sigma=1e-3, specials=False) for _ in range(ws)] for _ in range(ws)]
        ins = [[to_dev(x, F32) for x in row] for row in host]
        outs = [torch.empty(n, device=DEV) for _ in range(ws)]
        g.reduce_scatter(outs, ins, op)
        torch.cuda.synchronize()
        for d in range(ws):
            want = host[d][d].copy()
            for src in range(ws):
                if src != d:
                    oracle.fold2(want, host[src][d], F32, OP_SUM if op == OP_AVG else op)
            assert np.array_equal(bits(to_np(outs[d], F32)), bits(want)), (op, d)
    if ws > 1:
        assert g.stats()["last_algo"] == ("reduce_scatter_star" if ws >= 3 else "reduce_scatter_ring")
    with pytest.raises(RuntimeError, match="Input tensor list size must equal world_size"):
        g.reduce_scatter([torch.empty(4, device=DEV) for _ in range(ws)],
                         [[torch.empty(4, device=DEV)] * (ws + 1) for _ in range(ws)], OP_SUM)


def test_argument_checks(C):
    g = C.LoopbackGroup(3)
    with pytest.raises(RuntimeError, match="one tensor per rank expected"):
        g.allreduce([torch.ones(4, device=DEV)] * 2, OP_SUM)
    t = torch.ones(4, device=DEV)
    with pytest.raises(RuntimeError, match="each rank needs a buffer of its own"):
        g.allreduce([t, t, t], OP_SUM)
    with pytest.raises(RuntimeError, match="Shape mismatch in collective"):
        g.allreduce([torch.ones(4, device=DEV), torch.ones(5, device=DEV), torch.ones(4, device=DEV)], OP_SUM)
    with pytest.raises(RuntimeError, match="Unsupported ReduceOp"):
        g.allreduce_ring([torch.ones(400, device=DEV) for _ in range(3)], 7, True)
