"""The reference's own kernel tests (tests/test_local_kernels.py) run against
mccl_amd._C on a ROCm device, plus the device-resident compressor's state rules
(csrc/compression/TopKCompression.cpp:57-67,:160-179) and the two-bucket
residual isolation of tests/test_compression_e2e.py:33-75."""
import numpy as np
import pytest
import torch
import torch.distributed  # noqa: F401

import oracle
from tests._gpu_util import DEV, bits, student_t

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def k():
    from mccl_amd import _C
    return {"accumulate": _C._metal_accumulate_chunk, "min": _C._metal_elementwise_min,
            "max": _C._metal_elementwise_max, "product": _C._metal_elementwise_product,
            "scale": _C._metal_scale_inplace, "acc_scale": _C._metal_accumulate_and_scale, "C": _C}


def t(v, dt=torch.float32):
    return torch.tensor(v, device=DEV, dtype=dt)


class TestAccumulateChunk:
    def test_f32_basic(self, k):
        a = t([1.0, 2.0, 3.0]); b = t([4.0, 5.0, 6.0])
        r = k["accumulate"](a, b)
        assert r is a and torch.equal(r, t([5.0, 7.0, 9.0]))

    def test_f32_zeros(self, k):
        b = torch.ones(256, device=DEV) * 3.0
        assert torch.equal(k["accumulate"](torch.zeros(256, device=DEV), b), b)

    def test_f32_non_aligned_size(self, k):
        for size in (1, 3, 7, 13, 97, 997):
            r = k["accumulate"](torch.ones(size, device=DEV) * 2.0, torch.ones(size, device=DEV) * 3.0)
            assert torch.equal(r, torch.ones(size, device=DEV) * 5.0), size

    def test_f32_large(self, k):
        a = torch.randn(1_000_000, device=DEV); b = torch.randn(1_000_000, device=DEV)
        want = a.cpu() + b.cpu()
        assert torch.equal(k["accumulate"](a, b).cpu(), want)

    def test_f16_and_bf16(self, k):
        for dt in (torch.float16, torch.bfloat16):
            assert torch.equal(k["accumulate"](t([1., 2., 3.], dt), t([4., 5., 6.], dt)), t([5., 7., 9.], dt))
            for size in (1, 3, 7, 13):
                r = k["accumulate"](torch.ones(size, device=DEV, dtype=dt) * 2, torch.ones(size, device=DEV, dtype=dt) * 3)
                assert torch.equal(r, torch.ones(size, device=DEV, dtype=dt) * 5)

    def test_i64_non_aligned(self, k):
        for size in (1, 3, 7, 13):
            a = torch.arange(size, device=DEV, dtype=torch.int64)
            b = torch.full((size,), 3, device=DEV, dtype=torch.int64)
            assert torch.equal(k["accumulate"](a.clone(), b), a + b)


class TestMinMaxProduct:
    def test_basic(self, k):
        assert torch.equal(k["min"](t([1., 5., 3.]), t([4., 2., 6.])), t([1., 2., 3.]))
        assert torch.equal(k["max"](t([1., 5., 3.]), t([4., 2., 6.])), t([4., 5., 6.]))
        assert torch.equal(k["product"](t([2., 3., 4.]), t([5., 6., 7.])), t([10., 18., 28.]))
        a = torch.ones(100, device=DEV) * -1.0
        assert torch.equal(k["min"](a.clone(), torch.ones(100, device=DEV)), a)

    def test_non_aligned_vs_torch(self, k):
        for size in (1, 3, 7, 13, 97):
            a = torch.randn(size, device=DEV); b = torch.randn(size, device=DEV)
            assert torch.equal(k["min"](a.clone(), b), torch.minimum(a, b))
            assert torch.equal(k["max"](a.clone(), b), torch.maximum(a, b))
            assert torch.equal(k["product"](a.clone(), b), a * b)

    def test_f16(self, k):
        h = torch.float16
        assert torch.equal(k["min"](t([1., 5., 3.], h), t([4., 2., 6.], h)), t([1., 2., 3.], h))
        assert torch.equal(k["max"](t([1., 5., 3.], h), t([4., 2., 6.], h)), t([4., 5., 6.], h))
        assert torch.equal(k["product"](t([2., 3., 4.], h), t([5., 6., 7.], h)), t([10., 18., 28.], h))


class TestScaleAndFused:
    def test_scale(self, k):
        assert torch.equal(k["scale"](t([2., 4., 6.]), 0.5), t([1., 2., 3.]))
        a = torch.randn(1000, device=DEV)
        assert torch.equal(k["scale"](a.clone(), 1.0), a)
        for ws in (2, 3, 4, 8):
            r = k["scale"](torch.ones(256, device=DEV) * float(ws), 1.0 / ws)
            assert torch.allclose(r, torch.ones(256, device=DEV), rtol=1e-5, atol=1e-5)
        for size in (1, 3, 7, 13, 97):
            a = torch.randn(size, device=DEV)
            assert torch.equal(k["scale"](a.clone(), 0.25), a * 0.25)
        assert torch.equal(k["scale"](t([2., 4., 6.], torch.float16), 0.5), t([1., 2., 3.], torch.float16))

    def test_integral_avg_semantics(self, k):
        for size in (1, 3, 7, 13):
            exp = torch.arange(1, size + 1, device=DEV, dtype=torch.int64)
            assert torch.equal(k["scale"](exp * 3, 1.0 / 3.0), exp)
        assert torch.equal(k["scale"](t([True, False, True], torch.bool), 0.5), torch.zeros(3, device=DEV, dtype=torch.bool))
        for dt in (torch.int64, torch.int32):
            r = k["acc_scale"](t([1, 3, 5, 7, 9], dt), t([3, 5, 7, 9, 11], dt), 0.5)
            assert torch.equal(r, t([2, 4, 6, 8, 10], dt))
        r = k["acc_scale"](t([True, True, False], torch.bool), t([True, False, True], torch.bool), 0.5)
        assert torch.equal(r, t([True, False, False], torch.bool))

    def test_fused(self, k):
        assert torch.equal(k["acc_scale"](t([1., 3., 5.]), t([3., 5., 7.]), 0.5), t([2., 4., 6.]))
        for size in (1, 3, 7, 13, 97):
            a = torch.randn(size, device=DEV); b = torch.randn(size, device=DEV)
            assert torch.equal(k["acc_scale"](a.clone(), b, 0.5), (a + b) * 0.5)
        h = torch.float16
        assert torch.equal(k["acc_scale"](t([1., 3., 5.], h), t([3., 5., 7.], h), 0.5), t([2., 4., 6.], h))


def test_reduce_op_batch_equals_reduce_op_pair_by_pair(k):
    C = k["C"]
    g = torch.Generator(device=DEV).manual_seed(5)
    sizes = [1, 7, 4096, 100_003, 5]
    for dt in (torch.float32, torch.bfloat16, torch.int64):
        def mk():
            if dt == torch.int64:
                return [torch.randint(-10**9, 10**9, (n,), generator=g, device=DEV) for n in sizes]
            return [torch.randn(n, generator=g, device=DEV).to(dt) for n in sizes]
        d0, s0 = mk(), mk()
        for op in (0, 3, 4):  # SUM, MIN, MAX
            one = [x.clone() for x in d0]
            many = [x.clone() for x in d0]
            for d, s_ in zip(one, s0):
                C._metal_reduce_op(d, s_, op)
            C._hip_reduce_op_batch(many, s0, op)
            for a, b in zip(one, many):
                assert torch.equal(a, b)
    x = torch.zeros(100, device=DEV)
    with pytest.raises(RuntimeError):
        C._hip_reduce_op_batch([x[:60], x[50:]], [torch.ones(60, device=DEV), torch.ones(50, device=DEV)], 0)
    with pytest.raises(RuntimeError, match="Dtype mismatch"):
        C._hip_reduce_op_batch([x], [torch.ones(100, device=DEV, dtype=torch.float16)], 0)
    C._hip_reduce_op_batch([], [], 0)


def test_errors_and_fenced_reduce(k):
    C = k["C"]
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        C._metal_accumulate_chunk(torch.zeros(3, device=DEV), torch.zeros(4, device=DEV))
    with pytest.raises(RuntimeError, match="Dtype mismatch"):
        C._metal_accumulate_chunk(torch.zeros(3, device=DEV), torch.zeros(3, device=DEV, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="contiguous"):
        C._metal_accumulate_chunk(torch.zeros(4, 4, device=DEV).t(), torch.zeros(4, 4, device=DEV))
    with pytest.raises(RuntimeError, match="Unsupported ReduceOp"):
        C._metal_reduce_op(torch.zeros(3, device=DEV), torch.zeros(3, device=DEV), 5)
    with pytest.raises(RuntimeError, match="No HIP accumulate kernel for dtype"):
        C._metal_accumulate_chunk(torch.zeros(3, device=DEV, dtype=torch.float64), torch.zeros(3, device=DEV, dtype=torch.float64))
    a = torch.ones(1 << 20, device=DEV); b = torch.ones(1 << 20, device=DEV)
    ticket = C._metal_reduce_op_fenced(a, b, 1)  # AVG folds like SUM
    assert C._event_sync_available() and ticket > 0
    C._wait_for_mccl_fence(ticket)
    assert float(a.sum()) == 2.0 * (1 << 20)
    assert torch.equal(C._cpu_reduce_op(t([1., 5.]), t([4., 2.]), 4), t([4., 5.]))  # MAX
    # ring fold through the C++ entry: 3 constant ranks, AVG -> exactly 2.0
    ins = [torch.full((70_001,), float(r + 1), device=DEV) for r in range(3)]
    out = C._hip_ring_fold(torch.empty(70_001, device=DEV), ins, 1)
    assert torch.equal(out, torch.full((70_001,), 2.0, device=DEV))


def test_compressor_state_rules(k):
    C = k["C"]
    n = 100_000
    rng = np.random.default_rng(0)
    comp = C.TopKCompressor(0.01)
    res_o = np.zeros(n, np.float32)
    for step in range(3):  # error feedback carried inside the compressor, keyed by the id
        g = student_t(rng, n)
        wire = comp.compress(torch.from_numpy(g).to(DEV), stable_id=42)
        w, rc = oracle.topk_compress(g, res_o, 0.01)
        assert wire.numel() == rc and wire.cpu().numpy().tobytes() == w.tobytes(), step
        assert np.array_equal(bits(comp.error_feedback_buffer(42).cpu().numpy()), bits(res_o))
    assert comp.error_feedback_buffer_count() == 1
    # another id starts from a zero residual; the first id's state is untouched
    g2 = student_t(rng, n)
    w2, _ = oracle.topk_compress(g2, np.zeros(n, np.float32), 0.01)
    assert comp.compress(torch.from_numpy(g2).to(DEV), stable_id=43).cpu().numpy().tobytes() == w2.tobytes()
    assert comp.error_feedback_buffer_count() == 2
    assert np.array_equal(bits(comp.error_feedback_buffer(42).cpu().numpy()), bits(res_o))
    # a changed element count resets that id's residual
    g3 = student_t(rng, n // 2)
    w3, _ = oracle.topk_compress(g3, np.zeros(n // 2, np.float32), 0.01)
    assert comp.compress(torch.from_numpy(g3).to(DEV), stable_id=42).cpu().numpy().tobytes() == w3.tobytes()
    comp.reset_error_feedback_for_tensor(43)
    assert float(comp.error_feedback_buffer(43).abs().sum()) == 0.0 and comp.error_feedback_buffer_count() == 2
    comp.reset_error_feedback()
    assert comp.error_feedback_buffer_count() == 0
    # default id = storage address + offset: two views of one storage are two tensors
    base = torch.from_numpy(student_t(rng, 2000)).to(DEV)
    comp.compress(base[:1000]); comp.compress(base[1000:])
    assert comp.error_feedback_buffer_count() == 2
    assert C._compression_stable_id(base[1000:]) == C._compression_stable_id(base) + 4000
    # the map is cleared when a 1025th id arrives
    small = torch.from_numpy(student_t(rng, 64)).to(DEV)
    comp.reset_error_feedback()
    for i in range(1024):
        comp.compress(small, stable_id=10_000 + i)
    assert comp.error_feedback_buffer_count() == 1024
    comp.compress(small, stable_id=5)
    assert comp.error_feedback_buffer_count() == 1


def test_compressor_errors_and_decompress(k):
    C = k["C"]
    comp = C.TopKCompressor(0.1)
    g = torch.from_numpy(student_t(np.random.default_rng(1), 1000)).to(DEV)
    with pytest.raises(RuntimeError, match="buffer too small"):
        comp.compress(g, capacity=4 + 8 * 100 - 1)
    with pytest.raises(RuntimeError, match="float32 only"):
        comp.compress(g.half())
    wire = comp.compress(g, stable_id=1)
    dense = comp.decompress(wire, 1000)
    want, _ = oracle.topk_decompress(wire.cpu().numpy(), 1000)
    assert np.array_equal(bits(dense.cpu().numpy()), bits(want))
    with pytest.raises(RuntimeError, match="size mismatch"):
        comp.decompress(wire, 1000, compressed_size=wire.numel() - 8)
    idx_max = int(oracle.parse_wire(wire.cpu().numpy())[1].max())
    with pytest.raises(RuntimeError, match="index out of bounds"):
        comp.decompress(wire, idx_max)


def test_compressor_reports_a_give_up_of_the_compress_launch(k):
    """compress() is asynchronous; a launch that gives up (every wait forced into its limit from
    the host, all kernels exit normally) is reported by the calls that wait for the stream:
    check_compress_status() and decompress() raise, and the payload is rejected."""
    from mccl_amd import hip_ops as ops
    C = k["C"]
    comp = C.TopKCompressor(0.01)
    g = torch.from_numpy(student_t(np.random.default_rng(3), 400_000)).to(DEV)
    good = comp.compress(g, stable_id=1)
    comp.check_compress_status()
    try:
        ops.set_tuning("topk_stall_test", 1)
        ops.set_tuning("topk_barrier_ms", 1)
        bad = comp.compress(g, stable_id=1)
        torch.cuda.synchronize()
    finally:
        ops.set_tuning("topk_stall_test", 0)
        ops.set_tuning("topk_barrier_ms", 2000)
    with pytest.raises(RuntimeError, match="Timeout"):
        comp.check_compress_status()
    comp.check_compress_status()   # reported once
    with pytest.raises(RuntimeError, match="size mismatch"):
        comp.decompress(bad, 400_000)
    comp.decompress(good, 400_000)


def test_two_bucket_residual_isolation(k):
    # tests/test_compression_e2e.py:33-75: alternate two buckets of very different scale
    # through one compressor; each bucket's residual must only ever see its own gradients.
    C = k["C"]
    comp = C.TopKCompressor(0.1)
    n = 10_000
    rng = np.random.default_rng(2)
    res = {1: np.zeros(n, np.float32), 2: np.zeros(n, np.float32)}
    bufs = {1: torch.empty(n, device=DEV), 2: torch.empty(n, device=DEV)}
    for step in range(5):
        for bid, scale in ((1, 1.0), (2, 1e-3)):
            g = (rng.standard_normal(n) * scale).astype(np.float32)
            bufs[bid].copy_(torch.from_numpy(g))
            wire = comp.compress(bufs[bid])  # identity = storage address
            w, _ = oracle.topk_compress(g, res[bid], 0.1)
            assert wire.cpu().numpy().tobytes() == w.tobytes(), (step, bid)
    assert float(comp.error_feedback_buffer(C._compression_stable_id(bufs[2])).abs().max()) < 1e-2


def test_compress_many_equals_per_bucket_calls_and_the_oracle(k):
    # a coalesced list of buckets of different sizes, error feedback carried over two steps
    C = k["C"]
    rng = np.random.default_rng(9)
    sizes = [655_360] * 6 + [300_001, 65_537, 4_097, 1_000_003, 13]
    many, single = C.TopKCompressor(0.01), C.TopKCompressor(0.01)
    res_o = [np.zeros(n, np.float32) for n in sizes]
    bufs = [torch.empty(n, device=DEV) for n in sizes]
    for step in range(2):
        grads = [student_t(rng, n) * np.float32(10.0 ** (i % 3)) for i, n in enumerate(sizes)]
        for buf, g in zip(bufs, grads):
            buf.copy_(torch.from_numpy(g))
        ids = [100 + i for i in range(len(sizes))]
        payloads = many.compress_many(bufs, stable_ids=ids)
        torch.cuda.synchronize()
        for i, (g, p) in enumerate(zip(grads, payloads)):
            w, rc = oracle.topk_compress(g, res_o[i], 0.01)
            assert p.numel() == rc and p.cpu().numpy().tobytes() == w.tobytes(), (step, i)
            assert np.array_equal(bits(many.error_feedback_buffer(ids[i]).cpu().numpy()), bits(res_o[i])), (step, i)
            one = single.compress(bufs[i], stable_id=ids[i])
            assert torch.equal(one, p), (step, i)
    assert many.error_feedback_buffer_count() == len(sizes)
    # default ids = storage addresses; an id twice in one call is refused
    assert len(many.compress_many(bufs[:3])) == 3
    with pytest.raises(RuntimeError, match="same stable id twice"):
        many.compress_many(bufs[:2], stable_ids=[1, 1])
    with pytest.raises(RuntimeError, match="float32 only"):
        many.compress_many([bufs[0].half()])
    assert many.compress_many([]) == []
