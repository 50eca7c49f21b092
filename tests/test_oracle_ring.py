"""Pins the ring fold order: the closed form (left fold starting at the chunk's
first rank) against a brute-force run of the reference's step plan, and against
the exact answers the reference's own multi-rank tests hold."""
import numpy as np
import pytest

import oracle
from oracle import F16, BF16, F32, OP_SUM, OP_AVG, OP_MIN, OP_MAX, OP_PRODUCT, RING_BASIC, RING_CHUNKED


def _ranks(ws, n, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal(n) * scale).astype(np.float32) for _ in range(ws)]


@pytest.mark.parametrize("schedule", [RING_BASIC, RING_CHUNKED])
@pytest.mark.parametrize("ws", [2, 3, 4, 5, 6, 8])
def test_closed_form_equals_step_plan_simulation(schedule, ws):
    for n in (1, 3, ws - 1, 2 * ws + 1, 1023, 4097, 70_001):
        if n < 1:
            continue
        ins = _ranks(ws, n, seed=ws * 1000 + n)
        for op in (OP_SUM, OP_MIN, OP_MAX, OP_PRODUCT):
            sim = oracle.ring_simulate_f32(ins, op, schedule)
            closed = oracle.ring_fold(ins, F32, op, schedule)
            assert np.array_equal(sim.view(np.uint32), closed.view(np.uint32)), (ws, n, op)


def test_fold_order_is_observable():
    # a + b + c in fp32 depends on association; make sure the closed form really
    # is the left fold from the chunk's first rank and not a fixed rank order.
    ws, n = 3, 3  # basic ring: one element per chunk, chunk c starts at rank c
    big, tiny = np.float32(2.0 ** 24), np.float32(1.0)
    ins = [np.array([big, tiny, tiny], np.float32),
           np.array([tiny, big, tiny], np.float32),
           np.array([tiny, tiny, big], np.float32)]
    out = oracle.ring_fold(ins, F32, OP_SUM, RING_BASIC)
    # chunk 0: (big + tiny) + tiny = 2^24 (each tiny is lost)
    # chunk 1: (big + tiny) + tiny, starting at rank 1 -> also 2^24
    # chunk 2: starts at rank 2 (big), same.  A fixed order 0,1,2 would give
    # chunk 2 = (tiny + tiny) + big = 2^24 + 2.
    assert out.tolist() == [2.0 ** 24, 2.0 ** 24, 2.0 ** 24]
    fixed = (ins[0] + ins[1]) + ins[2]
    assert fixed[2] == np.float32(2.0 ** 24 + 2)
    assert oracle.lib.orc_ring_first_rank(2, 3, RING_BASIC) == 2
    # chunked ring: chunks 2q and 2q-1 both start at rank q
    for ws_ in (2, 3, 8):
        for q in range(ws_):
            assert oracle.lib.orc_ring_first_rank(2 * q, ws_, RING_CHUNKED) == q
            assert oracle.lib.orc_ring_first_rank((2 * q - 1) % (2 * ws_), ws_, RING_CHUNKED) == q


@pytest.mark.parametrize("schedule", [RING_BASIC, RING_CHUNKED])
@pytest.mark.parametrize("n", [70_000, 70_001])
def test_reference_three_rank_exact_answers(schedule, n):
    # tests/test_process_group_local.py:478-578, :635-647: constants rank+1,
    # SUM == 6, AVG == 2.0 (6 * float(1/3) rounds to 2.0f), MIN == 1, MAX == 3,
    # all at rtol=0, atol=0.
    ins = [np.full(n, float(r + 1), dtype=np.float32) for r in range(3)]
    assert np.all(oracle.ring_fold(ins, F32, OP_SUM, schedule) == 6.0)
    third = float(np.float32(1.0 / 3.0))
    assert np.all(oracle.ring_fold(ins, F32, OP_AVG, schedule, scale_by=third) == 2.0)
    assert np.all(oracle.ring_fold(ins, F32, OP_MIN, schedule) == 1.0)
    assert np.all(oracle.ring_fold(ins, F32, OP_MAX, schedule) == 3.0)


@pytest.mark.parametrize("dt,npcast", [(F32, None), (F16, "f16"), (BF16, "bf16")])
@pytest.mark.parametrize("ws", [2, 3, 4, 6])
def test_reference_pattern_allreduce(dt, npcast, ws):
    # tests/test_correctness_vs_reference.py:36-78: arange(n) % 13 - 6 + rank + 1,
    # exactly representable in every dtype so SUM / AVG / MAX are exact.
    for n in (1, 3, 1023, 4097, 70_001, 262_147):
        base = np.arange(n, dtype=np.float64) % 13 - 6.0
        contribs = [base + float(r + 1) for r in range(ws)]
        if dt == F32:
            ins = [c.astype(np.float32) for c in contribs]
            dec = lambda x: x.astype(np.float64)
        elif dt == F16:
            ins = [oracle.f32_to_f16_bits(c.astype(np.float32)) for c in contribs]
            dec = lambda x: oracle.f16_bits_to_f32(x).astype(np.float64)
        else:
            ins = [oracle.f32_to_bf16_bits(c.astype(np.float32)) for c in contribs]
            dec = lambda x: oracle.bf16_bits_to_f32(x).astype(np.float64)
        for schedule in (RING_BASIC, RING_CHUNKED):
            for stepwise in (False, True):
                got = dec(oracle.ring_fold(ins, dt, OP_SUM, schedule, stepwise=stepwise))
                assert np.array_equal(got, sum(contribs))
                got = dec(oracle.ring_fold(ins, dt, OP_MAX, schedule, stepwise=stepwise))
                assert np.array_equal(got, np.max(contribs, axis=0))
            inv = float(np.float32(1.0 / ws))
            got = dec(oracle.ring_fold(ins, dt, OP_AVG, schedule, scale_by=inv))
            tol = {F32: 1e-6, F16: 1e-2, BF16: 1e-1}[dt]  # the reference's tolerances
            assert np.allclose(got, sum(contribs) / ws, rtol=tol, atol=tol)


def test_avg_scale_value_float_of_double_equals_float_division():
    # Callers pass 1.0/ws as double (cast to float at the kernel boundary) on one
    # path and 1.0f/ws on the other (csrc/backend/ProcessGroupMCCL.cpp:1950,:1955).
    for ws in range(1, 1025):
        assert np.float32(1.0 / ws) == np.float32(1.0) / np.float32(ws)


def test_half_stepwise_vs_single_rounding_within_one_ulp():
    ws, n = 4, 200_000
    rng = np.random.default_rng(5)
    vals = [(rng.standard_normal(n) * 1e-3).astype(np.float32) for _ in range(ws)]
    for dt, enc, dec in ((F16, oracle.f32_to_f16_bits, oracle.f16_bits_to_f32),
                         (BF16, oracle.f32_to_bf16_bits, oracle.bf16_bits_to_f32)):
        ins = [enc(v) for v in vals]
        single = oracle.ring_fold(ins, dt, OP_SUM, RING_BASIC, stepwise=False)
        # correctly rounded ring-order sum: fp64 holds the 4-term sum of 16-bit
        # values exactly here (spread of exponents is small), round once to T
        exact = sum(dec(i).astype(np.float64) for i in ins)
        best = enc(exact.astype(np.float32))
        # single rounding of an fp32 accumulate is within 1 ulp(T) of the exact sum
        d = np.abs(single.astype(np.int64) - best.astype(np.int64))
        same_sign = (single & 0x8000) == (best & 0x8000)
        assert np.all(d[same_sign] <= 1)
        # MAX never rounds: both variants identical
        a = oracle.ring_fold(ins, dt, OP_MAX, RING_BASIC, stepwise=False)
        b = oracle.ring_fold(ins, dt, OP_MAX, RING_BASIC, stepwise=True)
        assert np.array_equal(a, b)
