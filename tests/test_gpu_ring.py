"""W-way ring-order fold on the GPU vs the oracle's closed form (itself checked
against a brute-force run of the reference's step plan), and vs the step-wise
drop-in sequence of binary folds on chunk views."""
import numpy as np
import pytest
import torch

import oracle
from oracle import F32, F16, BF16, OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX, RING_BASIC, RING_CHUNKED
from tests._gpu_util import DEV, to_dev, to_np, bits, rand_vals

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


@pytest.mark.parametrize("schedule", [RING_BASIC, RING_CHUNKED])
@pytest.mark.parametrize("ws", [2, 3, 4, 5, 8])
def test_fp32_ring_fold_matches_oracle(ops, schedule, ws):
    rng = np.random.default_rng(ws * 7 + schedule)
    for n in (1, 5, 2 * ws + 1, 4097, 70_001, 1_000_003):
        ins = [rand_vals(rng, n, F32, sigma=1e-3, specials=False) for _ in range(ws)]
        for op in (OP_SUM, OP_MIN, OP_MAX, OP_PRODUCT):
            want = oracle.ring_fold(ins, F32, op, schedule)
            dins = [to_dev(x, F32, pad_front=(r % 3)) for r, x in enumerate(ins)]
            out = torch.empty(n + 1, device=DEV)[1:]  # misaligned output too
            ops.ring_fold(out, dins, op, schedule)
            assert np.array_equal(bits(to_np(out, F32)), bits(want)), (n, op)
        inv = float(np.float32(1.0 / ws))
        want = oracle.ring_fold(ins, F32, OP_AVG, schedule, scale_by=inv)
        out = torch.empty(n, device=DEV)
        ops.ring_fold(out, [to_dev(x, F32) for x in ins], OP_AVG, schedule, scale_by=inv)
        assert np.array_equal(bits(to_np(out, F32)), bits(want)), n


def test_bucketed_ring_fold_equals_per_bucket_oracle(ops):
    # a gradient cut into buckets, every bucket into ws chunks; last bucket shorter and odd
    ws, n, be = 8, 3_000_017, 655_360
    rng = np.random.default_rng(3)
    ins = [rand_vals(rng, n, F32, sigma=1e-3, specials=False) for _ in range(ws)]
    want = np.empty(n, np.float32)
    for s in range(0, n, be):
        e = min(n, s + be)
        want[s:e] = oracle.ring_fold([x[s:e].copy() for x in ins], F32, OP_SUM, RING_BASIC, scale_by=0.125)
    out = torch.empty(n, device=DEV)
    ops.ring_fold(out, [to_dev(x, F32) for x in ins], OP_SUM, RING_BASIC, bucket_elems=be, scale_by=0.125)
    assert np.array_equal(bits(to_np(out, F32)), bits(want))


def test_ring_fold_equals_stepwise_binary_folds_on_chunk_views(ops):
    # the drop-in sequence: for every chunk, ws-1 calls of fold2(local chunk, incoming partial), then scale
    ws, n = 4, 1_000_003
    rng = np.random.default_rng(11)
    ins = [rand_vals(rng, n, F32, sigma=1e-3, specials=False) for _ in range(ws)]
    dins = [to_dev(x, F32) for x in ins]
    out = torch.empty(n, device=DEV)
    ops.ring_fold(out, dins, OP_SUM, RING_BASIC, scale_by=0.25)
    ce = (n + ws - 1) // ws
    step = torch.empty(n, device=DEV)
    for c in range(ws):
        lo, hi = c * ce, min(n, (c + 1) * ce)
        partial = dins[c][lo:hi].clone()
        for j in range(1, ws):
            local = dins[(c + j) % ws][lo:hi].clone()
            ops.fold2(local, partial, OP_SUM)      # local (op)= incoming
            partial = local
        step[lo:hi] = partial
    ops.scale(step, 0.25)
    assert torch.equal(out.view(torch.int32), step.view(torch.int32))


@pytest.mark.parametrize("dt,op", [(F32, OP_SUM), (oracle.BF16, OP_SUM), (oracle.F16, oracle.OP_MAX), (oracle.I32, OP_SUM)])
def test_batched_folds_equal_the_per_call_sequence(ops, dt, op):
    # the same step-wise sequence with the folds of one ring step handed over as one list: ws rank
    # buffers, 3 buckets (the last one shorter and odd), every bucket in ws chunks; ring step j
    # folds chunk (r - j) of rank r - 1's partial into rank r's copy, for all r and buckets at once
    ws, n, be = 4, 700_003, 262_144
    rng = np.random.default_rng(17)
    if dt == oracle.I32:
        ins = [rng.integers(-2**31, 2**31, n, dtype=np.int64).astype(np.int32) for _ in range(ws)]
    else:
        ins = [rand_vals(rng, n, dt, sigma=1e-3, specials=False) for _ in range(ws)]
    one = [to_dev(x, dt, pad_front=r % 3) for r, x in enumerate(ins)]     # folded call by call
    many = [to_dev(x, dt, pad_front=r % 3) for r, x in enumerate(ins)]    # folded list by list
    for j in range(1, ws):
        dsts, srcs, d1, s1 = [], [], [], []
        for lo in range(0, n, be):
            hi = min(n, lo + be)
            ce = (hi - lo + ws - 1) // ws
            for r in range(ws):
                c = (r - j) % ws
                a, b = lo + c * ce, min(hi, lo + (c + 1) * ce)
                if a >= b:
                    continue
                dsts.append(many[r][a:b]); srcs.append(many[(r - 1) % ws][a:b])
                d1.append(one[r][a:b]); s1.append(one[(r - 1) % ws][a:b])
        ops.fold2_batch(dsts, srcs, op)
        for d, s_ in zip(d1, s1):
            ops.fold2(d, s_, op)
    for a, b in zip(one, many):
        assert np.array_equal(bits(to_np(a, dt)), bits(to_np(b, dt)))


def test_batched_folds_refuse_overlapping_destinations(ops):
    x = torch.zeros(1000, device=DEV)
    y = torch.ones(1000, device=DEV)
    with pytest.raises(Exception):
        ops.fold2_batch([x[:600], x[500:]], [y[:600], y[500:]], OP_SUM)      # two destinations overlap
    with pytest.raises(Exception):
        ops.fold2_batch([x[:500], y[:500]], [y[:500], x[500:]], OP_SUM)      # a destination is another fold's source
    assert float(x.sum()) == 0.0 and float(y.sum()) == 1000.0                  # nothing was launched
    ops.fold2_batch([], [], OP_SUM)
    ops.fold2_batch([x[:0], x[:500]], [y[:0], y[:500]], OP_SUM)               # empty folds are skipped
    assert float(x.sum()) == 500.0


@pytest.mark.parametrize("dt", [F16, BF16])
@pytest.mark.parametrize("stepwise", [False, True])
def test_half_ring_fold_matches_oracle(ops, dt, stepwise):
    ws = 4
    rng = np.random.default_rng(dt + int(stepwise))
    for n in (9, 4099, 500_009):
        x32 = [(rng.standard_normal(n) * 1e-3).astype(np.float32) for _ in range(ws)]
        for x in x32:  # 0.1 % outliers x 1e3
            m = rng.random(n) < 1e-3
            x[m] *= 1e3
        enc = oracle.f32_to_f16_bits if dt == F16 else oracle.f32_to_bf16_bits
        ins = [enc(x) for x in x32]
        for op, sc in ((OP_SUM, None), (OP_SUM, 0.25), (OP_MAX, None), (OP_MIN, None)):
            for schedule in (RING_BASIC, RING_CHUNKED):
                want = oracle.ring_fold(ins, dt, op, schedule, scale_by=sc, stepwise=stepwise)
                out = to_dev(np.zeros(n, np.uint16), dt, pad_front=1)
                ops.ring_fold(out, [to_dev(x, dt, pad_front=r) for r, x in enumerate(ins)], op, schedule,
                              scale_by=sc, stepwise=stepwise)
                assert np.array_equal(to_np(out, dt), want), (n, op, sc, schedule)


def test_ring_fold_rejects_bad_arguments(ops):
    from mccl_amd._lib import MCCLHipError
    a = torch.zeros(8, device=DEV)
    with pytest.raises(MCCLHipError):
        ops.ring_fold(a, [a.clone()] * 2, 5)
    with pytest.raises(MCCLHipError):
        ops.ring_fold(a, [a.clone()] * 65, OP_SUM)
