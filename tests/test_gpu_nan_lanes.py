"""NaN lanes of the folds, compared on the device instead of masked out.

What an IEEE machine fixes and what it leaves open:
  * which lanes are NaN is fixed (inf + -inf, 0 * inf, any NaN operand) and must
    agree with the oracle everywhere;
  * a NaN made by an invalid operation has the platform's default sign: set on
    the x86 host the oracle runs on, clear on gfx950.  For those lanes the
    comparison drops the sign bit and checks the canonical pattern;
  * a NaN operand met by a number propagates with its own sign on both machines,
    so there every bit is compared.
The 16-bit narrowing then writes sign | 0x7E00 (fp16) or 0x7FC0 (bf16) for every
NaN, the c10 conversions' forms, which the oracle's casts are pinned to."""
import numpy as np
import pytest
import torch

import oracle
from oracle import F32, F16, BF16, OP_SUM, OP_PRODUCT, RING_BASIC
from tests._gpu_util import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


def make_inputs(rng, n, dt, ws):
    """ws arrays (bit representation of dt): ordinary values, with lanes that make
    NaN by an invalid operation (lane class 1), lanes with one NaN operand of
    either sign (class 2), and ordinary lanes (class 0)."""
    xs = [(rng.standard_normal(n)).astype(np.float32) for _ in range(ws)]
    cls = np.zeros(n, np.int8)
    lanes = rng.permutation(n)
    q = max(1, n // 8)
    inv, prop = lanes[:q], lanes[q:2 * q]
    cls[inv] = 1
    cls[prop] = 2
    # invalid operations: (+inf, -inf) for SUM, (0, inf) for PRODUCT both give NaN in one of the two ops;
    # use inf/-inf in ranks 0/1 and 0 in rank 0 for a second half
    half = inv[: len(inv) // 2]
    rest = inv[len(inv) // 2:]
    xs[0][half] = np.inf
    xs[1][half] = -np.inf
    xs[0][rest] = 0.0
    xs[1][rest] = np.inf
    if dt == F32:
        enc = [x.copy() for x in xs]
    elif dt == F16:
        enc = [oracle.f32_to_f16_bits(x) for x in xs]
    else:
        enc = [oracle.f32_to_bf16_bits(x) for x in xs]
    # one NaN operand per lane of class 2, in a random rank, random sign, canonical quiet pattern
    who = rng.integers(0, ws, len(prop))
    neg = rng.random(len(prop)) < 0.5
    for r in range(ws):
        sel = prop[who == r]
        sg = neg[who == r]
        if dt == F32:
            enc[r].view(np.uint32)[sel] = np.where(sg, 0xFFC00000, 0x7FC00000).astype(np.uint32)
        elif dt == F16:
            enc[r][sel] = np.where(sg, 0xFE00, 0x7E00).astype(np.uint16)
        else:
            enc[r][sel] = np.where(sg, 0xFFC0, 0x7FC0).astype(np.uint16)
    return enc, cls


def isnan_bits(a, dt):
    if dt == F32:
        return np.isnan(a)
    if dt == F16:
        return (a & 0x7FFF) > 0x7C00
    return (a & 0x7FFF) > 0x7F80


def compare(want, got, dt, cls, where):
    wn, gn = isnan_bits(want, dt), isnan_bits(got, dt)
    assert np.array_equal(wn, gn), (where, "NaN lanes differ")
    w = want.view(np.uint32) if dt == F32 else want
    g = got.view(np.uint32) if dt == F32 else got
    assert np.array_equal(w[~wn], g[~wn]), (where, "ordinary lanes")
    # a NaN operand propagates with its sign: every bit must agree
    p = wn & (cls == 2)
    assert np.array_equal(w[p], g[p]), (where, "propagated NaN")
    # NaN from an invalid operation: default sign is the machine's, the rest is canonical
    inv = wn & (cls != 2)
    mask = 0x7FFFFFFF if dt == F32 else 0x7FFF
    assert np.array_equal(w[inv] & mask, g[inv] & mask), (where, "default NaN")
    if dt == F16:
        assert np.all((g[wn] & 0x7FFF) == 0x7E00)
    elif dt == BF16:
        assert np.all(g[wn] == 0x7FC0) and np.all(w[wn] == 0x7FC0)
    else:
        assert np.all((g[inv] & 0x7FFFFFFF) == 0x7FC00000)


@pytest.mark.parametrize("dt", [F32, F16, BF16])
@pytest.mark.parametrize("op", [OP_SUM, OP_PRODUCT])
def test_fold2_nan_lanes(ops, dt, op):
    rng = np.random.default_rng(500 + dt + op)
    for n in (64, 4097, 300_001):
        (a, b), cls = make_inputs(rng, n, dt, 2)
        want = a.copy()
        assert oracle.fold2(want, b, dt, op) == oracle.OK
        d = to_dev(a, dt, 1)
        ops.fold2(d, to_dev(b, dt), op)
        compare(want, to_np(d, dt), dt, cls, (n, "fold2"))
        assert isnan_bits(want, dt).sum() >= n // 8   # the lanes under test exist
    if op == OP_SUM:
        (a, b), cls = make_inputs(rng, 100_003, dt, 2)
        want = a.copy()
        oracle.fold2_scale(want, b, dt, 0.5)
        d = to_dev(a, dt)
        ops.fold2_scale(d, to_dev(b, dt, 3), 0.5)
        compare(want, to_np(d, dt), dt, cls, "fold2_scale")


@pytest.mark.parametrize("dt", [F32, F16, BF16])
@pytest.mark.parametrize("op", [OP_SUM, OP_PRODUCT])
@pytest.mark.parametrize("ws", [2, 3, 4, 8])
def test_ring_fold_nan_lanes(ops, dt, op, ws):
    rng = np.random.default_rng(900 + dt + 7 * op + ws)
    n = 200_003
    ins, cls = make_inputs(rng, n, dt, ws)
    for stepwise in ((False, True) if dt != F32 else (False,)):
        for sc in (None, 0.5):
            want = oracle.ring_fold(ins, dt, op, RING_BASIC, scale_by=sc, stepwise=stepwise)
            out = torch.empty(n, device=DEV, dtype=torch.float32 if dt == F32 else
                              (torch.float16 if dt == F16 else torch.bfloat16))
            ops.ring_fold(out, [to_dev(x, dt, pad_front=r % 3) for r, x in enumerate(ins)], op, RING_BASIC,
                          scale_by=sc, stepwise=stepwise)
            compare(want, to_np(out, dt), dt, cls, (ws, stepwise, sc))
