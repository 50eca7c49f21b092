"""Sparse accumulate on hand-built payloads (csrc/backend/ProcessGroupMCCL.cpp:1692-1709,
:2272-2296: decompress every rank, fold the dense buffers in rank order): the cases
that decide whether the GPU walk over the payloads is exact.

    values    subnormals, both zeros, infinities, NaN, sums that overflow, many
              ranks on one element: the adds happen in rank order, in IEEE single
              precision with subnormals kept
    density   from a handful of pairs per bucket to 4.5 % (a rank's pairs of one
              tile no longer fit the registers requested up front), clustered
              payloads, one to eight ranks, short last bucket, misaligned output
    order     a payload out of order (or with a repeated index) at any position,
              lane 15/16, 31/32 and 63/64 included, is flagged; sorted payloads
              whose first index is 0 or whose k is a multiple of 64 are not
"""
import numpy as np
import pytest
import torch

import oracle
from tests._gpu_util import DEV, to_np, bits

pytestmark = pytest.mark.gpu
F32 = oracle.F32


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


def payload(idx, val, kcap):
    """[u32 k][k x (u32 index, f32 value)] padded with stale bytes to kcap pairs."""
    k = len(idx)
    body = np.empty((kcap, 2), "<u4")
    body[:] = 0xDEADBEEF                       # what lies past k is never looked at
    body[:k, 0] = np.asarray(idx, "<u4")
    body[:k, 1] = np.asarray(val, np.float32).view("<u4")
    return np.concatenate([np.array([k], "<u4").view(np.uint8), body.reshape(-1).view(np.uint8)])


def run_case(ops, per_rank, n, be, scale, expect_status=0, pad_front=0, paths=("auto", "tiles", None)):
    """per_rank[r][b] = (idx, val) of rank r's bucket-b payload.  Returns the GPU result."""
    ws = len(per_rank)
    nb = (n + be - 1) // be
    kcap = max(max(len(p[0]) for p in ranks) for ranks in per_rank)
    kcap = max(kcap, 1)
    stride = 4 + 8 * kcap
    wires, want = [], np.empty(n, np.float32)
    for r in range(ws):
        buf = np.concatenate([payload(*per_rank[r][b], kcap) for b in range(nb)])
        wires.append(torch.from_numpy(buf).to(DEV))
    rc_all = oracle.OK
    for b in range(nb):
        s, e = b * be, min(n, (b + 1) * be)
        pl = [payload(*per_rank[r][b], len(per_rank[r][b][0])) for r in range(ws)]
        acc, rc = oracle.sparse_accumulate(pl, e - s, scale_by=scale)
        want[s:e] = acc
        rc_all = rc_all or rc
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    got = None
    for path in paths:
        big = torch.full((n + pad_front + 8,), 3.0, device=DEV)
        acc = big[pad_front:pad_front + n]
        status.zero_()
        if path == "tiles":
            ops.set_tuning("sparse_path", 1)
        try:
            ops.sparse_accumulate(acc, wires, stride, bucket_elems=be, scale_by=scale, status=status,
                                  workspace=None if path is None else "auto")
        finally:
            ops.set_tuning("sparse_path", 0)
        assert int(status) == expect_status, (path, int(status))
        if expect_status == 0:
            assert rc_all == oracle.OK
            g = to_np(acc, F32)
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(g), nan), path
            assert np.array_equal(bits(g)[~nan], bits(want)[~nan]), path
            assert float(big[pad_front + n]) == 3.0 and (pad_front == 0 or float(big[pad_front - 1]) == 3.0)
            got = g
    return got


SPECIALS = np.array([0.0, -0.0, 1e-40, -1e-40, 1e-45, -1e-45, 5.877e-39, -5.877e-39, 1.17549435e-38, -1.17549435e-38,
                     3e38, -3e38, 3.4028235e38, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-30, -1e-30, 0.1, 16777216.0],
                    dtype=np.float32)


@pytest.mark.parametrize("ws", [2, 3, 8])
def test_special_values_add_in_rank_order(ops, ws):
    rng = np.random.default_rng(100 + ws)
    n, be = 40_000, 16_384
    nb = (n + be - 1) // be
    per_rank = []
    for r in range(ws):
        ranks = []
        for b in range(nb):
            bn = min(be, n - b * be)
            # every rank hits the first 64 elements (all ranks collide there) plus its own random picks
            own = rng.choice(np.arange(64, bn), size=300, replace=False)
            idx = np.sort(np.concatenate([np.arange(64), own])).astype(np.uint32)
            val = rng.choice(SPECIALS, size=idx.size)
            mix = rng.random(idx.size) < 0.3
            val[mix] = (rng.standard_normal(int(mix.sum())) * 1e-38).astype(np.float32)   # around the subnormal edge
            ranks.append((idx, val.astype(np.float32)))
        per_rank.append(ranks)
    for scale in (None, 1.0 / ws, 0.5):
        run_case(ops, per_rank, n, be, scale)


def test_three_way_sums_need_rank_order(ops):
    # (a + b) + c differs from (a + c) + b: only the rank order gives the oracle's bits
    n = 4096
    a, b, c = np.float32(1.0), np.float32(2.0 ** -24), np.float32(2.0 ** -24)
    assert np.float32(np.float32(a + b) + c) != np.float32(np.float32(b + c) + a)
    idx = np.arange(0, n, 7, dtype=np.uint32)
    for order in ((a, b, c), (b, c, a), (c, a, b)):
        per_rank = [[(idx, np.full(idx.size, v, np.float32))] for v in order]
        got = run_case(ops, per_rank, n, n, None)
        assert np.all(got[idx] == np.float32(np.float32(order[0] + order[1]) + order[2]))


@pytest.mark.parametrize("ws,n,be,density", [
    (1, 10_000, 10_000, 0.01), (2, 70_001, 32_768, 0.001), (5, 200_000, 65_536, 0.03),
    (8, 150_000, 65_536, 0.045), (3, 2048 * 5 + 1, 2048 * 5 + 1, 0.02), (4, 9, 4, 0.5), (8, 300_000, 100_000, 0.0001)])
def test_densities_worlds_and_geometries(ops, ws, n, be, density):
    rng = np.random.default_rng(ws * 1000 + n)
    nb = (n + be - 1) // be
    per_rank = []
    for r in range(ws):
        ranks = []
        for b in range(nb):
            bn = min(be, n - b * be)
            k = max(1, int(bn * density))
            idx = np.sort(rng.choice(bn, size=k, replace=False)).astype(np.uint32)
            ranks.append((idx, rng.standard_normal(k).astype(np.float32)))
        per_rank.append(ranks)
    run_case(ops, per_rank, n, be, 1.0 / ws)
    run_case(ops, per_rank, n, be, None, pad_front=1, paths=("auto",))       # output not 16-byte aligned


def test_clustered_payloads(ops):
    # all of a rank's pairs inside a few tiles (many windows of one rank per tile), nothing elsewhere;
    # another rank empty; another with one pair at each end
    n = 500_000
    rng = np.random.default_rng(7)
    k = 4000
    r0 = np.sort(rng.choice(np.arange(100_000, 104_500), size=k, replace=False)).astype(np.uint32)
    r1 = np.sort(rng.choice(np.arange(101_000, 101_000 + 2 * k), size=k, replace=False)).astype(np.uint32)
    r3 = np.array([0, n - 1], np.uint32)
    r4 = np.arange(n - k, n, dtype=np.uint32)                                   # the bucket's last k elements
    per_rank = [[(r0, rng.standard_normal(k).astype(np.float32))],
                [(r1, rng.standard_normal(k).astype(np.float32))],
                [(np.zeros(0, np.uint32), np.zeros(0, np.float32))],
                [(r3, np.array([1.5, -2.5], np.float32))],
                [(r4, rng.standard_normal(k).astype(np.float32))]]
    run_case(ops, per_rank, n, n, 0.2)


def sorted_payload(rng, n, k, first_zero):
    idx = np.sort(rng.choice(np.arange(1, n), size=k, replace=False)).astype(np.uint32)
    if first_zero:
        idx[0] = 0
    return idx, rng.standard_normal(k).astype(np.float32)


@pytest.mark.parametrize("k", [64, 128, 192, 200, 1000])
def test_sorted_payloads_are_not_flagged(ops, k):
    rng = np.random.default_rng(k)
    n = 100_000
    for first_zero in (True, False):
        per_rank = [[sorted_payload(rng, n, k, first_zero)] for _ in range(3)]
        run_case(ops, per_rank, n, n, None, paths=("auto",))
    # the largest index the bucket allows
    idx, val = sorted_payload(rng, n, k, False)
    idx[-1] = n - 1
    run_case(ops, [[(idx, val)]], n, n, None, paths=("auto",))


@pytest.mark.parametrize("pos", [0, 14, 15, 16, 31, 32, 47, 48, 62, 63, 64, 65, 127, 128, 191, 192, 193, 255, 256, 300, 998])
def test_order_violation_at_any_position_is_flagged(ops, pos):
    rng = np.random.default_rng(pos)
    n, k = 60_000, 1000
    good = [[sorted_payload(rng, n, k, False)] for _ in range(2)]
    for kind in ("swap", "repeat"):
        idx, val = good[1][0][0].copy(), good[1][0][1]
        if kind == "swap":
            idx[pos], idx[pos + 1] = idx[pos + 1], idx[pos]
        else:
            idx[pos + 1] = idx[pos]
        run_case(ops, [good[0], [(idx, val)]], n, n, None, expect_status=oracle.ERR_INDEX, paths=("auto",))
    # an index equal to the bucket's size, in the middle of the payload's last window
    idx, val = good[1][0][0].copy(), good[1][0][1]
    idx[k - 1] = n
    run_case(ops, [good[0], [(idx, val)]], n, n, None, expect_status=oracle.ERR_INDEX, paths=("auto",))


def test_buckets_that_start_off_a_16_byte_boundary(ops):
    # an odd bucket length puts every second bucket's first element off the vector alignment:
    # those buckets' tiles take the element-wise write-out
    rng = np.random.default_rng(77)
    n, be, ws = 50_003, 10_001, 3
    nb = (n + be - 1) // be
    per_rank = []
    for r in range(ws):
        ranks = []
        for b in range(nb):
            bn = min(be, n - b * be)
            k = max(1, bn // 50)
            idx = np.sort(rng.choice(bn, size=k, replace=False)).astype(np.uint32)
            ranks.append((idx, rng.standard_normal(k).astype(np.float32)))
        per_rank.append(ranks)
    run_case(ops, per_rank, n, be, 1.0 / 3.0)


def test_random_shapes_and_payload_shapes(ops):
    # seeded sweep: world size, bucket length (aligned or not), last bucket, density and clustering all vary
    rng = np.random.default_rng(20260)
    for case in range(40):
        ws = int(rng.integers(1, 9))
        be = int(rng.choice([1, 3, 64, 2047, 2048, 2049, 4096, 10_000, 33_333, 70_000]))
        nb = int(rng.integers(1, 5))
        n = max(1, be * (nb - 1) + int(rng.integers(1, be + 1)))
        density = float(rng.choice([0.0005, 0.005, 0.01, 0.02, 0.04]))
        per_rank = []
        for r in range(ws):
            ranks = []
            for b in range((n + be - 1) // be):
                bn = min(be, n - b * be)
                k = min(bn, max(int(rng.integers(0, 2)), int(bn * density)))
                if rng.random() < 0.3 and bn > 4 * max(k, 1):          # all pairs in one stretch of the bucket
                    lo = int(rng.integers(0, bn - 2 * max(k, 1)))
                    pool = np.arange(lo, lo + 2 * max(k, 1))
                else:
                    pool = bn
                idx = np.sort(rng.choice(pool, size=k, replace=False)).astype(np.uint32)
                ranks.append((idx, (rng.standard_normal(k) * 10.0 ** rng.integers(-20, 20)).astype(np.float32)))
            per_rank.append(ranks)
        scale = [None, 1.0 / ws, 0.3][case % 3]
        run_case(ops, per_rank, n, be, scale, paths=("auto", None))
