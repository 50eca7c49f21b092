"""Pins the oracle's top-k compressor / decompressor: brute force on small
inputs, the reference's own compiled TopKCompression.cpp (oracle/_ref) on
tie-free inputs, conservation invariants, and the reference tests' wire-format
and error-feedback properties (tests/test_compression.py:46-127)."""
import struct

import numpy as np
import pytest

import oracle

needs_ref = pytest.mark.skipif(not oracle.RefCompressor.available(),
                               reason="oracle/_ref not built (reference checkout absent)")


def brute_force(grad, residual, ratio):
    """Independent statement: sort by (|v| descending, index ascending)."""
    adj = (grad + residual).astype(np.float32)
    n = adj.size
    k = max(1, int(np.uint32(int(float(n) * ratio))))
    key = adj.view(np.uint32) & np.uint32(0x7FFFFFFF)
    order = np.lexsort((np.arange(n), -(key.astype(np.int64))))
    picks = np.sort(order[:k]).astype(np.uint32)
    new_res = adj.copy()
    new_res[picks] = 0.0
    return k, picks, adj[picks], new_res


def _student_t(rng, n, ties=0.0):
    x = (rng.standard_normal(n) / np.sqrt(rng.chisquare(3, n) / 3) * 1e-3).astype(np.float32)
    m = int(n * ties)
    if m:
        dst = rng.integers(0, n, m); src = rng.integers(0, n, m)
        sign = np.where(rng.random(m) < 0.5, -1.0, 1.0).astype(np.float32)
        x[dst] = x[src] * sign
    return x


def _tie_free(rng, n, res):
    """Student-t gradient redrawn at colliding positions until all |g + res|
    are pairwise distinct (bounded number of rounds)."""
    g = _student_t(rng, n)
    for _ in range(200):
        mag = np.abs(g + res)
        order = np.argsort(mag, kind="stable")
        dup = order[1:][mag[order][1:] == mag[order][:-1]]
        if dup.size == 0:
            return g
        g[dup] = _student_t(rng, dup.size)
    raise AssertionError("could not build a tie-free input")


@pytest.mark.parametrize("seed", range(12))
def test_matches_brute_force_with_heavy_ties(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 5000))
    ratio = float(rng.choice([0.001, 0.01, 0.1, 0.5, 1.0]))
    # few distinct magnitudes -> many ties, including at the threshold and +-0
    g = rng.choice(np.array([0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 2.0, 3.0], np.float32), n)
    r = rng.choice(np.array([0.0, 0.5, -0.5, 1.0], np.float32), n)
    k, picks, vals, new_res = brute_force(g, r, ratio)
    res = r.copy()
    wire, rc = oracle.topk_compress(g, res, ratio)
    assert rc == 4 + 8 * k
    kk, idx, val = oracle.parse_wire(wire)
    assert kk == k and np.array_equal(idx, picks)
    assert np.array_equal(val.view(np.uint32), vals.view(np.uint32))
    assert np.array_equal(res.view(np.uint32), new_res.view(np.uint32))


@pytest.mark.parametrize("n,ratio", [(1, 0.01), (99, 0.01), (100, 0.01), (101, 0.01), (65_537, 0.01),
                                     (300_000, 0.01), (300_000, 0.1), (1000, 1.0)])
def test_matches_brute_force_student_t_with_duplicates(n, ratio):
    rng = np.random.default_rng(n)
    g = _student_t(rng, n, ties=0.01)
    r = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    k, picks, vals, new_res = brute_force(g, r, ratio)
    res = r.copy()
    wire, rc = oracle.topk_compress(g, res, ratio)
    kk, idx, val = oracle.parse_wire(wire)
    assert (kk, rc) == (k, 4 + 8 * k)
    assert np.array_equal(idx, picks) and np.array_equal(val.view(np.uint32), vals.view(np.uint32))
    assert np.array_equal(res.view(np.uint32), new_res.view(np.uint32))


def test_k_formula_and_sizes():
    # k = max(1, uint32(count * ratio)) in double (csrc/compression/TopKCompression.cpp:45-47)
    assert oracle.topk_k(6_553_600, 0.01) == 65_536
    assert oracle.topk_k(4_759_624, 0.01) == 47_596
    assert oracle.topk_k(50, 0.01) == 1
    assert oracle.topk_k(100, 0.29) == int(100 * 0.29)  # 28, not 29: double truncation
    assert oracle.topk_max_compressed_size(6_553_600 * 4, 0.01) == 4 + 8 * 65_537
    g = np.ones(100, np.float32)
    wire, rc = oracle.topk_compress(g, np.zeros(100, np.float32), 0.1, capacity=4 + 8 * 10 - 1)
    assert rc == oracle.ERR_CAPACITY and wire is None


def test_invariants_conservation_and_order():
    rng = np.random.default_rng(1)
    n = 500_000
    g = _student_t(rng, n, ties=0.01)
    r = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    adj = g + r
    res = r.copy()
    wire, _ = oracle.topk_compress(g, res, 0.01)
    k, idx, val = oracle.parse_wire(wire)
    assert np.all(np.diff(idx.astype(np.int64)) > 0)            # strictly ascending
    dense = np.zeros(n, np.float32); dense[idx] = val
    # every element is either moved to the wire or kept: bitwise conservation
    moved = np.zeros(n, bool); moved[idx] = True
    assert np.array_equal(np.where(moved, dense, res).view(np.uint32), adj.view(np.uint32))
    assert np.all(res[idx].view(np.uint32) == 0)                # +0.0 at the picks
    thr = np.abs(val).min()
    assert np.all(np.abs(res) <= thr)                           # nothing larger was left behind
    above = np.nonzero(np.abs(adj) > thr)[0]
    assert np.all(moved[above])
    # ties at the threshold went to the lowest indices
    at = np.nonzero(np.abs(adj) == thr)[0]
    taken = at[moved[at]]
    assert np.array_equal(taken, at[: taken.size])


def test_reference_test_properties():
    # tests/test_compression.py:46-106: sparsity, error feedback keeps what was
    # not sent, 1000-step conservation below 1e-4
    rng = np.random.default_rng(42)
    data = rng.standard_normal(100).astype(np.float32)
    res = np.zeros(100, np.float32)
    wire, _ = oracle.topk_compress(data, res, 0.1)
    k, idx, val = oracle.parse_wire(wire)
    assert k == 10 and set(idx.tolist()) == set(np.argsort(-np.abs(data))[:10].tolist())
    assert np.count_nonzero(res) == 90
    error = np.zeros(100, np.float32)
    total_sent = np.zeros(100, np.float64); total_data = np.zeros(100, np.float64)
    for _ in range(1000):
        d = rng.standard_normal(100).astype(np.float32)
        total_data += d
        wire, _ = oracle.topk_compress(d, error, 0.1)
        _, idx, val = oracle.parse_wire(wire)
        total_sent[idx] += val
    assert np.max(np.abs(total_data - total_sent - error)) < 1e-4


def test_wire_format_is_the_reference_struct_layout():
    # tests/test_compression.py:108-127: "<I" then k x "<If"
    pairs = [(5, 1.5), (10, -2.0), (42, 3.14)]
    buf = struct.pack("<I", 3) + b"".join(struct.pack("<If", i, v) for i, v in pairs)
    dense, rc = oracle.topk_decompress(np.frombuffer(buf, np.uint8).copy(), 64)
    assert rc == oracle.OK
    want = np.zeros(64, np.float32)
    for i, v in pairs:
        want[i] = np.float32(v)
    assert np.array_equal(dense, want)
    g = np.zeros(64, np.float32); g[[5, 10, 42]] = [1.5, -2.0, 3.14]
    wire, _ = oracle.topk_compress(g, np.zeros(64, np.float32), 3 / 64)
    assert wire.tobytes() == buf


def test_decompress_errors():
    buf = struct.pack("<I", 2) + struct.pack("<If", 1, 1.0) + struct.pack("<If", 9, 2.0)
    w = np.frombuffer(buf, np.uint8).copy()
    assert oracle.topk_decompress(w, 10)[1] == oracle.OK
    assert oracle.topk_decompress(w, 9)[1] == oracle.ERR_INDEX        # index == count
    assert oracle.topk_decompress(w, 10, size=w.size - 1)[1] == oracle.ERR_SIZE
    assert oracle.topk_decompress(w, 10, size=w.size + 8)[1] == oracle.ERR_SIZE


@needs_ref
@pytest.mark.parametrize("n,ratio", [(1000, 0.01), (65_537, 0.01), (250_000, 0.05), (6_553_600, 0.01)])
def test_against_compiled_reference_tie_free(n, ratio):
    """On inputs whose magnitudes are pairwise distinct every valid
    std::nth_element outcome is the same set, so the reference's output is unique."""
    rng = np.random.default_rng(n + 1)
    ref = oracle.RefCompressor(2, ratio)
    res = np.zeros(n, np.float32)
    for step in range(3):  # error feedback carried across steps on both sides
        g = _tie_free(rng, n, res)
        want = ref.compress(g, stable_id=7)
        wire, rc = oracle.topk_compress(g, res, ratio)
        assert rc == want.size and wire.tobytes() == want.tobytes(), step
        assert ref.max_compressed_size(n * 4) == oracle.topk_max_compressed_size(n * 4, ratio)


@needs_ref
def test_against_compiled_reference_with_ties_everything_but_the_tie_choice():
    rng = np.random.default_rng(3)
    n = 200_000
    g = _student_t(rng, n, ties=0.05)
    ref = oracle.RefCompressor(2, 0.01)
    want = ref.compress(g, stable_id=1)
    res = np.zeros(n, np.float32)
    wire, _ = oracle.topk_compress(g, res, 0.01)
    k1, i1, v1 = oracle.parse_wire(wire)
    k2, i2, v2 = oracle.parse_wire(want)
    assert k1 == k2
    thr = np.abs(v1).min()
    assert thr == np.abs(v2).min()
    strict1 = i1[np.abs(v1) > thr]; strict2 = i2[np.abs(v2) > thr]
    assert np.array_equal(strict1, strict2)
    assert np.array_equal(np.sort(np.abs(v1)), np.sort(np.abs(v2)))


@needs_ref
def test_reference_decompress_and_errors_agree():
    rng = np.random.default_rng(9)
    n = 10_000
    g = _student_t(rng, n)
    wire, _ = oracle.topk_compress(g, np.zeros(n, np.float32), 0.01)
    ref = oracle.RefCompressor(2, 0.01)
    d_ref, rc_ref = ref.decompress(wire, n)
    d, rc = oracle.topk_decompress(wire, n)
    assert rc == rc_ref == 0 and np.array_equal(d.view(np.uint32), d_ref.view(np.uint32))
    _, idx, _ = oracle.parse_wire(wire)
    small = int(idx.max())  # count == max index -> out of bounds
    assert ref.decompress(wire, small)[1] == -1 and oracle.topk_decompress(wire, small)[1] == oracle.ERR_INDEX
    assert ref.decompress(wire, n, size=wire.size - 8)[1] == -1
    assert oracle.topk_decompress(wire, n, size=wire.size - 8)[1] == oracle.ERR_SIZE
    # fp32 only (csrc/compression/TopKCompression.cpp:42-43)
    assert ref.compress(g, dtype=oracle.F16) is None


def test_sparse_accumulate_is_rank_ordered_dense_form():
    rng = np.random.default_rng(4)
    n, ws = 20_000, 8
    wires = []
    for r in range(ws):
        g = _student_t(rng, n)
        w, _ = oracle.topk_compress(g, np.zeros(n, np.float32), 0.05)
        wires.append(w)
    acc, rc = oracle.sparse_accumulate(wires, n, scale_by=0.125)
    assert rc == oracle.OK
    want = np.zeros(n, np.float32)
    for w in wires:  # plain python restatement: scatter-add in rank order
        _, idx, val = oracle.parse_wire(w)
        want[idx] = want[idx] + val
    want = want * np.float32(0.125)
    assert np.array_equal(acc.view(np.uint32), want.view(np.uint32))
    touched = np.zeros(n, bool)
    for w in wires:
        touched[oracle.parse_wire(w)[1]] = True
    assert np.all(acc[~touched].view(np.uint32) == 0)
