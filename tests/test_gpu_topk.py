"""Top-k compress / decompress / sparse accumulate on the GPU vs the oracle:
wire bytes and residual bits must be identical (ties -> lower index)."""
import numpy as np
import pytest
import torch

import oracle
from tests._gpu_util import DEV, to_dev, to_np, bits, student_t

pytestmark = pytest.mark.gpu
F32 = oracle.F32


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


def oracle_buckets(g, r, ratio, be):
    """Per-bucket oracle compress; returns (list of wire arrays, new residual)."""
    n = g.size
    res = r.copy()
    wires = []
    for s in range(0, n, be):
        e = min(n, s + be)
        sub = res[s:e].copy()
        w, rc = oracle.topk_compress(g[s:e].copy(), sub, ratio)
        assert rc > 0
        res[s:e] = sub
        wires.append(w)
    return wires, res


PATHS = {"exact": 1, "single-pass": 2}  # both must give the oracle's bytes on every input


def check_compress(ops, g, r, ratio, be=None, pad=0):
    n = g.size
    be = be or n
    want_wires, want_res = oracle_buckets(g, r, ratio, be)
    try:
        for name, path in PATHS.items():
            ops.set_tuning("topk_path", path)
            dg = to_dev(g, F32, pad); dr = to_dev(r, F32, pad)
            ws = ops.topk_workspace(n, min(be, n), ratio, DEV)
            wire, stride = ops.topk_compress(dg, dr, ratio, bucket_elems=be, workspace=ws)
            if path == 2:
                ops.topk_path_report(ws, n, min(be, n), ratio)   # raises if a bucket barrier timed out
            torch.cuda.synchronize()
            got_res = to_np(dr, F32)
            assert np.array_equal(bits(got_res), bits(want_res)), name
            assert np.array_equal(bits(to_np(dg, F32)), bits(g)), name  # gradient untouched
            w = wire.cpu().numpy()
            for b, ww in enumerate(want_wires):
                got = w[b * stride: b * stride + ww.size]
                assert got.tobytes() == ww.tobytes(), f"{name}: bucket {b}"
    finally:
        ops.set_tuning("topk_path", 0)
    return wire, stride, want_wires


@pytest.mark.parametrize("n,ratio", [(1, 0.01), (2, 1.0), (99, 0.01), (100, 0.01), (101, 0.5), (4095, 0.01),
                                     (4096, 0.01), (4097, 0.1), (65_537, 0.01), (300_001, 0.01),
                                     (300_001, 0.25), (1000, 1.0)])
def test_compress_single_bucket(ops, n, ratio):
    rng = np.random.default_rng(n)
    g = student_t(rng, n, ties=0.01)
    r = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    check_compress(ops, g, r, ratio)
    check_compress(ops, g, np.zeros(n, np.float32), ratio, pad=1)


@pytest.mark.parametrize("seed", range(6))
def test_compress_heavy_ties(ops, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 200_000))
    ratio = float(rng.choice([0.001, 0.01, 0.1, 0.5, 1.0]))
    g = rng.choice(np.array([0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 2.0, 3.0], np.float32), n)
    r = rng.choice(np.array([0.0, 0.5, -0.5, 1.0], np.float32), n)
    check_compress(ops, g, r, ratio)


def test_compress_degenerate_inputs(ops):
    n = 50_000
    check_compress(ops, np.zeros(n, np.float32), np.zeros(n, np.float32), 0.01)        # all equal: pure tie-break
    check_compress(ops, np.full(n, -2.5, np.float32), np.zeros(n, np.float32), 0.1)
    g = np.zeros(n, np.float32); g[n - 1] = 1.0; g[0] = -1.0
    check_compress(ops, g, np.zeros(n, np.float32), 2 / n)
    big = np.array([3e38, -3e38, 1e-45, -1e-45, np.inf, 0.0, 1.0], np.float32)
    check_compress(ops, np.tile(big, 1000), np.zeros(7000, np.float32), 0.3)


def test_single_pass_path_on_clustered_and_tied_inputs(ops):
    """Inputs that stress the candidate machinery: all large values in one corner
    (sub-list overflow -> per-bucket fallback), a threshold shared by thousands of
    equal keys (tie-break by index), and a bucket whose sample misleads."""
    rng = np.random.default_rng(77)
    n = 600_000
    g = student_t(rng, n, ties=0.0) * np.float32(1e-3)
    g[:20_000] = student_t(rng, 20_000, ties=0.0) * np.float32(10.0)     # clustered picks
    check_compress(ops, g, np.zeros(n, np.float32), 0.01)
    g = student_t(rng, n, ties=0.0)
    thr = np.sort(np.abs(g))[-6000]
    tie_pos = rng.choice(n, 5000, replace=False)
    g[tie_pos] = thr * np.where(rng.random(5000) < 0.5, -1, 1).astype(np.float32)   # 5000 keys == T
    check_compress(ops, g, np.zeros(n, np.float32), 0.01)
    g = np.zeros(n, np.float32)
    g[::512 * 4] = 1.0                      # the sample sees only these
    g[1::7] = 2.0
    check_compress(ops, g, np.zeros(n, np.float32), 0.01)
    check_compress(ops, student_t(rng, n), (rng.standard_normal(n) * 1e-4).astype(np.float32), 0.001)
    check_compress(ops, student_t(rng, n), np.zeros(n, np.float32), 0.3, be=300_000)
    # half of the sampled elements (32-element runs, 7812 apart at this size; every second run
    # coincides with one of these) are 5.0 and nothing else is large: the candidate window sits
    # at 5.0, there are fewer candidates (12,288) than k = 20,000, and the bucket falls back to
    # the exact selection
    n = 2_000_000
    g = student_t(rng, n, ties=0.0) * np.float32(1e-6)
    for i in range(384):
        g[5208 * i: 5208 * i + 32] = 5.0
    check_compress(ops, g, np.zeros(n, np.float32), 0.01)
    ws = ops.topk_workspace(n, n, 0.01, DEV)
    try:
        ops.set_tuning("topk_path", 2)
        ops.topk_compress(to_dev(g, F32), to_dev(np.zeros(n, np.float32), F32), 0.01, workspace=ws)
        assert ops.topk_path_report(ws, n, n, 0.01) == (0, 1)   # the scenario really takes the fallback
    finally:
        ops.set_tuning("topk_path", 0)


def test_compress_many_buckets_short_last(ops):
    rng = np.random.default_rng(8)
    n, be = 1_000_003, 131_072
    g = student_t(rng, n, ties=0.01)
    r = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    check_compress(ops, g, r, 0.01, be=be)
    check_compress(ops, g, r, 0.01, be=be + 1, pad=3)  # buckets at odd element offsets


def test_config4_full_bucket_and_error_feedback_over_steps(ops):
    # one 25 MiB bucket, Student-t nu=3 x 1e-3 with 1 % exact duplicates, k = 65,536
    n = 6_553_600
    rng = np.random.default_rng(2024)
    res_o = np.zeros(n, np.float32)
    dres = to_dev(res_o, F32)
    ws = ops.topk_workspace(n, n, 0.01, DEV)
    for step in range(3):
        g = student_t(rng, n, ties=0.01)
        w, rc = oracle.topk_compress(g, res_o, 0.01)
        wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, workspace=ws)
        assert wire.cpu().numpy()[:rc].tobytes() == w.tobytes(), step
        assert np.array_equal(bits(to_np(dres, F32)), bits(res_o)), step
        # this is the workload the single-pass path is built for: it must have taken it
        assert ops.topk_path_report(ws, n, n, 0.01) == (1, 1), step
    assert oracle.parse_wire(w)[0] == 65_536


def test_every_call_samples_afresh_across_scale_jumps(ops):
    """The window of a call comes from a sample of that call's own gradient: jumps in scale from
    one call to the next (same workspace) stay on the single-pass path and give the oracle's bytes."""
    n = 2_000_000
    rng = np.random.default_rng(31)
    ws = ops.topk_workspace(n, n, 0.01, DEV)
    for step, sc in enumerate([1.0, 1.05, 100.0, 95.0, 1e-3, 1.0]):
        g = student_t(rng, n, ties=0.01) * np.float32(sc)
        res_o = (rng.standard_normal(n) * 1e-5 * sc).astype(np.float32)
        dres = to_dev(res_o, F32)
        w, rc = oracle.topk_compress(g, res_o, 0.01)
        wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, workspace=ws)
        assert wire.cpu().numpy()[:rc].tobytes() == w.tobytes(), step
        assert np.array_equal(bits(to_np(dres, F32)), bits(res_o)), step
        assert ops.topk_path_report(ws, n, n, 0.01) == (1, 1), step


def test_workspace_with_foreign_contents_is_harmless(ops):
    """A workspace whose words were overwritten between calls (it is scratch: a caller may lend
    the memory to something else): whatever it holds, the result is exact."""
    n = 600_000
    rng = np.random.default_rng(32)
    ws = ops.topk_workspace(n, n, 0.01, DEV)
    g = student_t(rng, n)
    ops.topk_compress(to_dev(g, F32), to_dev(np.zeros(n, np.float32), F32), 0.01, workspace=ws)
    for fill in (0xFF, 0x00, 0x5A, None):
        if fill is None:
            ws.copy_(torch.randint(0, 256, (ws.numel(),), dtype=torch.uint8, device=DEV))
        else:
            ws.fill_(fill)
        for _ in range(2):
            g = student_t(rng, n)
            res_o = (rng.standard_normal(n) * 1e-4).astype(np.float32)
            dres = to_dev(res_o, F32)
            w, rc = oracle.topk_compress(g, res_o, 0.01)
            wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, workspace=ws)
            assert wire.cpu().numpy()[:rc].tobytes() == w.tobytes(), fill
            assert np.array_equal(bits(to_np(dres, F32)), bits(res_o)), fill
            assert ops.topk_path_report(ws, n, n, 0.01) == (1, 1)


def _with_bits(x, positions, patterns):
    v = x.view(np.uint32)
    v[positions] = np.asarray(patterns, np.uint32)
    return x


def test_compress_orders_nan_and_inf_by_bit_pattern(ops):
    """Selection orders magnitudes by `bits & 0x7FFFFFFF`: infinities above every finite value,
    NaN patterns above infinity (by payload), ties to the lower index.  A gradient that carries
    NaN or inf therefore gives a defined payload, the same on both paths as in the oracle: NaNs
    spread over the bucket, a NaN inside a cluster of large values (a tile with more candidates
    than slots), and a threshold that falls among equal NaN patterns (tie-break by index)."""
    rng = np.random.default_rng(606)
    n = 400_000
    qnan, qnan2, neg_qnan, top = 0x7FC00000, 0x7FC00123, 0xFFC00001, 0x7FFFFFFF
    pinf, ninf = 0x7F800000, 0xFF800000
    # (a) a few specials spread over the bucket
    g = student_t(rng, n, ties=0.0)
    pos = rng.choice(n, 12, replace=False)
    g = _with_bits(g, pos, [qnan, qnan2, neg_qnan, top, pinf, ninf, qnan, qnan, pinf, neg_qnan, qnan2, ninf])
    r = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    check_compress(ops, g.copy(), r.copy(), 0.01)
    # (b) a cluster of large values with NaN and inf in its middle: more candidates than a tile has slots
    g = student_t(rng, n, ties=0.0) * np.float32(1e-3)
    g[200_000:203_000] = student_t(rng, 3_000, ties=0.0) * np.float32(50.0)
    g = _with_bits(g, [200_500, 201_000, 201_001, 202_999], [qnan, pinf, neg_qnan, top])
    check_compress(ops, g.copy(), np.zeros(n, np.float32), 0.01)
    # (c) the threshold falls among equal NaN patterns: k = 4000, 6000 identical NaNs, 1000 larger patterns
    g = student_t(rng, n, ties=0.0)
    same = rng.choice(n, 6_000, replace=False)
    g = _with_bits(g, same, np.full(6_000, qnan, np.uint32))
    bigger = rng.choice(np.setdiff1d(np.arange(n), same), 1_000, replace=False)
    g = _with_bits(g, bigger, np.full(1_000, qnan2, np.uint32))
    check_compress(ops, g.copy(), np.zeros(n, np.float32), 0.01)
    # (d) the same with the threshold among infinities of both signs
    g = student_t(rng, n, ties=0.0)
    g = _with_bits(g, same, np.where(rng.random(6_000) < 0.5, pinf, ninf).astype(np.uint32))
    check_compress(ops, g.copy(), np.zeros(n, np.float32), 0.01)


def _state_words(ws, nbuckets):
    """The per-bucket state words inside a top-k workspace (32 words per bucket, behind the
    4096-word histograms of all buckets), as a view."""
    w32 = ws.view(torch.int32)
    off = (nbuckets * 4096 + 3) & ~3
    return w32[off: off + nbuckets * 32].view(nbuckets, 32)


S_TIMEOUT = 13  # word of a bucket's state that a block sets when it gives up waiting


def test_timeout_word_is_reported(ops):
    """The reporting path without any stuck kernel: the host sets the give-up word of a finished
    call's workspace, and the path report returns the timeout."""
    from mccl_amd._lib import MCCLHipError
    n, be = 1_000_000, 262_144
    rng = np.random.default_rng(41)
    ws = ops.topk_workspace(n, be, 0.01, DEV)
    ops.topk_compress(to_dev(student_t(rng, n), F32), torch.zeros(n, device=DEV), 0.01, bucket_elems=be, workspace=ws)
    assert ops.topk_path_report(ws, n, be, 0.01) == (4, 4)
    _state_words(ws, 4)[2, S_TIMEOUT] = 1
    with pytest.raises(MCCLHipError, match="timed out"):
        ops.topk_path_report(ws, n, be, 0.01)


def test_give_up_path_poisons_the_payload_and_sets_the_status(ops):
    """Every wait of the single-pass path runs into its limit (the sample blocks are told to
    publish a number nobody waits for; every kernel still exits normally): the status word
    receives the timeout, the path report raises, every payload header holds 0xFFFFFFFF, and
    decompress / sparse accumulate reject such a payload.  The next ordinary call on the same
    workspace is exact again."""
    from mccl_amd._lib import MCCLHipError
    n, be = 1_000_000, 262_144
    nb = 4
    rng = np.random.default_rng(42)
    g = student_t(rng, n)
    ws = ops.topk_workspace(n, be, 0.01, DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    try:
        ops.set_tuning("topk_stall_test", 1)
        ops.set_tuning("topk_barrier_ms", 1)
        wire, stride = ops.topk_compress(to_dev(g, F32), torch.zeros(n, device=DEV), 0.01, bucket_elems=be,
                                         workspace=ws, status=status)
        torch.cuda.synchronize()
    finally:
        ops.set_tuning("topk_stall_test", 0)
        ops.set_tuning("topk_barrier_ms", 2000)
    assert int(status) == -9   # MCCL_HIP_ERR_TIMEOUT
    with pytest.raises(MCCLHipError, match="timed out"):
        ops.topk_path_report(ws, n, be, 0.01)
    hdr = wire.view(torch.int32)[:: stride // 4][:nb].cpu().numpy().view(np.uint32)
    assert (hdr == 0xFFFFFFFF).all()
    dstat = torch.zeros(1, dtype=torch.int32, device=DEV)
    ops.topk_decompress(wire[:stride], stride, be, status=dstat)
    assert int(dstat) == oracle.ERR_SIZE
    dstat.zero_()
    ops.sparse_accumulate(torch.empty(n, device=DEV), [wire], stride, bucket_elems=be, status=dstat)
    assert int(dstat) == oracle.ERR_SIZE
    # the same workspace, an ordinary call
    status.zero_()
    res_o = np.zeros(n, np.float32)
    dres = to_dev(res_o, F32)
    wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, bucket_elems=be, workspace=ws, status=status)
    want, want_res = oracle_buckets(g, res_o, 0.01, be)
    w = wire.cpu().numpy()
    for b, ww in enumerate(want):
        assert w[b * stride: b * stride + ww.size].tobytes() == ww.tobytes(), b
    assert np.array_equal(bits(to_np(dres, F32)), bits(want_res))
    assert int(status) == 0 and ops.topk_path_report(ws, n, be, 0.01) == (nb, nb)


def test_more_buckets_than_the_gpu_holds_blocks_for(ops):
    """48 buckets of 300,000 elements in one call, and a list of 64 buckets: far more bin and
    select blocks than are resident at once.  Nothing in the streaming launch waits for a later
    block, and the select launch goes out in groups of 16 buckets: exact bytes, no give-up."""
    rng = np.random.default_rng(48)
    be, nb = 300_000, 48
    n = be * nb - 12_345
    g = student_t(rng, n, ties=0.01)
    res_o = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    want, want_res = oracle_buckets(g, res_o, 0.01, be)
    dres = to_dev(res_o, F32)
    ws = ops.topk_workspace(n, be, 0.01, DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    try:
        ops.set_tuning("topk_path", 2)
        wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, bucket_elems=be, workspace=ws, status=status)
        assert ops.topk_path_report(ws, n, be, 0.01) == (nb, nb)
    finally:
        ops.set_tuning("topk_path", 0)
    w = wire.cpu().numpy()
    for b, ww in enumerate(want):
        assert w[b * stride: b * stride + ww.size].tobytes() == ww.tobytes(), b
    assert np.array_equal(bits(to_np(dres, F32)), bits(want_res)) and int(status) == 0
    # a list of 64 buckets of different lengths
    sizes = [int(s) for s in rng.integers(200_000, 400_000, 64)]
    grads = [student_t(rng, m) * np.float32(10.0 ** (i % 3 - 1)) for i, m in enumerate(sizes)]
    res = [np.zeros(m, np.float32) for m in sizes]
    dres = [to_dev(r, F32) for r in res]
    wires = ops.topk_compress_list([to_dev(x, F32) for x in grads], dres, 0.01, status=status)
    torch.cuda.synchronize()
    assert int(status) == 0
    for i, (x, wv) in enumerate(zip(grads, wires)):
        ww, rc = oracle.topk_compress(x, res[i], 0.01)
        assert wv.cpu().numpy()[:rc].tobytes() == ww.tobytes(), i
        assert np.array_equal(bits(to_np(dres[i], F32)), bits(res[i])), i


def test_one_large_bucket(ops):
    # 20 M elements in one bucket: more tiles per group than a block keeps in registers (its generic sweep)
    n = 20_000_003
    rng = np.random.default_rng(99)
    g = student_t(rng, n, ties=0.001)
    res_o = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    dres = to_dev(res_o, F32)
    ws = ops.topk_workspace(n, n, 0.01, DEV)
    w, rc = oracle.topk_compress(g, res_o, 0.01)
    wire, stride = ops.topk_compress(to_dev(g, F32), dres, 0.01, workspace=ws)
    assert ops.topk_path_report(ws, n, n, 0.01) == (1, 1)
    assert wire.cpu().numpy()[:rc].tobytes() == w.tobytes()
    assert np.array_equal(bits(to_np(dres, F32)), bits(res_o))


def test_compress_argument_errors(ops):
    from mccl_amd._lib import MCCLHipError
    g = torch.zeros(1000, device=DEV); r = torch.zeros(1000, device=DEV)
    with pytest.raises(MCCLHipError, match="buffer too small"):
        ops.topk_compress(g, r, 0.1, wire_stride=4 + 8 * 100 - 4)
    with pytest.raises(MCCLHipError):
        ops.topk_compress(g, r, 0.0)
    with pytest.raises(MCCLHipError):
        ops.topk_compress(g, r, 1.5)
    with pytest.raises(MCCLHipError, match="float32 only"):
        ops.topk_compress(g.half(), r.half(), 0.1)
    with pytest.raises(MCCLHipError, match="workspace"):
        ops.topk_compress(g, r, 0.1, workspace=torch.empty(16, dtype=torch.uint8, device=DEV))


def test_decompress_matches_oracle_and_reports_errors(ops):
    rng = np.random.default_rng(5)
    n = 200_003
    g = student_t(rng, n)
    w, rc = oracle.topk_compress(g, np.zeros(n, np.float32), 0.01)
    want, _ = oracle.topk_decompress(w, n)
    dw = torch.from_numpy(w).to(DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    dense = torch.full((n + 1,), 7.0, device=DEV)[1:]  # stale contents, misaligned
    ops.topk_decompress(dw, rc, n, dense=dense, status=status)
    assert np.array_equal(bits(to_np(dense, F32)), bits(want)) and int(status) == 0
    # index out of bounds: count == largest index
    idx_max = int(oracle.parse_wire(w)[1].max())
    ops.topk_decompress(dw, rc, idx_max, dense=dense[:idx_max], status=status)
    assert int(status) == oracle.ERR_INDEX
    # size mismatch: the size that arrived disagrees with the stored k
    status.zero_()
    ops.topk_decompress(dw, rc - 8, n, dense=dense, status=status)
    assert int(status) == oracle.ERR_SIZE
    from mccl_amd._lib import MCCLHipError
    with pytest.raises(MCCLHipError, match="size mismatch"):
        ops.topk_decompress(dw, rc - 3, n, dense=dense, status=status)


@pytest.mark.parametrize("ws,n,be", [(8, 300_007, 65_536), (3, 4096, 4096), (2, 5, 5), (8, 1_000_000, 1_000_000),
                                      (3, 20_000, 20_000), (12, 50_000, 16_384)])
def test_sparse_accumulate_matches_dense_reference_form(ops, ws, n, be):
    rng = np.random.default_rng(ws + n)
    ratio = 0.01 if n > 1000 else 0.5
    if n == 20_000:
        ratio = 0.5  # more than 256 pairs of one rank per 4096-element tile
    nb = (n + be - 1) // be
    stride = ops.topk_wire_stride(be, ratio)
    # ~30 % of a rank's picks shared with other ranks: a common pool of large entries
    shared = rng.random(n) < 0.004
    dev_wires, per_bucket = [], [[] for _ in range(nb)]
    for r in range(ws):
        g = student_t(rng, n, ties=0.0)
        g[shared] *= 50.0
        buf = np.zeros(nb * stride, np.uint8)
        for b in range(nb):
            s, e = b * be, min(n, (b + 1) * be)
            w, rc = oracle.topk_compress(g[s:e].copy(), np.zeros(e - s, np.float32), ratio)
            buf[b * stride: b * stride + rc] = w
            per_bucket[b].append(w)
        dev_wires.append(torch.from_numpy(buf).to(DEV))
    want = np.empty(n, np.float32)
    for b in range(nb):
        s, e = b * be, min(n, (b + 1) * be)
        acc, rc = oracle.sparse_accumulate(per_bucket[b], e - s, scale_by=1.0 / ws)
        assert rc == oracle.OK
        want[s:e] = acc
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    for workspace in ("auto", None):   # with the tile-bounds scratch, and the scratch-free kernel
        acc = torch.full((n,), 3.0, device=DEV)
        ops.sparse_accumulate(acc, dev_wires, stride, bucket_elems=be, scale_by=1.0 / ws, status=status,
                              workspace=workspace)
        assert int(status) == 0
        assert np.array_equal(bits(to_np(acc, F32)), bits(want)), workspace


def test_sparse_accumulate_flags_bad_payloads(ops):
    n = 10_000
    stride = 4 + 8 * 16
    good = np.zeros(stride, np.uint8)
    good[:4] = np.array([2], "<u4").view(np.uint8)
    good[4:20] = np.array([5, 0x3F800000, 9_999, 0x40000000], "<u4").view(np.uint8)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    acc = torch.empty(n, device=DEV)
    for workspace in ("auto", None):
        status.zero_()
        ops.sparse_accumulate(acc, [torch.from_numpy(good).to(DEV)], stride, status=status, workspace=workspace)
        assert int(status) == 0 and float(acc[5]) == 1.0 and float(acc[9_999]) == 2.0 and float(acc.sum()) == 3.0
        bad = good.copy(); bad[12:16] = np.array([10_000], "<u4").view(np.uint8)   # index == count
        ops.sparse_accumulate(acc, [torch.from_numpy(bad).to(DEV)], stride, status=status, workspace=workspace)
        assert int(status) == oracle.ERR_INDEX
        status.zero_()
        bad = good.copy(); bad[:4] = np.array([17], "<u4").view(np.uint8)           # k beyond the stride
        ops.sparse_accumulate(acc, [torch.from_numpy(bad).to(DEV)], stride, status=status, workspace=workspace)
        assert int(status) == oracle.ERR_SIZE
    # descending indices: flagged, never out of bounds
    status.zero_()
    bad = good.copy(); bad[4:20] = np.array([9_999, 0x3F800000, 5, 0x40000000], "<u4").view(np.uint8)
    ops.sparse_accumulate(acc, [torch.from_numpy(bad).to(DEV)], stride, status=status)
    assert int(status) == oracle.ERR_INDEX


def test_tensor_layer_checks_secondary_buffers(ops):
    # a short or mistyped buffer raises in the ctypes layer, before the library sees a pointer
    g = torch.zeros(1000, device=DEV)
    with pytest.raises(ValueError, match="residual holds"):
        ops.topk_compress(g, torch.zeros(999, device=DEV), 0.1)
    with pytest.raises(ValueError, match="wire holds"):
        ops.topk_compress(g, g.clone(), 0.1, wire=torch.empty(16, dtype=torch.uint8, device=DEV))
    with pytest.raises(ValueError, match="workspace must live on the GPU"):
        ops.topk_compress(g, g.clone(), 0.1, workspace=torch.empty(1 << 20, dtype=torch.uint8))
    wire, stride = ops.topk_compress(g, g.clone(), 0.1)
    with pytest.raises(ValueError, match="wire holds"):
        ops.topk_decompress(wire, wire.numel() + 8, 1000)
    with pytest.raises(ValueError, match="dense holds"):
        ops.topk_decompress(wire, 4 + 8 * 100, 1000, dense=torch.empty(999, device=DEV))
    with pytest.raises(ValueError, match="status must be torch.int32"):
        ops.topk_decompress(wire, 4 + 8 * 100, 1000, status=torch.zeros(1, device=DEV))
    acc = torch.empty(1000, device=DEV)
    with pytest.raises(ValueError, match=r"wires\[1\] holds"):
        ops.sparse_accumulate(acc, [wire, wire[:100]], stride)
    with pytest.raises(ValueError, match=r"wires\[0\] must live on the GPU"):
        ops.sparse_accumulate(acc, [wire.cpu()], stride)
    with pytest.raises(ValueError, match="dst holds"):
        ops.cast_f32_to_f16(g, torch.empty(10, dtype=torch.float16, device=DEV))
    with pytest.raises(ValueError, match="dst must be torch.float32"):
        ops.cast_f16_to_f32(g.half(), torch.empty(1000, dtype=torch.float16, device=DEV))


def test_compress_list_equals_one_call_per_bucket(ops):
    """Separate bucket buffers of different lengths (one of them misaligned, one with a single
    element) through the list entry point: the bytes of one call per bucket, two steps."""
    from mccl_amd._lib import MCCLHipError
    rng = np.random.default_rng(12)
    sizes = [655_360, 300_001, 1, 65_537, 4_097, 1_000_003, 13, 262_144]
    res_o = [(rng.standard_normal(n) * 1e-4).astype(np.float32) for n in sizes]
    dres = [to_dev(r, F32, i % 2) for i, r in enumerate(res_o)]
    for step in range(2):
        grads = [student_t(rng, n) * np.float32(10.0 ** (i % 4 - 2)) for i, n in enumerate(sizes)]
        dg = [to_dev(g, F32, (i + 1) % 3) for i, g in enumerate(grads)]
        wires = ops.topk_compress_list(dg, dres, 0.01)
        for i, (g, w) in enumerate(zip(grads, wires)):
            ww, rc = oracle.topk_compress(g, res_o[i], 0.01)
            assert w.cpu().numpy()[:rc].tobytes() == ww.tobytes(), (step, i)
            assert np.array_equal(bits(to_np(dres[i], F32)), bits(res_o[i])), (step, i)
            assert np.array_equal(to_np(dg[i], F32), g)
    with pytest.raises(MCCLHipError, match="buffer too small"):
        ops.topk_compress_list(dg[:2], dres[:2], 0.01, wires=[wires[0], torch.empty(8, dtype=torch.uint8, device=DEV)])
    with pytest.raises(MCCLHipError):
        ops.topk_compress_list([dg[0]] * 65, [dres[0]] * 65, 0.01)
    with pytest.raises(ValueError, match="residuals\\[1\\] holds"):
        ops.topk_compress_list(dg[:2], [dres[0], dres[0]], 0.01)
