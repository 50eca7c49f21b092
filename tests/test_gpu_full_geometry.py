"""The benchmark's own launch geometries checked bit for bit against the oracle:
the 96,510,024-element gradient in 25 MiB buckets (14 full buckets and one of
4,759,624 elements), exactly as bench.py launches it.

    fold      8 ranks, basic ring, 15 buckets x 8 chunks in one launch, AVG x 1/8
    16-bit    bf16 / fp16, 4 ranks, SUM x 0.25 (stepwise and single rounding), MAX
    top-k     15 buckets in one launch, residual carried over two steps
    sparse    8 ranks' payloads, 15 buckets, ~30 % index overlap, AVG x 1/8
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import F32, F16, BF16, OP_SUM, OP_AVG, OP_MAX, RING_BASIC
from tests._gpu_util import DEV, to_np, bits

pytestmark = pytest.mark.gpu

N = 96_510_024
BUCKET = 6_553_600
NB = (N + BUCKET - 1) // BUCKET


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


def cpu_randn(seed, sigma):
    return torch.randn(N, generator=torch.Generator().manual_seed(seed)).mul_(sigma)


def test_config2_fp32_ring_fold_w8_whole_gradient(ops):
    ws = 8
    host = [cpu_randn(1000 + r, 1e-3).numpy() for r in range(ws)]
    want = np.empty(N, np.float32)
    for s in range(0, N, BUCKET):
        e = min(N, s + BUCKET)
        want[s:e] = oracle.ring_fold([x[s:e] for x in host], F32, OP_SUM, RING_BASIC, scale_by=0.125)
    dins = [torch.from_numpy(x).to(DEV) for x in host]
    out = torch.empty(N, device=DEV)
    ops.ring_fold(out, dins, OP_AVG, RING_BASIC, bucket_elems=BUCKET, scale_by=0.125)
    assert np.array_equal(bits(out.cpu().numpy()), bits(want))
    # size-independent property at the same geometry: adding zeros is exact in every fold
    # order, so one rank's buffer folded with seven zero buffers comes back times 1/8
    zero = torch.zeros(N, device=DEV)
    for r in (0, 3, 7):
        ins = [zero] * ws
        ins[r] = dins[r]
        ops.ring_fold(out, ins, OP_AVG, RING_BASIC, bucket_elems=BUCKET, scale_by=0.125)
        assert torch.equal(out.view(torch.int32), (dins[r] * 0.125).view(torch.int32)), r


@pytest.mark.parametrize("dt", [BF16, F16])
def test_config3_16bit_ring_fold_w4_whole_gradient(ops, dt):
    ws = 4
    tdt = torch.bfloat16 if dt == BF16 else torch.float16
    ins_t = []
    for r in range(ws):
        g = torch.Generator().manual_seed(3000 + r)
        x = torch.randn(N, generator=g).mul_(1e-3)
        m = torch.rand(N, generator=g) < 1e-3          # 0.1 % outliers x 1e3
        x[m] *= 1e3
        ins_t.append(x.to(tdt))
        del x, m
    ins = [t.view(torch.int16).numpy().view(np.uint16) for t in ins_t]
    dins = [t.to(DEV) for t in ins_t]
    out = torch.empty(N, device=DEV, dtype=tdt)
    be = 2 * BUCKET                                    # 25 MiB of 16-bit elements
    for op, sc, stepwise in ((OP_SUM, 0.25, True), (OP_SUM, 0.25, False), (OP_MAX, None, False)):
        want = np.empty(N, np.uint16)
        for s in range(0, N, be):
            e = min(N, s + be)
            want[s:e] = oracle.ring_fold([x[s:e] for x in ins], dt, op, RING_BASIC, scale_by=sc,
                                         stepwise=stepwise)
        ops.ring_fold(out, dins, OP_AVG if sc else op, RING_BASIC, bucket_elems=be, scale_by=sc,
                      stepwise=stepwise)
        got = to_np(out, dt)
        assert np.array_equal(got, want), (op, sc, stepwise)


def bench_gradient(seed):
    """Student-t (nu = 3) x 1e-3 with 1 % exact duplicates (random sign), built on
    the device like bench.py's, returned as (device tensor, host array)."""
    gen = torch.Generator(device=DEV).manual_seed(seed)
    g = torch.randn(N, generator=gen, device=DEV)
    chi = sum(torch.randn(N, generator=gen, device=DEV).square_() for _ in range(3)).div_(3).sqrt_()
    grad = g.div_(chi).mul_(1e-3)
    del chi
    m = N // 100
    dst = torch.randint(0, N, (m,), generator=gen, device=DEV)
    src = torch.randint(0, N, (m,), generator=gen, device=DEV)
    sign = torch.where(torch.rand(m, generator=gen, device=DEV) < 0.5, -1.0, 1.0)
    grad[dst] = grad[src] * sign
    return grad, grad.cpu().numpy()


def test_config4_topk_15_buckets_two_steps(ops):
    stride = ops.topk_wire_stride(BUCKET, 0.01)
    wsb = ops.topk_workspace(N, BUCKET, 0.01, DEV)
    wire = torch.empty(NB * stride, dtype=torch.uint8, device=DEV)
    res_h = torch.randn(N, generator=torch.Generator().manual_seed(7)).mul_(1e-4).numpy()
    dres = torch.from_numpy(res_h).to(DEV)
    for step in range(2):
        dgrad, grad_h = bench_gradient(40 + step)
        ops.topk_compress(dgrad, dres, 0.01, bucket_elems=BUCKET, wire=wire, workspace=wsb, wire_stride=stride)
        w = wire.cpu().numpy()
        for b in range(NB):
            s, e = b * BUCKET, min(N, (b + 1) * BUCKET)
            sub = res_h[s:e]
            ww, rc = oracle.topk_compress(grad_h[s:e], sub, 0.01)
            assert w[b * stride: b * stride + rc].tobytes() == ww.tobytes(), (step, b)
        assert np.array_equal(bits(dres.cpu().numpy()), bits(res_h)), step
        assert ops.topk_path_report(wsb, N, BUCKET, 0.01) == (NB, NB), step
        del dgrad


def test_config5_sparse_accumulate_8_ranks_15_buckets(ops):
    ws = 8
    stride = ops.topk_wire_stride(BUCKET, 0.01)
    wsb = ops.topk_workspace(N, BUCKET, 0.01, DEV)
    shared = torch.rand(N, generator=torch.Generator(device=DEV).manual_seed(5), device=DEV) < 0.004
    wires = []
    for r in range(ws):
        gr = torch.randn(N, generator=torch.Generator(device=DEV).manual_seed(50 + r), device=DEV).mul_(1e-2)
        gr[shared] *= 50.0
        rz = torch.zeros(N, device=DEV)
        wr = torch.empty(NB * stride, dtype=torch.uint8, device=DEV)
        ops.topk_compress(gr, rz, 0.01, bucket_elems=BUCKET, wire=wr, workspace=wsb, wire_stride=stride)
        wires.append(wr)
        del gr, rz
    host = [w.cpu().numpy() for w in wires]
    want = np.empty(N, np.float32)
    overlap = 0
    for b in range(NB):
        s, e = b * BUCKET, min(N, (b + 1) * BUCKET)
        payloads = []
        for r in range(ws):
            k = int(host[r][b * stride: b * stride + 4].view("<u4")[0])
            payloads.append(host[r][b * stride: b * stride + 4 + 8 * k])
        acc, rc = oracle.sparse_accumulate(payloads, e - s, scale_by=0.125)
        assert rc == oracle.OK
        want[s:e] = acc
        if b == 0:
            i0 = oracle.parse_wire(payloads[0])[1]
            others = np.concatenate([oracle.parse_wire(p)[1] for p in payloads[1:]])
            overlap = np.isin(i0, others).mean()
    assert 0.15 < overlap < 0.6          # the workload's index overlap across ranks is present
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    acc = torch.full((N,), 3.0, device=DEV)
    ops.sparse_accumulate(acc, wires, stride, bucket_elems=BUCKET, scale_by=0.125, status=status)
    assert int(status) == 0
    assert np.array_equal(bits(acc.cpu().numpy()), bits(want))
