"""Properties that hold at any size, checked at the benchmark's full size
(96,510,024 elements, 25 MiB buckets) without the oracle in the loop:

    top-k     what leaves the residual is exactly what the payload carries:
              decompress(payload) + residual_after == grad + residual_before,
              bit for bit; indices strictly ascending; k entries per bucket;
              every kept magnitude >= every magnitude left behind
              (csrc/compression/TopKCompression.cpp:38-120)
    sparse    accumulate of one rank's payloads == their decompress; accumulate is
              additive over ranks whose index sets do not overlap
              (csrc/backend/ProcessGroupMCCL.cpp:2272-2296)
    fold      x + x is 2x exactly and its average is x; MAX of a buffer with itself
              is the buffer; the fold of zeros is zero
"""
import numpy as np
import pytest
import torch

from tests._gpu_util import DEV

pytestmark = pytest.mark.gpu

N = 96_510_024
BUCKET = 6_553_600
NB = (N + BUCKET - 1) // BUCKET


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


def gradient(seed, scale):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    g = torch.randn(N, generator=gen, device=DEV)
    g.mul_(torch.rand(N, generator=gen, device=DEV).mul_(4.0).exp_()).mul_(scale)   # heavy-tailed magnitudes
    return g


def parse(wire_bucket):
    """device payload -> (k, idx int64, val float32), tensors on the device."""
    k = int(wire_bucket[:4].view(torch.int32)[0])
    body = wire_bucket[4:4 + 8 * k].view(torch.int32).view(k, 2)
    return k, body[:, 0].to(torch.int64), body[:, 1].contiguous().view(torch.float32)


def test_topk_moves_exactly_the_payload_out_of_the_residual(ops):
    stride = ops.topk_wire_stride(BUCKET, 0.01)
    wsb = ops.topk_workspace(N, BUCKET, 0.01, DEV)
    wire = torch.empty(NB * stride, dtype=torch.uint8, device=DEV)
    residual = gradient(1, 1e-5)
    for step in range(2):
        grad = gradient(10 + step, 1e-3)
        total = grad + residual                                   # the single fp32 add the kernel does
        ops.topk_compress(grad, residual, 0.01, bucket_elems=BUCKET, wire=wire, workspace=wsb, wire_stride=stride)
        assert ops.topk_path_report(wsb, N, BUCKET, 0.01) == (NB, NB)
        rebuilt = residual.clone()
        for b in range(NB):
            s, e = b * BUCKET, min(N, (b + 1) * BUCKET)
            k, idx, val = parse(wire[b * stride:(b + 1) * stride])
            assert k == ops.topk_k(e - s, 0.01), (step, b)
            assert bool((idx[1:] > idx[:-1]).all()) and int(idx[-1]) < e - s, (step, b)
            sub = rebuilt[s:e]
            assert bool((sub[idx] == 0).all()), (step, b)          # picked elements left the residual
            kept_min = float(val.abs().min())
            assert float(residual[s:e].abs().max()) <= kept_min, (step, b)
            sub[idx] = val
        assert torch.equal(rebuilt.view(torch.int32), total.view(torch.int32)), step
        # decompress of every bucket gives the same dense picture
        dense = torch.empty(BUCKET, device=DEV)
        status = torch.zeros(1, dtype=torch.int32, device=DEV)
        for b in (0, NB - 1):
            s, e = b * BUCKET, min(N, (b + 1) * BUCKET)
            k = ops.topk_k(e - s, 0.01)
            ops.topk_decompress(wire[b * stride:(b + 1) * stride], 4 + 8 * k, e - s, dense=dense[:e - s], status=status)
            assert int(status) == 0
            assert torch.equal((dense[:e - s] + residual[s:e]).view(torch.int32), total[s:e].view(torch.int32)), (step, b)
        del grad, total, rebuilt


def test_sparse_accumulate_of_one_rank_is_its_decompress_and_disjoint_ranks_add_up(ops):
    stride = ops.topk_wire_stride(BUCKET, 0.01)
    wsb = ops.topk_workspace(N, BUCKET, 0.01, DEV)
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    # two ranks whose picks cannot collide: rank 0 only has mass on even elements, rank 1 on odd ones
    wires, dense = [], []
    for r in range(2):
        g = gradient(20 + r, 1e-3)
        g[(1 - r)::2] = 0.0
        w = torch.empty(NB * stride, dtype=torch.uint8, device=DEV)
        ops.topk_compress(g, torch.zeros(N, device=DEV), 0.01, bucket_elems=BUCKET, wire=w, workspace=wsb, wire_stride=stride)
        wires.append(w)
        d = torch.zeros(N, device=DEV)
        for b in range(NB):
            s, e = b * BUCKET, min(N, (b + 1) * BUCKET)
            k, idx, val = parse(w[b * stride:(b + 1) * stride])
            d[s:e][idx] = val
        dense.append(d)
        del g
    acc = torch.full((N,), 7.0, device=DEV)
    for r in range(2):
        ops.sparse_accumulate(acc, [wires[r]], stride, bucket_elems=BUCKET, status=status)
        assert int(status) == 0 and torch.equal(acc.view(torch.int32), dense[r].view(torch.int32)), r
    ops.sparse_accumulate(acc, wires, stride, bucket_elems=BUCKET, scale_by=0.5, status=status)
    assert int(status) == 0
    assert torch.equal(acc.view(torch.int32), ((dense[0] + dense[1]) * 0.5).view(torch.int32))
    ops.sparse_accumulate(acc, wires[::-1], stride, bucket_elems=BUCKET, scale_by=0.5, status=status)
    assert torch.equal(acc.view(torch.int32), ((dense[0] + dense[1]) * 0.5).view(torch.int32))


def test_fold_closed_forms(ops):
    from mccl_amd.hip_ops import SUM, MAX, AVG
    import oracle
    x = gradient(30, 1e-3)
    out = torch.empty(N, device=DEV)
    ops.ring_fold(out, [x, x], SUM, oracle.RING_BASIC, bucket_elems=BUCKET)
    assert torch.equal(out.view(torch.int32), (x * 2.0).view(torch.int32))                   # doubling is exact
    ops.ring_fold(out, [x, x], AVG, oracle.RING_CHUNKED, bucket_elems=BUCKET, scale_by=0.5)
    assert torch.equal(out.view(torch.int32), x.view(torch.int32))
    for ws in (3, 8):
        ops.ring_fold(out, [x] * ws, MAX, oracle.RING_BASIC, bucket_elems=BUCKET)
        assert torch.equal(out.view(torch.int32), x.view(torch.int32)), ws
    z = torch.zeros(N, device=DEV)
    ops.ring_fold(out, [z] * 6, SUM, oracle.RING_CHUNKED, bucket_elems=BUCKET)
    assert int(out.view(torch.int32).abs().max()) == 0
