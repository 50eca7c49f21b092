"""The entry points only enqueue kernels on the caller's stream (no host
synchronisation, no allocation, no memset nodes), so a launch-bound sequence
such as the launches of a one-bucket top-k compress (two on the single-pass path, six on the
exact path) can be captured in a HIP
graph.  Every replay is checked against the eager result and the oracle, with
eager work and synchronisations in between."""
import numpy as np
import pytest
import torch

import oracle
from oracle import F32
from tests._gpu_util import DEV, to_np, bits, student_t

pytestmark = pytest.mark.gpu


def test_topk_compress_and_fold_replay_from_a_graph():
    from mccl_amd import hip_ops as ops
    n, ratio = 1_000_003, 0.01
    rng = np.random.default_rng(5)
    grad = torch.empty(n, device=DEV)
    res = torch.zeros(n, device=DEV)
    other = torch.empty(n, device=DEV)
    ws = ops.topk_workspace(n, n, ratio, DEV)
    stride = ops.topk_wire_stride(n, ratio)
    wire = torch.zeros(stride, dtype=torch.uint8, device=DEV)
    # warm-up outside capture (library init, first-use paths)
    grad.copy_(torch.from_numpy(student_t(rng, n)))
    other.copy_(grad)
    ops.topk_compress(grad, res, ratio, wire=wire, workspace=ws)
    ops.fold2_scale(other, grad, 0.5)
    torch.cuda.synchronize()

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            ops.topk_compress(grad, res, ratio, wire=wire, workspace=ws)
            ops.fold2_scale(other, grad, 0.5)
    torch.cuda.current_stream().wait_stream(side)

    res_o = np.zeros(n, np.float32)
    res.zero_()
    for step in range(4):
        gh = student_t(rng, n, ties=0.01)
        oh = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        grad.copy_(torch.from_numpy(gh))
        other.copy_(torch.from_numpy(oh))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        w, rc = oracle.topk_compress(gh, res_o, ratio)
        assert wire.cpu().numpy()[:rc].tobytes() == w.tobytes(), step
        assert np.array_equal(bits(to_np(res, F32)), bits(res_o)), step
        want = oh.copy()
        oracle.fold2_scale(want, gh, F32, 0.5)
        assert np.array_equal(bits(to_np(other, F32)), bits(want)), step
        # eager work between replays
        assert float((other - torch.from_numpy(want).to(DEV)).abs().max()) == 0.0
