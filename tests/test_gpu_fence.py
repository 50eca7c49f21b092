"""Fence tickets (the analogue of csrc/metal/EventSync.mm:189-206) across streams.

The library holds the newest 1024 tickets' events.  A ticket pushed out of that
window must read as complete only when its stream's work really is: here stream A
carries a ticket behind a long queue of folds, an idle stream B then signals more
than 1024 times, and a wait on A's old ticket must still cover A's work."""
import pytest
import torch

from tests._gpu_util import DEV

pytestmark = pytest.mark.gpu


def test_ticket_pushed_out_of_the_event_window_still_orders_its_stream():
    from mccl_amd import hip_ops as ops
    n = 1 << 25
    a = torch.zeros(n, device=DEV)
    one = torch.ones(n, device=DEV)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    reps = 150                                   # ~0.1 ms each: stream A stays busy for >10 ms
    with torch.cuda.stream(sa):
        for _ in range(reps):
            ops.fold2(a, one, ops.SUM)
        old = ops.fence_signal()
    with torch.cuda.stream(sb):
        last = old
        for _ in range(1100):                    # wraps the 1024-event window on an idle stream
            last = ops.fence_signal()
    assert last >= old + 1100
    ops.fence_wait(old)
    assert ops.fence_query(old) is True
    # no further synchronisation: the wait above has to have covered stream A's folds
    with torch.cuda.stream(sb):
        head, tail = float(a[0]), float(a[-1])
    assert head == reps and tail == reps
    torch.cuda.synchronize()


def test_block_stream_orders_a_second_stream_behind_the_ticket():
    from mccl_amd import hip_ops as ops
    from mccl_amd import _lib
    n = 1 << 24
    a = torch.zeros(n, device=DEV)
    one = torch.ones(n, device=DEV)
    b = torch.empty(n, device=DEV)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(sa):
        for _ in range(40):
            ops.fold2(a, one, ops.SUM)
        t = ops.fence_signal()
    with torch.cuda.stream(sb):
        _lib.check(_lib.load().mccl_hip_fence_block_stream(t, sb.cuda_stream), "fence_block_stream")
        b.copy_(a)
    sb.synchronize()
    assert float(b[0]) == 40.0 and float(b[-1]) == 40.0
    torch.cuda.synchronize()
