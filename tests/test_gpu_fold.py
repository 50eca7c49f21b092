"""HIP folds vs the CPU oracle, bit for bit, through the C ABI.
Shapes follow the reference's kernel tests (tests/test_local_kernels.py: sizes
1,3,7,13,97,997, 1 M random) plus misaligned chunk views and the 25 MiB bucket."""
import numpy as np
import pytest
import torch

import oracle
from oracle import F32, F16, BF16, I32, I64, BOOL, OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX
from tests._gpu_util import DEV, to_dev, to_np, bits, rand_vals, NP_DT

pytestmark = pytest.mark.gpu

SIZES = (1, 3, 7, 13, 97, 997, 4097, 1_000_003)
OPS = (OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX)


@pytest.fixture(scope="module")
def ops():
    from mccl_amd import hip_ops
    return hip_ops


@pytest.mark.parametrize("dt", [F32, F16, BF16])
@pytest.mark.parametrize("op", OPS)
def test_fold2_matches_oracle(ops, dt, op):
    rng = np.random.default_rng(100 + dt * 10 + op)
    for n in SIZES:
        for pad_d, pad_s in ((0, 0), (1, 0), (0, 3), (5, 2)):
            a = rand_vals(rng, n, dt); b = rand_vals(rng, n, dt)
            want = a.copy()
            assert oracle.fold2(want, b, dt, op) == oracle.OK
            d = to_dev(a, dt, pad_d); s = to_dev(b, dt, pad_s)
            ops.fold2(d, s, op)
            got = to_np(d, dt)
            w32, g32 = (want, got) if dt != F32 else (bits(want), bits(got))
            if dt == F32:
                nan = np.isnan(want)
            elif dt == F16:
                nan = np.isnan(oracle.f16_bits_to_f32(want))
            else:
                nan = np.isnan(oracle.bf16_bits_to_f32(want))
            assert np.array_equal(w32[~nan], g32[~nan]), (n, pad_d, pad_s)
            assert np.array_equal(to_np(s, dt), b)  # src untouched


@pytest.mark.parametrize("dt", [F32, F16, BF16])
def test_scale_and_fused_match_oracle(ops, dt):
    rng = np.random.default_rng(7 + dt)
    for n in SIZES:
        for s in (0.5, 0.25, 0.125, float(np.float32(1.0 / 3.0)), float(np.float32(1.0 / 7.0))):
            a = rand_vals(rng, n, dt, specials=False); b = rand_vals(rng, n, dt, specials=False)
            want = a.copy(); oracle.scale(want, dt, s)
            d = to_dev(a, dt, 1)
            ops.scale(d, s)
            assert np.array_equal(bits(to_np(d, dt)), bits(want)), (n, s)
            want = a.copy(); oracle.fold2_scale(want, b, dt, s)
            d = to_dev(a, dt, 2); src = to_dev(b, dt, 1)
            ops.fold2_scale(d, src, s)
            assert np.array_equal(bits(to_np(d, dt)), bits(want)), (n, s)


def test_config1_bucket_fp32_sum_then_avg(ops):
    # one 25 MiB bucket per rank, N(0, 1e-2), seeds seed + rank; acc = x0 + x1; acc *= 0.5
    n = 6_553_600
    xs = [torch.randn(n, generator=torch.Generator().manual_seed(1234 + r)).mul_(1e-2).numpy() for r in range(2)]
    want = xs[0].copy(); oracle.fold2(want, xs[1], F32, OP_SUM); oracle.scale(want, F32, 0.5)
    acc = to_dev(xs[0], F32); x1 = to_dev(xs[1], F32)
    ops.fold2(acc, x1, OP_SUM); ops.scale(acc, 0.5)
    assert np.array_equal(bits(to_np(acc, F32)), bits(want))
    fused = to_dev(xs[0], F32)
    ops.fold2_scale(fused, x1, 0.5)
    assert np.array_equal(bits(to_np(fused, F32)), bits(want))  # x0.5 is exact: same bits


def test_reference_kernel_known_answers(ops):
    # tests/test_local_kernels.py:67-73,:133-139,:167-173,:205-211,:228-233,:287-294
    t = lambda v, dt=torch.float32: torch.tensor(v, dtype=dt, device=DEV)
    assert ops.fold2(t([1., 2., 3.]), t([4., 5., 6.]), OP_SUM).tolist() == [5., 7., 9.]
    assert ops.fold2(t([1., 5., 3.]), t([4., 2., 6.]), OP_MIN).tolist() == [1., 2., 3.]
    assert ops.fold2(t([1., 5., 3.]), t([4., 2., 6.]), OP_MAX).tolist() == [4., 5., 6.]
    assert ops.fold2(t([2., 3., 4.]), t([5., 6., 7.]), OP_PRODUCT).tolist() == [10., 18., 28.]
    assert ops.scale(t([2., 4., 6.]), 0.5).tolist() == [1., 2., 3.]
    assert ops.fold2_scale(t([1., 3., 5.]), t([3., 5., 7.]), 0.5).tolist() == [2., 4., 6.]
    for dt in (torch.float16, torch.bfloat16):
        assert ops.fold2(t([1., 2., 3.], dt), t([4., 5., 6.], dt), OP_SUM).tolist() == [5., 7., 9.]
        assert ops.fold2_scale(t([1., 3., 5.], dt), t([3., 5., 7.], dt), 0.5).tolist() == [2., 4., 6.]
    for ws in (2, 3, 4, 8):
        r = ops.scale(torch.full((256,), float(ws), device=DEV), float(np.float32(1.0 / ws)))
        assert torch.allclose(r, torch.ones(256, device=DEV), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt,npdt", [(I32, np.int32), (I64, np.int64), (BOOL, np.uint8)])
def test_integral_folds_and_scale(ops, dt, npdt):
    rng = np.random.default_rng(dt)
    for n in (1, 3, 7, 13, 1001, 100_003):
        hi = 2 if dt == BOOL else 1000
        a = rng.integers(0, hi, n).astype(npdt); b = rng.integers(0, hi, n).astype(npdt)
        for op in (OP_SUM, OP_PRODUCT, OP_MIN, OP_MAX):
            want = a.copy(); oracle.fold2(want, b, dt, op)
            d = to_dev(a, dt, 1); ops.fold2(d, to_dev(b, dt, 3), op)
            assert np.array_equal(to_np(d, dt), want), (n, op)
        for s in (0.5, float(np.float32(1.0 / 3.0))):
            want = a.copy(); oracle.scale(want, dt, s, round_i32=True)
            d = to_dev(a, dt); ops.scale(d, s)
            assert np.array_equal(to_np(d, dt), want), (n, s)
    # reference answers: tests/test_local_kernels.py:268-281,:315-337
    v = ops.scale(torch.arange(1, 14, device=DEV, dtype=torch.int64) * 3, 1.0 / 3.0)
    assert torch.equal(v, torch.arange(1, 14, device=DEV, dtype=torch.int64))
    a = torch.tensor([1, 3, 5, 7, 9], device=DEV, dtype=torch.int32)
    b = torch.tensor([3, 5, 7, 9, 11], device=DEV, dtype=torch.int32)
    assert ops.fold2_scale(a, b, 0.5).tolist() == [2, 4, 6, 8, 10]
    a = torch.tensor([True, True, False], device=DEV); b = torch.tensor([True, False, True], device=DEV)
    assert ops.fold2_scale(a, b, 0.5).tolist() == [True, False, False]
    assert ops.scale(torch.tensor([True, False, True], device=DEV), 0.5).tolist() == [False, False, False]


def test_errors(ops):
    from mccl_amd._lib import MCCLHipError
    a = torch.zeros(4, device=DEV); b = torch.zeros(4, device=DEV)
    with pytest.raises(MCCLHipError, match="Unsupported ReduceOp"):
        ops.fold2(a, b, 5)
    with pytest.raises(MCCLHipError, match="element type"):
        ops.fold2(a.double(), b.double(), OP_SUM)
    # empty tensors are no-ops
    e = torch.zeros(0, device=DEV)
    ops.fold2(e, e.clone(), OP_SUM); ops.scale(e, 0.5)


def test_fence_orders_completion(ops):
    a = torch.ones(1 << 22, device=DEV); b = torch.ones(1 << 22, device=DEV)
    ops.fold2(a, b, OP_SUM)
    t = ops.fence_signal()
    assert t > 0
    ops.fence_wait(t)
    assert ops.fence_query(t) is True
    assert float(a[0]) == 2.0 and float(a[-1]) == 2.0
