"""The raw-pointer fold family (csrc/metal/AccelerateOps.hpp:18-59: cpu_accumulate,
cpu_scale_inplace, cpu_accumulate_and_scale, cpu_elementwise_{min,max,product},
cpu_reduce_op and the _half / _bf16 / _integral forms) against the oracle, and
its pointer rule: the reference passes memory that CPU and GPU share; here a
buffer has to be reachable by a kernel (device or pinned host memory), and
pageable host memory raises before anything is launched."""
import numpy as np
import pytest
import torch
import torch.distributed  # noqa: F401

import oracle
from oracle import F32, F16, BF16, I32, I64, BOOL, OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX
from tests._gpu_util import DEV, to_dev, to_np, bits, rand_vals

pytestmark = pytest.mark.gpu
SIZES = (1, 3, 13, 997, 100_003)


@pytest.fixture(scope="module")
def C():
    from mccl_amd import _C
    return _C


@pytest.mark.parametrize("dt", [F32, F16, BF16])
def test_float_forms_match_oracle(C, dt):
    rng = np.random.default_rng(40 + dt)
    for n in SIZES:
        a = rand_vals(rng, n, dt, specials=False); b = rand_vals(rng, n, dt, specials=False)
        for op in (OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX):    # cpu_reduce_op / _half / _bf16
            want = a.copy(); oracle.fold2(want, b, dt, op)
            got = C._cpu_reduce_op(to_dev(a, dt, 1), to_dev(b, dt), op)
            assert np.array_equal(bits(to_np(got, dt)), bits(want)), (n, op)
        for s in (0.5, float(np.float32(1.0 / 3.0))):
            want = a.copy(); oracle.scale(want, dt, s)                  # cpu_scale_inplace*
            assert np.array_equal(bits(to_np(C._cpu_scale_inplace(to_dev(a, dt), s), dt)), bits(want)), (n, s)
            want = a.copy(); oracle.fold2_scale(want, b, dt, s)         # cpu_accumulate_and_scale*
            got = C._cpu_accumulate_and_scale(to_dev(a, dt, 3), to_dev(b, dt, 1), s)
            assert np.array_equal(bits(to_np(got, dt)), bits(want)), (n, s)


def test_named_f32_forms_match_oracle(C):
    rng = np.random.default_rng(41)
    for n in SIZES:
        a = rand_vals(rng, n, F32); b = rand_vals(rng, n, F32)
        for fn, op in ((C._cpu_accumulate, OP_SUM), (C._cpu_elementwise_min, OP_MIN),
                       (C._cpu_elementwise_max, OP_MAX), (C._cpu_elementwise_product, OP_PRODUCT)):
            want = a.copy(); oracle.fold2(want, b, F32, op)
            got = to_np(fn(to_dev(a, F32), to_dev(b, F32, 2)), F32)
            ok = ~np.isnan(want)
            assert np.array_equal(np.isnan(got), ~ok) and np.array_equal(bits(got)[ok], bits(want)[ok]), (n, op)


@pytest.mark.parametrize("dt,npdt", [(I32, np.int32), (I64, np.int64), (BOOL, np.uint8)])
def test_integral_forms_match_oracle(C, dt, npdt):
    rng = np.random.default_rng(42 + dt)
    for n in SIZES:
        hi = 2 if dt == BOOL else 1000
        a = rng.integers(0, hi, n).astype(npdt); b = rng.integers(0, hi, n).astype(npdt)
        for op in (OP_SUM, OP_PRODUCT, OP_MIN, OP_MAX):                # cpu_reduce_op_integral
            want = a.copy(); oracle.fold2(want, b, dt, op)
            assert np.array_equal(to_np(C._cpu_reduce_op(to_dev(a, dt), to_dev(b, dt, 1), op), dt), want), (n, op)
        want = a.copy(); oracle.scale(want, dt, 0.5, round_i32=True)    # cpu_scale_inplace_integral
        assert np.array_equal(to_np(C._cpu_scale_inplace(to_dev(a, dt), 0.5), dt), want), n
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        C._cpu_reduce_op(torch.zeros(4, device=DEV, dtype=torch.float64),
                         torch.zeros(4, device=DEV, dtype=torch.float64), OP_SUM)


def test_pinned_host_memory_is_accepted(C):
    # the closest thing to the reference's shared CPU/GPU buffers: the kernel works on the
    # pinned pages directly and the call has completed when it returns
    a = torch.arange(10_000, dtype=torch.float32).pin_memory()
    b = torch.full((10_000,), 0.5).pin_memory()
    r = C._cpu_reduce_op(a, b, OP_SUM)
    assert r.device.type == "cpu" and torch.equal(r, torch.arange(10_000, dtype=torch.float32) + 0.5)
    assert torch.equal(C._cpu_scale_inplace(a, 2.0), (torch.arange(10_000, dtype=torch.float32) + 0.5) * 2)
    # mixed: device destination, pinned source
    d = torch.ones(10_000, device=DEV)
    assert torch.equal(C._cpu_accumulate(d, b).cpu(), torch.full((10_000,), 1.5))


def test_pageable_host_memory_and_bad_ranges_raise_before_any_launch(C):
    a = torch.ones(1000); b = torch.ones(1000)                          # pageable host memory
    for call in (lambda: C._cpu_reduce_op(a, b, OP_SUM), lambda: C._cpu_scale_inplace(a, 0.5),
                 lambda: C._cpu_accumulate_and_scale(a, b, 0.5), lambda: C._cpu_accumulate(a, b),
                 lambda: C._cpu_elementwise_max(a, b),
                 lambda: C._cpu_reduce_op(a.half(), b.half(), OP_SUM),
                 lambda: C._cpu_reduce_op(a.long(), b.long(), OP_SUM)):
        with pytest.raises(RuntimeError, match="not memory a GPU kernel can reach"):
            call()
    assert float(a.sum()) == 1000.0                                     # untouched
    # device destination, pageable source
    with pytest.raises(RuntimeError, match="not memory a GPU kernel can reach"):
        C._cpu_accumulate(torch.ones(1000, device=DEV), b)
    # a count that runs past the end of the device allocation
    d = torch.ones(1000, device=DEV); s = torch.ones(1 << 20, device=DEV)
    with pytest.raises(RuntimeError, match="not memory a GPU kernel can reach"):
        C._cpu_reduce_op_ptr(d.data_ptr(), s.data_ptr(), 1 << 28, OP_SUM)
    # ... and past the end of a pinned host allocation (its extent is checked like device memory's)
    hp = torch.ones(1000).pin_memory()
    with pytest.raises(RuntimeError, match="not memory a GPU kernel can reach"):
        C._cpu_reduce_op_ptr(hp.data_ptr(), hp.data_ptr(), 1 << 28, OP_SUM)
    assert float(hp.sum()) == 1000.0
    with pytest.raises(RuntimeError, match="Unsupported ReduceOp"):
        C._cpu_reduce_op(d, d.clone(), 5)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        C._cpu_reduce_op(d, s, OP_SUM)
    torch.cuda.synchronize()
    assert float(d.sum()) == 1000.0


def test_decompress_bindings_validate_the_payload(C):
    comp = C.TopKCompressor(0.1)
    g = torch.randn(1000, device=DEV)
    wire = comp.compress(g, stable_id=1)
    with pytest.raises(RuntimeError, match="ROCm GPU device"):
        comp.decompress(wire.cpu(), 1000)
    with pytest.raises(RuntimeError, match="uint8"):
        comp.decompress(wire.view(torch.int32)[: wire.numel() // 4], 1000)
    with pytest.raises(RuntimeError, match="exceeds the payload tensor"):
        comp.decompress(wire, 1000, compressed_size=wire.numel() + 8)
    half = C.FP16Compressor()
    w16 = half.compress(g)
    with pytest.raises(RuntimeError, match="ROCm GPU device"):
        half.decompress(w16.cpu(), 1000)
    with pytest.raises(RuntimeError, match="exceeds the payload tensor"):
        half.decompress(w16, 1000, compressed_size=w16.numel() + 2)
    with pytest.raises(RuntimeError, match="output tensor's GPU"):
        C._compressed_unpack(comp, wire.numel(), wire.cpu(), torch.empty(1000, device=DEV))
