"""Pins the oracle's folds against torch's CPU kernels (independent library
routines) and the reference tests' known answers
(tests/test_local_kernels.py, tests/test_process_group_local.py:243-468)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import F16, BF16, F32, I32, I64, BOOL, OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX

SIZES = (1, 3, 7, 13, 97, 997, 4097, 1_000_000, 2_500_003)


def _bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


TORCH_OPS = {
    OP_SUM: lambda a, b: a + b,
    OP_AVG: lambda a, b: a + b,
    OP_PRODUCT: lambda a, b: a * b,
    OP_MIN: torch.minimum,
    OP_MAX: torch.maximum,
}


@pytest.mark.parametrize("op", [OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX])
def test_fp32_fold_matches_torch_cpu_bitwise(op):
    g = torch.Generator().manual_seed(11)
    for n in SIZES:
        a = torch.randn(n, generator=g)
        b = torch.randn(n, generator=g)
        want = TORCH_OPS[op](a, b).numpy()
        dst = a.numpy().copy()
        assert oracle.fold2(dst, b.numpy(), F32, op) == oracle.OK
        assert np.array_equal(dst.view(np.uint32), want.view(np.uint32)), n


def test_fp32_fold_thread_split_is_invisible():
    g = torch.Generator().manual_seed(3)
    a = torch.randn(9_000_001, generator=g).numpy()
    b = torch.randn(9_000_001, generator=g).numpy()
    one = a.copy(); oracle.fold2(one, b, F32, OP_SUM, threads=1)
    ref_split = a.copy(); oracle.fold2(ref_split, b, F32, OP_SUM, threads=0)
    many = a.copy(); oracle.fold2(many, b, F32, OP_SUM, threads=5)
    assert np.array_equal(one, ref_split) and np.array_equal(one, many)


def test_fp32_scale_and_fused_match_torch():
    g = torch.Generator().manual_seed(5)
    for n in SIZES:
        a = torch.randn(n, generator=g)
        b = torch.randn(n, generator=g)
        for s in (0.5, 0.25, 1.0 / 3.0, 1.0 / 7.0, 0.125):
            sf = float(np.float32(s))
            buf = a.numpy().copy()
            oracle.scale(buf, F32, sf)
            assert np.array_equal(buf, (a * torch.tensor(sf)).numpy())
            dst = a.numpy().copy()
            oracle.fold2_scale(dst, b.numpy(), F32, sf)
            want = ((a + b) * torch.tensor(sf)).numpy()  # two roundings, no FMA
            assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))


def test_fused_is_not_an_fma():
    # (a+b) must be rounded before the multiply: pick a, b whose exact sum needs
    # more than 24 bits so an FMA-style evaluation would differ.
    a = np.array([1.0], dtype=np.float32)
    b = np.array([2.0 ** -24], dtype=np.float32)
    s = float(np.float32(3.0))
    dst = a.copy()
    oracle.fold2_scale(dst, b, F32, s)
    assert dst[0] == np.float32(np.float32(a[0] + b[0]) * np.float32(s)) == np.float32(3.0)


def test_reference_known_answers_fp32():
    # tests/test_local_kernels.py:67-73,:133-139,:167-173,:205-211,:228-233,:287-294
    a = np.array([1, 2, 3], dtype=np.float32); b = np.array([4, 5, 6], dtype=np.float32)
    d = a.copy(); oracle.fold2(d, b, F32, OP_SUM); assert d.tolist() == [5, 7, 9]
    a = np.array([1, 5, 3], dtype=np.float32)
    d = a.copy(); oracle.fold2(d, b, F32, OP_MIN); assert d.tolist() == [1, 5, 3]
    b2 = np.array([4, 2, 6], dtype=np.float32)
    d = a.copy(); oracle.fold2(d, b2, F32, OP_MIN); assert d.tolist() == [1, 2, 3]
    d = a.copy(); oracle.fold2(d, b2, F32, OP_MAX); assert d.tolist() == [4, 5, 6]
    d = np.array([2, 3, 4], dtype=np.float32)
    oracle.fold2(d, np.array([5, 6, 7], dtype=np.float32), F32, OP_PRODUCT); assert d.tolist() == [10, 18, 28]
    d = np.array([2, 4, 6], dtype=np.float32); oracle.scale(d, F32, 0.5); assert d.tolist() == [1, 2, 3]
    d = np.array([1, 3, 5], dtype=np.float32)
    oracle.fold2_scale(d, np.array([3, 5, 7], dtype=np.float32), F32, 0.5); assert d.tolist() == [2, 4, 6]
    for ws in (2, 3, 4, 8):  # :243-249 scale by 1/ws gives ones within 1e-5
        d = np.full(256, float(ws), dtype=np.float32)
        oracle.scale(d, F32, float(np.float32(1.0 / ws)))
        assert np.allclose(d, 1.0, rtol=1e-5, atol=1e-5)


def test_unsupported_op_is_an_error():
    d = np.zeros(4, dtype=np.float32)
    assert oracle.fold2(d, d.copy(), F32, 5) == oracle.ERR_OP  # BAND
    assert oracle.fold2(d, d.copy(), F32, 8) == oracle.ERR_OP  # PREMUL_SUM


@pytest.mark.parametrize("dt,tdt", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("op", [OP_SUM, OP_PRODUCT, OP_MIN, OP_MAX])
def test_half_fold_all_values_times_partners(dt, tdt, op):
    """Every 16-bit encoding against 64 partners: widen, fp32 op, one RNE
    narrow == torch's own half arithmetic (computed in fp32 and rounded)."""
    rng = np.random.default_rng(op * 31 + dt)
    allbits = np.arange(65536, dtype=np.uint16)
    f = torch.from_numpy(allbits.view(np.int16)).view(tdt)
    keep = torch.isfinite(f.float())
    f = f[keep]
    for _ in range(64):
        partner = f[torch.from_numpy(rng.permutation(f.numel()))]
        want32 = TORCH_OPS[op](f.float(), partner.float())
        want = _bits(want32.to(tdt))
        dst = _bits(f).copy()
        assert oracle.fold2(dst, _bits(partner).copy(), dt, op) == oracle.OK
        nan = torch.isnan(want32).numpy()
        # inf-inf / 0*inf NaNs are outside every parity gate
        assert np.array_equal(dst[~nan], want[~nan])


@pytest.mark.parametrize("dt,tdt", [(F16, torch.float16), (BF16, torch.bfloat16)])
def test_half_native_add_equals_fp32_accumulate(dt, tdt):
    """The innocuous-double-rounding theorem the fold relies on: T(a)+T(b) done
    natively in T equals fp32 add followed by RNE to T."""
    g = torch.Generator().manual_seed(99)
    a = (torch.randn(400_000, generator=g) * 3).to(tdt)
    b = (torch.randn(400_000, generator=g) * 0.01).to(tdt)
    dst = _bits(a).copy()
    oracle.fold2(dst, _bits(b).copy(), dt, OP_SUM)
    assert np.array_equal(dst, _bits(a + b))


@pytest.mark.parametrize("dt,tdt", [(F16, torch.float16), (BF16, torch.bfloat16)])
def test_half_scale_and_fused(dt, tdt):
    g = torch.Generator().manual_seed(17)
    a = torch.randn(100_003, generator=g).to(tdt)
    b = torch.randn(100_003, generator=g).to(tdt)
    for s in (0.5, 0.25, 1.0 / 3.0):
        sf = float(np.float32(s))
        buf = _bits(a).copy(); oracle.scale(buf, dt, sf)
        assert np.array_equal(buf, _bits((a.float() * torch.tensor(sf)).to(tdt)))
        dst = _bits(a).copy(); oracle.fold2_scale(dst, _bits(b).copy(), dt, sf)
        assert np.array_equal(dst, _bits(((a.float() + b.float()) * torch.tensor(sf)).to(tdt)))
    # reference known answers (tests/test_local_kernels.py:103-119,:260-266,:307-313)
    x = _bits(torch.tensor([1.0, 3.0, 5.0], dtype=tdt)).copy()
    oracle.fold2_scale(x, _bits(torch.tensor([3.0, 5.0, 7.0], dtype=tdt)).copy(), dt, 0.5)
    assert np.array_equal(x, _bits(torch.tensor([2.0, 4.0, 6.0], dtype=tdt)))


def test_integral_known_answers():
    # tests/test_local_kernels.py:121-127 (int64 add), :268-281 (int64 x 1/3, bool x 0.5),
    # :315-337 (int64/int32/bool AVG of two ranks)
    for size in (1, 3, 7, 13):
        a = np.arange(size, dtype=np.int64); b = np.full(size, 3, dtype=np.int64)
        d = a.copy(); oracle.fold2(d, b, I64, OP_SUM); assert np.array_equal(d, a + b)
        exp = np.arange(1, size + 1, dtype=np.int64); v = exp * 3
        oracle.scale(v, I64, float(np.float32(1.0 / 3.0)))
        assert np.array_equal(v, exp)
    v = np.array([1, 0, 1], dtype=np.uint8); oracle.scale(v, BOOL, 0.5); assert v.tolist() == [0, 0, 0]
    for dt, npdt in ((I64, np.int64), (I32, np.int32)):
        a = np.array([1, 3, 5, 7, 9], dtype=npdt); b = np.array([3, 5, 7, 9, 11], dtype=npdt)
        oracle.fold2(a, b, dt, OP_SUM); oracle.scale(a, dt, 0.5, round_i32=True)
        assert a.tolist() == [2, 4, 6, 8, 10]
    a = np.array([1, 1, 0], dtype=np.uint8); b = np.array([1, 0, 1], dtype=np.uint8)
    oracle.fold2(a, b, BOOL, OP_SUM); oracle.scale(a, BOOL, 0.5)
    assert a.tolist() == [1, 0, 0]


def test_integral_folds_match_numpy():
    rng = np.random.default_rng(2)
    for dt, npdt in ((I32, np.int32), (I64, np.int64), (BOOL, np.uint8)):
        hi = 2 if dt == BOOL else 1000
        a = rng.integers(0, hi, 10_001).astype(npdt); b = rng.integers(0, hi, 10_001).astype(npdt)
        for op, f in ((OP_SUM, np.add), (OP_PRODUCT, np.multiply), (OP_MIN, np.minimum), (OP_MAX, np.maximum)):
            d = a.copy(); oracle.fold2(d, b, dt, op)
            assert np.array_equal(d, f(a, b).astype(npdt))
    # int32 scale: round half away from zero on the GPU rule, truncation on the CPU rule
    v = np.array([5, -5, 7, -7, 1], dtype=np.int32)
    r = v.copy(); oracle.scale(r, I32, 0.5, round_i32=True); assert r.tolist() == [3, -3, 4, -4, 1]
    t = v.copy(); oracle.scale(t, I32, 0.5, round_i32=False); assert t.tolist() == [2, -2, 3, -3, 0]
