"""Pins the oracle's fp16/bf16 conversions against torch's CPU casts (an
independent implementation of c10::Half / c10::BFloat16) over every encoding
and every rounding boundary."""
import numpy as np
import torch

import oracle


def _t_f16_bits(x32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x32).to(torch.float16).view(torch.int16).numpy().view(np.uint16)


def _t_bf16_bits(x32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_f16_widen_all_encodings():
    bits = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.float16).float().numpy()
    got = oracle.f16_bits_to_f32(bits)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bf16_widen_all_encodings():
    bits = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = oracle.bf16_bits_to_f32(bits)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _finite(x):
    return x[np.isfinite(x) | np.isinf(x)]  # drops NaN only


def test_f16_narrow_every_boundary():
    # every finite half, its fp32 neighbours, and the exact midpoints between
    # adjacent halves (ties) with their fp32 neighbours
    h = np.arange(0x7C00, dtype=np.uint16)
    v = oracle.f16_bits_to_f32(h).astype(np.float64)
    nxt = oracle.f16_bits_to_f32((h + 1).astype(np.uint16)).astype(np.float64)
    nxt[-1] = 65536.0
    mid = ((v + nxt) / 2).astype(np.float32)  # exact: halves have 11 bits
    cands = [v.astype(np.float32), mid]
    for base in list(cands):
        cands.append(np.nextafter(base, np.float32(np.inf)))
        cands.append(np.nextafter(base, np.float32(-np.inf)))
    x = np.concatenate(cands + [np.array([65504, 65519.99, 65520, 65536, 1e6, np.inf, 2.0 ** -25,
                                         2.0 ** -24, 2.0 ** -26, 1e-10, 0.0], dtype=np.float32)])
    x = np.concatenate([x, -x]).astype(np.float32)
    assert np.array_equal(oracle.f32_to_f16_bits(x), _t_f16_bits(x))


def test_bf16_narrow_every_boundary():
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    u = (hi[:, None] | lows[None, :]).ravel().astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    assert np.array_equal(oracle.f32_to_bf16_bits(x), _t_bf16_bits(x))


def test_narrow_random_wide_range():
    rng = np.random.default_rng(7)
    u = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    assert np.array_equal(oracle.f32_to_f16_bits(x), _t_f16_bits(x))
    assert np.array_equal(oracle.f32_to_bf16_bits(x), _t_bf16_bits(x))


def test_nan_canonical_forms():
    nan = np.array([np.nan], dtype=np.float32)
    assert oracle.f32_to_bf16_bits(nan)[0] == 0x7FC0
    assert oracle.f32_to_f16_bits(nan)[0] & 0x7FFF == 0x7E00
