"""Helpers shared by the GPU parity tests: seeded inputs, numpy <-> device
round trips that preserve bit patterns, and oracle wrappers."""
import numpy as np
import torch

import oracle

DEV = "cuda:0"
TORCH_DT = {oracle.F32: torch.float32, oracle.F16: torch.float16, oracle.BF16: torch.bfloat16,
            oracle.I32: torch.int32, oracle.I64: torch.int64, oracle.BOOL: torch.bool, oracle.U8: torch.uint8}
NP_DT = {oracle.F32: np.float32, oracle.F16: np.uint16, oracle.BF16: np.uint16,
         oracle.I32: np.int32, oracle.I64: np.int64, oracle.BOOL: np.uint8, oracle.U8: np.uint8}


def to_dev(a: np.ndarray, dt: int, pad_front: int = 0) -> torch.Tensor:
    """numpy bits -> device tensor of dtype dt; pad_front shifts the start by
    that many elements (a view into a larger allocation) to break alignment."""
    if dt in (oracle.F16, oracle.BF16):
        t = torch.from_numpy(a.view(np.int16)).view(TORCH_DT[dt])
    elif dt == oracle.BOOL:
        t = torch.from_numpy(a).view(torch.bool)
    else:
        t = torch.from_numpy(a)
    if pad_front:
        big = torch.empty(t.numel() + pad_front + 64, dtype=t.dtype, device=DEV)
        view = big[pad_front:pad_front + t.numel()]
        view.copy_(t)
        return view
    return t.to(DEV)


def to_np(t: torch.Tensor, dt: int) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if dt in (oracle.F16, oracle.BF16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    if dt == oracle.BOOL:
        return t.view(torch.uint8).numpy().copy()
    return t.numpy().copy()


def bits(a: np.ndarray) -> np.ndarray:
    if a.dtype == np.float32:
        return a.view(np.uint32)
    return a


def rand_vals(rng, n, dt, sigma=1.0, specials=True):
    """Seeded values in the element type's bit representation."""
    x = (rng.standard_normal(n) * sigma).astype(np.float32)
    if specials and n >= 16:
        # denormals, zeros of both signs, large magnitudes, infinities
        sp = np.array([0.0, -0.0, 1e-40, -1e-40, 1e-45, 3e38, -3e38, np.inf, -np.inf,
                       65504.0, 65520.0, 6e-8, -6e-8, 1.0, -1.0, 0.5], dtype=np.float32)
        pos = rng.choice(n, size=sp.size, replace=False)
        x[pos] = sp
    if dt == oracle.F32:
        return x
    if dt == oracle.F16:
        return oracle.f32_to_f16_bits(x)
    return oracle.f32_to_bf16_bits(x)


def student_t(rng, n, ties=0.01, scale=1e-3):
    x = (rng.standard_normal(n) / np.sqrt(rng.chisquare(3, n) / 3) * scale).astype(np.float32)
    m = int(n * ties)
    if m:
        dst = rng.integers(0, n, m); src = rng.integers(0, n, m)
        sign = np.where(rng.random(m) < 0.5, -1.0, 1.0).astype(np.float32)
        x[dst] = x[src] * sign
    return x
