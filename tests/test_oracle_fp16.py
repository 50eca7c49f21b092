"""Pins the oracle's FP16 compressor (csrc/compression/FP16Compression.cpp).

Three independent checks:
  * the reference's own C++ (portable branch, compiled from its sources) on
    every input whose half result is not subnormal -- the one place the two
    branches of the reference differ;
  * numpy's float16 casts, the proxy the reference's unit tests use
    (tests/test_compression.py:14-40), everywhere except NaN payloads;
  * the reference's end-to-end vectors (tests/test_compression_e2e.py:20-30).
"""
import numpy as np
import pytest

import oracle

needs_ref = pytest.mark.skipif(not oracle.RefCompressor.available(), reason="compiled reference not built")


def _boundary_inputs() -> np.ndarray:
    """Every finite half, the midpoints between neighbours, and the fp32
    values either side of each; NaNs of several payloads; infinities."""
    h = np.arange(0x7C00, dtype=np.uint16)
    v = oracle.f16_bits_to_f32(h).astype(np.float64)
    nxt = np.append(v[1:], 65536.0)
    mid = ((v + nxt) / 2).astype(np.float32)
    parts = [v.astype(np.float32), mid]
    for base in list(parts):
        parts.append(np.nextafter(base, np.float32(np.inf)))
        parts.append(np.nextafter(base, np.float32(-np.inf)))
    nan_bits = np.array([0x7FC00000, 0x7F800001, 0x7FA55555, 0x7FFFFFFF, 0x7F802000, 0x7F801FFF], dtype=np.uint32)
    parts.append(nan_bits.view(np.float32))
    parts.append(np.array([np.inf, 65519.99, 65520.0, 1e9, 1e-10, 2.0 ** -25, 2.0 ** -26], dtype=np.float32))
    x = np.concatenate(parts).astype(np.float32)
    return np.concatenate([x, (x.view(np.uint32) ^ np.uint32(0x80000000)).view(np.float32)])


@needs_ref
def test_compress_matches_reference_outside_subnormal_range():
    x = _boundary_inputs()
    got = oracle.fp16_compress(x).view(np.uint16)
    ref = oracle.RefCompressor(mode=1).compress(x).view(np.uint16)
    sub = (got & 0x7FFF) <= 0x0400  # zero, subnormal, or rounded up to the smallest normal
    # the portable branch flushes: exp <= 0 -> signed zero
    flush = np.abs(x) < np.float32(2.0 ** -14)
    assert np.array_equal(got[~flush], ref[~flush])
    assert np.all((ref[flush] & 0x7FFF) == 0)
    assert np.array_equal(got[flush] & 0x8000, ref[flush] & 0x8000)
    assert np.all(sub[flush])


def test_compress_matches_numpy_float16():
    x = _boundary_inputs()
    x = x[~np.isnan(x)]
    got = oracle.fp16_compress(x).view(np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_nan_keeps_sign_payload_top_bits_and_quiet_bit():
    bits = np.array([0x7F800001, 0xFF800001, 0x7FA55555, 0x7FFFFFFF, 0xFFC00000, 0x7F802000], dtype=np.uint32)
    got = oracle.fp16_compress(bits.view(np.float32)).view(np.uint16)
    want = ((bits >> 16) & 0x8000) | 0x7C00 | ((bits & 0x7FFFFF) >> 13) | 0x200
    assert np.array_equal(got, want.astype(np.uint16))


@needs_ref
def test_decompress_matches_reference_on_normals_inf_and_quiet_nan():
    h = np.arange(65536, dtype=np.uint16)
    e = (h >> 10) & 0x1F
    m = h & 0x3FF
    keep = ~((e == 0) & (m != 0)) & ~((e == 31) & (m != 0) & ((m & 0x200) == 0))
    hk = h[keep]
    got, rc = oracle.fp16_decompress(hk.view(np.uint8), hk.size)
    assert rc == 0
    ref, rrc = oracle.RefCompressor(mode=1).decompress(hk.view(np.uint8), hk.size)
    assert rrc == 0
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_decompress_matches_numpy_float16():
    h = np.arange(65536, dtype=np.uint16)
    got, rc = oracle.fp16_decompress(h.view(np.uint8), h.size)
    assert rc == 0
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(got[nan]))


@pytest.mark.parametrize("n", [1024, 70_001])
@pytest.mark.parametrize("ws", [2, 3])
def test_reference_e2e_vectors_are_lossless(n, ws):
    # tests/test_compression_e2e.py:20-30: rank r holds (r+1)*0.5; the SUM of the
    # round-tripped contributions equals the exact sum.
    total = np.zeros(n, dtype=np.float32)
    for r in range(ws):
        x = np.full(n, (r + 1) * 0.5, dtype=np.float32)
        wire = oracle.fp16_compress(x)
        assert wire.nbytes == n * 2
        back, rc = oracle.fp16_decompress(wire, n)
        assert rc == 0
        total += back
    assert np.all(total == 0.5 * sum(r + 1 for r in range(ws)))


def test_half_passthrough_and_size_checks():
    h = np.array([0x3C00, 0x0001, 0x7E00, 0xFBFF], dtype=np.uint16)
    wire = oracle.fp16_compress(h, dtype=oracle.F16)
    assert np.array_equal(wire.view(np.uint16), h)
    back, rc = oracle.fp16_decompress(wire, h.size, dtype=oracle.F16)
    assert rc == 0 and np.array_equal(back, h)
    x = np.ones(8, dtype=np.float32)
    assert oracle.fp16_compress(x, capacity=15) == oracle.ERR_CAPACITY
    assert oracle.fp16_compress(h, dtype=oracle.F16, capacity=7) == oracle.ERR_CAPACITY
    assert oracle.fp16_decompress(np.zeros(14, np.uint8), 8)[1] == oracle.ERR_SIZE
    assert oracle.fp16_decompress(np.zeros(6, np.uint8), 4, dtype=oracle.F16)[1] == oracle.ERR_SIZE
    assert oracle.fp16_compress(np.zeros(4, np.int32), dtype=oracle.I32) == oracle.ERR_DTYPE


@needs_ref
def test_reference_errors_agree():
    ref = oracle.RefCompressor(mode=1)
    x = np.ones(8, dtype=np.float32)
    assert ref.compress(x, capacity=15) is None
    assert ref.decompress(np.zeros(14, np.uint8), 8)[1] == -1
    assert ref.max_compressed_size(4096) == 4096
