"""GPU parity of the FP16 compressor's casts with the oracle
(csrc/compression/FP16Compression.cpp:16-165): bit-exact over every half
encoding, every rounding boundary, NaN payloads, ragged and misaligned sizes;
the compressor class on top, with the reference's error messages and its
end-to-end vectors (tests/test_compression_e2e.py:20-30)."""
import numpy as np
import pytest
import torch
import torch.distributed  # noqa: F401

import oracle
from mccl_amd import hip_ops
from tests._gpu_util import DEV, to_dev, to_np
from tests.test_oracle_fp16 import _boundary_inputs

pytestmark = pytest.mark.gpu


def _narrow_ok(x: np.ndarray, pad: int = 0):
    src = to_dev(x, oracle.F32, pad_front=pad)
    got = to_np(hip_ops.cast_f32_to_f16(src), oracle.F16)
    want = oracle.fp16_compress(x).view(np.uint16)
    assert np.array_equal(got, want)


def test_narrow_every_boundary():
    _narrow_ok(_boundary_inputs())


def test_widen_every_encoding():
    h = np.arange(65536, dtype=np.uint16)
    got = to_np(hip_ops.cast_f16_to_f32(to_dev(h, oracle.F16)), oracle.F32)
    want, rc = oracle.fp16_decompress(h.view(np.uint8), h.size)
    assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 63, 2047, 2049, 70_001, 1 << 20, (1 << 22) + 5])
@pytest.mark.parametrize("pad", [0, 1, 3])
def test_ragged_and_misaligned(n, pad):
    rng = np.random.default_rng(n * 7 + pad)
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-9, 5, n)).astype(np.float32)
    _narrow_ok(x, pad)
    h = rng.integers(0, 65536, n).astype(np.uint16)
    got = to_np(hip_ops.cast_f16_to_f32(to_dev(h, oracle.F16, pad_front=pad)), oracle.F32)
    want, _ = oracle.fp16_decompress(h.view(np.uint8), n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_all_f32_exponents_random_mantissas():
    rng = np.random.default_rng(11)
    u = rng.integers(0, 1 << 32, 1 << 21, dtype=np.uint64).astype(np.uint32)
    _narrow_ok(u.view(np.float32))


def test_full_size_round_trip_properties():
    # 96,510,024 elements: narrowing is idempotent through a round trip, and
    # values already representable in half survive exactly.
    n = 96_510_024
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(n, device=DEV, generator=g)
    h = hip_ops.cast_f32_to_f16(x)
    back = hip_ops.cast_f16_to_f32(h)
    h2 = hip_ops.cast_f32_to_f16(back)
    assert torch.equal(h.view(torch.int16), h2.view(torch.int16))
    assert torch.equal(h, x.to(torch.float16))  # no NaNs here: torch's cast is the same RNE
    del back, h2
    sl = slice(n - 100_003, n)
    want = oracle.fp16_compress(x[sl].cpu().numpy()).view(np.uint16)
    assert np.array_equal(to_np(h[sl], oracle.F16), want)


class TestCompressor:
    @pytest.fixture(scope="class")
    def C(self):
        from mccl_amd import _C
        return _C

    def test_round_trip_and_payload(self, C):
        c = C.make_compressor(C.CompressionMode.FP16, 0.0)
        rng = np.random.default_rng(5)
        x = rng.standard_normal(70_001).astype(np.float32)
        wire = c.compress(torch.from_numpy(x).to(DEV))
        assert wire.dtype == torch.uint8 and wire.numel() == x.size * 2
        assert np.array_equal(wire.cpu().numpy(), oracle.fp16_compress(x))
        back = c.decompress(wire, x.size)
        want, _ = oracle.fp16_decompress(wire.cpu().numpy(), x.size)
        assert np.array_equal(back.cpu().numpy().view(np.uint32), want.view(np.uint32))

    @pytest.mark.parametrize("n", [1024, 70_001])
    def test_reference_e2e_vectors(self, C, n):
        c = C.FP16Compressor()
        ws = 3
        total = torch.zeros(n, device=DEV)
        for r in range(ws):
            t = torch.full((n,), (r + 1) * 0.5, device=DEV)
            total += c.decompress(c.compress(t), n)
        assert int((total != 0.5 * sum(r + 1 for r in range(ws))).sum()) == 0

    def test_half_passthrough(self, C):
        c = C.FP16Compressor()
        h = torch.randn(4097, device=DEV).to(torch.float16)
        wire = c.compress(h)
        assert wire.numel() == h.numel() * 2 and torch.equal(wire.view(torch.float16), h)
        assert torch.equal(c.decompress(wire, h.numel(), dtype=torch.float16), h)

    def test_errors(self, C):
        c = C.FP16Compressor()
        x = torch.ones(8, device=DEV)
        with pytest.raises(RuntimeError, match="FP16 compress: buffer too small"):
            c.compress(x, capacity=15)
        with pytest.raises(RuntimeError, match="FP16 compress: buffer too small"):
            c.compress(x.to(torch.float16), capacity=15)
        with pytest.raises(RuntimeError, match="FP16 compression only supports float32 input"):
            c.compress(x.to(torch.bfloat16))
        wire = c.compress(x)
        with pytest.raises(RuntimeError, match="FP16 decompress: compressed size mismatch"):
            c.decompress(wire, 7)
        with pytest.raises(RuntimeError, match="FP16 decompress: size mismatch"):
            c.decompress(wire, 7, dtype=torch.float16)
        with pytest.raises(RuntimeError, match="FP16 decompression only supports float32 output"):
            c.decompress(wire, 4, dtype=torch.bfloat16)


needs_ref = pytest.mark.skipif(not oracle.RefCompressor.available(), reason="compiled reference not built")


@needs_ref
def test_portable_mode_is_the_compiled_reference_bit_for_bit():
    # "fp16_portable" follows the branch of FP16Compression.cpp that a non-ARM build runs
    # (:38-73, :96-111): checked against that very code, compiled from the reference's sources,
    # over every half encoding, every rounding boundary and random bit patterns.
    ref = oracle.RefCompressor(mode=1)
    hip_ops.set_tuning("fp16_portable", 1)
    try:
        h = np.arange(65536, dtype=np.uint16)
        got = to_np(hip_ops.cast_f16_to_f32(to_dev(h, oracle.F16)), oracle.F32)
        want, rc = ref.decompress(h.view(np.uint8), h.size)
        assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
        rng = np.random.default_rng(5)
        rand = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
        tiny = (rng.standard_normal(1 << 16) * 6e-5).astype(np.float32)          # around the smallest normal half
        for x in (_boundary_inputs(), rand, tiny):
            got = to_np(hip_ops.cast_f32_to_f16(to_dev(x, oracle.F32, pad_front=1)), oracle.F16)
            want = ref.compress(x).view(np.uint16)
            assert np.array_equal(got, want)
        # the two modes differ exactly where the portable branch says they do
        sub = np.array([1e-7, -3e-6, 6.0e-8, 6.2e-5, 6.1e-5], np.float32)        # 2^-14 = 6.1035e-5
        flushed = to_np(hip_ops.cast_f32_to_f16(to_dev(sub, oracle.F32)), oracle.F16)
        hip_ops.set_tuning("fp16_portable", 0)
        kept = to_np(hip_ops.cast_f32_to_f16(to_dev(sub, oracle.F32)), oracle.F16)
        assert list(flushed & 0x7FFF) == [0, 0, 0, int(kept[3] & 0x7FFF), 0] and all(kept & 0x7FFF)
        assert list(flushed & 0x8000) == list(kept & 0x8000)
    finally:
        hip_ops.set_tuning("fp16_portable", 0)
