"""The torch extension mirrors the reference's pybind surface for this path
(csrc/backend/Registration.cpp:220-312) and its host-side error behaviour;
everything here runs without a GPU."""
import pytest
import torch
import torch.distributed  # noqa: F401  (registers c10d base types)


@pytest.fixture(scope="module")
def C():
    from mccl_amd import _C
    return _C


def test_names_and_constants(C):
    assert C.__version__ == "0.5.0" and C.__protocol_version__ == 5
    for name in ("_metal_accumulate_chunk", "_metal_elementwise_min", "_metal_elementwise_max",
                 "_metal_elementwise_product", "_metal_scale_inplace", "_metal_accumulate_and_scale",
                 "CompressionMode", "MCCLOptions", "TopKCompressor", "make_compressor"):
        assert hasattr(C, name), name
    assert int(C.CompressionMode.NONE) == 0 and int(C.CompressionMode.FP16) == 1 and int(C.CompressionMode.TOPK) == 2


def test_options_defaults(C):
    o = C.MCCLOptions()
    assert (o.transport, o.listen_addr, o.port_base, o.chunk_bytes) == ("auto", "0.0.0.0", 20100, 16 << 20)
    assert (o.small_msg_threshold, o.transport_crc, o.fast_math, o.gpu_threshold) == (262144, False, True, 4096)
    assert (o.overlap_comm, o.max_queue_depth, o.topk_ratio) == (True, 1024, 0.01)
    assert o.compression == C.CompressionMode.NONE
    o.compression = C.CompressionMode.TOPK
    o.topk_ratio = 0.05
    assert o.compression == C.CompressionMode.TOPK and o.topk_ratio == 0.05
    assert isinstance(o, torch._C._distributed_c10d.Backend.Options)


def test_make_compressor_rules(C):
    # csrc/compression/Compression.cpp:8-20, TopKCompression.cpp:12-15,:154-158
    assert C.make_compressor(C.CompressionMode.NONE, 0.5) is None
    c = C.make_compressor(C.CompressionMode.TOPK, 0.0)          # param <= 0 -> 0.01
    assert c.name() == "topk" and c.max_compressed_size(6_553_600 * 4) == 4 + 8 * 65_537
    assert C.make_compressor(C.CompressionMode.TOPK, 0.1).max_compressed_size(4000) == 4 + 8 * 101
    h = C.make_compressor(C.CompressionMode.FP16, 0.0)          # FP16Compression.cpp:165-168
    assert isinstance(h, C.FP16Compressor) and h.name() == "fp16" and h.max_compressed_size(4096) == 4096
    for bad in (0.0, -1.0, 1.5):
        with pytest.raises(RuntimeError, match=r"k_ratio must be in \(0, 1\]"):
            C.TopKCompressor(bad)
    assert c.error_feedback_buffer_count() == 0


def test_cpu_tensors_are_rejected_loudly(C):
    if torch.cuda.is_available():
        pytest.skip("host-only check")
    with pytest.raises(RuntimeError, match=r"\[MCCL\]"):
        C._metal_accumulate_chunk(torch.zeros(3), torch.zeros(3))


def test_compressor_from_env(monkeypatch):
    import mccl_amd
    monkeypatch.delenv("MCCL_COMPRESSION", raising=False)
    assert mccl_amd.compressor_from_env() is None
    mccl_amd.init(compression="topk", topk_ratio=0.1)
    c = mccl_amd.compressor_from_env()
    assert c.name() == "topk" and c.max_compressed_size(4000) == 4 + 8 * 101
    monkeypatch.setenv("MCCL_COMPRESSION", "none")
    assert mccl_amd.compressor_from_env() is None
