"""MCCLConfig / init behave like the reference's config API: the reference's own
test file (tests/test_config_profiles.py:10-36) restated against mccl_amd, plus
the defaults, env mapping and validation read from mccl/config.py:23-172."""
import os

import pytest

import mccl_amd
from mccl_amd.config import MCCLConfig, _coerce


@pytest.fixture(autouse=True)
def clean_env(monkeypatch):
    for k in list(os.environ):
        if k.startswith("MCCL_"):
            monkeypatch.delenv(k, raising=False)
    yield


def test_for_world_size_invariant():
    for ws in (4, 8, 16):
        cfg = MCCLConfig.for_world_size(ws)
        assert cfg.ring_algo == "auto"
        assert cfg.collective_concurrency == 1
        assert cfg.pipeline_depth == 1
        assert cfg.port_base == 20100
        assert cfg.fast_math is True
        assert cfg.unified_collective is True
        assert cfg.demux_inflight_budget_bytes == 1 * 1024 * 1024 * 1024
        assert cfg.ddp_bucket_mb == 25


def test_apply_to_env_only_if_unset(monkeypatch):
    monkeypatch.delenv("MCCL_RING_ALGO", raising=False)
    monkeypatch.setenv("MCCL_COLLECTIVE_CONCURRENCY", "3")
    cfg = MCCLConfig.for_world_size(8)
    applied = cfg.apply_to_env(only_if_unset=True)
    assert os.environ.get("MCCL_RING_ALGO") is None  # "auto" skipped
    assert os.environ.get("MCCL_COLLECTIVE_CONCURRENCY") == "3"
    assert "MCCL_COLLECTIVE_CONCURRENCY" not in applied


def test_perf_mode():
    cfg = MCCLConfig.for_world_size(8, mode="perf")
    assert cfg.ring_algo == "chunked"
    assert cfg.collective_concurrency == 3 and cfg.pipeline_depth == 3
    assert MCCLConfig.for_world_size(2, link_profile="thunderbolt").link_profile == "thunderbolt"


def test_defaults_table():
    c = MCCLConfig()
    want = dict(transport="auto", listen_addr="auto", port_base=20100, ifname="", chunk_bytes=16 << 20,
                small_msg_threshold=262144, connect_timeout_ms=30000, transport_crc=False, fast_math=True,
                gpu_threshold=4096, shader_path="", overlap_comm=True, ring_algo="auto", ring_pipeline=True,
                pipeline_depth=1, collective_concurrency=1, max_collective_concurrency=8,
                demux_park_bytes=512 << 20, demux_inflight_budget_bytes=1 << 30, credit_min_chunk=1 << 20,
                fp32_cpu_reduce=False, cpu_write_sync="auto", event_sync=True, link_profile="",
                unified_collective=True, compression="none", topk_ratio=0.01, watchdog_timeout_ms=300000,
                heartbeat_interval_ms=5000, max_queue_depth=1024, log_level="WARN", ddp_bucket_mb=25)
    assert c.to_dict() == want
    assert len(c._ENV_MAP) == 31 and "MCCL_TOPK_RATIO" in c._ENV_MAP and "ddp_bucket_mb" not in c._ENV_MAP.values()
    assert "_ENV_MAP" not in repr(c)
    assert str(c).startswith("MCCLConfig(\n  transport='auto',\n") and str(c).endswith(")")


@pytest.mark.parametrize("kw,msg", [
    (dict(transport="udp"), "transport must be one of ['auto', 'rdma', 'tcp'], got 'udp'"),
    (dict(compression="zstd"), "compression must be one of ['fp16', 'none', 'topk'], got 'zstd'"),
    (dict(ring_algo="tree"), "ring_algo must be one of"),
    (dict(pipeline_depth=0), "pipeline_depth must be in [1, 8], got 0"),
    (dict(collective_concurrency=9), "collective_concurrency must be in [1, 8], got 9"),
    (dict(max_collective_concurrency=17), "max_collective_concurrency must be in [1, 16], got 17"),
    (dict(cpu_write_sync="half"), "cpu_write_sync must be one of"),
    (dict(log_level="LOUD"), "log_level must be one of"),
    (dict(port_base=0), "port_base must be in [1, 65535], got 0"),
    (dict(gpu_threshold=-1), "gpu_threshold must be >= 0, got -1"),
    (dict(topk_ratio=0.0), "topk_ratio must be in (0.0, 1.0], got 0.0"),
    (dict(topk_ratio=1.5), "topk_ratio must be in (0.0, 1.0], got 1.5"),
    (dict(max_queue_depth=0), "max_queue_depth must be >= 1, got 0"),
    (dict(chunk_bytes=0), "chunk_bytes must be >= 1, got 0"),
    (dict(watchdog_timeout_ms=0), "watchdog_timeout_ms must be >= 1, got 0"),
])
def test_validation(kw, msg):
    with pytest.raises(ValueError) as e:
        MCCLConfig(**kw)
    assert msg in str(e.value)


def test_log_level_is_case_insensitive_and_ratio_one_is_valid():
    assert MCCLConfig(log_level="debug").log_level == "debug"
    assert MCCLConfig(topk_ratio=1.0).topk_ratio == 1.0


def test_env_round_trip(monkeypatch):
    cfg = MCCLConfig(compression="topk", topk_ratio=0.05, fast_math=False, gpu_threshold=8192, ifname="en0")
    out = cfg.to_env()
    assert out["MCCL_COMPRESSION"] == "topk" and out["MCCL_TOPK_RATIO"] == "0.05"
    assert out["MCCL_FAST_MATH"] == "0" and out["MCCL_EVENT_SYNC"] == "1" and out["MCCL_IFNAME"] == "en0"
    for skipped in ("MCCL_TRANSPORT", "MCCL_LISTEN_ADDR", "MCCL_RING_ALGO", "MCCL_SHADER_PATH", "MCCL_LINK_PROFILE"):
        assert skipped not in out and skipped not in os.environ
    back = MCCLConfig.from_env()
    assert back.to_dict() == cfg.to_dict()
    monkeypatch.setenv("MCCL_TRANSPORT_CRC", "no")
    monkeypatch.setenv("MCCL_OVERLAP_COMM", "yes")
    monkeypatch.setenv("MCCL_PORT_BASE", "31000")
    c2 = MCCLConfig.from_env()
    assert c2.transport_crc is False and c2.overlap_comm is True and c2.port_base == 31000
    assert _coerce("FALSE", bool) is False and _coerce("1", "bool") is True and _coerce("2.5", float) == 2.5


def test_from_dict_ignores_unknown_keys():
    c = MCCLConfig.from_dict({"compression": "topk", "topk_ratio": 0.05, "not_a_field": 1})
    assert c.compression == "topk" and c.topk_ratio == 0.05


def test_init_precedence(monkeypatch):
    assert mccl_amd.get_config() is None or isinstance(mccl_amd.get_config(), MCCLConfig)
    c = mccl_amd.init(compression="topk", topk_ratio=0.02)
    assert mccl_amd.get_config() is c and os.environ["MCCL_COMPRESSION"] == "topk"
    c = mccl_amd.init({"compression": "fp16"}, fast_math=False)
    assert c.compression == "fp16" and c.fast_math is False
    monkeypatch.setenv("MCCL_GPU_THRESHOLD", "123")
    assert mccl_amd.init().gpu_threshold == 123
    cfg = MCCLConfig()
    assert mccl_amd.init(cfg, log_level="INFO") is cfg and os.environ["MCCL_LOG_LEVEL"] == "INFO"
    assert mccl_amd.__version__ == "0.5.0"
