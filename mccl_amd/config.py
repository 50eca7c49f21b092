"""MCCLConfig: every MCCL tunable in one dataclass, exported to the native layer
through ``MCCL_*`` environment variables.

Drop-in for the reference's ``mccl.config.MCCLConfig`` (mccl/config.py:18-284):
same fields, defaults, validation, env names and helper methods.  The class is
generated from one table (field, type, default, env name) so that fields, env
mapping and coercion cannot drift apart.  On this build only ``compression``,
``topk_ratio``, ``event_sync`` and ``log_level`` reach native code; the transport
and engine fields are carried for API compatibility.
"""
from __future__ import annotations

import dataclasses
import os
from typing import Any, Callable, Dict, List, Optional, Tuple

_MiB = 1024 * 1024

# (field, type, default, env name or None)
_SPEC: List[Tuple[str, type, Any, Optional[str]]] = [
    # transport
    ("transport", str, "auto", "MCCL_TRANSPORT"),
    ("listen_addr", str, "auto", "MCCL_LISTEN_ADDR"),
    ("port_base", int, 20100, "MCCL_PORT_BASE"),
    ("ifname", str, "", "MCCL_IFNAME"),
    ("chunk_bytes", int, 16 * _MiB, "MCCL_CHUNK_BYTES"),
    ("small_msg_threshold", int, 262144, "MCCL_SMALL_MSG_THRESHOLD"),
    ("connect_timeout_ms", int, 30000, "MCCL_CONNECT_TIMEOUT_MS"),
    ("transport_crc", bool, False, "MCCL_TRANSPORT_CRC"),
    # compute
    ("fast_math", bool, True, "MCCL_FAST_MATH"),
    ("gpu_threshold", int, 4096, "MCCL_GPU_THRESHOLD"),
    ("shader_path", str, "", "MCCL_SHADER_PATH"),
    ("overlap_comm", bool, True, "MCCL_OVERLAP_COMM"),
    ("ring_algo", str, "auto", "MCCL_RING_ALGO"),
    ("ring_pipeline", bool, True, "MCCL_RING_PIPELINE"),
    ("pipeline_depth", int, 1, "MCCL_PIPELINE_DEPTH"),
    ("collective_concurrency", int, 1, "MCCL_COLLECTIVE_CONCURRENCY"),
    ("max_collective_concurrency", int, 8, "MCCL_MAX_COLLECTIVE_CONCURRENCY"),
    ("demux_park_bytes", int, 512 * _MiB, "MCCL_DEMUX_PARK_BYTES"),
    ("demux_inflight_budget_bytes", int, 1024 * _MiB, "MCCL_DEMUX_INFLIGHT_BUDGET_BYTES"),
    ("credit_min_chunk", int, _MiB, "MCCL_CREDIT_MIN_CHUNK"),
    ("fp32_cpu_reduce", bool, False, "MCCL_FP32_CPU_REDUCE"),
    ("cpu_write_sync", str, "auto", "MCCL_CPU_WRITE_SYNC"),
    ("event_sync", bool, True, "MCCL_EVENT_SYNC"),
    ("link_profile", str, "", "MCCL_LINK_PROFILE"),
    ("unified_collective", bool, True, "MCCL_UNIFIED_COLLECTIVE"),
    # compression
    ("compression", str, "none", "MCCL_COMPRESSION"),
    ("topk_ratio", float, 0.01, "MCCL_TOPK_RATIO"),
    # runtime
    ("watchdog_timeout_ms", int, 300000, "MCCL_WATCHDOG_TIMEOUT_MS"),
    ("heartbeat_interval_ms", int, 5000, "MCCL_HEARTBEAT_INTERVAL_MS"),
    ("max_queue_depth", int, 1024, "MCCL_MAX_QUEUE_DEPTH"),
    ("log_level", str, "WARN", "MCCL_LOG_LEVEL"),
    # integration hint, never exported
    ("ddp_bucket_mb", int, 25, None),
]

_TYPES: Dict[str, type] = {name: typ for name, typ, _, _ in _SPEC}
_FALSE_WORDS = ("0", "false", "FALSE", "no", "NO", "")


def _one_of(field: str, allowed: set, fold: Callable[[str], str] = lambda s: s):
    def rule(cfg) -> Optional[str]:
        value = getattr(cfg, field)
        if fold(value) not in allowed:
            return f"{field} must be one of {sorted(allowed)}, got {value!r}"
        return None
    return rule


def _in_range(field: str, lo: int, hi: int):
    def rule(cfg) -> Optional[str]:
        value = getattr(cfg, field)
        if not (lo <= value <= hi):
            return f"{field} must be in [{lo}, {hi}], got {value}"
        return None
    return rule


def _at_least(field: str, lo: int):
    def rule(cfg) -> Optional[str]:
        value = getattr(cfg, field)
        if value < lo:
            return f"{field} must be >= {lo}, got {value}"
        return None
    return rule


def _ratio(cfg) -> Optional[str]:
    if not (0.0 < cfg.topk_ratio <= 1.0):
        return f"topk_ratio must be in (0.0, 1.0], got {cfg.topk_ratio}"
    return None


# checked in this order; the first failing rule raises
_RULES = [
    _one_of("transport", {"auto", "tcp", "rdma"}),
    _one_of("compression", {"none", "fp16", "topk"}),
    _one_of("ring_algo", {"auto", "chunked", "basic", "ring", "plain"}),
    _in_range("pipeline_depth", 1, 8),
    _in_range("collective_concurrency", 1, 8),
    _in_range("max_collective_concurrency", 1, 16),
    _one_of("cpu_write_sync", {"auto", "none", "full"}),
    _one_of("log_level", {"TRACE", "DEBUG", "INFO", "WARN", "ERROR", "FATAL", "OFF"}, str.upper),
    _in_range("port_base", 1, 65535),
    _at_least("gpu_threshold", 0),
    _ratio,
    _at_least("max_queue_depth", 1),
    _at_least("chunk_bytes", 1),
    _at_least("watchdog_timeout_ms", 1),
]


def _coerce(raw: str, target_type: Any) -> Any:
    """Environment string -> field type (bools: anything but 0/false/no/empty)."""
    if target_type in (bool, "bool"):
        return raw not in _FALSE_WORDS
    if target_type in (int, "int"):
        return int(raw)
    if target_type in (float, "float"):
        return float(raw)
    return raw


def _env_text(value: Any) -> str:
    if isinstance(value, bool):
        return "1" if value else "0"
    return str(value)


class _Methods:
    """Behaviour of MCCLConfig; the fields are attached by make_dataclass below."""

    def __post_init__(self) -> None:
        self._ENV_MAP = {env: name for name, _, _, env in _SPEC if env}
        self._validate()

    def _validate(self) -> None:
        for rule in _RULES:
            problem = rule(self)
            if problem:
                raise ValueError(problem)

    @classmethod
    def from_env(cls) -> "MCCLConfig":
        """Defaults overridden by every MCCL_* variable that is set."""
        cfg = cls()
        for env, name in cfg._ENV_MAP.items():
            raw = os.environ.get(env)
            if raw is not None:
                setattr(cfg, name, _coerce(raw, _TYPES[name]))
        return cfg

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MCCLConfig":
        """From a plain mapping (parsed YAML / JSON); unknown keys are ignored."""
        return cls(**{k: v for k, v in d.items() if k in _TYPES})

    def _export(self, skip_if_set: bool) -> Dict[str, str]:
        written: Dict[str, str] = {}
        for env, name in self._ENV_MAP.items():
            if skip_if_set and os.environ.get(env) is not None:
                continue
            text = _env_text(getattr(self, name))
            # "" and "auto" mean "built-in default": leave the environment alone
            if text and text != "auto":
                os.environ[env] = text
                written[env] = text
        return written

    def to_env(self) -> Dict[str, str]:
        """Writes the values into os.environ and returns what was written."""
        return self._export(skip_if_set=False)

    def apply_to_env(self, only_if_unset: bool = True) -> Dict[str, str]:
        """Like to_env, but variables the user already set are kept."""
        return self._export(skip_if_set=only_if_unset)

    def to_dict(self) -> Dict[str, Any]:
        return {name: getattr(self, name) for name in _TYPES}

    @classmethod
    def for_world_size(cls, world_size: int, *, mode: str = "lab", link_profile: str = "") -> "MCCLConfig":
        """Defaults do not depend on the world size; mode="perf" selects the
        chunked ring with three collectives in flight and depth-3 pipelines."""
        del world_size
        cfg = cls()
        if link_profile:
            cfg.link_profile = link_profile
        if mode == "perf":
            cfg.ring_algo = "chunked"
            cfg.collective_concurrency = 3
            cfg.pipeline_depth = 3
        return cfg

    def __str__(self) -> str:
        body = "".join(f"  {k}={v!r},\n" for k, v in self.to_dict().items())
        return "MCCLConfig(\n" + body + ")"


MCCLConfig = dataclasses.make_dataclass(
    "MCCLConfig",
    [(name, typ, dataclasses.field(default=default)) for name, typ, default, _ in _SPEC]
    + [("_ENV_MAP", dict, dataclasses.field(default_factory=dict, repr=False, init=False))],
    bases=(_Methods,),
)
MCCLConfig.__module__ = __name__
MCCLConfig.__doc__ = "All MCCL tunables in one place."
