"""mccl_amd -- MI355X-native implementation of MCCL's per-rank data-parallel
compute path (chunk fold, AVG scale, top-k compression with error feedback,
decompress / accumulate), behind MCCL's own config and local-kernel API.

    import mccl_amd as mccl
    mccl.init(compression="topk", topk_ratio=0.01)
    comp = mccl.compressor_from_env()          # what the backend builds at start-up

``mccl_amd._C`` is the native extension (same helper names as the reference's
``mccl._C``); ``mccl_amd.hip_ops`` talks to the C ABI directly.
"""
from __future__ import annotations

import os
from typing import Any, Dict, Optional

from mccl_amd.config import MCCLConfig
from mccl_amd.version import COMPATIBILITY_MATRIX, __version__

_active_config: Optional[MCCLConfig] = None


def init(config: "MCCLConfig | Dict[str, Any] | None" = None, **kwargs: Any) -> MCCLConfig:
    """Resolves the configuration and exports it as ``MCCL_*`` variables.

    Same precedence as the reference's ``mccl.init`` (mccl/__init__.py:70-110):
    keyword arguments alone build a fresh config; a dict is merged with the
    keywords; no arguments reads the environment; an MCCLConfig object is
    updated with the keywords.  Returns the active config.
    """
    global _active_config
    if config is None and kwargs:
        config = MCCLConfig(**kwargs)
    elif isinstance(config, dict):
        config = MCCLConfig.from_dict({**config, **kwargs})
    elif config is None:
        config = MCCLConfig.from_env()
    elif kwargs:
        for key, value in kwargs.items():
            setattr(config, key, value)
    config.to_env()
    _active_config = config
    return config


def get_config() -> Optional[MCCLConfig]:
    """The config of the last init() call, or None."""
    return _active_config


def compressor_from_env():
    """The compressor the backend creates at start-up from MCCL_COMPRESSION /
    MCCL_TOPK_RATIO (csrc/backend/ProcessGroupMCCL.cpp:729-741): None for
    "none", a device-resident FP16Compressor for "fp16", TopKCompressor for "topk"."""
    import torch.distributed  # noqa: F401  (registers c10d base types for the extension)
    from mccl_amd import _C

    mode = _C.CompressionMode.NONE
    text = os.environ.get("MCCL_COMPRESSION", "")
    if text in ("fp16", "FP16"):
        mode = _C.CompressionMode.FP16
    elif text in ("topk", "TOPK"):
        mode = _C.CompressionMode.TOPK
    ratio = 0.01
    if os.environ.get("MCCL_TOPK_RATIO") is not None:
        try:
            ratio = float(os.environ["MCCL_TOPK_RATIO"])
        except ValueError:
            ratio = 0.0  # atof() of garbage; make_compressor falls back to 0.01
    return _C.make_compressor(mode, ratio)


__all__ = ["__version__", "COMPATIBILITY_MATRIX", "MCCLConfig", "init", "get_config", "compressor_from_env"]
