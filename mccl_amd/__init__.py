"""mccl_amd -- MI355X-native implementation of MCCL's per-rank data-parallel
compute path (chunk fold, AVG scale, top-k compression with error feedback,
decompress / accumulate), behind MCCL's own config and local-kernel API."""
from __future__ import annotations

from mccl_amd.version import __version__

__all__ = ["__version__"]
