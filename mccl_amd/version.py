"""Version of the MCCL API this package implements (mccl/version.py:1-16)."""
__version__ = "0.5.0"

COMPATIBILITY_MATRIX = {
    "rocm": ["7.0", "7.2"],
    "python": ["3.10", "3.11", "3.12"],
    "pytorch": ["2.10.x (ROCm)"],
    "hardware": "AMD Instinct MI355X (gfx950)",
    "backend_name": "mccl",
    "supported_devices": ["cuda (ROCm)"],
    "scope": "per-rank compute path: chunk fold, AVG scale, top-k compress, decompress/accumulate",
    "compression_modes": ["none", "topk"],
}
