"""Version of the MCCL API this package implements and what it was built for
(the reference keeps the same two names in mccl/version.py)."""
__version__ = "0.5.0"


def _matrix():
    m = dict(backend_name="mccl", hardware="AMD Instinct MI355X (gfx950)")
    m["rocm"] = ["7.0", "7.2"]
    m["python"] = [f"3.{minor}" for minor in (10, 11, 12)]
    m["pytorch"] = ["2.10.x (ROCm)"]
    m["supported_devices"] = ["cuda (ROCm)"]
    m["compression_modes"] = ["none", "fp16", "topk"]
    m["scope"] = ("per-rank compute path: chunk fold, AVG scale, top-k and fp16 compression, "
                  "decompress/accumulate, ring-step driver for ranks on one GPU")
    return m


COMPATIBILITY_MATRIX = _matrix()
