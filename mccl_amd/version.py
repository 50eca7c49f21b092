# Mirrors mccl/version.py:1 of the reference (same release line of the API).
__version__ = "0.5.0"
