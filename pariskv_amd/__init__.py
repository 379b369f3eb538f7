"""pariskv_amd: ParisKV's per-decode-step KV retrieval path on MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (``libpariskv_hip.so``), reached from
Python through ctypes; ``cache_hub`` / ``attn_hub`` mirror the reference's call
surface so the package drops in under ``attn_hub/polar_attn.py``.
"""
from . import _lib, ops  # noqa: F401

__all__ = ["_lib", "ops"]
