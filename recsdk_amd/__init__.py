"""recsdk_amd - MI355X-native sparse-embedding hot path (key dedup, key->slot hash tables, row gather,
segment-reduced sparse optimizer updates) behind the reference's operator surface.

`recsdk_amd.capi` binds the C ABI (include/recsdk_hip.h); `recsdk_amd.host` mirrors the reference's
host interfaces on top of it.  The HIP library must be built first (`python -m recsdk_amd.build`).
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
