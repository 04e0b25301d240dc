"""Runtime flags of the fused-MoE path (reference: python/lightop/envs.py:26-65).

The reference evaluates these at import and queries the GPU while doing so
(envs.py:16-19); here they are module attributes computed on access, and nothing
touches a device.
"""
from __future__ import annotations

import os

_INT_FLAGS = {
    "LMSLIM_FUSED_MOE_CHUNK_SIZE": (("LMSLIM_FUSED_MOE_CHUNK_SIZE", "VLLM_FUSED_MOE_CHUNK_SIZE"), 16 * 1024),
}
_BOOL_FLAGS = {
    "LMSLIM_USE_GLOBAL_MOE_CACHE": (("LMSLIM_USE_GLOBAL_MOE_CACHE", "VLLM_USE_GLOBAL_CACHE13"), False),
    "LMSLIM_USE_FUSED_RMS_QUANT": (("LMSLIM_USE_FUSED_RMS_QUANT", "USE_FUSED_RMS_QUANT"), False),
    "LMSLIM_USE_FUSE_SILU_AND_MUL": (("LMSLIM_USE_FUSE_SILU_AND_MUL", "VLLM_USE_FUSE_SILU_AND_MUL"), False),
}

SUPPORTED_DEVICES = ["gfx950_256cu"]
LMSLIM_GPU_NAME = "gfx950_256cu"
device_name = "gfx950"
number_cu = 256


def _first(names):
    for n in names:
        raw = os.getenv(n)
        if raw is not None and raw != "":
            return raw
    return None


def __getattr__(name: str):
    if name == "LMSLIM_USE_LIGHTOP":
        # The native kernels are the only implementation; the flag is kept for callers
        # that read it.
        return int(os.getenv("LMSLIM_USE_LIGHTOP", 1))
    if name in _INT_FLAGS:
        names, default = _INT_FLAGS[name]
        raw = _first(names)
        return default if raw is None else int(raw)
    if name in _BOOL_FLAGS:
        names, default = _BOOL_FLAGS[name]
        raw = _first(names)
        return default if raw is None else raw.strip().lower() in ("1", "true", "yes", "on")
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


__all__ = [
    "SUPPORTED_DEVICES", "device_name", "number_cu", "LMSLIM_GPU_NAME", "LMSLIM_USE_LIGHTOP",
    "LMSLIM_FUSED_MOE_CHUNK_SIZE", "LMSLIM_USE_GLOBAL_MOE_CACHE", "LMSLIM_USE_FUSED_RMS_QUANT",
    "LMSLIM_USE_FUSE_SILU_AND_MUL",
]
