"""Process-wide ``cache13`` workspaces of the fused-MoE path.

The reference keeps one module-level tensor and hands it to every caller
(python/lightop/_lmslim_native/vllm_compat/fused_moe_cache.py:19-24); a later call with another
device, dtype or a larger layer gets the first call's buffer there.  Here a buffer is kept per
(device, dtype) and replaced by a larger one when a call needs more, so every caller receives a
tensor that is on its device, has its dtype and holds at least what it asked for.
"""
from __future__ import annotations

import logging
import threading
from typing import Dict, Optional, Tuple

import torch

from .. import envs

logger = logging.getLogger(__name__)

_lock = threading.Lock()
_buffers: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}

# Name kept for callers that look at the reference's global: the buffer handed out last.
moe_cache_singleton: Optional[torch.Tensor] = None


def _key(device, dtype) -> Tuple[str, torch.dtype]:
    dev = torch.device(device)
    if dev.type == "cuda" and dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    return str(dev), dtype


def get_moe_cache(top_k_num: int, N: int, K: int, device, dtype) -> torch.Tensor:
    """A 1-D buffer of at least ``CHUNK * top_k_num * max(N, K)`` elements of ``dtype`` on ``device``
    (``CHUNK`` = ``LMSLIM_FUSED_MOE_CHUNK_SIZE``), shared by every call with that device and dtype.
    Callers that overlap on different streams must not share it; give those their own ``cache13``."""
    global moe_cache_singleton
    need = int(envs.LMSLIM_FUSED_MOE_CHUNK_SIZE) * int(top_k_num) * max(int(N), int(K))
    key = _key(device, dtype)
    with _lock:
        buf = _buffers.get(key)
        if buf is None or buf.numel() < need:
            buf = torch.empty(need, device=device, dtype=dtype)
            _buffers[key] = buf
            logger.info("moe cache13 for %s / %s: %d elements, %.2f MB", key[0], dtype, need,
                        need * buf.element_size() / 2 ** 20)
        moe_cache_singleton = buf
        return buf


def release_moe_cache() -> None:
    """Drop every cached buffer (their memory returns to the allocator)."""
    global moe_cache_singleton
    with _lock:
        _buffers.clear()
        moe_cache_singleton = None
