"""Tile tables read from tuning files, ahead of the table compiled into the library.

The reference resolves the tile configuration of both GEMMs from per-device JSON files
(W8a8GetCacheJSON, python/lightop/_lmslim_native/vllm_compat/w8a8_get_cache_json.py:12-174;
lookup get_w8a8moe_json, layers/fused_moe/int8.py:220-256) and lets the user point it at a directory
of his own with ``TRITON_JSON_DIR`` (w8a8_get_cache_json.py:24).  ``python -m lightop_amd.tune --out DIR``
writes files of that layout for the GPU at hand; with ``TRITON_JSON_DIR=DIR`` set, the block size they
hold for a problem wins over the compiled-in pick.  File name and keys are the reference's:

    MOE_<kind>_E=<E>_N1=<2I>_N2=<H>_K=<I>_TOPK<k>_<device>.json        kind: BLOCKINT8[128,128], W8A8INT8,
    {"<2I>_<H>_<I>": {"<M>": {"config1": {...}, "config2": {...}}}}           W4A8INT8[1,128], W4A8INT8

The reference maps a token count onto the handful of counts its own files were tuned at
(int8.py:232-245).  A file written by the tuner holds whatever counts it was run with, so the lookup
here takes the tuned count nearest to ``m`` on a logarithmic scale (the larger one on a tie).
Nothing is read, and no environment variable is looked at, before the first lookup.
"""
from __future__ import annotations

import json
import math
import os
import threading
from typing import Dict, List, Optional, Tuple

from .. import envs

_lock = threading.Lock()
_files: Dict[str, Optional[Dict[int, Tuple[dict, dict]]]] = {}   # path -> {M: (config1, config2)} or None


def json_dir() -> Optional[str]:
    """Directory of the tuning files, or None when the compiled-in table is all there is."""
    d = os.getenv("TRITON_JSON_DIR", "")
    return d if d else None


def file_name(E: int, n1: int, n2: int, k: int, topk: int, block_shape: Optional[List[int]], int4: bool,
              device: Optional[str] = None) -> str:
    """Name of the file for one layer shape (get_moeint8json_name, w8a8_get_cache_json.py:133-149)."""
    if int4:
        kind = "W4A8INT8" if block_shape is None else f"W4A8INT8[{block_shape[0]},{block_shape[1]}]"
    else:
        kind = "W8A8INT8" if block_shape is None else f"BLOCKINT8[{block_shape[0]},{block_shape[1]}]"
    return f"MOE_{kind}_E={E}_N1={n1}_N2={n2}_K={k}_TOPK{topk}_{device or envs.LMSLIM_GPU_NAME}.json"


def _load(path: str, shape_key: str) -> Optional[Dict[int, Tuple[dict, dict]]]:
    with _lock:
        if path in _files:
            return _files[path]
    table: Optional[Dict[int, Tuple[dict, dict]]] = None
    if os.path.exists(path):
        with open(path, "r") as f:
            doc = json.load(f)
        rows = doc.get(shape_key, {})
        table = {}
        for m_key, pair in rows.items():
            if "config1" in pair and "config2" in pair:
                table[int(m_key)] = (dict(pair["config1"]), dict(pair["config2"]))
        if not table:
            table = None
    with _lock:
        _files[path] = table
    return table


def forget() -> None:
    """Drop everything read so far (a test that rewrites a file, a tuner that has just written one)."""
    with _lock:
        _files.clear()


def lookup(m: int, E: int, n1: int, n2: int, k: int, topk: int, block_shape: Optional[List[int]],
           int4: bool = False) -> Optional[Tuple[dict, dict]]:
    """(config1, config2) of the tuned token count nearest to ``m`` for this layer shape, or None when
    ``TRITON_JSON_DIR`` is unset or holds no file for the shape."""
    d = json_dir()
    if d is None:
        return None
    table = _load(os.path.join(d, file_name(E, n1, n2, k, topk, block_shape, int4)), f"{n1}_{n2}_{k}")
    if not table:
        return None
    lm = math.log(max(int(m), 1))
    best = min(table, key=lambda t: (abs(math.log(max(t, 1)) - lm), -t))
    return table[best]


def block_size_m(m: int, E: int, n1: int, n2: int, k: int, topk: int, block_shape: Optional[List[int]],
                 int4: bool = False) -> int:
    """BLOCK_SIZE_M a tuning file holds for the problem (both GEMMs share it: the alignment is done once,
    as the reference asserts for its own tables, int8.py:217), or 0."""
    hit = lookup(m, E, n1, n2, k, topk, block_shape, int4)
    if hit is None or hit[0].get("lightop_amd_two_launch"):  # the tuner's mark: the library's own pick was fastest
        return 0
    return int(hit[0].get("BLOCK_SIZE_M", 0))
