"""Compressed-dim index rules, restated for checking.  TEST INFRASTRUCTURE ONLY.

Pinned against every raw/splithead pair the reference ships under
``compressed_dims_file/`` (``tests/test_masks.py``, skipped where the reference
tree is not mounted) and against the small committed extracts in
``tests/golden/``.
"""
from __future__ import annotations

from bisect import bisect_left
from typing import Dict, List, Sequence


def splithead_layer(raw_k: Sequence[int], raw_v: Sequence[int], num_kv_heads: int, head_dim: int) -> Dict[str, List[int]]:
    """Rule that maps one layer of the raw search output to the cache's on-disk format.

    Raw lists hold flat KV-hidden indices (``h*D + d``) of the compressed
    ("non-critical") dims in rank order (compressed_dim_search.py:386-390).
    The cache consumes (cache_utils_fourier.py:444-452):
    ``kc_list`` = sorted raw list, ``kn_list`` = sorted complement in
    ``[0, Hkv*D)``, and ``k?_h_list[h]`` = number of list entries below
    ``(h+1)*D`` (cumulative per-head counts, no leading zero on disk).
    """
    hidden = num_kv_heads * head_dim
    out: Dict[str, List[int]] = {}
    for tag, raw in (("k", raw_k), ("v", raw_v)):
        c = sorted(int(i) for i in raw)
        cs = set(c)
        n = [i for i in range(hidden) if i not in cs]
        out[f"{tag}c_list"] = c
        out[f"{tag}n_list"] = n
        out[f"{tag}c_h_list"] = [bisect_left(c, (h + 1) * head_dim) for h in range(num_kv_heads)]
        out[f"{tag}n_h_list"] = [bisect_left(n, (h + 1) * head_dim) for h in range(num_kv_heads)]
    return out


def select_noncritical(mean_mse: Sequence[float], percent: float) -> List[int]:
    """Selection rule of the offline search (compressed_dim_search.py:367-390):
    rank dims by ``abs(mean MSE)`` ascending (stable for ties) and keep the first
    ``int(percent * n)``."""
    order = sorted(range(len(mean_mse)), key=lambda i: (abs(mean_mse[i]), i))
    return order[: int(percent * len(mean_mse))]


def percent_schedule(layer: int, tensor: str) -> float:
    """Per-layer compressed fraction (compressed_dim_search.py:342-353)."""
    if 20 <= layer <= 27:
        return 0.5 if tensor == "k" else 0.7
    if 0 <= layer <= 3:
        return 0.9 if tensor == "k" else 0.95
    return 0.8
