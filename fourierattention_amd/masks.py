"""Compressed-dim masks: the on-disk ``*_splithead.json`` format the cache consumes
(cache_utils_fourier.py:403-455), the raw -> splithead conversion, and a seeded
synthetic generator for benchmarks.

A mask file maps ``"Layer_<i>"`` to eight integer lists.  ``kc_list`` / ``vc_list``
hold the flat KV-hidden indices (``head * head_dim + dim``) of the dims that are
stored as Fourier coefficients, ascending; ``kn_list`` / ``vn_list`` the complement;
``k?_h_list[h]`` counts the entries that belong to heads ``0..h`` (cumulative, no
leading zero on disk - the cache prepends it, cache_utils_fourier.py:449-452).
"""
from __future__ import annotations

import json
from bisect import bisect_left
from typing import Dict, Iterable, List, Sequence

import numpy as np

LAYER_KEYS = ("kc_list", "vc_list", "kc_h_list", "vc_h_list", "kn_list", "vn_list", "kn_h_list", "vn_h_list")


def load_masks(path: str) -> Dict[str, Dict[str, List[int]]]:
    with open(path, "r") as f:
        return json.load(f)


def save_masks(masks: Dict[str, Dict[str, List[int]]], path: str) -> None:
    with open(path, "w") as f:
        json.dump(masks, f)


def _cumulative(sorted_list: Sequence[int], num_kv_heads: int, head_dim: int) -> List[int]:
    return [bisect_left(sorted_list, (h + 1) * head_dim) for h in range(num_kv_heads)]


def layer_from_compressed(k_compressed: Iterable[int], v_compressed: Iterable[int], num_kv_heads: int,
                          head_dim: int) -> Dict[str, List[int]]:
    """Build one layer entry from the sets of compressed flat dims (any order)."""
    hidden = num_kv_heads * head_dim
    entry: Dict[str, List[int]] = {}
    for tag, comp in (("k", k_compressed), ("v", v_compressed)):
        c = sorted({int(i) for i in comp})
        if c and (c[0] < 0 or c[-1] >= hidden):
            raise ValueError(f"compressed dim out of range [0, {hidden})")
        member = np.zeros(hidden, dtype=bool)
        member[c] = True
        n = np.nonzero(~member)[0].tolist()
        entry[f"{tag}c_list"] = c
        entry[f"{tag}n_list"] = n
        entry[f"{tag}c_h_list"] = _cumulative(c, num_kv_heads, head_dim)
        entry[f"{tag}n_h_list"] = _cumulative(n, num_kv_heads, head_dim)
    return entry


def splithead_from_raw(raw: Dict[str, Dict[str, List[int]]], num_kv_heads: int, head_dim: int):
    """Convert the search's raw output (``self_attn.k_proj`` / ``self_attn.v_proj`` rank-ordered
    lists per layer, compressed_dim_search.py:386-390) to the splithead format."""
    out = {}
    for i in range(len(raw)):
        key = f"Layer_{i}"
        if key not in raw:
            raise ValueError(f"{key} missing from raw mask data")
        out[key] = layer_from_compressed(raw[key]["self_attn.k_proj"], raw[key]["self_attn.v_proj"], num_kv_heads, head_dim)
    return out


def synthetic_masks(num_layers: int, num_kv_heads: int, head_dim: int, k_per_head, v_per_head=None, seed: int = 0):
    """Seeded masks compressing exactly ``k_per_head`` / ``v_per_head`` dims of every head (an int, or one count per
    head for masks whose heads differ)."""
    v_per_head = k_per_head if v_per_head is None else v_per_head
    per = lambda c: [int(c)] * num_kv_heads if np.isscalar(c) else [int(x) for x in c]
    k_cnt, v_cnt = per(k_per_head), per(v_per_head)
    if len(k_cnt) != num_kv_heads or len(v_cnt) != num_kv_heads:
        raise ValueError(f"one count per KV head expected ({num_kv_heads})")
    rng = np.random.default_rng(seed)
    out = {}
    for i in range(num_layers):
        kc, vc = [], []
        for h in range(num_kv_heads):
            kc += (h * head_dim + np.sort(rng.choice(head_dim, k_cnt[h], replace=False))).tolist()
            vc += (h * head_dim + np.sort(rng.choice(head_dim, v_cnt[h], replace=False))).tolist()
        out[f"Layer_{i}"] = layer_from_compressed(kc, vc, num_kv_heads, head_dim)
    return out


def validate_layer(entry: Dict[str, List[int]], num_kv_heads: int, head_dim: int) -> None:
    """Raise ``ValueError`` unless the eight lists are mutually consistent."""
    hidden = num_kv_heads * head_dim
    for tag in ("k", "v"):
        c, n = entry[f"{tag}c_list"], entry[f"{tag}n_list"]
        ch, nh = entry[f"{tag}c_h_list"], entry[f"{tag}n_h_list"]
        if sorted(c) != list(c) or sorted(n) != list(n):
            raise ValueError(f"{tag}: index lists must be ascending")
        if sorted(list(c) + list(n)) != list(range(hidden)):
            raise ValueError(f"{tag}: compressed and stored dims must partition [0, {hidden})")
        if len(ch) != num_kv_heads or len(nh) != num_kv_heads:
            raise ValueError(f"{tag}: per-head lists need {num_kv_heads} entries")
        if ch != _cumulative(c, num_kv_heads, head_dim) or nh != _cumulative(n, num_kv_heads, head_dim):
            raise ValueError(f"{tag}: per-head cumulative counts do not match the index lists")
