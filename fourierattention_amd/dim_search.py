"""Offline search for the head dimensions that tolerate spectral compression
(compressed_dims_search/compressed_dim_search.py:135-161, 239-269, 321-397 with the transform of
compressed_dims_search/hippo_function_approx_legt_fourier_awq.py:335-393), restated on this package's kernels.

``search`` takes the projection outputs as an argument (``(B, S, Hkv*D)`` tensors per layer), so it runs on
whatever produced them; ``search_model`` is the reference's driver: it hooks ``k_proj`` / ``v_proj`` of a model that
runs calibration samples (compressed_dim_search.py:195-291) and feeds the same scoring.  Per dim the search
measures how well the middle of the sequence survives compress -> reconstruct -> mean / maximum-deviation
matching, ranks the dims by that error and marks the best ``percent`` of them as compressible.  The output is
the reference's raw mask format; ``masks.splithead_from_raw`` turns it into what the cache loads.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from . import ops


def percent_schedule(layer: int, tensor: str, num_layers: int) -> float:
    """Fraction of the dims to compress (compressed_dim_search.py:342-353, written there for a 28-layer model:
    layers 0-3 keep the most, the last eight the least; the shipped 32-layer masks follow the same rule with the
    last eight layers, 24-31)."""
    if layer >= num_layers - 8:
        return 0.5 if tensor == "k" else 0.7
    if layer <= 3:
        return 0.9 if tensor == "k" else 0.95
    return 0.8


@torch.no_grad()
def reconstruction_mse(x: torch.Tensor, numinittokens: int = 4, maxlocallen: int = 1024,
                       maxmidstates: int = 1024) -> torch.Tensor:
    """``x (B, S, C)`` projection output -> ``(B, C)`` float32: mean squared error per dim between the middle rows
    ``x[:, I:S-W]`` and their reconstruction from ``maxmidstates // 2`` frequencies over a period of exactly
    their length (``dt = 1 / L``, ``T = 1``: compressed_dim_search.py:252-258), after the reconstruction has been
    given the mean and the maximum deviation of the original (compressed_dim_search.py:137-147; each sample with
    its own statistics - the reference handles one sample at a time)."""
    assert x.dim() == 3 and x.shape[1] > numinittokens + maxlocallen, f"{tuple(x.shape)}: nothing between sink and window"
    mid = x[:, numinittokens: x.shape[1] - maxlocallen, :]
    L = mid.shape[1]
    coef = ops.mat_fourier(mid if mid.stride(2) == 1 else mid.contiguous(), maxmidstates // 2, L)
    rec = ops.mat_fourier_inv(coef, L, L)                       # (B, L, C) fp32, carries the 1 / N_f
    orig = mid.float()
    mean_r, mean_o = rec.mean(dim=1, keepdim=True), orig.mean(dim=1, keepdim=True)
    scale = (rec - mean_r).abs().amax(dim=1, keepdim=True) / (orig - mean_o).abs().amax(dim=1, keepdim=True)
    matched = (rec - mean_r) / scale + mean_o
    return ((orig - matched) ** 2).mean(dim=1)


def rank_dims(mean_mse: torch.Tensor) -> torch.Tensor:
    """Dims in ascending order of ``|mean error|`` (compressed_dim_search.py:367-368); ties keep index order."""
    return torch.argsort(mean_mse.abs(), stable=True)


def select_noncritical(mean_mse: torch.Tensor, percent: float) -> List[int]:
    """The first ``int(percent * n)`` dims of the ranking (compressed_dim_search.py:386-390)."""
    return rank_dims(mean_mse)[: int(percent * mean_mse.numel())].tolist()


@torch.no_grad()
def search(layers_kv: Iterable[Tuple[Sequence[torch.Tensor], Sequence[torch.Tensor]]], num_layers: Optional[int] = None,
           numinittokens: int = 4, maxlocallen: int = 1024, maxmidstates: int = 1024,
           percents: Optional[Dict[Tuple[int, str], float]] = None):
    """``layers_kv[i] = (k_samples, v_samples)``: the ``k_proj`` / ``v_proj`` outputs of layer ``i`` for every
    calibration sample (each ``(1, S, Hkv*D)``; lengths may differ).  Returns ``(raw, errors)``: ``raw`` in the
    reference's format ``{"Layer_i": {"self_attn.k_proj": [...], "self_attn.v_proj": [...]}}`` (rank-ordered
    compressible dims) and ``errors[(i, "k" | "v")]`` the mean error per dim over the samples."""
    layers_kv = list(layers_kv)
    n_layers = num_layers if num_layers is not None else len(layers_kv)
    errors = {}
    for i, (ks, vs) in enumerate(layers_kv):
        for tag, samples in (("k", ks), ("v", vs)):
            acc = None
            for sample in samples:
                e = reconstruction_mse(sample, numinittokens, maxlocallen, maxmidstates)[0]
                acc = e if acc is None else acc + e
            if acc is not None:
                errors[(i, tag)] = acc / len(samples)
    return _select(errors, n_layers, percents), errors


def _select(errors, n_layers: int, percents) -> dict:
    """The raw mask of every measured layer from its mean errors (compressed_dim_search.py:321-397); ``n_layers`` is
    the depth of the model the layers belong to (it places them in the schedule of fractions)."""
    raw = {}
    for i in sorted({layer for layer, _ in errors}):
        raw[f"Layer_{i}"] = {}
        for tag, name in (("k", "self_attn.k_proj"), ("v", "self_attn.v_proj")):
            if (i, tag) not in errors:
                continue
            pct = percents[(i, tag)] if percents and (i, tag) in percents else percent_schedule(i, tag, n_layers)
            raw[f"Layer_{i}"][name] = select_noncritical(errors[(i, tag)], pct)
    return raw


@torch.no_grad()
def search_model(model, samples: Sequence[torch.Tensor], numinittokens: int = 4, maxlocallen: int = 1024,
                 maxmidstates: int = 1024, percents: Optional[Dict[Tuple[int, str], float]] = None):
    """The reference's driver (compressed_dim_search.py:164-291) on a decoder of ``fourierattention_amd.llama``:
    every calibration sample (token ids ``(1, S)``, ``S > numinittokens + maxlocallen``) runs through the model's
    prompt pass with a forward hook on ``k_proj`` and ``v_proj`` of every layer.  The hook recomputes the projection
    from the module's input and weight (before the rotary embedding, compressed_dim_search.py:243-247) and scores
    it at once, so no projection output outlives its layer; the errors are averaged over the samples and the best
    dims of every layer selected (compressed_dim_search.py:321-397).  Returns ``(raw, errors)`` like ``search``."""
    import torch.nn.functional as F
    from . import masks as pm
    from .cache import DynamicCache, ExtraConfig
    cfg = model.config
    layers = model.model.layers
    sums: Dict[Tuple[int, str], torch.Tensor] = {}

    def hook(module, inputs, output, layer_idx, tag):
        proj = F.linear(inputs[0], module.weight)                  # independent of the module's own output
        e = reconstruction_mse(proj, numinittokens, maxlocallen, maxmidstates)[0]
        key = (layer_idx, tag)
        sums[key] = e if key not in sums else sums[key] + e

    handles = []
    for i, layer in enumerate(layers):
        for tag, mod in (("k", layer.self_attn.k_proj), ("v", layer.self_attn.v_proj)):
            handles.append(mod.register_forward_hook(lambda m, a, o, i=i, tag=tag: hook(m, a, o, i, tag)))
    fused = model.model.fused_elementwise
    model.model.fused_elementwise = False     # the module chain calls k_proj / v_proj themselves
    try:
        placeholder = pm.synthetic_masks(len(layers), cfg.num_key_value_heads, cfg.head_dim, cfg.head_dim // 2, seed=0)
        for sample in samples:
            assert sample.dim() == 2 and sample.shape[0] == 1, "one calibration sample at a time: (1, S) token ids"
            # a cache whose window holds the whole sample: the prompt pass is plain causal attention
            ec = ExtraConfig(numinittokens=0, maxlocallen=sample.shape[1] + 1, maxmidstates=2, non_critical_dims=placeholder,
                             non_critical_dims_path=None, max_position_embeddings=sample.shape[1] + 128,
                             num_key_value_heads=cfg.num_key_value_heads, max_new_tokens=64, model_type="llama")
            model.model(sample, DynamicCache(ec, device=sample.device))
    finally:
        model.model.fused_elementwise = fused
        for h in handles:
            h.remove()
    errors = {key: total / len(samples) for key, total in sums.items()}
    return _select(errors, len(layers), percents), errors
