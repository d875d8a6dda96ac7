"""Attention forward of the modified LLaMA layer
(fourier_attn_triton/modeling_llama_fourier.py:565-667) on top of the Fourier cache.

``fourier_attention`` is the part after RoPE: ``cache.update`` then the dispatch between
exact attention (prefill, or layers that only keep a window) and Fourier decode attention.
``LlamaSdpaAttention`` wraps it with the projections and keeps the reference's forward
signature and return triple.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .cache import CacheParts, DynamicCache


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
    """HF convention (modeling_llama_fourier.py:213-244): ``x*cos + rotate_half(x)*sin``."""
    cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def _exact_attention(query_states, k_local, v_local, num_kv_heads, head_dim):
    """Causal attention over full keys (the ``flash_attn_func(..., causal=True)`` call at
    modeling_llama_fourier.py:633; bottom-right aligned when ``q_len < kv_len``)."""
    B, Hq, q_len, D = query_states.shape
    S = k_local.shape[1]
    if ops.prefill_attention_supported(query_states, k_local, head_dim) and v_local.stride() == k_local.stride():
        return ops.prefill_attention(query_states, k_local, v_local, num_kv_heads)   # (B, q_len, Hq, D)
    if query_states.is_cuda and query_states.dtype == torch.float32 and head_dim in (64, 128):
        # float32 storage: the reference casts q, k and v to half for this call whatever the model's type
        # (modeling_llama_fourier.py:633); the caller casts the result back
        qh, kh, vh = query_states.half().contiguous(), k_local.half().contiguous(), v_local.half().contiguous()
        if ops.prefill_attention_supported(qh, kh, head_dim):
            return ops.prefill_attention(qh, kh, vh, num_kv_heads)
    # other head dims and the host-only tests: the framework's attention
    k = k_local.view(B, S, num_kv_heads, head_dim).transpose(1, 2)
    v = v_local.view(B, S, num_kv_heads, head_dim).transpose(1, 2)
    if q_len == S:
        o = F.scaled_dot_product_attention(query_states, k, v, is_causal=True, enable_gqa=True)
    else:
        idx_q = torch.arange(q_len, device=query_states.device)[:, None] + (S - q_len)
        mask = torch.arange(S, device=query_states.device)[None, :] <= idx_q
        o = F.scaled_dot_product_attention(query_states, k, v, attn_mask=mask, enable_gqa=True)
    return o.transpose(1, 2)  # (B, q_len, Hq, D)


def fourier_attention(query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                      past_key_value: DynamicCache, layer_idx: int, num_heads: int, num_key_value_heads: int,
                      cache_kwargs=None) -> torch.Tensor:
    """``query_states (B, Hq, q_len, D)``, ``key_states / value_states (B, Hkv, q_len, D)`` after RoPE.
    Returns ``(B, q_len, Hq*D)`` in the query dtype (modeling_llama_fourier.py:618-663)."""
    bsz, _, q_len, head_dim = query_states.shape
    k_parts, v_parts = past_key_value.update(key_states, value_states, layer_idx, cache_kwargs)
    if k_parts["k_init"] is None and k_parts["k_compressed"] is None and k_parts["k_uncompressed"] is None:
        if q_len == 1 and query_states.is_cuda:
            o = past_key_value.decode_attention(query_states, layer_idx, num_heads, num_key_value_heads,
                                                out_dtype=query_states.dtype)
            o = o.transpose(1, 2)
        else:
            o = _exact_attention(query_states, k_parts["k_local"], v_parts["v_local"], num_key_value_heads, head_dim)
    elif isinstance(k_parts, CacheParts):
        o = past_key_value.decode_attention(query_states, layer_idx, num_heads, num_key_value_heads,
                                            out_dtype=query_states.dtype).transpose(1, 2)
    else:  # plain tensors in the reference's layout
        pkv = past_key_value
        o = ops.triton_fourier_attn(
            q=query_states.transpose(1, 2).reshape(bsz, q_len, num_heads * head_dim).contiguous(),
            k_il=torch.cat([k_parts["k_init"], k_parts["k_local"]], dim=1).contiguous(),
            v_il=torch.cat([v_parts["v_init"], v_parts["v_local"]], dim=1).contiguous(),
            k_mc=k_parts["k_compressed"], v_mc=v_parts["v_compressed"],
            k_mn=k_parts["k_uncompressed"], v_mn=v_parts["v_uncompressed"],
            avg_k_u=pkv.k_layer_average[layer_idx], avg_k_d=pkv.kd_layer_average[layer_idx], scale_k=pkv.k_scale[layer_idx],
            avg_v_u=pkv.v_layer_average[layer_idx], avg_v_d=pkv.vd_layer_average[layer_idx], scale_v=pkv.v_scale[layer_idx],
            kc_list=pkv.k_non_critical_dims[layer_idx], kc_h_list=pkv.k_non_critical_head_dims[layer_idx],
            kn_list=pkv.k_critical_dims[layer_idx], kn_h_list=pkv.k_critical_head_dims[layer_idx],
            vc_list=pkv.v_non_critical_dims[layer_idx], vc_h_list=pkv.v_non_critical_head_dims[layer_idx],
            vn_list=pkv.v_critical_dims[layer_idx], vn_h_list=pkv.v_critical_head_dims[layer_idx],
            num_head_q=num_heads, num_head_kv=num_key_value_heads, seq_len_m=k_parts["k_uncompressed"].size(1),
            T=pkv.maxtokens - pkv.numinittokens - pkv.maxlocallen).transpose(1, 2)
    return o.reshape(bsz, q_len, -1).to(query_states.dtype)


class LlamaRotaryEmbedding(nn.Module):
    """Plain ("default") rotary tables: ``inv_freq = theta^(-2i/D)``, angles in fp32, tables in the
    activation dtype (modeling_llama_fourier.py:165-187).  ``config`` needs ``head_dim`` (or ``hidden_size`` and
    ``num_attention_heads``) and optionally ``rope_theta`` (default 10000, as the stock config)."""

    def __init__(self, config):
        super().__init__()
        d = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        theta = float(getattr(config, "rope_theta", 10000.0))
        inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    @torch.no_grad()
    def forward(self, x, position_ids):
        freqs = position_ids[:, :, None].float() * self.inv_freq[None, None, :].float().to(position_ids.device)
        emb = torch.cat((freqs, freqs), dim=-1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


class LlamaSdpaAttention(nn.Module):
    """Projection + RoPE + Fourier-cache attention with the reference's forward contract
    (modeling_llama_fourier.py:547-667).  ``config`` needs ``hidden_size``, ``num_attention_heads``,
    ``num_key_value_heads`` and optionally ``head_dim`` / ``attention_bias``."""

    def __init__(self, config, layer_idx: Optional[int] = None):
        super().__init__()
        self.config, self.layer_idx = config, layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = getattr(config, "head_dim", None) or self.hidden_size // self.num_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        bias = getattr(config, "attention_bias", False)
        self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=bias)
        self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
        self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=bias)
        # only used when a caller passes position_ids instead of position_embeddings
        # (modeling_llama_fourier.py:332, 604-612)
        self.rotary_emb = LlamaRotaryEmbedding(config)

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                position_ids: Optional[torch.LongTensor] = None, past_key_value: Optional[DynamicCache] = None,
                output_attentions: bool = False, use_cache: bool = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, **kwargs):
        if output_attentions:
            raise NotImplementedError("attention weights are never materialised on this path")
        if past_key_value is None:
            raise ValueError("a Fourier DynamicCache must be passed as past_key_value")
        if position_embeddings is None and position_ids is None:
            raise ValueError("either position_embeddings (cos, sin) or position_ids must be passed")
        bsz, q_len, _ = hidden_states.size()
        q = self.q_proj(hidden_states).view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        if position_embeddings is None:   # modeling_llama_fourier.py:604-612
            cos, sin = self.rotary_emb(v, position_ids)
        else:
            cos, sin = position_embeddings
        q, k = apply_rotary_pos_emb(q, k, cos, sin)
        cache_kwargs = {"sin": sin, "cos": cos, "cache_position": cache_position}
        o = fourier_attention(q, k, v, past_key_value, self.layer_idx, self.num_heads, self.num_key_value_heads,
                              cache_kwargs)
        return self.o_proj(o), None, past_key_value
