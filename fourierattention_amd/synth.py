"""Seeded synthetic inputs of the benchmark configurations: N(0,1) Q/K/V with plain RoPE
(base 500000, HF half-rotation layout) on Q and K, and per-head masks."""
from __future__ import annotations

import torch


def rope_tables(positions: torch.Tensor, head_dim: int, base: float = 500000.0):
    inv = base ** (-torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim)
    ang = positions.to(torch.float64)[:, None] * inv[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos().float(), emb.sin().float()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``x (B, H, S, D)`` float32; ``cos, sin (S, D)``."""
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos[None, None] + rot * sin[None, None]


def make_qkv(batch: int, num_q_heads: int, num_kv_heads: int, head_dim: int, context: int, dtype=torch.bfloat16,
             seed: int = 0, device="cpu", chunk: int = 8192):
    """Prompt K, V ``(B, Hkv, context, D)`` plus one decode step ``q (B, Hq, 1, D)``,
    ``k_new, v_new (B, Hkv, 1, D)`` at position ``context``.  Generated on the CPU generator in
    chunks over the sequence so that every size reproduces the same leading values."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    k = torch.empty((batch, num_kv_heads, context, head_dim), dtype=dtype, device=device)
    v = torch.empty_like(k)
    for s0 in range(0, context, chunk):
        s1 = min(context, s0 + chunk)
        kk = torch.randn((batch, num_kv_heads, s1 - s0, head_dim), generator=g)
        vv = torch.randn((batch, num_kv_heads, s1 - s0, head_dim), generator=g)
        cos, sin = rope_tables(torch.arange(s0, s1), head_dim)
        k[:, :, s0:s1] = apply_rope(kk, cos, sin).to(dtype).to(device)
        v[:, :, s0:s1] = vv.to(dtype).to(device)
    q = torch.randn((batch, num_q_heads, 1, head_dim), generator=g)
    kn = torch.randn((batch, num_kv_heads, 1, head_dim), generator=g)
    vn = torch.randn((batch, num_kv_heads, 1, head_dim), generator=g)
    cos, sin = rope_tables(torch.tensor([context]), head_dim)
    q = apply_rope(q, cos, sin).to(dtype).to(device)
    kn = apply_rope(kn, cos, sin).to(dtype).to(device)
    return k, v, q, kn, vn.to(dtype).to(device)
