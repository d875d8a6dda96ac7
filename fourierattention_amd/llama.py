"""Minimal LLaMA decoder around the Fourier cache: what runs either side of the attention path in one
decode step (fourier_attn_triton/modeling_llama_fourier.py:78-98 RMSNorm, 100-190 rotary embedding,
246-283 SwiGLU MLP, 677-754 decoder layer, 912-1033 model forward, 1090-1200 LM head) and the greedy loop
of models/fourier.py:155-203.

Stock math only: the projections and the MLP are ``torch`` GEMMs, the attention module is
``fourierattention_amd.attention.LlamaSdpaAttention``.  Weights are random (no checkpoint can be fetched
here); ``synthetic_prefill`` fills the cache of every layer with a random prompt of the requested length
through the cache's own prefill branch, so a decode benchmark at a long context does not have to run the
quadratic prompt pass of a random model first.
"""
from __future__ import annotations

from dataclasses import dataclass
from types import SimpleNamespace
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops, synth
from .attention import LlamaRotaryEmbedding, LlamaSdpaAttention, fourier_attention
from .cache import DynamicCache


@dataclass
class LlamaConfig:
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: Optional[int] = None
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    attention_bias: bool = False
    mlp_bias: bool = False
    tie_word_embeddings: bool = False

    def __post_init__(self):
        if self.head_dim is None:
            self.head_dim = self.hidden_size // self.num_attention_heads


PRESETS = {
    "llama-3.1-8b": dict(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=128),
    "llama-3.2-3b": dict(hidden_size=3072, intermediate_size=8192, num_hidden_layers=28, num_attention_heads=24,
                         num_key_value_heads=8, head_dim=128, tie_word_embeddings=True),
}


class LlamaRMSNorm(nn.Module):
    """Variance in fp32, scale in the input dtype (modeling_llama_fourier.py:78-95)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, x):
        dt = x.dtype
        x = x.float()
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * x.to(dt)


class LlamaMLP(nn.Module):
    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=config.mlp_bias)
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=config.mlp_bias)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=config.mlp_bias)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class LlamaDecoderLayer(nn.Module):
    def __init__(self, config: LlamaConfig, layer_idx: int):
        super().__init__()
        self.self_attn = LlamaSdpaAttention(config, layer_idx)
        self.mlp = LlamaMLP(config)
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self._qkv_weight = self._gate_up_weight = None
        self._packed = {}   # "qkv", "o", "gate_up", "down" -> ops.PackedLinearWeight (decode steps of at most 16 rows)

    def pack_projections(self):
        """Keeps a second copy of the four weight groups in the order ``ops.linear_packed`` streams them (16-bit GPU
        weights without bias).  A decode step of at most 16 rows then runs its projections on those copies; prompts
        keep using the row-major weights through the GEMM library.  Doubles the memory of the layer's weights."""
        at, mlp = self.self_attn, self.mlp
        w = at.q_proj.weight
        if at.q_proj.bias is not None or mlp.gate_proj.bias is not None or not w.is_cuda or w.dtype not in (torch.bfloat16, torch.float16):
            return
        groups = {"qkv": (at.q_proj, at.k_proj, at.v_proj), "o": (at.o_proj,), "gate_up": (mlp.gate_proj, mlp.up_proj),
                  "down": (mlp.down_proj,)}
        for name, mods in groups.items():
            n_out, k = sum(m.weight.shape[0] for m in mods), mods[0].weight.shape[1]
            if n_out % 16 or k % 1024:
                continue
            fused = mods[0].weight.data if len(mods) == 1 else torch.cat([m.weight.data for m in mods], dim=0)
            self._packed[name] = ops.PackedLinearWeight(fused.contiguous(), sources=[m.weight for m in mods])

    def _packed_weight(self, name):
        """The packed copy of a weight group, or ``None``: a copy whose source parameters have been written or
        replaced since it was made (``load_state_dict``, ``.to()``, an in-place update) is dropped, and the layer goes
        back to the modules' own weights until ``pack_projections`` is called again."""
        w = self._packed.get(name)
        if w is not None and w.stale():
            del self._packed[name]
            return None
        return w

    def _linear(self, name, x, fallback):
        w = self._packed_weight(name)
        return ops.linear_packed(x, w) if w is not None and w.covers(x) else fallback(x)

    def fuse_projections(self, max_rows: int = 16384):
        """Moves the q/k/v weights into one tensor and the gate/up weights into another; the five modules keep
        views of them (same values, same state dict), ``forward_fused`` runs one GEMM per group.  A decode step
        reads every weight once, so five short launches become two that stream the same bytes.  A group whose
        fused weight would have more than ``max_rows`` rows stays as it is: for a handful of tokens the GEMM
        library answers a very wide output with a tile shape that streams the weights at half the rate of the two
        separate calls (measured at 2 x 14336 rows of 4096)."""
        at, mlp = self.self_attn, self.mlp
        if at.q_proj.bias is not None or mlp.gate_proj.bias is not None:
            return
        for name, mods in (("_qkv_weight", (at.q_proj, at.k_proj, at.v_proj)), ("_gate_up_weight", (mlp.gate_proj, mlp.up_proj))):
            if sum(m.weight.shape[0] for m in mods) > max_rows:
                continue
            fused = torch.cat([m.weight.data for m in mods], dim=0)
            row = 0
            for m in mods:
                n = m.weight.shape[0]
                m.weight.data = fused[row:row + n]
                row += n
            setattr(self, name, fused)

    def forward(self, hidden_states, position_embeddings, past_key_value, cache_position=None):
        h, _, _ = self.self_attn(self.input_layernorm(hidden_states), past_key_value=past_key_value, use_cache=True,
                                 cache_position=cache_position, position_embeddings=position_embeddings)
        hidden_states = hidden_states + h
        return hidden_states + self.mlp(self.post_attention_layernorm(hidden_states))

    def forward_fused(self, h, delta, position_embeddings, past_key_value, cache_position=None):
        """The same layer on the GPU with its elementwise chains in single launches.  ``h`` is the residual
        stream, updated in place; ``delta`` the branch output not yet added to it (``None`` for the first layer).
        Returns this layer's MLP output, to be added by whoever normalises next."""
        at = self.self_attn
        y = ops.add_rmsnorm(h, delta, self.input_layernorm.weight, self.input_layernorm.variance_epsilon)
        bsz, q_len, _ = y.shape
        nq, nk = at.num_heads * at.head_dim, at.num_key_value_heads * at.head_dim
        pk = self._packed_weight("qkv")
        if pk is not None and pk.covers(y):
            q, k, v = ops.linear_packed(y, pk).split((nq, nk, nk), dim=-1)
        elif self._qkv_weight is not None:
            q, k, v = F.linear(y, self._qkv_weight).split((nq, nk, nk), dim=-1)
        else:
            q, k, v = at.q_proj(y), at.k_proj(y), at.v_proj(y)
        cos, sin = position_embeddings
        q = ops.rope_qk(q, k, cos, sin, at.head_dim)
        split = lambda t, n: t.view(bsz, q_len, n, at.head_dim).transpose(1, 2)
        o = fourier_attention(split(q, at.num_heads), split(k, at.num_key_value_heads), split(v, at.num_key_value_heads),
                              past_key_value, at.layer_idx, at.num_heads, at.num_key_value_heads,
                              {"sin": sin, "cos": cos, "cache_position": cache_position})
        y = ops.add_rmsnorm(h, self._linear("o", o, at.o_proj), self.post_attention_layernorm.weight,
                            self.post_attention_layernorm.variance_epsilon)
        pk = self._packed_weight("gate_up")
        if pk is not None and pk.covers(y):
            gate, up = ops.linear_packed(y, pk).chunk(2, dim=-1)
        elif self._gate_up_weight is not None:
            gate, up = F.linear(y, self._gate_up_weight).chunk(2, dim=-1)
        else:
            gate, up = self.mlp.gate_proj(y), self.mlp.up_proj(y)
        return self._linear("down", ops.silu_mul(gate, up), self.mlp.down_proj)


class LlamaModel(nn.Module):
    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([LlamaDecoderLayer(config, i) for i in range(config.num_hidden_layers)])
        self.norm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self.rotary_emb = LlamaRotaryEmbedding(config)
        # on the GPU: residual add + RMSNorm, rotary embedding and the SwiGLU gate as one launch each (same
        # arithmetic and rounding points as the module chain below); False keeps the chain of tensor ops
        self.fused_elementwise = True

    def fuse_projections(self, max_rows: int = 16384):
        for layer in self.layers:
            layer.fuse_projections(max_rows)
        return self

    def pack_projections(self):
        for layer in self.layers:
            layer.pack_projections()
        return self

    def forward(self, input_ids, past_key_values: DynamicCache, position_ids=None):
        """A cache object is required (modeling_llama_fourier.py:946-949 would otherwise build one without
        its configuration and fail); positions continue from ``past_key_values.get_seq_length()``
        (modeling_llama_fourier.py:959-963)."""
        if past_key_values is None:
            raise ValueError("a Fourier DynamicCache must be passed as past_key_values")
        x = self.embed_tokens(input_ids)
        seen = past_key_values.get_seq_length()
        cache_position = torch.arange(seen, seen + x.shape[1], device=x.device)
        if position_ids is None:
            position_ids = cache_position.unsqueeze(0)
        pe = self.rotary_emb(x, position_ids)
        if x.is_cuda and self.fused_elementwise and not self.config.attention_bias and x.shape[-1] <= 8192:
            x, delta = x.contiguous(), None
            pe = tuple(t.expand(x.shape[0], -1, -1).contiguous() for t in pe)   # one table row per token, made once
            for layer in self.layers:
                delta = layer.forward_fused(x, delta, pe, past_key_values, cache_position)
            return ops.add_rmsnorm(x, delta, self.norm.weight, self.norm.variance_epsilon)
        for layer in self.layers:
            x = layer(x, pe, past_key_values, cache_position)
        return self.norm(x)


class LlamaForCausalLM(nn.Module):
    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.config = config
        self.model = LlamaModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight

    def forward(self, input_ids, past_key_values: DynamicCache, use_cache: bool = True, position_ids=None,
                num_logits_to_keep: int = 0):
        h = self.model(input_ids, past_key_values, position_ids)
        if num_logits_to_keep:
            h = h[:, -num_logits_to_keep:, :]
        return SimpleNamespace(logits=self.lm_head(h).float(), past_key_values=past_key_values)


def random_init(config: LlamaConfig, dtype=torch.bfloat16, device="cuda:0", seed: int = 0, std: float = 0.02):
    """A model of the given architecture with seeded normal weights (norm scales stay 1)."""
    with torch.device(device):
        prev = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            model = LlamaForCausalLM(config)
        finally:
            torch.set_default_dtype(prev)
    g = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() > 1:
                p.normal_(0.0, std, generator=g)
    return model.eval()


@torch.no_grad()
def greedy_generate(model: LlamaForCausalLM, input_ids: torch.Tensor, cache: DynamicCache, max_new_tokens: int,
                    eos_token_id: Optional[int] = None):
    """The loop of models/fourier.py:175-190: feed the prompt, then one argmax token per step with the cache
    threaded through.  Returns ``(B, prompt + generated)`` ids.  With ``eos_token_id`` the loop stops once
    every sequence of the batch has produced it (the reference handles batch 1 only)."""
    seq = input_ids
    done = torch.zeros(input_ids.shape[0], dtype=torch.bool, device=input_ids.device)
    for _ in range(max_new_tokens):
        out = model(input_ids=input_ids, past_key_values=cache, use_cache=True, num_logits_to_keep=1)
        input_ids = torch.argmax(out.logits[:, -1, :], dim=-1, keepdim=True)
        seq = torch.cat([seq, input_ids], dim=-1)
        if eos_token_id is not None:
            done |= input_ids[:, 0] == eos_token_id
            if bool(done.all()):
                break
    return seq


@torch.no_grad()
def synthetic_prefill(cache: DynamicCache, config: LlamaConfig, batch: int, prompt_len: int, dtype=torch.bfloat16,
                      device="cuda:0", seed: int = 0):
    """Fill every layer of ``cache`` with a random prompt: K, V ~ N(0, 1), rotary embedding on K, pushed
    through ``cache.update`` layer by layer in ascending order exactly as a prompt pass does."""
    g = torch.Generator(device=device).manual_seed(seed)
    cos, sin = synth.rope_tables(torch.arange(prompt_len), config.head_dim, config.rope_theta)
    cos, sin = cos.to(device), sin.to(device)
    shape = (batch, config.num_key_value_heads, prompt_len, config.head_dim)
    for layer in range(config.num_hidden_layers):
        k = synth.apply_rope(torch.randn(shape, generator=g, device=device, dtype=torch.float32), cos, sin).to(dtype)
        v = torch.randn(shape, generator=g, device=device, dtype=torch.float32).to(dtype)
        cache.update(k, v, layer)
        del k, v
