"""The cache object at the seam with the reference's model code: the three type tests the modified LLaMA
applies to ``past_key_values`` (modeling_llama_fourier.py:29, 946-951, 1052) restated here and fed with this
package's objects, and the rotary fallback of the attention forward (modeling_llama_fourier.py:604-612).
CPU only: nothing here computes on the GPU."""
import pytest
import torch

from tests.test_gpu_cache import _cfg, _masks


def _route_like_llama_model_forward(past_key_values, use_cache, Cache, DynamicCache):
    """modeling_llama_fourier.py:944-957, with the names the model imports at line 29 passed in."""
    return_legacy_cache = False
    if use_cache and not isinstance(past_key_values, Cache):
        return_legacy_cache = True
        if past_key_values is None:
            past_key_values = DynamicCache()                      # raises: extra_config is required
        else:
            past_key_values = DynamicCache.from_legacy_cache(past_key_values)
    return past_key_values, return_legacy_cache


def _cache():
    from fourierattention_amd import DynamicCache
    return DynamicCache(_cfg(_masks(2, 2, 16, [8, 8], [8, 8])), device="cpu")


def test_cache_passes_the_models_type_gates():
    import fourierattention_amd as fa
    from fourierattention_amd import Cache, DynamicCache, StaticCache     # the import line of the model, re-pointed
    cache = _cache()
    assert isinstance(cache, Cache) and isinstance(cache, torch.nn.Module)          # the reference's base is a Module
    got, legacy = _route_like_llama_model_forward(cache, True, Cache, DynamicCache)
    assert got is cache and legacy is False                                          # line 946: kept as it is
    assert isinstance(cache, StaticCache) is False                                   # line 1052: "not static"
    assert cache.get_max_cache_shape() is None and cache.get_seq_length() == 0       # lines 959, 1051
    assert cache.get_usable_length(5) == 0 and cache.seen_tokens == 0
    assert issubclass(StaticCache, Cache)
    with pytest.raises(NotImplementedError):
        StaticCache()
    # what the model does with anything that is not a Cache: both arms fail like the reference's do
    with pytest.raises(TypeError):
        _route_like_llama_model_forward(None, True, Cache, DynamicCache)
    with pytest.raises(NotImplementedError):
        _route_like_llama_model_forward(((None, None),), True, Cache, DynamicCache)
    assert {"Cache", "DynamicCache", "StaticCache"} <= set(fa.__all__)


def test_base_class_methods_raise_like_the_reference():
    from fourierattention_amd import Cache
    base = Cache()
    for call in (lambda: base.update(None, None, 0), base.get_seq_length, base.get_max_cache_shape):
        with pytest.raises(NotImplementedError):
            call()


def test_attention_forward_computes_rotary_tables_from_position_ids():
    """Without ``position_embeddings`` the forward builds cos / sin from ``position_ids`` with its own rotary
    module; the result equals the call that is handed the tables."""
    from fourierattention_amd import LlamaSdpaAttention
    from fourierattention_amd.llama import LlamaConfig
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=16, vocab_size=11, rope_theta=500000.0)
    torch.manual_seed(0)
    attn = LlamaSdpaAttention(cfg, layer_idx=0)
    x = torch.randn(2, 9, 64)
    pos = torch.arange(9)[None, :].expand(2, -1)
    cos, sin = attn.rotary_emb(x, pos)
    assert cos.shape == (2, 9, 16) and torch.allclose(cos[:, 0], torch.ones(2, 16)) and torch.allclose(sin[:, 0], torch.zeros(2, 16))
    a, _, ca = attn(x, position_ids=pos, past_key_value=_cache(), position_embeddings=(cos, sin))
    b, _, cb = attn(x, position_ids=pos, past_key_value=_cache())
    assert torch.equal(a, b) and ca.get_seq_length() == cb.get_seq_length() == 9
    with pytest.raises(ValueError):
        attn(x, past_key_value=_cache())


def test_shapes_off_the_matrix_cores_are_announced_once():
    """Long contexts whose shape only the any-shape vector kernels take (e.g. float32 storage, 384 frequencies) are
    about 50x slower: the operator says so, once per shape."""
    import warnings
    import torch
    from fourierattention_amd import ops
    ops._warned_shapes.clear()
    with warnings.catch_warnings(record=True) as got:
        warnings.simplefilter("always")
        ops._warn_if_off_the_matrix_cores(torch.bfloat16, 32, 8, 128, 512, True)      # covered: silent
        ops._warn_if_off_the_matrix_cores(torch.float32, 32, 8, 128, 512, True)
        ops._warn_if_off_the_matrix_cores(torch.float32, 32, 8, 128, 512, True)       # the same shape again: silent
        ops._warn_if_off_the_matrix_cores(torch.bfloat16, 32, 8, 128, 384, True)
        ops._warn_if_off_the_matrix_cores(torch.bfloat16, 72, 8, 128, 512, True)      # nine query heads per KV head
    assert len(got) == 3 and all(issubclass(w.category, RuntimeWarning) for w in got)
    assert "vector kernels" in str(got[0].message)
