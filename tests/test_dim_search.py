"""Offline dim search (fourierattention_amd/dim_search.py) against a numpy restatement of the reference's
measurement (hippo_function_approx_legt_fourier_awq.py:335-393 transform and reconstruction,
compressed_dim_search.py:137-161 matching and error) and of its selection rule."""
import numpy as np
import pytest
import torch

from oracle import masks_oracle as mo


def test_selection_rule_and_schedule_match_the_oracle():
    from fourierattention_amd import dim_search as ds
    r = np.random.default_rng(0)
    e = r.standard_normal(257) ** 2
    e[10] = e[200]                       # a tie: index order decides
    for pct in (0.5, 0.7, 0.8, 0.9, 0.95):
        assert ds.select_noncritical(torch.from_numpy(e), pct) == mo.select_noncritical(e.tolist(), pct)
    for layer in range(28):              # the 28-layer schedule the reference spells out
        for t in ("k", "v"):
            assert ds.percent_schedule(layer, t, 28) == mo.percent_schedule(layer, t)
    assert ds.percent_schedule(24, "k", 32) == 0.5 and ds.percent_schedule(23, "k", 32) == 0.8   # the shipped 8B masks


def _reference_mse(x, I, W, M):
    """float64 restatement: interleaved cos/sin basis over dt = 1/L, reconstruction / base_N, matching, MSE."""
    mid = x[:, I: x.shape[1] - W, :].astype(np.float64)
    L, n_f = mid.shape[1], M // 2
    ph = 2 * np.pi * np.arange(L)[:, None] * np.arange(n_f)[None, :] / L
    basis = np.stack([np.cos(ph), np.sin(ph)], axis=-1).reshape(L, -1)            # (L, 2 n_f) interleaved
    coef = np.einsum("bln,ld->bdn", mid, basis)
    rec = np.einsum("bdn,ld->bln", coef, basis) / n_f
    out = np.zeros((x.shape[0], x.shape[2]))
    for b in range(x.shape[0]):
        mr, mo_ = rec[b].mean(0), mid[b].mean(0)
        scale = np.abs(rec[b] - mr).max(0) / np.abs(mid[b] - mo_).max(0)
        out[b] = (((rec[b] - mr) / scale + mo_ - mid[b]) ** 2).mean(0)
    return out


@pytest.mark.gpu
def test_reconstruction_error_matches_the_reference_formulation_and_ranks_smooth_dims_first():
    from fourierattention_amd import dim_search as ds, masks
    r = np.random.default_rng(1)
    S, I, W, M, Hkv, D = 700, 4, 64, 32, 2, 16
    C = Hkv * D
    t = np.arange(S)[:, None]
    smooth = np.sin(2 * np.pi * t * r.integers(1, 6, C)[None, :] / (S - I - W) + r.uniform(0, 6, C)[None, :])
    x = r.standard_normal((1, S, C)) * 0.05 + smooth[None] * (np.arange(C) % 2 == 0)[None, None, :]   # even dims: few frequencies
    x += r.standard_normal((1, S, C)) * (np.arange(C) % 2 == 1)[None, None, :]                         # odd dims: noise
    xg = torch.from_numpy(x.astype(np.float32)).cuda()
    got = ds.reconstruction_mse(xg, I, W, M).cpu().numpy()
    want = _reference_mse(x.astype(np.float32), I, W, M)
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=1e-6)
    raw, errs = ds.search([([xg], [xg])] * 2, num_layers=28, numinittokens=I, maxlocallen=W, maxmidstates=M,
                          percents={(0, "k"): 0.5})
    assert sorted(raw["Layer_0"]["self_attn.k_proj"]) == list(range(0, C, 2))       # exactly the smooth dims
    assert len(raw["Layer_1"]["self_attn.v_proj"]) == int(0.95 * C)                 # the schedule of an early layer
    sp = masks.splithead_from_raw(raw, Hkv, D)
    masks.validate_layer(sp["Layer_0"], Hkv, D)
    assert sp["Layer_0"]["kc_h_list"] == [D // 2, D]


@pytest.mark.gpu
def test_model_hook_driver_scores_the_projections_before_the_rotary_embedding():
    """``search_model`` against ``search`` fed with the same projections taken by hand: the hooks see ``k_proj`` /
    ``v_proj`` of every layer for every sample, the flags of the model and its hooks are left as they were."""
    import torch.nn.functional as F
    from fourierattention_amd import dim_search
    from fourierattention_amd.llama import LlamaConfig, random_init
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=16, vocab_size=97)
    model = random_init(cfg, dtype=torch.bfloat16, device="cuda", seed=5, std=0.3)
    g = torch.Generator(device="cuda").manual_seed(0)
    samples = [torch.randint(0, 97, (1, n), generator=g, device="cuda") for n in (200, 260)]
    kw = dict(numinittokens=4, maxlocallen=64, maxmidstates=32)
    raw, errors = dim_search.search_model(model, samples, **kw)
    assert model.model.fused_elementwise is True
    assert all(len(m._forward_hooks) == 0 for m in model.modules())
    # the same projections by hand: the input of a layer's attention is its normalised residual stream
    taken = [([], []) for _ in range(3)]
    hooks = []
    for i, layer in enumerate(model.model.layers):
        def grab(m, a, o, i=i):
            x = a[0]
            taken[i][0].append(F.linear(x, model.model.layers[i].self_attn.k_proj.weight))
            taken[i][1].append(F.linear(x, model.model.layers[i].self_attn.v_proj.weight))
        hooks.append(layer.self_attn.q_proj.register_forward_hook(grab))
    model.model.fused_elementwise = False
    from fourierattention_amd import DynamicCache, ExtraConfig, masks as pm
    for s_ in samples:
        ec = ExtraConfig(numinittokens=0, maxlocallen=s_.shape[1] + 1, maxmidstates=2, non_critical_dims_path=None,
                         non_critical_dims=pm.synthetic_masks(3, 2, 16, 8), max_position_embeddings=s_.shape[1] + 128,
                         num_key_value_heads=2, max_new_tokens=64, model_type="llama")
        model.model(s_, DynamicCache(ec, device="cuda"))
    for h in hooks:
        h.remove()
    raw2, errors2 = dim_search.search(taken, **kw)
    assert raw == raw2 and set(raw) == {"Layer_0", "Layer_1", "Layer_2"}
    for key in errors:
        assert torch.equal(errors[key], errors2[key])
    assert len(raw["Layer_0"]["self_attn.k_proj"]) == int(dim_search.percent_schedule(0, "k", 3) * 32)
