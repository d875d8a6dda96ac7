"""The whole chain prefill -> statistics -> streaming step -> decode attention against the CPU restatement with
nothing handed from one side to the other, at the full lengths of the benchmark configurations, and the reference's
own decode arm of the attention forward restated over what ``update`` returns.

The other full-length tests compare the statistics within a unit of their storage type and then hand the GPU's
statistics to the oracle, so that the attention comparison sees identical inputs.  Here the oracle keeps its own:
the bound is the one stated for 16-bit attention against the fp32 / fp64 reference (2e-2)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import fourier_oracle as fo
from oracle.cache_oracle import OracleCache
from tests import helpers as H

pytestmark = pytest.mark.gpu

STAT_NAMES = ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average")


def _config(mask, Hkv, W, M, max_new=8, max_pos=1 << 20):
    from fourierattention_amd import ExtraConfig
    return ExtraConfig(numinittokens=4, maxlocallen=W, maxmidstates=M, non_critical_dims=mask, non_critical_dims_path=None,
                       max_position_embeddings=max_pos, num_key_value_heads=Hkv, max_new_tokens=max_new, model_type="llama")


def _ulps(got, want, dtype):
    """|got - want| in units of the last place of ``want`` in ``dtype`` (bf16: 8 bits of mantissa, fp16: 11, with
    fp16's subnormal spacing below 2^-14)."""
    bits = {torch.bfloat16: 8, torch.float16: 11, torch.float32: 24}[dtype]
    a = np.abs(want).astype(np.float64)
    expo = np.floor(np.log2(np.maximum(a, 1e-300)))
    if dtype == torch.float16:
        expo = np.maximum(expo, -14)
    return np.abs(got.astype(np.float64) - want) / 2.0 ** (expo - (bits - 1))


def _one_sequence(S, Hq, Hkv, D, W, M, dtype, mask, seed=0):
    """Prefill of one seeded sequence of S tokens on both sides, one streaming step, one query: returns what the two
    sides hold and compute, nothing exchanged between them."""
    from fourierattention_amd import DynamicCache
    cfg = _config(mask, Hkv, W, M)
    r = np.random.default_rng(seed)
    cos, sin = fo.rope_tables(np.arange(S), D)
    k = H.to_dtype_np(fo.apply_rope(r.standard_normal((1, Hkv, S, D)), cos, sin), dtype)
    v = H.to_dtype_np(r.standard_normal((1, Hkv, S, D)), dtype)
    gpu = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=mask, model_dtype=H.NP_ROUND[dtype])
    gpu.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    del k, v
    cq, sq = fo.rope_tables(np.array([S]), D)
    kn = H.to_dtype_np(fo.apply_rope(r.standard_normal((1, Hkv, 1, D)), cq, sq), dtype)
    vn = H.to_dtype_np(r.standard_normal((1, Hkv, 1, D)), dtype)
    q = H.to_dtype_np(fo.apply_rope(r.standard_normal((1, Hq, 1, D)), cq, sq), dtype)
    gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
    kw, vw = cpu.update(kn, vn, 0)
    want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
    got = gpu.decode_attention(H.to_gpu(q, dtype), 0, Hq, Hkv).cpu().numpy()
    return gpu, cpu, got, want


def test_config3_sequence_with_the_oracles_own_statistics():
    """BASELINE config 3 geometry, one of its sequences at full length (32768 tokens, 32 / 8 heads of 128 dims, 1024
    states, 1024-token window, bf16, 64 of 128 dims per head compressed)."""
    from fourierattention_amd import masks as pm
    mask = pm.synthetic_masks(1, 8, 128, 64, seed=0)
    gpu, cpu, got, want = _one_sequence(32768, 32, 8, 128, 1024, 1024, torch.bfloat16, mask)
    assert gpu._tables is not None and gpu.curr_tokennum == cpu.curr_tokennum
    err = np.abs(got - want).max()
    assert np.isfinite(got).all() and err <= 2e-2, err


def test_config4_sequence_at_65536_tokens():
    """BASELINE config 4 geometry, one of its sixteen sequences at full length: 64508 mid rows, 2016 pages (the
    longest chain of frame-to-frame rotations any configuration has), prefill + streaming step + attention."""
    from fourierattention_amd import masks as pm
    mask = pm.synthetic_masks(1, 8, 128, 64, seed=0)
    gpu, cpu, got, want = _one_sequence(65536, 32, 8, 128, 1024, 1024, torch.bfloat16, mask, seed=4)
    assert gpu._tables is not None and gpu.curr_tokennum == cpu.curr_tokennum == [64508 + 1]
    # stored rows bit for bit, coefficients as the matrix-core transform leaves them
    for tag, gp, cp in (("k", gpu.key_cache[0], cpu.key_cache[0]), ("v", gpu.value_cache[0], cpu.value_cache[0])):
        np.testing.assert_array_equal(gp[f"{tag}_uncompressed"].float().cpu().numpy(), cp[f"{tag}_uncompressed"].astype(np.float32))
        c, w = gp[f"{tag}_compressed"].cpu().numpy(), cp[f"{tag}_compressed"]
        assert np.linalg.norm(c - w) / np.linalg.norm(w) <= 5e-4
    err = np.abs(got - want).max()
    assert np.isfinite(got).all() and err <= 2e-2, err


@pytest.mark.parametrize("states", [1024, 512])
def test_reference_evaluation_settings_batch_one(states):
    """The settings the reference evaluates with (models/fourier.py:141-153, eval/eval_longbench_fourier.py:45-46):
    batch 1, 4 sink tokens, a local window of 1020, 1024 (or 512) states, and layer 31 of the mask it ships for
    Llama-3.1-8B at 32k (ragged heads, up to 127 stored dims: the wide kernel instance).  At batch 1 a workgroup's
    sixteen matrix-core columns hold the four query heads of one KV head only."""
    fx = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "masks_extract.json")))
    mask = {"Layer_0": fx["llama3.1-8b-fourier/compressed_dims_32k_1024states"]["layers"]["Layer_31"]["splithead"]}
    gpu, cpu, got, want = _one_sequence(32768, 32, 8, 128, 1020, states, torch.bfloat16, mask, seed=9)
    assert gpu._tables is not None and gpu.curr_tokennum == cpu.curr_tokennum == [32768 - 4 - 1020 + 1]
    assert gpu.period_reconstruct == cpu._t_x()
    err = np.abs(got - want).max()
    assert np.isfinite(got).all() and err <= 2e-2, err


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_statistics_at_full_length_in_units_of_the_last_place(dtype):
    """The statistics the prefill freezes (CACHE:564-569), at 32768 tokens, on columns that differ in offset and in
    scale (means between -3 and 3, deviations between 0.2 and 30): a kernel that returned zeros, or the wrong
    column, fails every one of them.  Bounds in units of the last place of the type each statistic is stored in
    (TRI:326, 461, CACHE:567).  The mean of the signal is an exact reduction rounded once: one unit.  The mean of
    the reconstruction is a sum of products whose operands are rounded to fp16 (2^-11 each, relative to the
    column's scale, not to the mean, which is a small difference of large terms), then rounded to fp16 itself.
    The scale is the quotient of two maximum deviations, each within a unit of its own type."""
    from fourierattention_amd import DynamicCache, masks as pm
    S, Hkv, D, W, M = 32768, 8, 128, 1024, 1024
    mask = pm.synthetic_masks(1, Hkv, D, 64, seed=2)
    cfg = _config(mask, Hkv, W, M)
    r = np.random.default_rng(7)
    off = r.uniform(-3, 3, (1, Hkv, 1, D))
    scl = r.uniform(0.2, 30.0, (1, Hkv, 1, D))
    data_scale = {"k": scl.reshape(-1), "v": scl[..., ::-1].reshape(-1)}
    k = H.to_dtype_np(r.standard_normal((1, Hkv, S, D)) * scl + off, dtype)
    v = H.to_dtype_np(r.standard_normal((1, Hkv, S, D)) * scl[..., ::-1] - off, dtype)
    gpu = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=mask, model_dtype=H.NP_ROUND[dtype])
    gpu.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    scale_dtype = torch.float16 if dtype == torch.float16 else torch.float32
    model_eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11      # half a unit, relative
    worst = {}
    for tag in ("k", "v"):
        cols = getattr(gpu, f"{tag}_non_critical_dims")[0].cpu().numpy()
        col_scale = data_scale[tag][cols][None, :]
        # mean of the signal
        g, w = getattr(gpu, f"{tag}_layer_average")[0], getattr(cpu, f"{tag}_layer_average")[0]
        assert g.dtype == dtype and tuple(g.shape) == w.shape and np.abs(w).max() > 1.0
        worst[f"{tag}_layer_average"] = u = _ulps(g.float().cpu().numpy(), w, dtype).max()
        assert u <= 1.0, (tag, u)
        # mean of the reconstruction
        g, w = getattr(gpu, f"{tag}d_layer_average")[0], getattr(cpu, f"{tag}d_layer_average")[0]
        assert g.dtype == torch.float16 and tuple(g.shape) == w.shape and np.abs(w).max() > 1.0
        e = np.abs(g.float().cpu().numpy() - w) / (2.0 ** -11 * (np.abs(w) + col_scale))
        worst[f"{tag}d_layer_average"] = e.max()
        assert e.max() <= 3.0, (tag, e.max())
        # scale
        g, w = getattr(gpu, f"{tag}_scale")[0], getattr(cpu, f"{tag}_scale")[0]
        assert g.dtype == scale_dtype and tuple(g.shape) == w.shape and w.min() > 0.05
        e = np.abs(g.float().cpu().numpy() - w) / w
        worst[f"{tag}_scale"] = e.max()
        assert e.max() <= 2 * model_eps + 3 * 2.0 ** -11, (tag, e.max())
    print("worst deviations:", {n: float(x) for n, x in worst.items()})


@pytest.mark.parametrize("prompt,M", [(3000, 256), (700, 64)])
def test_reference_decode_arm_over_the_returned_parts(prompt, M):
    """The decode arm of the reference's attention forward (MODEL:641-660) restated word for word over what
    ``update`` returns and over the cache's attribute lists: index the mapping, join sink and window, read the
    statistics and the index lists of the layer, call ``triton_fourier_attn``.  A model that keeps that body and only
    swaps the imports runs exactly this.  It must agree with the cache's own ``decode_attention`` (same arithmetic,
    other buffers: the parts are materialised, the mid rows re-paged or read token-major) and with the oracle."""
    from fourierattention_amd import DynamicCache, CacheParts, triton_fourier_attn
    dtype, B, Hq, Hkv, D, W = torch.bfloat16, 2, 8, 2, 128, 64
    from tests.test_gpu_cache import _masks
    mask = _masks(1, Hkv, D, [64, 40], [64, 96], seed=3)
    cfg = _config(mask, Hkv, W, M, max_new=16, max_pos=1 << 17)
    r = np.random.default_rng(21)
    k = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype)
    v = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)) + 0.1, dtype)
    past_key_value = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=mask, model_dtype=H.NP_ROUND[dtype])
    past_key_value.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    layer_idx, num_heads, num_key_value_heads, head_dim, bsz, q_len = 0, Hq, Hkv, D, B, 1
    for step in range(3):
        kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)) * 1.5, dtype)
        query_states = H.to_gpu(q, dtype)
        key_states, value_states = past_key_value.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), layer_idx, None)
        kw, vw = cpu.update(kn, vn, 0)
        assert isinstance(key_states, CacheParts)
        assert not (key_states["k_init"] is None and key_states["k_compressed"] is None and key_states["k_uncompressed"] is None)
        attn_output = triton_fourier_attn(
            q=query_states.transpose(1, 2).view(bsz, q_len, num_heads * head_dim).contiguous(),
            k_il=torch.cat([key_states["k_init"], key_states["k_local"]], dim=1).contiguous(),
            v_il=torch.cat([value_states["v_init"], value_states["v_local"]], dim=1).contiguous(),
            k_mc=key_states["k_compressed"], v_mc=value_states["v_compressed"],
            k_mn=key_states["k_uncompressed"], v_mn=value_states["v_uncompressed"],
            avg_k_u=past_key_value.k_layer_average[layer_idx], avg_k_d=past_key_value.kd_layer_average[layer_idx],
            scale_k=past_key_value.k_scale[layer_idx],
            avg_v_u=past_key_value.v_layer_average[layer_idx], avg_v_d=past_key_value.vd_layer_average[layer_idx],
            scale_v=past_key_value.v_scale[layer_idx],
            kc_list=past_key_value.k_non_critical_dims[layer_idx], kc_h_list=past_key_value.k_non_critical_head_dims[layer_idx],
            kn_list=past_key_value.k_critical_dims[layer_idx], kn_h_list=past_key_value.k_critical_head_dims[layer_idx],
            vc_list=past_key_value.v_non_critical_dims[layer_idx], vc_h_list=past_key_value.v_non_critical_head_dims[layer_idx],
            vn_list=past_key_value.v_critical_dims[layer_idx], vn_h_list=past_key_value.v_critical_head_dims[layer_idx],
            num_head_q=num_heads, num_head_kv=num_key_value_heads, seq_len_m=key_states["k_uncompressed"].size(1),
            T=past_key_value.maxtokens - past_key_value.numinittokens - past_key_value.maxlocallen)
        assert attn_output.dtype == torch.float32 and tuple(attn_output.shape) == (bsz, num_heads, 1, head_dim)
        own = past_key_value.decode_attention(query_states, layer_idx, num_heads, num_key_value_heads)
        want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
        assert (attn_output - own).abs().max().item() <= 5e-3
        assert np.abs(attn_output.cpu().numpy() - want).max() <= 2e-2
        # what the forward does with it (MODEL:661-663)
        out = attn_output.transpose(1, 2).contiguous().view(bsz, q_len, -1).to(query_states.dtype)
        assert tuple(out.shape) == (bsz, q_len, num_heads * head_dim)
