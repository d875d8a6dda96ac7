"""The benchmark's named configurations through the cache object on the GPU against the CPU restatement, each at
its literal size and convention:

* configuration 1: the reference's CPU-sized case with float32 storage (generic kernels, element-wise page pack);
* configuration 3 at its full batch of eight: two of the eight sequences against the restatement (sequences are
  independent there, so the other six need no oracle run);
* configuration 5 with the model's own ``max_position_embeddings = 131072``: the prompt fills the position range,
  ``maxtokens`` is clamped, the period pair is ``(130044, 130043)``, the transform drops the last mid row and the
  phase of every streamed token lies beyond the period of the update.
"""
import numpy as np
import pytest
import torch

from oracle import fourier_oracle as fo
from oracle.cache_oracle import OracleCache
from tests import helpers as H

pytestmark = pytest.mark.gpu

STAT_NAMES = ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average")


def _compare_rows(gpu_parts, cpu_parts, tag, dtype, rows, coef_tol):
    """Parts of the GPU cache at batch rows ``rows`` against the oracle's parts (whose batch is exactly those rows)."""
    for part in ("init", "compressed", "uncompressed", "local"):
        g, w = gpu_parts[f"{tag}_{part}"][rows], cpu_parts[f"{tag}_{part}"]
        assert tuple(g.shape) == tuple(w.shape), (tag, part, g.shape, w.shape)
        if part == "compressed":
            assert g.dtype == torch.float32
            err = np.linalg.norm(g.cpu().numpy() - w) / np.linalg.norm(w)
            assert err <= 1e-3 and err <= coef_tol, (tag, err)      # stated bound, then what the path really leaves
        else:
            assert g.dtype == dtype
            np.testing.assert_array_equal(g.float().cpu().numpy(), w.astype(np.float32))     # stored rows are copies


def _adopt_gpu_statistics(gpu, cpu, layer, rows, tol=(4e-3, 1e-2, 2e-3)):
    """Statistics within one unit of their storage type, then handed to the oracle so that the attention
    comparison sees identical statistics."""
    for name, t in zip(STAT_NAMES, tol * 2):
        g = getattr(gpu, name)[layer][rows].float().cpu().numpy()
        np.testing.assert_allclose(g, getattr(cpu, name)[layer], rtol=t, atol=t)
        getattr(cpu, name)[layer] = g


def _cfg(masks, **kw):
    from fourierattention_amd import ExtraConfig
    base = dict(numinittokens=4, non_critical_dims=masks, non_critical_dims_path=None, model_type="llama")
    base.update(kw)
    return ExtraConfig(**base)


def test_config1_float32_storage_full_size():
    """B=1, 24 query / 8 KV heads of 128 dims, 2048-token context, float32 storage, 256 states, 512-token window,
    rotary embedding on q and k, 64 of 128 dims per head compressed: prefill, streaming steps and attention."""
    from fourierattention_amd import DynamicCache, masks as pm
    dtype, B, Hq, Hkv, D, S = torch.float32, 1, 24, 8, 128, 2048
    m = pm.synthetic_masks(1, Hkv, D, 64, seed=0)
    cfg = _cfg(m, maxlocallen=512, maxmidstates=256, max_position_embeddings=131072, num_key_value_heads=Hkv, max_new_tokens=8)
    r = np.random.default_rng(0)
    cos, sin = fo.rope_tables(np.arange(S), D)
    k = H.to_dtype_np(fo.apply_rope(r.standard_normal((B, Hkv, S, D)), cos, sin), dtype)
    v = H.to_dtype_np(r.standard_normal((B, Hkv, S, D)), dtype)
    gpu, cpu = DynamicCache(cfg), OracleCache(cfg, masks=m, model_dtype="fp32")
    gpu.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    assert (gpu._book.t_x, gpu._book.t_c) == (cpu._t_x(), cpu.t_c) == (1540, 1540)
    assert gpu.curr_tokennum == cpu.curr_tokennum == [S - 4 - 512]
    rows = slice(None)
    _compare_rows(gpu.key_cache[0], cpu.key_cache[0], "k", dtype, rows, 2e-5)
    _compare_rows(gpu.value_cache[0], cpu.value_cache[0], "v", dtype, rows, 2e-5)
    assert gpu.k_scale[0].dtype == torch.float32 and gpu.k_layer_average[0].dtype == torch.float32
    assert gpu.kd_layer_average[0].dtype == torch.float16
    _adopt_gpu_statistics(gpu, cpu, 0, rows, tol=(2e-3, 1e-5, 2e-3))
    for step in range(2):
        cq, sq = fo.rope_tables(np.array([S + step]), D)
        kn = H.to_dtype_np(fo.apply_rope(r.standard_normal((B, Hkv, 1, D)), cq, sq), dtype)
        vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        q = H.to_dtype_np(fo.apply_rope(r.standard_normal((B, Hq, 1, D)), cq, sq), dtype)
        kp, vp = gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
        kw, vw = cpu.update(kn, vn, 0)
        _compare_rows(kp, kw, "k", dtype, rows, 2e-5)
        _compare_rows(vp, vw, "v", dtype, rows, 2e-5)
        assert gpu.get_seq_length(0) == cpu.get_seq_length(0) == S + step + 1
        want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
        got = gpu.decode_attention(H.to_gpu(q, dtype), 0, Hq, Hkv)
        assert got.dtype == torch.float32
        err = np.abs(got.cpu().numpy() - want).max()
        assert err <= 2e-4, (step, err)


def test_config3_full_batch_two_sequences_against_the_oracle():
    """B=8, 32768-token context, 32 query / 8 KV heads of 128 dims, bf16, 1024 states, 1024-token window: the
    first and the last sequence of the batch against the restatement run on those two sequences."""
    from fourierattention_amd import DynamicCache, masks as pm, synth
    dtype, B, Hq, Hkv, D, S = torch.bfloat16, 8, 32, 8, 128, 32768
    picked = [0, 7]
    m = pm.synthetic_masks(1, Hkv, D, 64, seed=0)
    cfg = _cfg(m, maxlocallen=1024, maxmidstates=1024, max_position_embeddings=131072, num_key_value_heads=Hkv, max_new_tokens=8)
    r = np.random.default_rng(3)
    cos, sin = fo.rope_tables(np.arange(S), D)
    k2 = H.to_dtype_np(fo.apply_rope(r.standard_normal((2, Hkv, S, D)), cos, sin), dtype)
    v2 = H.to_dtype_np(r.standard_normal((2, Hkv, S, D)), dtype)
    g = torch.Generator(device="cuda").manual_seed(5)
    tc, ts = synth.rope_tables(torch.arange(S), D)
    kg = synth.apply_rope(torch.randn((B, Hkv, S, D), generator=g, device="cuda"), tc.cuda(), ts.cuda()).to(dtype)
    vg = torch.randn((B, Hkv, S, D), generator=g, device="cuda").to(dtype)
    for i, b in enumerate(picked):
        kg[b], vg[b] = H.to_gpu(k2[i], dtype), H.to_gpu(v2[i], dtype)
    gpu, cpu = DynamicCache(cfg), OracleCache(cfg, masks=m, model_dtype="bf16")
    gpu.update(kg, vg, 0)
    cpu.update(k2, v2, 0)
    del kg, vg, k2, v2
    assert gpu._tables is not None
    assert (gpu._book.t_x, gpu._book.t_c) == (cpu._t_x(), cpu.t_c) == (31748, 31748)
    _compare_rows(gpu.key_cache[0], cpu.key_cache[0], "k", dtype, picked, 5e-4)
    _compare_rows(gpu.value_cache[0], cpu.value_cache[0], "v", dtype, picked, 5e-4)
    _adopt_gpu_statistics(gpu, cpu, 0, picked)
    cq, sq = fo.rope_tables(np.array([S]), D)
    kn2 = H.to_dtype_np(fo.apply_rope(r.standard_normal((2, Hkv, 1, D)), cq, sq), dtype)
    vn2 = H.to_dtype_np(r.standard_normal((2, Hkv, 1, D)), dtype)
    q2 = H.to_dtype_np(fo.apply_rope(r.standard_normal((2, Hq, 1, D)), cq, sq), dtype)
    kn = torch.randn((B, Hkv, 1, D), generator=g, device="cuda").to(dtype)
    vn = torch.randn((B, Hkv, 1, D), generator=g, device="cuda").to(dtype)
    q = torch.randn((B, Hq, 1, D), generator=g, device="cuda").to(dtype)
    for i, b in enumerate(picked):
        kn[b], vn[b], q[b] = H.to_gpu(kn2[i], dtype), H.to_gpu(vn2[i], dtype), H.to_gpu(q2[i], dtype)
    kp, vp = gpu.update(kn, vn, 0)
    kw, vw = cpu.update(kn2, vn2, 0)
    _compare_rows(kp, kw, "k", dtype, picked, 5e-4)
    _compare_rows(vp, vw, "v", dtype, picked, 5e-4)
    assert gpu.get_seq_length(0) == cpu.get_seq_length(0) == S + 1
    want = cpu.attend(q2, kw, vw, 0, Hq, Hkv)
    got = gpu.decode_attention(q, 0, Hq, Hkv)
    assert torch.isfinite(got).all()
    err = np.abs(got[picked].cpu().numpy() - want).max()
    assert err <= 2e-2 and err <= 2e-3, err


def test_config5_literal_position_limit_truncated_transform_and_wrapped_phase():
    """131072-token prompt with ``max_position_embeddings = 131072`` (the streaming configuration as the reference
    would run it: cache_utils_fourier.py:542-547, 566, 732-733; fourier_triton_valid4_v2.py:856-859), 2048 states,
    1024-token window, one sequence and two KV heads (three query heads each) to bound the oracle's time."""
    from fourierattention_amd import DynamicCache, masks as pm
    dtype, B, Hq, Hkv, D, S = torch.bfloat16, 1, 6, 2, 128, 131072
    m = pm.synthetic_masks(1, Hkv, D, 64, seed=0)
    cfg = _cfg(m, maxlocallen=1024, maxmidstates=2048, max_position_embeddings=131072, num_key_value_heads=Hkv,
               max_new_tokens=512)
    r = np.random.default_rng(4)
    cos, sin = fo.rope_tables(np.arange(S), D)
    k = H.to_dtype_np(fo.apply_rope(r.standard_normal((B, Hkv, S, D)), cos, sin), dtype)
    v = H.to_dtype_np(r.standard_normal((B, Hkv, S, D)), dtype)
    del cos, sin
    gpu, cpu = DynamicCache(cfg), OracleCache(cfg, masks=m, model_dtype="bf16")
    gpu.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    del k, v
    L = S - 4 - 1024
    assert gpu.maxtokens == cpu.maxtokens == 131072                                       # clamped at the position limit
    assert (gpu._book.t_x, gpu._book.t_c) == (cpu._t_x(), cpu.t_c) == (130044, 130043)   # int(1 / (1 / T_x)) = T_x - 1
    assert L == 130044 > gpu._book.t_c                      # the transform reads T_c rows: the last mid row is dropped
    assert gpu.curr_tokennum == cpu.curr_tokennum == [L]
    assert gpu._tables is not None
    rows = slice(None)
    _compare_rows(gpu.key_cache[0], cpu.key_cache[0], "k", dtype, rows, 5e-4)
    _compare_rows(gpu.value_cache[0], cpu.value_cache[0], "v", dtype, rows, 5e-4)
    _adopt_gpu_statistics(gpu, cpu, 0, rows)
    for step in range(3):
        kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)), dtype)
        kp, vp = gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
        kw, vw = cpu.update(kn, vn, 0)
        assert gpu.curr_tokennum == cpu.curr_tokennum == [L + step + 1]
        assert gpu.curr_tokennum[0] > gpu._book.t_c           # the phase of the update has wrapped past its period
        _compare_rows(kp, kw, "k", dtype, rows, 5e-4)
        _compare_rows(vp, vw, "v", dtype, rows, 5e-4)
        assert gpu.get_seq_length(0) == cpu.get_seq_length(0) == S + step + 1
        want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
        got = gpu.decode_attention(H.to_gpu(q, dtype), 0, Hq, Hkv).cpu().numpy()
        err = np.abs(got - want).max()
        assert err <= 2e-2 and err <= 2e-3, (step, err)
