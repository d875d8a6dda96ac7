#!/usr/bin/env python3
"""Benchmark of the Fourier-cache decode hot path on one MI355X.

One "step" = one decode-attention pass of one layer over a resident Fourier cache
(BASELINE config 3: B=8, ctx 32768, Hq=32, Hkv=8, D=128, 4 sink + 1024 window rows full,
64 of 128 dims per head stored as M=1024 coefficients, bf16).  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# max_position_embeddings of Llama-3.1-8B and Llama-3.2-3B: the cache clamps prompt + max_new_tokens to it
# (cache_utils_fourier.py:542).  Only the 131072-token prompt of configuration 5 reaches it: there the periods are
# T_x = 130044 and T_c = int(1 / (1 / T_x)) = 130043, as the reference would run that configuration.
MODEL_MAX_POSITIONS = 131072

WORKLOADS = {
    # name: B, ctx, Hq, Hkv, D, I, W, M, compressed dims per head, max_new_tokens
    "config3_decode_attn_8b_32k": dict(B=8, ctx=32768, Hq=32, Hkv=8, D=128, I=4, W=1024, M=1024, cper=64, max_new=128),
    # the per-layer attention of BASELINE configs 4 and 5 (their end-to-end runs are under --e2e)
    "config4_decode_attn_8b_64k": dict(B=16, ctx=65536, Hq=32, Hkv=8, D=128, I=4, W=1024, M=1024, cper=64, max_new=128),
    "config5_decode_attn_3b_128k": dict(B=4, ctx=131072, Hq=24, Hkv=8, D=128, I=4, W=1024, M=2048, cper=64, max_new=512),
    "config1_cpu_geometry_3b_2k": dict(B=1, ctx=2048, Hq=24, Hkv=8, D=128, I=4, W=512, M=256, cper=64, max_new=64),
}
# Config 3 with the head-by-head counts of three layers of the mask the reference ships for this model and
# context (compressed_dims_32k_1024states_splithead.json: compressed dims per KV head, K and V; which dims of a head
# they are is drawn from a seed, the kernels only see the counts and the gathers)
_RAGGED = {
    "layer0": ([121, 124, 103, 127, 128, 117, 83, 118], [115, 122, 119, 126, 122, 125, 122, 121]),
    "layer15": ([83, 116, 117, 96, 122, 88, 116, 81], [120, 128, 110, 111, 8, 122, 128, 92]),
    "layer31": ([47, 86, 44, 60, 75, 64, 69, 67], [82, 127, 124, 61, 114, 1, 81, 126]),
}
for _name, (_kc, _vc) in _RAGGED.items():
    WORKLOADS[f"config3_ragged_{_name}"] = dict(WORKLOADS["config3_decode_attn_8b_32k"], cper=None, kc_heads=_kc, vc_heads=_vc)
# The settings the reference itself evaluates with (models/fourier.py:141-153, eval/eval_longbench_fourier.py:45-46,
# 72, 86): batch 1, 4 sink tokens, a window of 1020, 512 / 1024 / 2048 states, with the head-by-head counts of its own
# Llama-3.1-8B mask (layers 0, 15 and 31 at 1024 states; layer 15 at the other two)
_REF_EVAL = dict(B=1, ctx=32768, Hq=32, Hkv=8, D=128, I=4, W=1020, cper=None, max_new=128)
for _name, (_kc, _vc) in _RAGGED.items():
    WORKLOADS[f"ref_eval_b1_32k_m1024_{_name}"] = dict(_REF_EVAL, M=1024, kc_heads=_kc, vc_heads=_vc)
for _m in (512, 2048):
    WORKLOADS[f"ref_eval_b1_32k_m{_m}_layer15"] = dict(_REF_EVAL, M=_m, kc_heads=_RAGGED["layer15"][0], vc_heads=_RAGGED["layer15"][1])
# what the default run times besides its headline workload (one line each in "other_workloads")
OTHER_WORKLOADS = ["config3_ragged_layer0", "config3_ragged_layer15", "config3_ragged_layer31", "config4_decode_attn_8b_64k",
                   "config5_decode_attn_3b_128k"] + [n for n in WORKLOADS if n.startswith("ref_eval_")]


def compressed_counts(w):
    """Compressed dims of a whole row (all KV heads), K and V."""
    if w.get("kc_heads"):
        return sum(w["kc_heads"]), sum(w["vc_heads"])
    return w["cper"] * w["Hkv"], w["cper"] * w["Hkv"]


def workload_masks(w, layers, seed):
    from fourierattention_amd import masks
    if w.get("kc_heads"):
        return masks.synthetic_masks(layers, w["Hkv"], w["D"], w["kc_heads"], w["vc_heads"], seed=seed)
    return masks.synthetic_masks(layers, w["Hkv"], w["D"], w["cper"], seed=seed)


def algorithmic_bytes(w, coef_bytes=4, elem_bytes=2):
    """Compulsory HBM bytes of one decode-attention pass (per layer, whole batch):
    sink+window K,V (all dims) + stored dims of the mid rows (K,V) + coefficients (K,V) + q + out."""
    L = w["ctx"] - w["I"] - w["W"]
    hd = w["Hkv"] * w["D"]
    ck, cv = compressed_counts(w)
    per_b = 2 * (w["I"] + w["W"]) * hd * elem_bytes + L * (2 * hd - ck - cv) * elem_bytes + w["M"] * (ck + cv) * coef_bytes \
        + 2 * w["Hq"] * w["D"] * elem_bytes
    return per_b * w["B"]


def build_cache(w, dtype, device, seed=0, layers=1):
    """Random K/V of the workload's shape pushed through the cache's own prefill (split, spectral
    compression, statistics), so the timed decode reads exactly what a real prompt leaves behind."""
    from fourierattention_amd import DynamicCache, ExtraConfig, synth
    m = workload_masks(w, layers, seed)
    cfg = ExtraConfig(numinittokens=w["I"], maxlocallen=w["W"], maxmidstates=w["M"], non_critical_dims=m,
                      non_critical_dims_path=None, max_position_embeddings=MODEL_MAX_POSITIONS, num_key_value_heads=w["Hkv"],
                      max_new_tokens=w["max_new"], model_type="llama")
    cache = DynamicCache(cfg, device=device)
    g = torch.Generator(device=device).manual_seed(seed)
    B, Hkv, S, D = w["B"], w["Hkv"], w["ctx"], w["D"]
    cos, sin = synth.rope_tables(torch.arange(S), D)
    cos, sin = cos.to(device), sin.to(device)
    for layer in range(layers):
        k = torch.randn((B, Hkv, S, D), generator=g, device=device, dtype=torch.float32)
        k = synth.apply_rope(k, cos, sin).to(dtype)
        v = torch.randn((B, Hkv, S, D), generator=g, device=device, dtype=torch.float32).to(dtype)
        cache.update(k, v, layer)
        del k, v
    cq, sq = synth.rope_tables(torch.tensor([S]), D)
    q = torch.randn((B, w["Hq"], 1, D), generator=g, device=device, dtype=torch.float32)
    q = synth.apply_rope(q, cq.to(device), sq.to(device)).to(dtype)
    kn = synth.apply_rope(torch.randn((B, Hkv, 1, D), generator=g, device=device), cq.to(device), sq.to(device)).to(dtype)
    vn = torch.randn((B, Hkv, 1, D), generator=g, device=device).to(dtype)
    return cache, q, kn, vn


def attn_step_bench(name, device, steps=100, warmup=10):
    """Decode attention of one layer on workload ``name`` (cache built through its own prefill): time per step between
    events around ``steps`` calls, the compulsory bytes and what fraction of the HBM peak that is."""
    from fourierattention_amd import _lib
    w = WORKLOADS[name]
    cache, q, kn, vn = build_cache(w, torch.bfloat16, device)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # warm-up by time: at least ``warmup`` steps and 40 ms of them (the first tens of milliseconds after an idle
    # period run slower than the steady state of a decode loop)
    done_ms = 0.0
    while done_ms < 40.0:
        e0.record()
        for _ in range(warmup):
            out = cache.decode_attention(q, 0, w["Hq"], w["Hkv"])
        e1.record()
        torch.cuda.synchronize()
        done_ms += e0.elapsed_time(e1)
    e0.record()
    for _ in range(steps):
        out = cache.decode_attention(q, 0, w["Hq"], w["Hkv"])
    e1.record()
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    ms = e0.elapsed_time(e1) / steps
    nbytes = algorithmic_bytes(w)
    return {"us_per_step": round(ms * 1e3, 2), "algorithmic_bytes": nbytes, "GB_s": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "batch": w["B"], "context": w["ctx"],
            "window": w["W"], "coeff_rows": w["M"], "merge_inside_mid_row_launch": bool(_lib.load().fa_decode_attn_last_fused())}


def parity_check(device):
    """Small seeded case through the GPU cache and through the CPU oracle; returns max-abs error.  Part of the
    CPU-baseline leg: ``--no-cpu-baseline`` skips it together with the timing of the oracle."""
    from oracle.cache_oracle import OracleCache
    from oracle import fourier_oracle as fo
    from fourierattention_amd import DynamicCache, ExtraConfig, masks
    B, Hq, Hkv, D, S = 2, 8, 2, 128, 700
    m = masks.synthetic_masks(1, Hkv, D, 64, seed=3)
    cfg = ExtraConfig(numinittokens=4, maxlocallen=64, maxmidstates=64, non_critical_dims=m, non_critical_dims_path=None,
                      max_position_embeddings=MODEL_MAX_POSITIONS, num_key_value_heads=Hkv, max_new_tokens=16, model_type="llama")
    r = np.random.default_rng(0)
    rd = lambda a: fo.round_bf16(a).astype(np.float64)
    k, v = rd(r.standard_normal((B, Hkv, S, D))), rd(r.standard_normal((B, Hkv, S, D)))
    kn, vn, q = rd(r.standard_normal((B, Hkv, 1, D))), rd(r.standard_normal((B, Hkv, 1, D))), rd(r.standard_normal((B, Hq, 1, D)))
    g = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16).to(device)
    gpu = DynamicCache(cfg, device=device)
    cpu = OracleCache(cfg, masks=m, model_dtype="bf16")
    gpu.update(g(k), g(v), 0); cpu.update(k, v, 0)
    gpu.update(g(kn), g(vn), 0); kw, vw = cpu.update(kn, vn, 0)
    got = gpu.decode_attention(g(q), 0, Hq, Hkv).float().cpu().numpy()
    want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
    return float(np.abs(got - want).max())


def _oracle_step_times(w, batch, dtype_name, reps, warm):
    """Seconds per decode step (cache update + attention of one layer) of the CPU restatement on workload ``w`` with
    ``batch`` sequences, after its own prefill of the synthetic prompt."""
    from oracle.cache_oracle import OracleCache
    from oracle import fourier_oracle as fo
    from fourierattention_amd import ExtraConfig, masks
    m = masks.synthetic_masks(1, w["Hkv"], w["D"], w["cper"], seed=0)
    cfg = ExtraConfig(numinittokens=w["I"], maxlocallen=w["W"], maxmidstates=w["M"], non_critical_dims=m,
                      non_critical_dims_path=None, max_position_embeddings=MODEL_MAX_POSITIONS, num_key_value_heads=w["Hkv"],
                      max_new_tokens=w["max_new"], model_type="llama")
    r = np.random.default_rng(0)
    B, Hq, Hkv, D, S = batch, w["Hq"], w["Hkv"], w["D"], w["ctx"]
    cos, sin = fo.rope_tables(np.arange(S), D)
    rd = lambda a: fo.round_to(a, dtype_name).astype(np.float64)
    k = rd(fo.apply_rope(r.standard_normal((B, Hkv, S, D)), cos, sin))
    v = rd(r.standard_normal((B, Hkv, S, D)))
    cache = OracleCache(cfg, masks=m, model_dtype=dtype_name)
    cache.update(k, v, 0)
    del k, v
    cq, sq = fo.rope_tables(np.array([S]), D)
    times = []
    for rep in range(warm + reps):
        kn = rd(fo.apply_rope(r.standard_normal((B, Hkv, 1, D)), cq, sq))
        vn = rd(r.standard_normal((B, Hkv, 1, D)))
        q = rd(fo.apply_rope(r.standard_normal((B, Hq, 1, D)), cq, sq))
        t0 = time.perf_counter()
        kw, vw = cache.update(kn, vn, 0)
        cache.attend(q, kw, vw, 0, Hq, Hkv)
        times.append(time.perf_counter() - t0)
    return sorted(times[warm:])


def cpu_baseline():
    """The CPU restatement of the reference path (numpy, float64 arithmetic) timed on the host: one layer, one decode
    step = cache update (rank-1 coefficient update, eviction) + attention.  The figure is taken on a bounded sample
    of the benchmark's own workload - config 3 with ONE of its eight sequences (32k context, bf16-rounded inputs) -
    and BASELINE config 1 (the reference's CPU-sized case) is timed beside it."""
    w3 = WORKLOADS["config3_decode_attn_8b_32k"]
    t3 = _oracle_step_times(w3, 1, "bf16", reps=3, warm=1)
    med3 = t3[len(t3) // 2]
    bytes3 = algorithmic_bytes(w3) // w3["B"]
    w1 = WORKLOADS["config1_cpu_geometry_3b_2k"]
    t1 = _oracle_step_times(w1, w1["B"], "fp32", reps=10, warm=3)
    med1 = t1[len(t1) // 2]
    bytes1 = algorithmic_bytes(w1, coef_bytes=4, elem_bytes=4)
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = 1
    return {"value": round(bytes3 / med3 / 1e9, 4), "unit": "GB/s", "cores": int(threads), "kind": "port",
            "cores_note": "threads of the BLAS pool numpy's contractions run on; the rest of the restatement is single-threaded numpy",
            "sample": f"config 3 with 1 of its 8 sequences (ctx 32768, Hq=32, Hkv=8, D=128, bf16-rounded inputs, M=1024, W=1024): "
                      f"update + attention of one layer, one decode step, median of 3 after 1 warm-up = {med3 * 1e3:.1f} ms "
                      f"(min {t3[0] * 1e3:.1f} ms), {bytes3} algorithmic bytes; host has {os.cpu_count()} logical CPUs",
            "config1": {"value": round(bytes1 / med1 / 1e9, 4), "unit": "GB/s",
                        "sample": f"config 1 (B=1, ctx 2048, Hq=24, Hkv=8, D=128, fp32 inputs, M=256, W=512): median of 10 after 3 "
                                  f"warm-ups = {med1 * 1e3:.2f} ms (min {t1[0] * 1e3:.2f} ms), {bytes1} algorithmic bytes"}}


KERNEL_SOURCES = ("fa_decode.hip", "fa_decode_mfma.h", "fa_decode_fused.h", "fa_decode_mid_launch.h", "fa_mfma_util.h", "fa_common.h")


def kernel_source_digest():
    """sha256 over the sources of the decode kernels: ties a counter summary under profiles/ to the code it was
    taken from."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "fourierattention_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic(dom, workload):
    """HBM bytes per launch of the dominant kernel from the hardware-counter summary under profiles/ (rocprofv3
    --pmc runs cannot happen inside this process).  The summary names the digest of the kernel sources it was
    taken from; if the sources have changed since, the figure is stale and is not reported."""
    tpath = os.path.join(ROOT, "profiles", "decode_mid_rows_traffic.txt")
    if dom != "mid_rows" or not workload.startswith("config3") or not os.path.exists(tpath):
        return None, None
    traffic, digest = None, None
    for line in open(tpath):
        if line.startswith("hbm_bytes_per_launch:"):
            traffic = int(float(line.split(":", 1)[1]))
        if line.startswith("kernel_source_digest:"):
            digest = line.split(":", 1)[1].strip()
    now = kernel_source_digest()
    if digest != now:
        return None, f"profiles/decode_mid_rows_traffic.txt is stale: taken at kernel sources {digest}, now {now}"
    return traffic, f"profiles/decode_mid_rows_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, kernel sources {digest})"


def compress_bench(device, reps=20):
    """Spectral compression of one tensor of a 32k prompt (B=1, 32768 tokens, 8 KV heads x 128 dims of which
    64 per head are compressed, 1024 coefficient rows, bf16): matrix-core roofline of the whole call
    (basis table, gather/pack, GEMM, chunk reduction)."""
    from fourierattention_amd import ops
    L, HD, Mc, N = 32768, 1024, 512, 512
    g = torch.Generator(device=device).manual_seed(0)
    x = torch.randn((1, L, HD), device=device, generator=g).to(torch.bfloat16)
    cols = torch.sort(torch.randperm(HD, device=device, generator=g)[:Mc])[0].int()
    out = torch.empty((1, 2 * N, Mc), device=device)
    for _ in range(3):
        ops.mat_fourier(x, N, L, 0, cols=cols, out=out)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        ops.mat_fourier(x, N, L, 0, cols=cols, out=out)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    flops = 2.0 * (2 * N) * L * Mc
    tf = flops / (ms * 1e-3) / 1e12
    out_d = {"workload": "config2_compress_32k", "ms_per_tensor": round(ms, 5), "bound": "mfma", "achieved": round(tf, 1),
             "peak": 2500.0, "unit": "TFLOP/s", "frac": round(tf / 2500.0, 4), "algorithmic_flops": flops,
             "operand_dtype": "f16 (basis and data), fp32 accumulation"}
    # What the cache itself calls at prefill for one tensor (cache_utils_fourier.py:560-565): one read of the rows
    # gives the pages of the stored dims, the coefficients of the compressed dims and their column statistics
    try:
        from fourierattention_amd.midstore import MidStore
        Hkv, D = 8, 128
        head_of = (cols.long() // D)
        c_h = [0] + [int((head_of <= h).sum()) for h in range(Hkv)]
        keep = torch.ones(HD, dtype=torch.bool, device=device)
        keep[cols.long()] = False
        n_list = torch.nonzero(keep).flatten().int()
        n_head = (n_list.long() // D)
        n_h = [0] + [int((n_head <= h).sum()) for h in range(Hkv)]
        store = MidStore(1, n_list, torch.tensor(n_h, dtype=torch.int32, device=device), n_h, Hkv, D, L, torch.bfloat16,
                         device, False)
        c_h32 = torch.tensor(c_h, dtype=torch.int32, device=device)
        call = lambda: store.pack_and_compress(x, 0, L, L, cols, c_h32, N, L, torch.bfloat16)
        if call() is not None:
            for _ in range(2):
                call()
            e0.record()
            for _ in range(reps):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms2 = e0.elapsed_time(e1) / reps
            out_d["cache_prefill_call"] = {
                "entry_point": "fa_prefill_compress", "ms_per_tensor": round(ms2, 5),
                "does": "pages of the 512 stored dims + 1024 x 512 coefficients + column statistics from one read of the rows",
                "TFLOP_s": round(flops / (ms2 * 1e-3) / 1e12, 1), "frac_of_f16_peak": round(flops / (ms2 * 1e-3) / 1e12 / 2500.0, 4),
                "bytes_moved": int(L * HD * 2 + L * (HD - Mc) * 2 + 2 * N * Mc * 4)}
    except Exception as exc:   # the figure above stands on its own
        out_d["cache_prefill_call"] = {"error": f"{type(exc).__name__}: {exc}"}
    return out_d


def prefill_attn_bench(device, S=32768, reps=5):
    """Exact causal attention of the prompt pass (one layer of Llama-3.1-8B geometry, B=1, bf16) on the matrix-core
    kernel, both launches (the transposing pass over V and the attention itself): matrix-core roofline."""
    from fourierattention_amd import ops
    B, Hq, Hkv, D = 1, 32, 8, 128
    g = torch.Generator(device=device).manual_seed(0)
    q = torch.randn((B, Hq, S, D), device=device, generator=g).to(torch.bfloat16)
    k = torch.randn((B, S, Hkv * D), device=device, generator=g).to(torch.bfloat16)
    v = torch.randn((B, S, Hkv * D), device=device, generator=g).to(torch.bfloat16)
    for _ in range(2):
        ops.prefill_attention(q, k, v, Hkv)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        ops.prefill_attention(q, k, v, Hkv)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    flops = 4.0 * D * Hq * B * S * (S + 1) / 2     # QK^T and PV over the causal half
    tf = flops / (ms * 1e-3) / 1e12
    return {"workload": f"prompt attention, B=1, {S} tokens, Hq=32, Hkv=8, D=128, causal", "ms_per_layer": round(ms, 4),
            "bound": "mfma", "achieved": round(tf, 1), "peak": 2500.0, "unit": "TFLOP/s", "frac": round(tf / 2500.0, 4),
            "algorithmic_flops": flops, "operand_dtype": "bf16, fp32 accumulation"}


E2E = {
    # BASELINE configs 4 and 5: a random-init decoder with the Fourier cache on every layer
    "config4_e2e_8b_64k": dict(preset="llama-3.1-8b", B=16, prompt=65536, new=128, I=4, W=1024, M=1024, cper=64),
    "config5_e2e_3b_128k": dict(preset="llama-3.2-3b", B=4, prompt=131072, new=512, I=4, W=1024, M=2048, cper=64),
    # the reference's evaluation settings (one sequence, window 1020, 1024 states; about three quarters of the dims
    # compressed, as in its mask for this model)
    "refeval_e2e_8b_32k": dict(preset="llama-3.1-8b", B=1, prompt=32768, new=128, I=4, W=1020, M=1024, cper=96),
}


def e2e_bench(name, device, steps=None, warmup=3):
    """Greedy decode of a random-init LLaMA with the Fourier cache on every layer.  The prompt's K/V are
    synthetic (random rows pushed through the cache's own prefill, layer by layer): the quadratic prompt pass
    of a random model is not what this figure is about.  Every timed step is a full model step: embedding,
    all layers (projections, rotary embedding, cache update, Fourier attention, MLP), final norm, LM head,
    argmax."""
    from fourierattention_amd import DynamicCache, ExtraConfig, masks
    from fourierattention_amd.llama import PRESETS, LlamaConfig, random_init, synthetic_prefill
    e = E2E[name]
    cfg = LlamaConfig(**PRESETS[e["preset"]])
    steps = steps or e["new"]
    m = masks.synthetic_masks(cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.head_dim, e["cper"], seed=0)
    ec = ExtraConfig(numinittokens=e["I"], maxlocallen=e["W"], maxmidstates=e["M"], non_critical_dims=m,
                     non_critical_dims_path=None, max_position_embeddings=MODEL_MAX_POSITIONS,
                     num_key_value_heads=cfg.num_key_value_heads, max_new_tokens=e["new"] + warmup + 8, model_type="llama")
    model = random_init(cfg, torch.bfloat16, device, seed=0)
    model.model.fuse_projections()
    if not os.environ.get("FA_BENCH_LIBRARY_GEMM"):   # (set to time the decode with the GEMM library's projections)
        model.model.pack_projections()
    cache = DynamicCache(ec, device=device)
    cache.defer_coef_update = os.environ.get("FA_BENCH_UPDATE_INSIDE_ATTENTION", "0") == "1"   # (comparison)
    cache.fuse_decode = os.environ.get("FA_BENCH_NO_FUSE", "0") != "1"                         # (comparison)
    t0 = time.perf_counter()
    synthetic_prefill(cache, cfg, e["B"], e["prompt"], torch.bfloat16, device, seed=0)
    torch.cuda.synchronize()
    fill_s = time.perf_counter() - t0
    g = torch.Generator(device=device).manual_seed(1)
    ids = torch.randint(0, cfg.vocab_size, (e["B"], 1), generator=g, device=device)
    with torch.no_grad():
        for _ in range(warmup):
            ids = model(input_ids=ids, past_key_values=cache, num_logits_to_keep=1).logits[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            ids = model(input_ids=ids, past_key_values=cache, num_logits_to_keep=1).logits[:, -1].argmax(-1, keepdim=True)
        issued = time.perf_counter() - t0   # the host has queued every launch; what is left is the device catching up
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    assert cache.get_seq_length() == e["prompt"] + warmup + steps
    hd = cfg.num_key_value_heads * cfg.head_dim
    held = 0
    for layer in cache._layers:
        for t in (layer.k, layer.v):
            held += t.il.numel() * t.il.element_size() + t.coef.numel() * 4 + t.mid.data.numel() * t.mid.data.element_size()
    ctx = e["prompt"] + warmup + steps
    full = 2 * ctx * hd * 2 * cfg.num_hidden_layers * e["B"]
    L = ctx - e["I"] - e["W"]
    ck = e["cper"] * cfg.num_key_value_heads
    used = (2 * (e["I"] + e["W"]) * hd * 2 + 2 * L * (hd - ck) * 2 + 2 * e["M"] * ck * 4) * cfg.num_hidden_layers * e["B"]
    return {"metric": "end-to-end greedy decode tokens/s, random-init model, Fourier cache on every layer",
            "value": round(e["B"] * steps / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(dt / steps * 1e3, 3), "host_issue_ms_per_step": round(issued / steps * 1e3, 3),
            "higher_is_better": True, "dtype": "bf16",
            "data": "synthetic (random weights, random prompt K/V through the cache's prefill)",
            "config": {"workload": name, "model": e["preset"], "batch": e["B"], "prompt": e["prompt"],
                       "new_tokens": steps, "sink": e["I"], "window": e["W"], "coeff_rows": e["M"],
                       "compressed_dims_per_head": e["cper"], "T_x": cache.period_reconstruct, "T_c": cache._book.t_c,
                       "max_position_embeddings": MODEL_MAX_POSITIONS},
            "kv_cache_bytes": {"full_bf16": full, "fourier_in_use": used, "fourier_allocated": held,
                               "reduction_in_use": round(full / used, 3)},
            "synthetic_prefill_s": round(fill_s, 2),
            # the decode projections run on a second copy of the layer weights in matrix-core order
            # (LlamaModel.pack_projections): what that copy costs in memory
            "packed_projection_weights_bytes": sum(w.data.numel() * w.data.element_size()
                                                   for layer in model.model.layers for w in layer._packed.values())}


def prefill_e2e_bench(device, preset="llama-3.1-8b", prompt=32768, reps=2):
    """The prompt pass of a random-init decoder end to end (B=1): embedding, every layer with its projections, rotary
    embedding, exact causal attention on the matrix-core kernel, Fourier-cache prefill (split, page pack, spectral
    compression, statistics) and MLP, final norm, LM head of the last position.  The reference publishes this
    latency for Llama-3.1-8B / Llama-3.2-3B as a plot (hardware unstated); the value read off it is quoted beside."""
    from fourierattention_amd import DynamicCache, ExtraConfig, masks
    from fourierattention_amd.llama import PRESETS, LlamaConfig, random_init
    cfg = LlamaConfig(**PRESETS[preset])
    m = masks.synthetic_masks(cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.head_dim, 64, seed=0)
    ec = ExtraConfig(numinittokens=4, maxlocallen=1024, maxmidstates=1024, non_critical_dims=m, non_critical_dims_path=None,
                     max_position_embeddings=MODEL_MAX_POSITIONS, num_key_value_heads=cfg.num_key_value_heads,
                     max_new_tokens=128, model_type="llama")
    model = random_init(cfg, torch.bfloat16, device, seed=0)
    model.model.fuse_projections()
    g = torch.Generator(device=device).manual_seed(2)
    ids = torch.randint(0, cfg.vocab_size, (1, prompt), generator=g, device=device)
    times = []
    torch.cuda.reset_peak_memory_stats(device)
    with torch.no_grad():
        for rep in range(reps + 1):
            cache = DynamicCache(ec, device=device)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = model(input_ids=ids, past_key_values=cache, num_logits_to_keep=1)
            nxt = out.logits[:, -1].argmax(-1)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert cache.get_seq_length() == prompt and torch.isfinite(out.logits).all()
            del cache, out
    best = min(times[1:])
    published = {("llama-3.1-8b", 16384): 0.75, ("llama-3.1-8b", 32768): 1.8, ("llama-3.2-3b", 32768): 1.03}
    return {"model": preset, "batch": 1, "prompt": prompt, "seconds": round(best, 4), "first_call_seconds": round(times[0], 4),
            "tokens_per_s": round(prompt / best, 1), "peak_memory_GB": round(torch.cuda.max_memory_allocated(device) / 1e9, 2),
            "reference_published_seconds": published.get((preset, prompt)),
            "reference_note": "read off the reference's efficiency plot (about +-0.1 s), hardware not stated there"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-priming", action="store_true",
                    help="skip the 60 ms of untimed steps that bring an idle device to the state of a running decode loop "
                         "before the warm-up steps (comparison: the first 30 ms or so after an idle period run about 8 %% slower)")
    ap.add_argument("--workload", default="config3_decode_attn_8b_32k", choices=list(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the leg that uses the CPU restatement: the parity check before the timed region and the "
                         "CPU baseline after it (for profiler runs)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end decodes of configs 4 and 5 in the default run")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the ragged-mask, config 4 / 5 and batch-1 workloads the default run times besides its headline")
    ap.add_argument("--layers", type=int, default=32, help="layers assumed for the attention-only tok/s figure")
    ap.add_argument("--even-splits", action="store_true",
                    help="give every KV head the same number of splits of the mid rows (default: heads that store more dims "
                         "get more; no difference with a uniform mask)")
    ap.add_argument("--no-fuse", action="store_true",
                    help="run sink/window tiles, mid rows and merge as launches of their own where the library would run the "
                         "merge inside the mid-row launch (for comparison)")
    ap.add_argument("--update-inside-attention", action="store_true",
                    help="update_plus_attn: the streaming update leaves the rank-1 coefficient update to the attention that "
                         "follows, which applies it while it streams the coefficients (comparison: measured no faster than the update launch)")
    ap.add_argument("--no-sub-splits", action="store_true",
                    help="a batch of one sequence: one page stream per workgroup instead of four sub-splits (comparison)")
    ap.add_argument("--e2e", choices=list(E2E), default=None,
                    help="run the end-to-end decode of a random-init model instead (its own JSON line); --steps caps the "
                         "number of timed tokens per sequence")
    ap.add_argument("--prefill-e2e", type=int, default=None, metavar="TOKENS",
                    help="only run the end-to-end prompt pass of the 8B decoder at this prompt length (its own JSON line)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run ten 1 GiB device-to-device copies (reference point for rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives exist on this path); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path exists only as HIP kernels", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    from fourierattention_amd import _lib
    _lib.load()
    if args.e2e:
        explicit = any(x == "--steps" or x.startswith("--steps=") for x in sys.argv[1:])
        print(json.dumps(e2e_bench(args.e2e, device, steps=args.steps if explicit else None)))
        return
    if args.prefill_e2e:
        print(json.dumps(prefill_e2e_bench(device, prompt=args.prefill_e2e)))
        return
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_per_copy": 1 << 30, "copies": 10}))
        return

    w = WORKLOADS[args.workload]
    dtype = torch.bfloat16
    # the CPU-baseline leg starts here: the same CPU restatement that is timed at the end first checks the GPU path
    # on a small seeded case, so that no number is reported for kernels that do not agree with it
    parity = None
    if not args.no_cpu_baseline:
        parity = parity_check(device)
        if not parity <= 2e-2:
            print(f"bench.py: parity check failed (max abs err {parity})", file=sys.stderr)
            sys.exit(1)
    cache, q, kn, vn = build_cache(w, dtype, device)
    cache.balance_heads = not args.even_splits
    cache.fuse_decode = not args.no_fuse
    cache.sub_splits = not args.no_sub_splits
    Hq, Hkv = w["Hq"], w["Hkv"]
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # A decode loop runs for thousands of steps; a device that has been idle takes its first 30 ms or so of work
    # about 8 % slower (both launches of the step, by the kernel trace) and a few hundred steps to settle.  The figure
    # of merit is the settled one, so the same step first runs untimed for 60 ms, whatever --warmup and --steps say.
    priming = {"steps": 0, "ms": 0.0}
    while not args.no_priming and priming["ms"] < 60.0:
        start.record()
        for _ in range(50):
            out = cache.decode_attention(q, 0, Hq, Hkv)
        stop.record()
        torch.cuda.synchronize()
        priming["steps"] += 50
        priming["ms"] = round(priming["ms"] + start.elapsed_time(stop), 2)
    for _ in range(args.warmup):
        out = cache.decode_attention(q, 0, Hq, Hkv)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        out = cache.decode_attention(q, 0, Hq, Hkv)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = start.elapsed_time(stop) / args.steps
    assert torch.isfinite(out).all()

    nbytes = algorithmic_bytes(w)
    gbs = nbytes / (ms * 1e-3) / 1e9
    L = w["ctx"] - w["I"] - w["W"]
    hd = w["Hkv"] * w["D"]
    ck, cv = compressed_counts(w)
    # per-kernel durations, HIP events recorded inside the library on the launch stream
    reps = max(10, min(50, args.steps))
    per = np.zeros(4)
    for _ in range(reps):
        tm = []
        cache.decode_attention(q, 0, Hq, Hkv, timings=tm)
        per += np.array(tm)
    per /= reps
    merge_in_mid_rows = bool(_lib.load().fa_decode_attn_last_fused())
    # three launches: the coefficient-domain query shares one with the sink/window tiles (the third slot is the
    # gap left between the event pairs, a few microseconds of event overhead)
    # (with the merge inside the mid-row launch the step has two launches and the last slot is event overhead only)
    kernel_ms = {"query_and_sink_window": per[0] + per[2], "mid_rows_and_merge" if merge_in_mid_rows else "mid_rows": per[1]}
    if merge_in_mid_rows:
        kernel_ms["empty_event_pair"] = per[3]
    else:
        kernel_ms["merge"] = per[3]
    # algorithmic bytes of each kernel's own launch
    kbytes = {
        "query_and_sink_window": w["B"] * w["M"] * ck * 4 + w["B"] * Hq * w["M"] * 4 + w["B"] * 2 * (w["I"] + w["W"]) * hd * 2,
        "mid_rows": w["B"] * L * (2 * hd - ck - cv) * 2,
        "mid_rows_and_merge": w["B"] * L * (2 * hd - ck - cv) * 2 + w["B"] * w["M"] * cv * 4,
        "merge": w["B"] * w["M"] * cv * 4,
    }
    dom = max(kernel_ms, key=kernel_ms.get)
    dom_gbs = kbytes[dom] / (kernel_ms[dom] * 1e-3) / 1e9
    traffic, traffic_source = recorded_traffic("mid_rows" if dom.startswith("mid_rows") else dom, args.workload)
    full = 2 * w["ctx"] * hd * 2
    fourier = 2 * (w["I"] + w["W"]) * hd * 2 + L * (2 * hd - ck - cv) * 2 + w["M"] * (ck + cv) * 4
    result = {
        "metric": "Fourier decode attn HBM GB/s (% peak) + tok/s, Llama-3.1-8B geometry, 32k ctx",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "batch": w["B"], "context": w["ctx"], "q_heads": Hq, "kv_heads": Hkv,
                   "head_dim": w["D"], "sink": w["I"], "window": w["W"], "coeff_rows": w["M"],
                   "compressed_dims_per_head": w["cper"] if w["cper"] else {"k": w["kc_heads"], "v": w["vc_heads"]},
                   "coeff_dtype": "f32"},
        "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "attn_only_tok_s": round(w["B"] / (args.layers * ms * 1e-3), 1),
        "kv_bytes_per_layer_per_seq": {"full_bf16": full, "fourier": fourier, "reduction": round(full / fourier, 3)},
        "algorithmic_bytes_per_step": nbytes,
        "parity_max_abs_err": parity,
        "wall_ms_per_step": round(wall * 1e3 / args.steps, 5),
        "untimed_steps_before_warmup": priming,
        "kernel_ms": {k: round(float(v), 5) for k, v in kernel_ms.items()},
        "merge_inside_mid_row_launch": merge_in_mid_rows,
        # each launch of kernel_ms sits between its own pair of HIP events; the pairs cost a few microseconds each,
        # which is why the three figures add up to more than ms_per_step (timed without events inside)
        "event_overhead_ms": round(float(sum(kernel_ms.values())) - ms, 5),
        "roofline": {"bound": "hbm", "achieved": round(dom_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom_gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": dom,
                     "algorithmic_bytes_per_launch": kbytes[dom], "kernel_ms": round(float(kernel_ms[dom]), 5),
                     "whole_step_frac": round(gbs / HBM_PEAK_GBS, 4)},
    }
    if merge_in_mid_rows and dom.startswith("mid_rows"):
        # kernel_ms is the distance between two HIP events with the launch between them; two events with nothing between
        # them are `empty_event_pair` apart.  Beside the figure as measured: the same with that distance taken off (the
        # kernel trace of the profiler, which has no events in the stream, reads about that much less per launch)
        net = float(kernel_ms[dom] - kernel_ms["empty_event_pair"])
        result["roofline"]["minus_empty_event_pair"] = {
            "kernel_ms": round(net, 5), "achieved": round(kbytes[dom] / (net * 1e-3) / 1e9, 2),
            "frac": round(kbytes[dom] / (net * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if merge_in_mid_rows:
        # The dominant launch now ends with the merge and the output rows, so its time is not comparable with the
        # mid-row kernel of a step whose merge is a launch of its own: the same step that way, timed beside it
        cache.fuse_decode = False
        for _ in range(5):
            cache.decode_attention(q, 0, Hq, Hkv)
        start.record()
        for _ in range(reps):
            cache.decode_attention(q, 0, Hq, Hkv)
        stop.record()
        torch.cuda.synchronize()
        ms_sep = start.elapsed_time(stop) / reps
        per_sep = np.zeros(4)
        for _ in range(reps):
            tm = []
            cache.decode_attention(q, 0, Hq, Hkv, timings=tm)
            per_sep += np.array(tm)
        per_sep /= reps
        cache.fuse_decode = not args.no_fuse
        sep_gbs = kbytes["mid_rows"] / (per_sep[1] * 1e-3) / 1e9
        result["roofline"]["merge_as_a_launch_of_its_own"] = {
            "ms_per_step": round(ms_sep, 5), "whole_step_frac": round(nbytes / (ms_sep * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "kernel_ms": {"query_and_sink_window": round(float(per_sep[0] + per_sep[2]), 5), "mid_rows": round(float(per_sep[1]), 5),
                          "merge": round(float(per_sep[3]), 5)},
            "mid_rows_achieved": round(sep_gbs, 2), "mid_rows_frac": round(sep_gbs / HBM_PEAK_GBS, 4),
            "mid_rows_algorithmic_bytes_per_launch": kbytes["mid_rows"]}
    # the streaming update that precedes every decode-attention pass in use (one launch: rank-1 coefficient
    # update, evicted row into the page store, new token into the window); read + write of the coefficients
    # (fewer streamed tokens in all than the workload's max_new_tokens: the page store is sized for those and would
    # be re-paged, a one-off of about a millisecond, inside one of the loops below)
    assert 3 + 40 + 30 + 3 + 50 <= w["max_new"] or w["max_new"] < 128
    # (the update on its own, as one launch: what a caller pays who does not attend right after it)
    cache.defer_coef_update = False
    for _ in range(3):
        cache.update(kn, vn, 0)
    torch.cuda.synchronize()
    # The launch is shorter than the host takes to issue it.  For the device-side figure the 40 updates are queued
    # behind a few milliseconds of other work, so that the device runs them back to back; the wall figure is the
    # host-paced loop.
    busy = torch.empty((8192, 8192), dtype=torch.bfloat16, device=device).normal_()
    for _ in range(4):
        busy = busy @ busy
    start.record()
    for _ in range(40):
        cache.update(kn, vn, 0)
    stop.record()
    torch.cuda.synchronize()
    upd_ms = start.elapsed_time(stop) / 40
    del busy
    t0 = time.perf_counter()
    for _ in range(30):
        cache.update(kn, vn, 0)
    torch.cuda.synchronize()
    upd_wall = (time.perf_counter() - t0) / 30
    upd_bytes = w["B"] * 2 * w["M"] * (ck + cv) * 4
    # a decode step in use: the streaming update, then the attention over the updated cache
    # (--update-inside-attention: the attention applies the rank-1 update of the coefficients while it streams them)
    cache.defer_coef_update = bool(args.update_inside_attention)
    for _ in range(3):
        cache.update(kn, vn, 0)
        cache.decode_attention(q, 0, Hq, Hkv)
    start.record()
    for _ in range(50):
        cache.update(kn, vn, 0)
        cache.decode_attention(q, 0, Hq, Hkv)
    stop.record()
    torch.cuda.synchronize()
    both_ms = start.elapsed_time(stop) / 50
    result["update_plus_attn"] = {"ms_per_step": round(both_ms, 5), "coefficient_update_inside_attention": bool(cache.defer_coef_update),
                                  "algorithmic_bytes": upd_bytes + nbytes,
                                  "GB_s": round((upd_bytes + nbytes) / (both_ms * 1e-3) / 1e9, 1),
                                  "pct_hbm_peak": round(100.0 * (upd_bytes + nbytes) / (both_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)}
    result["stream_update"] = {"ms_per_step": round(upd_ms, 5), "wall_ms_per_step": round(upd_wall * 1e3, 5),
                               "algorithmic_bytes": upd_bytes, "GB_s": round(upd_bytes / (upd_ms * 1e-3) / 1e9, 1)}
    del cache, q, kn, vn, out
    if args.workload == "config3_decode_attn_8b_32k" and not args.no_other_workloads:
        # the same kernels on the reference's own ragged masks, on the per-layer attention of configs 4 and 5 and
        # in the reference's evaluation settings (batch 1): latency and fraction of the HBM peak of the whole step
        result["other_workloads"] = {}
        for name in OTHER_WORKLOADS:
            torch.cuda.empty_cache()
            try:
                result["other_workloads"][name] = attn_step_bench(name, device)
            except Exception as exc:
                result["other_workloads"][name] = {"error": f"{type(exc).__name__}: {exc}"}
    result["prefill_compress"] = compress_bench(device)
    result["prefill_attn"] = prefill_attn_bench(device)
    if not args.no_e2e and args.workload.startswith("config3"):
        # BASELINE configs 4 and 5 end to end (a few seconds each); the headline value above stays config 3
        result["e2e"] = {}
        torch.cuda.empty_cache()
        try:
            result["e2e"]["prefill_8b_32k"] = prefill_e2e_bench(device)
        except Exception as exc:
            result["e2e"]["prefill_8b_32k"] = {"error": f"{type(exc).__name__}: {exc}"}
        for name in E2E:
            torch.cuda.empty_cache()
            try:
                r = e2e_bench(name, device)
                result["e2e"][name.split("_")[0]] = {
                    "tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "steps": r["steps"], "warmup": r["warmup"],
                    "batch": r["config"]["batch"], "prompt": r["config"]["prompt"], "model": r["config"]["model"],
                    "T_x": r["config"]["T_x"], "T_c": r["config"]["T_c"], "max_position_embeddings": MODEL_MAX_POSITIONS,
                    "kv_cache_bytes": r["kv_cache_bytes"], "synthetic_prefill_s": r["synthetic_prefill_s"],
                    "packed_projection_weights_bytes": r["packed_projection_weights_bytes"]}
            except Exception as exc:   # the headline figure above stands on its own; say what happened here
                result["e2e"][name.split("_")[0]] = {"error": f"{type(exc).__name__}: {exc}"}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
