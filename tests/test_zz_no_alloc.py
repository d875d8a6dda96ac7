"""``fa_decode_attn_noalloc``: the decode-attention entry point that keeps its partial results in a buffer built into
the library instead of a caller's workspace.  Called through the C ABI on the same operands as ``fa_decode_attn``,
twice in a row with the second call on a smaller input (the buffer keeps the first call's contents), it must give
the same result bit for bit: both run the same kernels with the same split of the work (the cache's default, more
splits for heads that store more dims, is switched off for the comparison)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle.cache_oracle import OracleCache
from tests import helpers as H
from tests.test_gpu_cache import _cfg, _masks


def test_header_and_binding_agree_on_the_buffer_size():
    import os
    import re
    from fourierattention_amd import _lib
    text = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "fourier_attn_hip.h")).read()
    m = re.search(r"#define FA_DECODE_NOALLOC_SCRATCH_BYTES \((\d+)u << (\d+)\)", text)
    assert m and int(m.group(1)) << int(m.group(2)) == _lib.DECODE_NOALLOC_SCRATCH_BYTES == 32 << 20


def test_oversized_shape_is_refused_before_anything_is_touched():
    """The streaming configuration (1024 frequencies, 131072 mid rows) needs about 100 MiB of partial results:
    refused with the workspace code and a message that names both sizes.  Needs no GPU: the check comes first."""
    from fourierattention_amd import _lib
    lib = _lib.load()
    a = _lib.DecodeArgs()
    a.B, a.Hq, a.Hkv, a.D, a.N, a.L_m, a.q_len, a.T = 4, 24, 8, 128, 1024, 131072, 1, 131072
    a.il_rows[0] = 1028
    need = lib.fa_decode_attn_workspace_bytes(4, 24, 8, 128, 1024, 1028, 131072)
    assert need > _lib.DECODE_NOALLOC_SCRATCH_BYTES
    assert lib.fa_decode_attn_noalloc(ctypes.byref(a), None) == -4          # FA_ERR_WORKSPACE
    msg = lib.fa_last_error_string().decode()
    # the size it names is that of a call with the same number of splits for every head (what this entry point
    # runs): above the buffer, and no more than the general workspace query, which leaves room for uneven shares
    import re
    sizes = [int(x) for x in re.findall(r"\d{6,}", msg)]
    assert _lib.DECODE_NOALLOC_SCRATCH_BYTES in sizes
    assert any(_lib.DECODE_NOALLOC_SCRATCH_BYTES < x <= need for x in sizes)
    assert lib.fa_decode_attn_noalloc(None, None) == -1                     # FA_ERR_NULL_POINTER


def _cache_case(dtype, B, Hq, Hkv, D, W, M, prompt, kcounts, vcounts, seed):
    from fourierattention_amd import DynamicCache
    masks = _masks(1, Hkv, D, kcounts, vcounts, seed=seed)
    cfg = _cfg(masks, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=16, max_position_embeddings=1 << 20)
    r = np.random.default_rng(seed)
    k = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype)
    v = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype)
    gpu, cpu = DynamicCache(cfg), OracleCache(cfg, masks=masks, model_dtype=H.NP_ROUND[dtype])
    gpu.update(H.to_gpu(k, dtype), H.to_gpu(v, dtype), 0)
    cpu.update(k, v, 0)
    kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
    vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
    q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)), dtype)
    gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
    kw, vw = cpu.update(kn, vn, 0)
    for n in ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average"):
        getattr(cpu, n)[0] = getattr(gpu, n)[0].float().cpu().numpy()
    want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
    return gpu, H.to_gpu(q, dtype), want


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-3), (torch.float32, 2e-4)])
def test_two_calls_in_a_row_match_the_entry_point_with_a_workspace(dtype, tol):
    """bf16: the matrix-core kernels over the paged store; float32: the generic kernels.  The second call is a
    smaller problem (fewer sequences, shorter context, fewer coefficient rows) that finds the first call's partial
    results in the buffer."""
    Hq, Hkv, D = 8, 2, 128
    big = _cache_case(dtype, 5, Hq, Hkv, D, 64, 512, 3000, [64, 40], [64, 96], seed=1)
    small = _cache_case(dtype, 2, Hq, Hkv, D, 32, 256, 700, [64, 64], [30, 64], seed=2)
    for gpu, q, want in (big, small):
        # the entry point under test gives every head the same number of splits; so does the reference call here
        # (with its default, shares by stored dims, the sums run in another order: checked to rounding below)
        shared = gpu.decode_attention(q, 0, Hq, Hkv)
        gpu.balance_heads = False
        ref = gpu.decode_attention(q, 0, Hq, Hkv)                               # fa_decode_attn, caller's workspace
        assert (shared - ref).abs().max().item() <= 1e-3 * max(1.0, ref.abs().max().item())
        out = torch.full_like(ref, float("nan"))
        got = gpu.decode_attention(q, 0, Hq, Hkv, out=out, no_alloc=True)       # fa_decode_attn_noalloc
        assert got is out and torch.equal(got, ref)
        err = np.abs(got.cpu().numpy() - want).max()
        assert err <= 2e-2 and err <= tol, err
    # and once more the larger one after the smaller: nothing of the smaller call's leftovers is read
    gpu, q, want = big
    out = torch.full((5, Hq, 1, D), float("nan"), device="cuda")
    assert torch.equal(gpu.decode_attention(q, 0, Hq, Hkv, out=out, no_alloc=True), gpu.decode_attention(q, 0, Hq, Hkv))


@pytest.mark.gpu
def test_calls_whose_mid_row_launch_merges_its_own_partials():
    """Eight KV heads: the teams of the mid-row launch fill the dies, so the merge runs inside that launch and its
    meeting counters live in the buffer too (cleared by the launch in front, every call).  A batch of four, then a
    single sequence (four sub-splits per workgroup), then the batch again: bit for bit as with a workspace.  (This
    entry point does not probe the device's workgroup placement itself, see the header: the calls with a workspace
    in front of it have.)"""
    from fourierattention_amd import _lib
    Hq, Hkv, D = 32, 8, 128
    big = _cache_case(torch.bfloat16, 4, Hq, Hkv, D, 64, 1024, 3000, [64] * 8, [64, 0, 128, 30, 64, 64, 100, 64], seed=5)
    one = _cache_case(torch.bfloat16, 1, Hq, Hkv, D, 32, 512, 1500, [64] * 8, [64] * 8, seed=6)
    for (gpu, q, want), mode in ((big, 1), (one, 2), (big, 1)):
        gpu.balance_heads = False
        ref = gpu.decode_attention(q, 0, Hq, Hkv)
        assert _lib.load().fa_decode_attn_last_fused() == mode
        out = torch.full_like(ref, float("nan"))
        got = gpu.decode_attention(q, 0, Hq, Hkv, out=out, no_alloc=True)
        assert _lib.load().fa_decode_attn_last_fused() == mode
        assert got is out and torch.equal(got, ref)
        err = np.abs(got.cpu().numpy() - want).max()
        assert err <= 2e-3, err


@pytest.mark.gpu
def test_two_calls_with_1024_frequencies():
    """1024 frequencies take the two-pass mid rows and the merge whose blocks hand over through counters in the
    buffer (cleared by the launch in front): two calls in a row, the second smaller, bit for bit as with a workspace."""
    Hq, Hkv, D = 6, 2, 128
    big = _cache_case(torch.bfloat16, 3, Hq, Hkv, D, 32, 2048, 4500, [64, 100], [64, 20], seed=3)
    small = _cache_case(torch.bfloat16, 2, Hq, Hkv, D, 32, 2048, 4200, [64, 64], [64, 64], seed=4)
    for gpu, q, want in (big, small, big):
        gpu.balance_heads = False
        ref = gpu.decode_attention(q, 0, Hq, Hkv)
        out = torch.full_like(ref, float("nan"))
        got = gpu.decode_attention(q, 0, Hq, Hkv, out=out, no_alloc=True)
        assert got is out and torch.equal(got, ref)
        err = np.abs(got.cpu().numpy() - want).max()
        assert err <= 2e-3, err


@pytest.mark.gpu
def test_captured_in_a_graph_and_replayed():
    """``fa_decode_attn_noalloc`` recorded into a graph (no allocation, no clearing of memory by the runtime: the
    counters of the merge are cleared by the launch in front of it) and replayed on new queries in the same buffers:
    every replay bit for bit what the eager call returns."""
    # the one-pass mid rows / the two passes of 1024 frequencies with the merge as a launch of its own (two KV heads);
    # the merge inside the mid-row launch (eight KV heads: its meeting counters are cleared by the launch in front on
    # every replay), for a batch and for a single sequence with its sub-splits.  (1024 frequencies on eight KV heads
    # need more than the built-in buffer holds.)
    shapes = [(3, 8, 2, 512, 2000, [64, 40], [64, 96], 0), (3, 8, 2, 2048, 4300, [64, 40], [64, 96], 0),
              (4, 32, 8, 1024, 3000, [64] * 8, [64, 0, 128, 30, 64, 64, 100, 64], 1), (1, 32, 8, 512, 1500, [64] * 8, [64] * 8, 2)]
    D = 128
    from fourierattention_amd import _lib
    for B, Hq, Hkv, M, prompt, kc, vc, mode in shapes:
        gpu, q, want = _cache_case(torch.bfloat16, B, Hq, Hkv, D, 64, M, prompt, kc, vc, seed=5)
        gpu.balance_heads = False
        ref = gpu.decode_attention(q, 0, Hq, Hkv)
        out = torch.full_like(ref, float("nan"))
        qbuf = q.clone()
        # first call outside the capture: the address of the built-in buffer is looked up once per device
        assert torch.equal(gpu.decode_attention(qbuf, 0, Hq, Hkv, out=out, no_alloc=True), ref)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            gpu.decode_attention(qbuf, 0, Hq, Hkv, out=out, no_alloc=True)
        assert _lib.load().fa_decode_attn_last_fused() == mode     # (what the recorded call runs)
        gen = torch.Generator(device="cuda").manual_seed(7)
        for _ in range(3):
            qk = (torch.randn(q.shape, generator=gen, device="cuda") * 1.5).to(q.dtype)
            eager = gpu.decode_attention(qk, 0, Hq, Hkv)
            qbuf.copy_(qk)
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
