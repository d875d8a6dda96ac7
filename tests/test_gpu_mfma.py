"""The MFMA decode path (paged mid store) against the CPU oracle and against the generic
kernels, on shapes that exercise ragged heads, several batch groups, partial last pages."""
import numpy as np
import pytest
import torch

from oracle.cache_oracle import OracleCache
from tests import helpers as H
from tests.test_gpu_cache import _cfg, _masks

pytestmark = pytest.mark.gpu


def test_mid_store_roundtrip_bit_exact():
    from fourierattention_amd.midstore import MidStore
    r = np.random.default_rng(0)
    B, Hkv, D, S = 3, 4, 128, 150
    for is_v in (False, True):
        n, _, _, _ = H.ragged_mask(r, Hkv, D, [0, 128, 37, 64])      # stored dims per head
        nh = [0] + [int((n < (h + 1) * D).sum()) for h in range(Hkv)]
        src = torch.randn((B, S, Hkv * D), device="cuda").to(torch.bfloat16)
        n32 = torch.from_numpy(n).int().cuda(); nh32 = torch.tensor(nh, dtype=torch.int32, device="cuda")
        st = MidStore(B, n32, nh32, nh, Hkv, D, 100, torch.bfloat16, "cuda", is_v)
        want = src[:, 7:100][:, :, torch.from_numpy(n).cuda()]
        for head_dims in (True, False):       # the head's slice read whole / every element by its column number
            st.data.zero_()
            st.pack(src, 7, 93, head_dims=head_dims)
            assert torch.equal(st.dense(93), want)
        st.append(src[:, 120, :], 93)                                   # one evicted row
        st.append(src[:, 121, :], 94)
        want2 = torch.cat([want, src[:, 120:122][:, :, torch.from_numpy(n).cuda()]], dim=1)
        assert torch.equal(st.dense(95), want2)
        st.grow(95, 400)                                                # re-paging keeps the rows
        assert st.cap_tokens >= 400 and torch.equal(st.dense(95), want2)
        # padded dims and unused slots stay zero
        assert st.data.float().abs().sum().item() == pytest.approx(want2.float().abs().sum().item(), rel=1e-6)


def test_mid_pack_of_rows_that_are_gathered_already():
    """An identity list over rows that hold the stored dims only (what re-paging and the function-level drop-in
    hand over), the rows being a column slice of a wider, 16-byte aligned buffer: the row stride is then at least
    ``Hkv * D`` and says nothing about what the list means."""
    from fourierattention_amd import _lib
    from fourierattention_amd.midstore import MidStore
    r = np.random.default_rng(1)
    B, Hkv, D, S = 2, 4, 64, 70
    n, _, _, _ = H.ragged_mask(r, Hkv, D, [20, 64, 0, 33])
    nh = [0] + [int((n < (h + 1) * D).sum()) for h in range(Hkv)]
    Cn = nh[-1]
    wide = torch.randn((B, S, 512), device="cuda").to(torch.bfloat16)      # 512 >= Hkv * D = 256
    gathered = wide[:, :, 8: 8 + Cn]                                       # (B, S, Cn) view, rows 1024 bytes apart
    assert gathered.stride(1) >= Hkv * D and gathered.data_ptr() % 16 == 0
    ident = torch.arange(Cn, dtype=torch.int32, device="cuda")
    nh32 = torch.tensor(nh, dtype=torch.int32, device="cuda")
    for is_v in (False, True):
        st = MidStore(B, ident, nh32, nh, Hkv, D, S, torch.bfloat16, "cuda", is_v)
        st.pack(gathered, 0, S)
        assert torch.equal(st.dense(S), gathered)
    # the other meaning of the list needs rows wide enough for every head
    st = MidStore(B, ident, nh32, nh, Hkv, D, S, torch.bfloat16, "cuda", False)
    with pytest.raises(_lib.FourierAttnError):
        st.pack(wide[:, :, :128].contiguous(), 0, S, head_dims=True)


MFMA_CASES = [
    # dtype, B, Hq, Hkv, D, I, W, M, prompt, steps, kcounts, vcounts
    (torch.bfloat16, 5, 8, 2, 128, 4, 32, 256, 700, 3, [64, 64], [64, 64]),          # two batch groups (4 + 1)
    (torch.bfloat16, 1, 24, 8, 128, 4, 48, 256, 611, 2, [64] * 8, [64] * 8),         # 3:1 grouping, B = 1
    (torch.bfloat16, 2, 8, 2, 128, 4, 32, 512, 1100, 2, [0, 128], [127, 5]),         # ragged: nothing / everything stored
    (torch.float16, 3, 4, 4, 64, 2, 16, 256, 420, 2, [10, 30, 64, 1], [3, 64, 33, 17]),  # MHA, head_dim 64, fp16
    (torch.bfloat16, 2, 32, 8, 128, 4, 64, 1024, 2200, 2, [64] * 8, [64] * 8),       # the benchmark's geometry, short
    (torch.bfloat16, 3, 16, 2, 128, 4, 200, 256, 900, 3, [64, 40], [64, 96]),        # 8:1 grouping, window of several tiles
    # the remaining instances of the mid-row kernel (256 frequencies with narrow pages, 512 with wide ones), an odd
    # number of pages per split and splits of a single page (nine pages, the last one ragged)
    (torch.bfloat16, 2, 8, 2, 128, 4, 32, 512, 1000, 2, [64, 70], [80, 64]),
    (torch.bfloat16, 2, 16, 4, 128, 4, 32, 1024, 2300, 2, [30, 64, 0, 100], [128, 3, 64, 20]),
    (torch.bfloat16, 1, 8, 2, 128, 4, 32, 256, 300, 2, [64, 64], [64, 64]),
    # 1024 frequencies: the mid rows run as a score pass and a value pass
    (torch.bfloat16, 5, 16, 4, 128, 4, 32, 2048, 4500, 2, [64] * 4, [64] * 4),
    (torch.float16, 2, 8, 2, 128, 4, 32, 2048, 4200, 2, [0, 128], [120, 7]),
    # ... whose partials meet in the merge cut along the coefficient rows: one, two and eight query heads per KV
    # head (one to eight classes of splits per block), head dims of 64, a head with nothing compressed
    (torch.bfloat16, 3, 2, 2, 128, 4, 32, 2048, 4300, 2, [64, 128], [50, 0]),
    (torch.bfloat16, 2, 4, 2, 64, 4, 32, 2048, 4300, 2, [32, 20], [64, 33]),
    (torch.bfloat16, 1, 16, 2, 128, 4, 32, 2048, 4400, 2, [64, 100], [64, 127]),
]


@pytest.mark.parametrize("case", range(len(MFMA_CASES)))
def test_mfma_decode_matches_oracle_and_generic(case):
    from fourierattention_amd import DynamicCache
    dtype, B, Hq, Hkv, D, I, W, M, prompt, steps, kcnt, vcnt = MFMA_CASES[case]
    masks = _masks(1, Hkv, D, kcnt, vcnt, seed=case)
    cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=64)
    gpu = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=masks, model_dtype=H.NP_ROUND[dtype])
    r = np.random.default_rng(50 + case)
    k0 = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype)
    v0 = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)) + 0.1, dtype)
    gpu.update(H.to_gpu(k0, dtype), H.to_gpu(v0, dtype), 0)
    cpu.update(k0, v0, 0)
    assert gpu._tables is not None, "this shape must be served by the MFMA kernels"
    for s in range(steps):
        kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype); vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
        q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)) * 1.5, dtype)
        kp, vp = gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
        kw, vw = cpu.update(kn, vn, 0)
        np.testing.assert_array_equal(kp["k_uncompressed"].float().cpu().numpy(), kw["k_uncompressed"].astype(np.float32))
        np.testing.assert_array_equal(vp["v_uncompressed"].float().cpu().numpy(), vw["v_uncompressed"].astype(np.float32))
        for n in ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average"):
            getattr(cpu, n)[0] = getattr(gpu, n)[0].float().cpu().numpy()
        want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
        qg = H.to_gpu(q, dtype)
        gpu.force_generic = False
        got = gpu.decode_attention(qg, 0, Hq, Hkv).cpu().numpy()
        gpu.force_generic = True
        ref = gpu.decode_attention(qg, 0, Hq, Hkv).cpu().numpy()
        gpu.force_generic = False
        assert np.isfinite(got).all()
        e_gen = np.abs(ref - want).max()
        e_mfma = np.abs(got - want).max()
        assert e_gen <= 1e-3, e_gen
        # stated bound for 16-bit attention vs the fp32/fp64 reference; f16 basis + bf16 probabilities
        # on the matrix cores land well inside it
        assert e_mfma <= 2e-2, e_mfma
        assert e_mfma <= 5e-3, e_mfma


@pytest.mark.parametrize("shape", ["ramp", "spike"])
def test_mfma_softmax_reference_moves(shape):
    """Key magnitudes that grow along the sequence (the running softmax reference has to move again and again)
    and a late burst of keys with scores far above everything before (it moves by much more than its slack)."""
    from fourierattention_amd import DynamicCache
    dtype, B, Hq, Hkv, D, I, W, M, prompt = torch.bfloat16, 2, 8, 2, 128, 4, 32, 256, 1500
    masks = _masks(1, Hkv, D, [64, 64], [64, 64], seed=11)
    cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=16)
    gpu = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=masks, model_dtype=H.NP_ROUND[dtype])
    r = np.random.default_rng(77)
    k0 = r.standard_normal((B, Hkv, prompt, D))
    if shape == "ramp":
        k0 *= (0.1 + 4.0 * np.arange(prompt) / prompt)[None, None, :, None]
    else:
        k0[:, :, 1100:1110, :] *= 12.0
    k0 = H.to_dtype_np(k0, dtype)
    v0 = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)) + 0.1, dtype)
    gpu.update(H.to_gpu(k0, dtype), H.to_gpu(v0, dtype), 0)
    cpu.update(k0, v0, 0)
    kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype); vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
    q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)) * 1.5, dtype)
    gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
    kw, vw = cpu.update(kn, vn, 0)
    for n in ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average"):
        getattr(cpu, n)[0] = getattr(gpu, n)[0].float().cpu().numpy()
    want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
    assert gpu._tables is not None
    got = gpu.decode_attention(H.to_gpu(q, dtype), 0, Hq, Hkv).cpu().numpy()
    assert np.isfinite(got).all()
    err = np.abs(got - want).max()
    assert err <= 2e-2, err        # the stated bound
    assert err <= 8e-3, err        # sharply peaked softmax: the bf16 probabilities dominate


def test_mfma_random_shapes_agree_with_the_generic_kernels():
    """Seeded random geometry (batch 1-9, 1-4 KV heads, grouping 1-8, head_dim 64 / 128, 128-1024 frequencies,
    ragged per-head masks, odd sink / window / prompt lengths): the matrix-core path against the plain kernels."""
    from fourierattention_amd import DynamicCache
    rng = np.random.default_rng(2024)
    for case in range(16):
        dtype = [torch.bfloat16, torch.float16][rng.integers(2)]
        D = [64, 128][rng.integers(2)]
        Hkv = int(rng.integers(1, 5)); G = int([1, 2, 3, 4, 6, 8][rng.integers(6)]); Hq = Hkv * G
        B = int(rng.integers(1, 10)); I = int(rng.integers(0, 6)); W = int(rng.integers(1, 70))
        M = int([256, 512, 1024, 2048][rng.integers(4)])
        prompt = int(I + W + M + rng.integers(1, 1500))
        kc = [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)]
        vc = [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)]
        tag = f"case {case}: {dtype} B={B} Hq={Hq} Hkv={Hkv} D={D} I={I} W={W} M={M} prompt={prompt} k={kc} v={vc}"
        print(tag, flush=True)
        masks = _masks(1, Hkv, D, kc, vc, seed=case)
        cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=8,
                   max_position_embeddings=1 << 20)
        gpu = DynamicCache(cfg)
        g = torch.Generator(device="cuda").manual_seed(case)
        rn = lambda *sh: torch.randn(*sh, generator=g, device="cuda")
        gpu.update(rn(B, Hkv, prompt, D).to(dtype), rn(B, Hkv, prompt, D).to(dtype), 0)
        assert gpu._tables is not None, tag
        for _ in range(2):
            gpu.update(rn(B, Hkv, 1, D).to(dtype), rn(B, Hkv, 1, D).to(dtype), 0)
            q = (rn(B, Hq, 1, D) * 1.5).to(dtype)
            got = gpu.decode_attention(q, 0, Hq, Hkv)
            gpu.force_generic = True
            ref = gpu.decode_attention(q, 0, Hq, Hkv)
            gpu.force_generic = False
            assert torch.isfinite(got).all(), tag
            err = (got - ref).abs().max().item()
            assert err <= 5e-3, (tag, err)



def test_merge_for_few_query_heads_agrees_with_the_generic_kernels():
    """The merge launch behind the matrix-core mid rows for up to four query heads per KV head and up to 512
    frequencies (16-byte loads where a head's columns are aligned, single values otherwise; shares of the dims per
    block): heads whose V dims are all compressed, all stored or none at all, odd totals of compressed dims (rows of
    the coefficient tensor that are no multiple of 16 bytes), no sink rows, batches that do not fill a group, windows
    of one tile, of many tiles, and of more tiles than that kernel takes (the general merge kernel runs then)."""
    from fourierattention_amd import DynamicCache
    rng = np.random.default_rng(77)
    fixed = [   # (D, Hkv, G, B, I, W, M, k dims compressed per head, v dims compressed per head)
        (128, 2, 4, 5, 0, 3, 256, [64, 64], [128, 0]),
        (128, 3, 3, 2, 4, 130, 512, [1, 127, 64], [1, 2, 3]),
        (64, 4, 4, 9, 2, 64, 1024, [32, 32, 32, 32], [64, 64, 64, 64]),
        (64, 1, 1, 1, 1, 1, 256, [64], [63]),
        (128, 4, 2, 3, 4, 70, 1024, [60, 64, 68, 4], [4, 8, 12, 124]),
        (128, 2, 4, 2, 4, 8200, 512, [64, 64], [64, 60]),      # 129 sink/window tiles: more than are requested ahead
        (128, 1, 4, 1, 4, 20000, 512, [64], [64]),             # more split weights than the kernel has threads for
    ]
    cases = [(*f, torch.bfloat16) for f in fixed]
    for _ in range(10):
        D = [64, 128][rng.integers(2)]
        Hkv = int(rng.integers(1, 5)); G = int(rng.integers(1, 5))
        cases.append((D, Hkv, G, int(rng.integers(1, 10)), int(rng.integers(0, 6)), int(rng.integers(1, 200)),
                      int([256, 512, 1024][rng.integers(3)]),
                      [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)],
                      [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)],
                      [torch.bfloat16, torch.float16][rng.integers(2)]))
    for case, (D, Hkv, G, B, I, W, M, kc, vc, dtype) in enumerate(cases):
        Hq = Hkv * G
        prompt = int(I + W + M + 40 + rng.integers(1, 1200))
        tag = f"case {case}: {dtype} B={B} Hq={Hq} Hkv={Hkv} D={D} I={I} W={W} M={M} prompt={prompt} k={kc} v={vc}"
        print(tag, flush=True)
        masks = _masks(1, Hkv, D, kc, vc, seed=100 + case)
        cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=8,
                   max_position_embeddings=1 << 20)
        gpu = DynamicCache(cfg)
        g = torch.Generator(device="cuda").manual_seed(1000 + case)
        rn = lambda *sh: torch.randn(*sh, generator=g, device="cuda")
        gpu.update(rn(B, Hkv, prompt, D).to(dtype), rn(B, Hkv, prompt, D).to(dtype), 0)
        assert gpu._tables is not None, tag
        gpu.update(rn(B, Hkv, 1, D).to(dtype), rn(B, Hkv, 1, D).to(dtype), 0)
        q = (rn(B, Hq, 1, D) * 1.5).to(dtype)
        got = gpu.decode_attention(q, 0, Hq, Hkv)
        gpu.force_generic = True
        ref = gpu.decode_attention(q, 0, Hq, Hkv)
        gpu.force_generic = False
        assert torch.isfinite(got).all(), tag
        err = (got - ref).abs().max().item()
        assert err <= 5e-3, (tag, err)


def test_full_size_properties():
    """BASELINE config 3 at full size (B=8, 32k context): properties that need no CPU oracle.
    (1) the matrix-core path and the generic path (independent kernels, each checked against the oracle at
    small sizes) agree; (2) swapping two batch elements of the query and of the cache-independent inputs
    swaps the output rows only where the cache rows are swapped too: here the query alone is permuted across
    the heads of a KV group, which must permute the output heads the same way (GQA heads share K/V)."""
    import bench
    w = bench.WORKLOADS["config3_decode_attn_8b_32k"]
    dev = torch.device("cuda", 0)
    cache, q, kn, vn = bench.build_cache(w, torch.bfloat16, dev)
    Hq, Hkv = w["Hq"], w["Hkv"]
    assert cache._tables is not None
    out = cache.decode_attention(q, 0, Hq, Hkv)
    cache.force_generic = True
    ref = cache.decode_attention(q, 0, Hq, Hkv)
    cache.force_generic = False
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max().item() <= 5e-3
    G = Hq // Hkv
    perm = torch.arange(Hq, device=dev).view(Hkv, G).flip(1).reshape(-1)     # reverse the heads inside every group
    out_p = cache.decode_attention(q[:, perm].contiguous(), 0, Hq, Hkv)
    # same rows, other MFMA columns: equal up to the accumulation order of the split merge (identical here)
    assert (out_p - out[:, perm]).abs().max().item() <= 1e-5
    # a streaming step keeps everything consistent: sequence length grows by one, output stays finite
    n0 = cache.get_seq_length(0)
    cache.update(kn, vn, 0)
    assert cache.get_seq_length(0) == n0 + 1
    out2 = cache.decode_attention(q, 0, Hq, Hkv)
    assert torch.isfinite(out2).all() and (out2 - out).abs().max().item() < 1.0


@pytest.mark.parametrize("workload", ["config4_decode_attn_8b_64k", "config5_decode_attn_3b_128k"])
def test_long_splits_agree_with_the_generic_kernels(workload):
    """The two long-context geometries of the benchmark at full size: a workgroup walks 252 pages (config 4) or
    127 pages in two passes with 1024 frequencies (config 5), so the page-to-page rotation of the
    coefficient-domain state is applied that many times in a row.  The generic kernels evaluate every phase from
    its exactly reduced integer argument instead; both must agree as they do on short contexts."""
    import bench
    w = bench.WORKLOADS[workload]
    dev = torch.device("cuda", 0)
    cache, q, kn, vn = bench.build_cache(w, torch.bfloat16, dev)
    Hq, Hkv = w["Hq"], w["Hkv"]
    assert cache._tables is not None
    out = cache.decode_attention(q, 0, Hq, Hkv)
    cache.force_generic = True
    ref = cache.decode_attention(q, 0, Hq, Hkv)
    cache.force_generic = False
    assert torch.isfinite(out).all()
    err = (out - ref).abs().max().item()
    assert err <= 5e-3, err
    del cache
    torch.cuda.empty_cache()
