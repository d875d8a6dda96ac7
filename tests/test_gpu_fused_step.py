"""The three ways ``fa_decode_attn`` runs a step on the one-pass matrix-core path must agree: mid rows and merge as
launches of their own, the merge inside the mid-row launch (teams of workgroups that meet through the L2 of their
die), and, for a batch of one sequence, the same with four sub-splits per workgroup in the places of four batch
elements.  Every case is also held against the CPU restatement (bound 2e-2 for 16-bit storage, as everywhere).

Geometries: eight KV heads so that the teams of a launch fill the eight dies (what the fused merge needs), one to
four query heads per KV head, batches that fill a group of four, leave it ragged or consist of one sequence, heads
that compress everything, nothing, or one to three dims, mid rows from a single page to a few hundred, 128 to 1024
frequencies (the last as two passes over the pages, the second of which then merges)."""
import numpy as np
import pytest
import torch

from oracle.cache_oracle import OracleCache
from tests import helpers as H
from tests.test_gpu_cache import _cfg, _masks

pytestmark = pytest.mark.gpu

U = [64] * 8
CASES = [
    # dtype, B, Hq, I, W, M, prompt, kcounts, vcounts (stored dims per KV head), what fa_decode_attn_last_fused reports
    # for the default call (1: merge inside the mid-row launch, 2: that with sub-splits)
    (torch.bfloat16, 1, 32, 4, 64, 1024, 9000, U, U, 2),                                   # the benchmark's geometry, one sequence
    (torch.bfloat16, 1, 32, 4, 60, 1024, 5000, [0, 128, 64, 3, 125, 127, 64, 96], [128, 0, 61, 64, 2, 64, 127, 1], 2),
    (torch.float16, 1, 24, 4, 48, 512, 3011, U, [40] * 8, 2),                              # three query heads per KV head
    (torch.bfloat16, 1, 16, 0, 33, 256, 2000, U, U, 2),                                    # two; no sink rows
    (torch.bfloat16, 1, 8, 4, 32, 256, 700, U, U, 2),                                      # one; splits of a few pages
    (torch.bfloat16, 1, 32, 4, 32, 256, 330, U, U, 2),                                     # two pages of mid rows: empty sub-splits
    (torch.bfloat16, 1, 32, 4, 32, 512, 1100 + 19, U, U, 2),                               # ragged last page
    (torch.bfloat16, 4, 32, 4, 64, 1024, 3000, U, U, 1),                                   # a full group of four
    (torch.bfloat16, 8, 32, 4, 64, 512, 1500, [64, 0, 128, 30, 64, 64, 100, 64], [1, 64, 2, 3, 128, 64, 0, 64], 1),
    (torch.float16, 2, 16, 4, 40, 512, 2500, U, U, 1),                                     # two sequences: no sub-splits
    # heads with few compressed V dims (8, 3, 0, 16, 64, 1, 28, 12): few outputs and many row classes in the tail's product
    (torch.bfloat16, 4, 32, 4, 64, 512, 2500, U, [120, 125, 128, 112, 64, 127, 100, 116], 1),
    (torch.bfloat16, 1, 32, 4, 64, 1024, 6000, U, [120, 125, 128, 112, 64, 127, 100, 116], 2),
    # 1024 frequencies: the value pass of the two merges its own partials
    (torch.bfloat16, 4, 24, 4, 40, 2048, 6000, U, U, 1),
    (torch.float16, 2, 32, 4, 64, 2048, 5000, [64, 0, 128, 30, 64, 64, 100, 64], [1, 64, 2, 3, 128, 64, 0, 64], 1),
    (torch.bfloat16, 1, 32, 4, 64, 2048, 7000, U, U, 1),                                   # one sequence there: no sub-splits either
]


def _step(case):
    from fourierattention_amd import DynamicCache
    dtype, B, Hq, I, W, M, prompt, kcnt, vcnt, mode = CASES[case]
    Hkv, D = 8, 128
    masks = _masks(1, Hkv, D, kcnt, vcnt, seed=case)
    cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=16)
    gpu = DynamicCache(cfg)
    cpu = OracleCache(cfg, masks=masks, model_dtype=H.NP_ROUND[dtype])
    r = np.random.default_rng(900 + case)
    k0 = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype)
    v0 = H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)) + 0.1, dtype)
    gpu.update(H.to_gpu(k0, dtype), H.to_gpu(v0, dtype), 0)
    cpu.update(k0, v0, 0)
    kn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
    vn = H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype)
    q = H.to_dtype_np(r.standard_normal((B, Hq, 1, D)) * 1.5, dtype)
    gpu.update(H.to_gpu(kn, dtype), H.to_gpu(vn, dtype), 0)
    kw, vw = cpu.update(kn, vn, 0)
    for n in ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average"):
        getattr(cpu, n)[0] = getattr(gpu, n)[0].float().cpu().numpy()
    want = cpu.attend(q, kw, vw, 0, Hq, Hkv)
    return gpu, H.to_gpu(q, dtype), want, Hq, Hkv, mode


@pytest.mark.parametrize("case", range(len(CASES)))
def test_the_ways_a_step_runs_agree(case):
    from fourierattention_amd import _lib
    gpu, q, want, Hq, Hkv, mode = _step(case)
    assert gpu._tables is not None, "this shape must be served by the matrix-core kernels"
    lib = _lib.load()
    got = {}
    for name, fuse, sub in (("launches", False, True), ("merged", True, False), ("default", True, True)):
        gpu.fuse_decode, gpu.sub_splits = fuse, sub
        print(f"case {case} {name}", flush=True)
        for rep in range(2):        # twice: the meeting counters are cleared by the launch in front, every call
            out = gpu.decode_attention(q, 0, Hq, Hkv).cpu().numpy()
            ran = lib.fa_decode_attn_last_fused()
            assert ran == {"launches": 0, "merged": 1, "default": mode}[name], (name, ran)
            assert np.isfinite(out).all(), name
            if rep:
                np.testing.assert_array_equal(out, got[name])     # fixed summation order: the same bits every time
            got[name] = out
    for name, out in got.items():
        err = np.abs(out - want).max()
        assert err <= 2e-2 and err <= 5e-3, (name, err)
    # Among each other: the merge is the same arithmetic in another place, but the three ways cut the mid rows into
    # splits differently (shares within bins of heads, sub-splits), which moves the softmax references of the pages
    # and with them the rounding of the 16-bit probabilities
    assert np.abs(got["merged"] - got["launches"]).max() <= 2e-3
    assert np.abs(got["default"] - got["launches"]).max() <= 2e-3


def test_fused_step_with_converted_output_rows():
    """``out_cast`` (the rows rounded to the model's type) from the launch that merges its own partials: the
    rounded fp32 rows, for a batch of one (sub-splits) and a batch of four."""
    for case in (0, 7):
        gpu, q, want, Hq, Hkv, mode = _step(case)
        f32 = gpu.decode_attention(q, 0, Hq, Hkv)
        cast = gpu.decode_attention(q, 0, Hq, Hkv, out_dtype=q.dtype)
        assert cast.dtype == q.dtype and torch.equal(cast, f32.to(q.dtype))


def test_random_geometries_with_the_merge_inside_the_launch_agree_with_the_generic_kernels():
    """Seeded random geometry on eight or sixteen KV heads (whole teams per die, so the merge runs inside the mid-row
    launch wherever the shape allows it): batches of 1 to 9 (groups of four, a last group that is not full, a single
    sequence with its sub-splits), one to four query heads per KV head, 128 to 1024 frequencies, ragged per-head
    masks, odd sink / window / prompt lengths, with and without a pending coefficient update; against the plain
    kernels on the same cache.  At least half of the cases must have taken the launch that merges."""
    from fourierattention_amd import DynamicCache, _lib
    rng = np.random.default_rng(4711)
    lib = _lib.load()
    merged = 0
    n_cases = 14
    for case in range(n_cases):
        dtype = [torch.bfloat16, torch.float16][rng.integers(2)]
        D = 128
        Hkv = int([8, 8, 8, 16][rng.integers(4)]); G = int(rng.integers(1, 5)); Hq = Hkv * G
        B = int([1, 1, 2, 3, 4, 5, 8, 9][rng.integers(8)]); I = int(rng.integers(0, 6)); W = int(rng.integers(1, 130))
        M = int([256, 512, 1024, 1024, 2048][rng.integers(5)])
        prompt = int(I + W + M + rng.integers(1, 4000))
        kc = [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)]
        vc = [int(rng.integers(1 if h == 0 else 0, D + 1)) for h in range(Hkv)]
        defer = bool(rng.integers(2))
        tag = (f"case {case}: {dtype} B={B} Hq={Hq} Hkv={Hkv} I={I} W={W} M={M} prompt={prompt} defer={defer} "
               f"k={kc} v={vc}")
        print(tag, flush=True)
        masks = _masks(1, Hkv, D, kc, vc, seed=case)
        cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=8,
                   max_position_embeddings=1 << 20)
        gpu = DynamicCache(cfg)
        gpu.defer_coef_update = defer
        g = torch.Generator(device="cuda").manual_seed(case)
        rn = lambda *sh: torch.randn(*sh, generator=g, device="cuda")
        gpu.update(rn(B, Hkv, prompt, D).to(dtype), rn(B, Hkv, prompt, D).to(dtype), 0)
        assert gpu._tables is not None, tag
        for _ in range(2):
            gpu.update(rn(B, Hkv, 1, D).to(dtype), rn(B, Hkv, 1, D).to(dtype), 0)
            q = (rn(B, Hq, 1, D) * 1.5).to(dtype)
            got = gpu.decode_attention(q, 0, Hq, Hkv)
            ran = lib.fa_decode_attn_last_fused()
            gpu.force_generic = True
            ref = gpu.decode_attention(q, 0, Hq, Hkv)
            gpu.force_generic = False
            assert torch.isfinite(got).all(), tag
            err = (got - ref).abs().max().item()
            assert err <= 5e-3, (tag, err, ran)
        merged += ran > 0
        assert ran != 2 or B == 1, tag
    assert merged >= n_cases // 2, merged
