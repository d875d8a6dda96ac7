"""The minimal LLaMA decoder and greedy loop around the cache (fourierattention_amd/llama.py).

CPU: with a window larger than the sequence nothing is compressed, so the cached decode must reproduce a full
recomputation of the sequence with the same weights (exact attention either way) — this pins positions, the
prefill / decode dispatch and the threading of the cache through the loop.
GPU: with a compressed cache, every decode step's logits are compared with the same weights run layer by layer
on the CPU through the oracle cache and the oracle attention.
"""
import numpy as np
import pytest
import torch

from tests.test_gpu_cache import _cfg, _masks


def _tiny(layers=2, hidden=64, heads=4, kv=2, hd=16, vocab=97):
    from fourierattention_amd.llama import LlamaConfig
    return LlamaConfig(hidden_size=hidden, intermediate_size=2 * hidden, num_hidden_layers=layers, num_attention_heads=heads,
                       num_key_value_heads=kv, head_dim=hd, vocab_size=vocab)


def test_greedy_loop_matches_full_recompute_cpu():
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import greedy_generate, random_init
    cfg = _tiny()
    model = random_init(cfg, dtype=torch.float32, device="cpu", seed=3, std=0.3)
    masks = _masks(cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.head_dim, [8, 8], [8, 8])
    ec = lambda: _cfg(masks, numinittokens=2, maxlocallen=64, maxmidstates=8, num_key_value_heads=cfg.num_key_value_heads,
                      max_new_tokens=16, max_position_embeddings=256)
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, cfg.vocab_size, (2, 11), generator=g)
    seq = greedy_generate(model, prompt, DynamicCache(ec(), device="cpu"), max_new_tokens=6)
    assert seq.shape == (2, 17) and torch.equal(seq[:, :11], prompt)
    # the same tokens one by one from scratch: a fresh cache and a prompt pass over everything so far
    cur = prompt
    for step in range(6):
        out = model(input_ids=cur, past_key_values=DynamicCache(ec(), device="cpu"), num_logits_to_keep=1)
        nxt = out.logits[:, -1, :].argmax(-1, keepdim=True)
        assert torch.equal(nxt, seq[:, 11 + step: 12 + step]), step
        cur = torch.cat([cur, nxt], dim=-1)
    # and the logits of a cached step agree with the recomputation
    cache = DynamicCache(ec(), device="cpu")
    model(input_ids=seq[:, :14], past_key_values=cache)
    a = model(input_ids=seq[:, 14:15], past_key_values=cache).logits[:, -1]
    b = model(input_ids=seq[:, :15], past_key_values=DynamicCache(ec(), device="cpu")).logits[:, -1]
    assert cache.get_seq_length() == 15
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)


def test_fused_projection_weights_keep_modules_and_state_dict():
    """After ``fuse_projections`` the five projection modules are views of two wider tensors: same values, the
    module chain computes the same logits, and a state dict loaded afterwards lands in the fused tensors."""
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import random_init
    cfg = _tiny()
    model = random_init(cfg, dtype=torch.float32, device="cpu", seed=3, std=0.3)
    other = random_init(cfg, dtype=torch.float32, device="cpu", seed=4, std=0.3)
    masks = _masks(cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.head_dim, [8, 8], [8, 8])
    ec = lambda: _cfg(masks, numinittokens=2, maxlocallen=64, maxmidstates=8, num_key_value_heads=cfg.num_key_value_heads,
                      max_new_tokens=16, max_position_embeddings=256)
    ids = torch.randint(0, cfg.vocab_size, (2, 9), generator=torch.Generator().manual_seed(0))
    want = model(input_ids=ids, past_key_values=DynamicCache(ec(), device="cpu")).logits
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    model.model.fuse_projections()
    assert all(torch.equal(v, sd[k]) for k, v in model.state_dict().items())
    assert torch.equal(model(input_ids=ids, past_key_values=DynamicCache(ec(), device="cpu")).logits, want)
    layer = model.model.layers[1]
    at, mlp = layer.self_attn, layer.mlp
    assert torch.equal(layer._qkv_weight, torch.cat([at.q_proj.weight, at.k_proj.weight, at.v_proj.weight]))
    assert torch.equal(layer._gate_up_weight, torch.cat([mlp.gate_proj.weight, mlp.up_proj.weight]))
    model.load_state_dict(other.state_dict())
    assert torch.equal(layer._qkv_weight[-at.v_proj.weight.shape[0]:], other.model.layers[1].self_attn.v_proj.weight)
    assert torch.equal(layer._gate_up_weight[:mlp.gate_proj.weight.shape[0]], other.model.layers[1].mlp.gate_proj.weight)


def test_packed_copies_are_dropped_when_their_weights_change():
    """A packed copy of a weight group (``pack_projections``) is a second tensor: once one of the parameters it was
    made from is written in place (``load_state_dict``, an update) or replaced, decode steps must go back to the
    modules' own weights instead of multiplying with the stale copy."""
    from fourierattention_amd import ops
    from fourierattention_amd.llama import LlamaDecoderLayer
    w1, w2 = torch.nn.Parameter(torch.randn(8, 4)), torch.nn.Parameter(torch.randn(8, 4))
    stamp = ops.WeightStamp([w1, w2])
    assert not stamp.changed()
    with torch.no_grad():
        w2.mul_(2.0)                                    # in place
    assert stamp.changed()
    stamp = ops.WeightStamp([w1, w2])
    w1.data = w1.data.clone()                           # replaced storage
    assert stamp.changed()

    class Copy:                                         # stands in for a packed weight (which needs the GPU)
        def __init__(self, sources):
            self.stamp = ops.WeightStamp(sources)

        def stale(self):
            return self.stamp.changed()

        def covers(self, x):
            return True

    layer = LlamaDecoderLayer(_tiny(), 0)
    layer._packed["o"] = Copy([layer.self_attn.o_proj.weight])
    assert layer._packed_weight("o") is layer._packed["o"]
    layer.load_state_dict(layer.state_dict())           # copies in place: every version moves on
    assert layer._packed_weight("o") is None and "o" not in layer._packed
    x = torch.randn(2, layer.self_attn.o_proj.weight.shape[1])
    assert torch.equal(layer._linear("o", x, layer.self_attn.o_proj), layer.self_attn.o_proj(x))


def test_model_requires_a_cache():
    from fourierattention_amd.llama import random_init
    model = random_init(_tiny(layers=1), dtype=torch.float32, device="cpu")
    with pytest.raises(ValueError):
        model(input_ids=torch.zeros((1, 3), dtype=torch.long), past_key_values=None)


def test_eos_stops_the_loop():
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import greedy_generate, random_init
    cfg = _tiny(layers=1)
    model = random_init(cfg, dtype=torch.float32, device="cpu", seed=1, std=0.3)
    masks = _masks(1, cfg.num_key_value_heads, cfg.head_dim, [8, 8], [8, 8])
    ec = lambda: _cfg(masks, numinittokens=2, maxlocallen=64, maxmidstates=8, num_key_value_heads=cfg.num_key_value_heads,
                      max_new_tokens=16, max_position_embeddings=256)
    prompt = torch.tensor([[5, 6, 7, 8]])
    free = greedy_generate(model, prompt, DynamicCache(ec(), device="cpu"), max_new_tokens=5)
    stop = greedy_generate(model, prompt, DynamicCache(ec(), device="cpu"), max_new_tokens=5, eos_token_id=int(free[0, 5]))
    assert stop.shape[1] == 6 and torch.equal(stop, free[:, :6])


def _oracle_forward(model, cfg, cache, ids, pos0, gpu_cache):
    """The model's forward on the CPU in float64 with the oracle cache and the oracle attention."""
    from oracle import fourier_oracle as fo
    f64 = lambda t: t.detach().double().cpu().numpy()
    x = f64(model.model.embed_tokens.weight)[ids.cpu().numpy()]                 # (B, q, hidden)
    B, q_len, _ = x.shape
    Hq, Hkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    cos, sin = fo.rope_tables(np.arange(pos0, pos0 + q_len), D, cfg.rope_theta)
    rms = lambda v, w: v / np.sqrt((v * v).mean(-1, keepdims=True) + cfg.rms_norm_eps) * f64(w)
    for li, layer in enumerate(model.model.layers):
        at = layer.self_attn
        h = rms(x, layer.input_layernorm.weight)
        proj = lambda lin, n: (h @ f64(lin.weight).T).reshape(B, q_len, n, D).transpose(0, 2, 1, 3)
        qh, kh, vh = proj(at.q_proj, Hq), proj(at.k_proj, Hkv), proj(at.v_proj, Hkv)
        qh, kh = fo.apply_rope(qh, cos, sin), fo.apply_rope(kh, cos, sin)
        kw, vw = cache.update(kh, vh, li)
        if kw["k_init"] is None and kw["k_compressed"] is None and kw["k_uncompressed"] is None:
            S = kw["k_local"].shape[1]
            k = kw["k_local"].reshape(B, S, Hkv, D).transpose(0, 2, 1, 3).repeat(Hq // Hkv, axis=1)
            v = vw["v_local"].reshape(B, S, Hkv, D).transpose(0, 2, 1, 3).repeat(Hq // Hkv, axis=1)
            # the reference computes the prompt attention on half-precision copies whatever the model's type and
            # casts the result back (flash_attn_func(q.half(), k.half(), v.half()), modeling_llama_fourier.py:633);
            # the cache above was given the unrounded keys and values, as there
            half = lambda a: a.astype(np.float16).astype(np.float64)
            qa, k, v = half(qh), half(k), half(v)
            s = np.einsum("bhqd,bhkd->bhqk", qa, k) / np.sqrt(D)
            s = np.where(np.arange(S)[None, :] <= np.arange(q_len)[:, None] + (S - q_len), s, -np.inf)
            p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
            o = half(np.einsum("bhqk,bhkd->bhqd", p, v))
        else:
            for n in ("k_scale", "k_layer_average", "kd_layer_average", "v_scale", "v_layer_average", "vd_layer_average"):
                getattr(cache, n)[li] = getattr(gpu_cache, n)[li].float().cpu().numpy()   # isolate the attention from the stats
            o = cache.attend(qh, kw, vw, li, Hq, Hkv)
        o = o.transpose(0, 2, 1, 3).reshape(B, q_len, Hq * D)
        x = x + o @ f64(at.o_proj.weight).T
        h2 = rms(x, layer.post_attention_layernorm.weight)
        gate = h2 @ f64(layer.mlp.gate_proj.weight).T
        x = x + ((gate / (1 + np.exp(-gate))) * (h2 @ f64(layer.mlp.up_proj.weight).T)) @ f64(layer.mlp.down_proj.weight).T
    return rms(x, model.model.norm.weight)[:, -1] @ f64(model.lm_head.weight).T


@pytest.mark.gpu
def test_compressed_decode_steps_match_the_oracle_model():
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import LlamaConfig, random_init
    from oracle.cache_oracle import OracleCache
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=64, vocab_size=211)
    model = random_init(cfg, dtype=torch.float32, device="cuda:0", seed=5, std=0.15)
    masks = _masks(2, 2, 64, [32, 20], [32, 40], seed=2)
    ec = _cfg(masks, numinittokens=4, maxlocallen=32, maxmidstates=64, num_key_value_heads=2, max_new_tokens=8,
              max_position_embeddings=1024)
    gpu, cpu = DynamicCache(ec), OracleCache(ec, masks=masks, model_dtype="fp32")
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, cfg.vocab_size, (2, 300), generator=g)
    with torch.no_grad():
        got = model(input_ids=ids.cuda(), past_key_values=gpu, num_logits_to_keep=1).logits[:, -1].cpu().numpy()
        want = _oracle_forward(model, cfg, cpu, ids, 0, gpu)
        np.testing.assert_allclose(got, want, rtol=3e-3, atol=3e-3)     # prompt pass: exact attention in half on both sides
        nxt = torch.from_numpy(want.argmax(-1))[:, None]
        for step in range(4):
            assert gpu.get_seq_length() == 300 + step == cpu.get_seq_length()
            got = model(input_ids=nxt.cuda(), past_key_values=gpu, num_logits_to_keep=1).logits[:, -1].cpu().numpy()
            want = _oracle_forward(model, cfg, cpu, nxt, 300 + step, gpu)
            # fp32 storage: the kernels' fp32 arithmetic against float64; logits are O(1)
            np.testing.assert_allclose(got, want, rtol=5e-3, atol=5e-3)
            nxt = torch.from_numpy(want.argmax(-1))[:, None]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fused_elementwise_kernels_match_the_tensor_op_chains(dtype):
    """fa_add_rmsnorm / fa_rope_qk / fa_silu_mul against the chains of tensor ops they replace
    (LlamaRMSNorm.forward after the residual add, apply_rotary_pos_emb, silu(gate) * up)."""
    from fourierattention_amd import ops
    from fourierattention_amd.attention import apply_rotary_pos_emb
    from fourierattention_amd.llama import LlamaRMSNorm
    g = torch.Generator(device="cuda").manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device="cuda", dtype=torch.float32)
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2e-6}[dtype]
    # residual add + RMSNorm (hidden not a multiple of the block size on purpose)
    for rows, hidden in ((5, 4096), (3, 1000), (2, 1001)):   # the last one takes the element-wise variant
        h, d = (rn(rows, 1, hidden) * 2).to(dtype), rn(rows, 1, hidden).to(dtype)
        norm = LlamaRMSNorm(hidden, 1e-5).cuda().to(dtype)
        norm.weight.data = (1 + 0.1 * rn(hidden)).to(dtype)
        want_h = h + d
        want_y = norm(want_h)
        h2 = h.clone()
        y = ops.add_rmsnorm(h2, d, norm.weight, 1e-5)
        assert torch.equal(h2, want_h)                                    # the add rounds exactly like the tensor add
        torch.testing.assert_close(y.float(), want_y.float(), rtol=ulp, atol=ulp)   # reduction order: last place only
        y0 = ops.add_rmsnorm(h2, None, norm.weight, 1e-5)                 # no delta: h untouched
        assert torch.equal(h2, want_h) and torch.equal(y0, y)
    # rotary embedding: no reduction anywhere, so bit for bit (head dims of 64 and at least 64 rows: 16 bytes per
    # thread with 16-bit storage; otherwise the element-wise variant)
    # 120 rows; a few rows (one block per head); odd head dim; one row (one token of one sequence: the slice of a
    # wider row is then "contiguous" and still reports the wider row's stride)
    for D, q_len, B in ((64, 40, 3), (64, 2, 3), (40, 2, 3), (64, 1, 1)):
        Hq, Hkv = 6, 2
        q, k = rn(B, q_len, Hq * D).to(dtype), rn(B, q_len, Hkv * D).to(dtype)
        ang = rn(B, q_len, D) * 3
        cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)
        wq, wk = apply_rotary_pos_emb(q.view(B, q_len, Hq, D).transpose(1, 2), k.view(B, q_len, Hkv, D).transpose(1, 2), cos, sin)
        q2, k2 = q.clone(), k.clone()
        ops.rope_qk_(q2, k2, cos, sin, D)
        assert torch.equal(q2.view(B, q_len, Hq, D).transpose(1, 2), wq) and torch.equal(k2.view(B, q_len, Hkv, D).transpose(1, 2), wk)
        # the same on column slices of one fused projection output: q comes back densely packed, k is rotated where it lies
        qkv = torch.cat([q, k, rn(B, q_len, Hkv * D).to(dtype)], dim=-1)
        qs, ks, vs = qkv.split((Hq * D, Hkv * D, Hkv * D), dim=-1)
        v_before = vs.clone()
        q3 = ops.rope_qk(qs, ks, cos, sin, D)
        assert q3.is_contiguous() and torch.equal(q3, q2) and torch.equal(ks, k2) and torch.equal(vs, v_before)
    # SwiGLU gate: the exponential may differ in the last place (1111 columns: element-wise; 2048: 16 bytes per thread)
    for cols in (1111, 2048):
        gate, up = (rn(7, 1, cols) * 3).to(dtype), rn(7, 1, cols).to(dtype)
        want = torch.nn.functional.silu(gate) * up
        got = ops.silu_mul(gate, up)
        torch.testing.assert_close(got.float(), want.float(), rtol=2 * ulp, atol=2 * ulp)
        g2, u2 = torch.cat([gate, up], dim=-1).chunk(2, dim=-1)              # column slices of one wider row
        got2 = ops.silu_mul(g2, u2)
        assert got2.is_contiguous() and torch.equal(got2, got)


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [2, 1])
def test_fused_decoder_path_matches_the_module_chain(batch):
    """The same bf16 model stepped with and without the fused elementwise launches. With one sequence the q slice of
    a step's fused q/k/v row is a single row whose view still reports the stride of the wider row."""
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import LlamaConfig, random_init
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=64, vocab_size=301)
    model = random_init(cfg, dtype=torch.bfloat16, device="cuda:0", seed=7, std=0.05)
    masks = _masks(3, 2, 64, [32, 32], [32, 32], seed=4)
    ec = lambda: _cfg(masks, numinittokens=4, maxlocallen=32, maxmidstates=64, num_key_value_heads=2, max_new_tokens=8,
                      max_position_embeddings=1024)
    ids = torch.randint(0, cfg.vocab_size, (batch, 200), generator=torch.Generator().manual_seed(3)).cuda()
    outs = []
    with torch.no_grad():
        for fused in (True, False, "projections"):
            model.model.fused_elementwise = bool(fused)
            if fused == "projections":       # q/k/v and gate/up as one GEMM each; the modules keep views of the weights
                before = {n: p.detach().clone() for n, p in model.named_parameters()}
                model.model.fuse_projections()
                assert all(torch.equal(p, before[n]) for n, p in model.named_parameters())
                at = model.model.layers[0].self_attn
                assert at.k_proj.weight.data_ptr() == at.q_proj.weight.data_ptr() + at.q_proj.weight.numel() * 2
            cache = DynamicCache(ec())
            logits = [model(input_ids=ids, past_key_values=cache, num_logits_to_keep=1).logits[:, -1]]
            tok = logits[0].argmax(-1, keepdim=True)
            for _ in range(3):
                logits.append(model(input_ids=tok, past_key_values=cache, num_logits_to_keep=1).logits[:, -1])
                tok = logits[-1].argmax(-1, keepdim=True)
            outs.append(torch.stack(logits))
    # identical rounding points; only reduction order (norm) and the exponential differ in the last place of bf16
    # (logits of magnitude 0.5 - 1.5: one place of bf16 there is 0.004 - 0.008; the mean difference stays below one)
    torch.testing.assert_close(outs[0], outs[1], rtol=3e-2, atol=3e-2)
    assert (outs[0] - outs[1]).abs().mean().item() < 5e-3
    # a wider GEMM may pick another tiling, hence another summation order inside the dot products
    torch.testing.assert_close(outs[2], outs[0], rtol=3e-2, atol=3e-2)
    assert (outs[2] - outs[0]).abs().mean().item() < 5e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_packed_linear_matches_the_library_product(dtype):
    """``fa_linear_packed`` (projections of a decode step on weights re-laid for the matrix cores) against the fp32
    product of the same 16-bit operands: fp32 accumulation either way, so what is left is the rounding of the result
    (half a unit in the last place of the storage type) plus the order of the sums."""
    from fourierattention_amd import ops
    g = torch.Generator(device="cuda").manual_seed(5)
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    for rows, K, n_out in ((16, 4096, 6144), (4, 3072, 5120), (1, 1024, 16), (7, 14336, 4096), (16, 2048, 28672)):
        w = (torch.randn(n_out, K, generator=g, device="cuda") * 0.05).to(dtype)
        x = torch.randn(rows, 1, K, generator=g, device="cuda").to(dtype)
        pw = ops.PackedLinearWeight(w)
        assert pw.covers(x)
        got = ops.linear_packed(x, pw)
        want = torch.nn.functional.linear(x.float(), w.float())
        assert got.shape == (rows, 1, n_out) and got.dtype == dtype
        bound = 0.75 * ulp * want.abs().max().item() + 1e-6
        assert (got.float() - want).abs().max().item() <= bound
        # rows that are slices of wider rows (a fused projection output, as the decoder hands them over)
        wide = torch.cat([x, torch.randn(rows, 1, 64, generator=g, device="cuda").to(dtype)], dim=-1)
        assert torch.equal(ops.linear_packed(wide[..., :K], pw), got)
    # shapes outside the kernel are for the GEMM library
    assert not pw.covers(torch.zeros(17, 2048, dtype=dtype, device="cuda"))
    assert not ops.PackedLinearWeight(torch.zeros(16, 1536, dtype=dtype, device="cuda")).covers(torch.zeros(1, 1536, dtype=dtype, device="cuda"))


@pytest.mark.gpu
def test_decoder_steps_on_packed_projections():
    """The same bf16 model stepped with the projections of its decode steps on the packed weights and through the
    GEMM library (the prompt goes through the library either way)."""
    from fourierattention_amd import DynamicCache
    from fourierattention_amd.llama import LlamaConfig, random_init
    cfg = LlamaConfig(hidden_size=1024, intermediate_size=2048, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=128, vocab_size=301)
    model = random_init(cfg, dtype=torch.bfloat16, device="cuda:0", seed=7, std=0.03)
    model.model.fuse_projections()
    masks = _masks(2, 2, 128, [64, 64], [64, 64], seed=4)
    ec = lambda: _cfg(masks, numinittokens=4, maxlocallen=32, maxmidstates=64, num_key_value_heads=2, max_new_tokens=8,
                      max_position_embeddings=1024)
    ids = torch.randint(0, cfg.vocab_size, (3, 200), generator=torch.Generator().manual_seed(3)).cuda()
    outs = []
    with torch.no_grad():
        for packed in (False, True):
            if packed:
                model.model.pack_projections()
                assert set(model.model.layers[0]._packed) == {"qkv", "o", "gate_up", "down"}
            cache = DynamicCache(ec())
            logits = [model(input_ids=ids, past_key_values=cache, num_logits_to_keep=1).logits[:, -1]]
            tok = logits[0].argmax(-1, keepdim=True)
            for _ in range(3):
                logits.append(model(input_ids=tok, past_key_values=cache, num_logits_to_keep=1).logits[:, -1])
                tok = logits[-1].argmax(-1, keepdim=True)
            outs.append(torch.stack(logits))
    assert torch.equal(outs[0][0], outs[1][0])                     # the prompt pass does not touch the packed weights
    torch.testing.assert_close(outs[1], outs[0], rtol=3e-2, atol=3e-2)   # another summation order inside the dot products
    assert (outs[1] - outs[0]).abs().mean().item() < 3e-3
