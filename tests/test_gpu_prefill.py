"""Exact causal attention of the prompt pass (``fa_prefill_attn``, the ``flash_attn_func(q, k, v, causal=True)`` of
modeling_llama_fourier.py:633) against the CPU restatement's textbook attention with a causal mask.

Small shapes compare every query row; at 4096 and 32768 tokens the oracle is run on a sample of rows (each row of
the result depends on its own query only, so a sample of rows checks the kernel at those rows exactly) that covers
the first rows, tile edges, rows in the middle and the last row.  Bound: 2e-2 max-abs for 16-bit storage (stated),
and what fp32 accumulation with 16-bit probabilities really leaves."""
import numpy as np
import pytest
import torch

from oracle import fourier_oracle as fo
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _oracle_rows(q, k, v, rows, Hq, Hkv, offset):
    """``q (B, Hq, q_len, D)``, ``k, v (B, S, Hkv*D)`` float64 -> ``(B, len(rows), Hq, D)``: row i sees keys 0 .. i + offset."""
    B, _, _, D = q.shape
    out = np.empty((B, len(rows), Hq, D))
    for n, i in enumerate(rows):
        qi = np.transpose(q[:, :, i, :], (0, 1, 2)).reshape(B, Hq * D)
        out[:, n] = fo.softmax_attention(qi, k[:, : i + offset + 1], v[:, : i + offset + 1], Hq, Hkv)
    return out


def _tight(want, dtype):
    """What the arithmetic really leaves: the result is rounded to the storage type (half a unit in the last place of
    the largest value) on top of f16 probabilities accumulated in fp32 - f16 for both storage types, as the reference
    computes this attention in half precision whatever the model's type (modeling_llama_fourier.py:633)."""
    top = float(np.abs(want).max())
    ulp = 2.0 ** (np.floor(np.log2(top)) - (7 if dtype == torch.bfloat16 else 10))   # of the largest value's binade
    return 0.5 * ulp + 1e-3


def _case(seed, B, Hq, Hkv, D, S, q_len, dtype, rope=True):
    r = np.random.default_rng(seed)
    q = r.standard_normal((B, Hq, q_len, D))
    k = r.standard_normal((B, Hkv, S, D))
    v = r.standard_normal((B, Hkv, S, D))
    if rope:
        cos, sin = fo.rope_tables(np.arange(S), D)
        k = fo.apply_rope(k, cos, sin)
        q = fo.apply_rope(q, cos[S - q_len:], sin[S - q_len:])
    q, k, v = (H.to_dtype_np(a, dtype) for a in (q, k, v))
    k_tm = np.transpose(k, (0, 2, 1, 3)).reshape(B, S, Hkv * D)
    v_tm = np.transpose(v, (0, 2, 1, 3)).reshape(B, S, Hkv * D)
    return q, k_tm, v_tm


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,D,S,q_len", [
    (2, 8, 2, 128, 200, 200),     # four query heads per KV head, ragged last tile
    (1, 6, 2, 128, 97, 97),       # three query heads per KV head (a workgroup of three waves)
    (2, 4, 4, 64, 130, 130),      # one query head per KV head, heads of 64 dims
    (1, 16, 2, 64, 75, 75),       # eight query heads per KV head
    (2, 4, 2, 128, 150, 37),      # fewer query rows than keys: the mask is aligned to the last key
    (1, 8, 2, 128, 33, 1),        # a single query row
])
def test_every_row_of_small_shapes(dtype, B, Hq, Hkv, D, S, q_len):
    from fourierattention_amd import ops
    q, k, v = _case(1, B, Hq, Hkv, D, S, q_len, dtype)
    want = _oracle_rows(q, k, v, range(q_len), Hq, Hkv, S - q_len)
    # the query as the attention forward holds it: a transposed view of the projection output
    qg = H.to_gpu(np.transpose(q, (0, 2, 1, 3)), dtype).transpose(1, 2)
    assert not qg.is_contiguous() or Hq == 1 or q_len == 1
    got = ops.prefill_attention(qg, H.to_gpu(k, dtype), H.to_gpu(v, dtype), Hkv)
    assert tuple(got.shape) == (B, q_len, Hq, D) and got.dtype == dtype
    err = np.abs(got.float().cpu().numpy() - want).max()
    assert err <= 2e-2 and err <= _tight(want, dtype), err


@pytest.mark.parametrize("S,B,Hq,Hkv", [(4096, 2, 32, 8), (32768, 1, 32, 8)])
def test_long_prompts_on_sampled_rows(S, B, Hq, Hkv):
    """Llama-3.1-8B head geometry, bf16, rotary embedding on q and k, 4096 and 32768 tokens."""
    from fourierattention_amd import ops
    dtype, D = torch.bfloat16, 128
    q, k, v = _case(2, B, Hq, Hkv, D, S, S, dtype)
    rows = sorted(set([0, 1, 15, 16, 31, 32, 33, 63, 64, 1000, S // 2 - 1, S // 2, S - 130, S - 33, S - 32, S - 2, S - 1]))
    want = _oracle_rows(q, k, v, rows, Hq, Hkv, 0)
    got = ops.prefill_attention(H.to_gpu(q, dtype), H.to_gpu(k, dtype), H.to_gpu(v, dtype), Hkv)
    assert torch.isfinite(got.float()).all()
    err = np.abs(got[:, rows].float().cpu().numpy() - want).max()
    assert err <= 2e-2 and err <= _tight(want, dtype), err


def test_attention_forward_takes_the_kernel_for_the_prompt():
    """``fourier_attention`` on a prompt (every layer returns ``*_local`` only): same result as the operator, for a
    prompt that is compressed afterwards and for one that stays in the window."""
    from fourierattention_amd import DynamicCache, fourier_attention, ops
    from tests.test_gpu_cache import _cfg, _masks
    dtype, B, Hq, Hkv, D = torch.bfloat16, 2, 8, 2, 128
    masks = _masks(1, Hkv, D, [64, 64], [64, 64])
    for S in (30, 300):
        q, k, v = _case(3, B, Hq, Hkv, D, S, S, dtype)
        cache = DynamicCache(_cfg(masks, num_key_value_heads=Hkv))
        qg = H.to_gpu(q, dtype)
        kg = H.to_gpu(k, dtype).view(B, S, Hkv, D).transpose(1, 2)
        vg = H.to_gpu(v, dtype).view(B, S, Hkv, D).transpose(1, 2)
        out = fourier_attention(qg, kg, vg, cache, 0, Hq, Hkv)
        assert tuple(out.shape) == (B, S, Hq * D) and out.dtype == dtype
        direct = ops.prefill_attention(qg, H.to_gpu(k, dtype), H.to_gpu(v, dtype), Hkv).reshape(B, S, Hq * D)
        assert torch.equal(out, direct)
        want = _oracle_rows(q, k, v, [0, S - 1], Hq, Hkv, 0).reshape(B, 2, Hq * D)
        assert np.abs(out[:, [0, S - 1]].float().cpu().numpy() - want).max() <= _tight(want, dtype)


def test_float32_prompt_is_computed_in_half_like_the_reference():
    """A float32 model: the reference casts q, k and v to half for the prompt attention whatever the model's type
    (modeling_llama_fourier.py:633) and casts the result back.  Same here, on the matrix-core kernel."""
    from fourierattention_amd import DynamicCache, fourier_attention, ops
    from tests.test_gpu_cache import _cfg, _masks
    B, Hq, Hkv, D, S = 1, 8, 2, 128, 200
    masks = _masks(1, Hkv, D, [64, 64], [64, 64])
    q, k, v = _case(5, B, Hq, Hkv, D, S, S, torch.float32)
    cache = DynamicCache(_cfg(masks, num_key_value_heads=Hkv))
    qg = H.to_gpu(q, torch.float32)
    kg = H.to_gpu(k, torch.float32).view(B, S, Hkv, D).transpose(1, 2)
    vg = H.to_gpu(v, torch.float32).view(B, S, Hkv, D).transpose(1, 2)
    out = fourier_attention(qg, kg, vg, cache, 0, Hq, Hkv)
    assert tuple(out.shape) == (B, S, Hq * D) and out.dtype == torch.float32
    direct = ops.prefill_attention(qg.half(), H.to_gpu(k, torch.float32).half(), H.to_gpu(v, torch.float32).half(), Hkv)
    assert torch.equal(out, direct.reshape(B, S, Hq * D).float())
    want = _oracle_rows(q, k, v, [0, S // 2, S - 1], Hq, Hkv, 0).reshape(B, 3, Hq * D)
    assert np.abs(out[:, [0, S // 2, S - 1]].cpu().numpy() - want).max() <= 4e-3      # inputs rounded to half


def test_argument_errors():
    from fourierattention_amd import _lib, ops
    q = torch.zeros((1, 4, 8, 128), dtype=torch.float32, device="cuda")
    k = torch.zeros((1, 8, 2 * 128), dtype=torch.float32, device="cuda")
    with pytest.raises(AssertionError):
        ops.prefill_attention(q, k, k, 2)                    # float32 storage has no matrix-core path
    lib = _lib.load()
    assert lib.fa_prefill_attn(None, 0, 0, 0, None, None, 0, 0, None, 0, 1, 4, 2, 128, 8, 8, -1.0, None, 0, None) == -1
    qh, kh = q.to(torch.bfloat16), k.to(torch.bfloat16)
    out = torch.empty((1, 8, 4, 128), dtype=torch.bfloat16, device="cuda")
    args = (qh.data_ptr(), qh.stride(0), qh.stride(1), qh.stride(2), kh.data_ptr(), kh.data_ptr(), kh.stride(0), kh.stride(1),
            out.data_ptr(), 0, 1, 4, 2, 128, 8)
    assert lib.fa_prefill_attn(*args, 9, -1.0, None, 0, None) == -2                      # more query rows than keys
    assert lib.fa_prefill_attn(*args, 8, -1.0, None, 0, None) == -4                      # no workspace
    assert lib.fa_prefill_attn_workspace_bytes(1, 2, 128, 8) == 2 * 32 * 128 * 2
