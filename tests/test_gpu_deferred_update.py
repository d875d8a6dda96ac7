"""Streaming steps whose rank-1 coefficient update is left to the decode attention that follows (``fa_stream_update``
with ``skip_coef``, then ``fa_decode_attn`` with ``upd_*``): the query preparation adds the evicted row's term to the K
coefficients it streams and the merge inside the mid-row launch to the V coefficients, where those kernels run; other
shapes give the update a launch of its own.  Held against the same cache with the update applied at once
(cache_utils_fourier.py:731-748 as written), step by step: same coefficients, same attention output."""
import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.test_gpu_cache import _cfg, _masks

pytestmark = pytest.mark.gpu

U = [64] * 8
CASES = [
    # dtype, B, Hq, Hkv, D, I, W, M, prompt, kcounts, vcounts (stored dims per KV head)
    (torch.bfloat16, 4, 32, 8, 128, 4, 64, 1024, 3000, U, U),                    # merge inside the mid-row launch
    (torch.bfloat16, 1, 32, 8, 128, 4, 60, 1024, 5000, [0, 128, 64, 3, 125, 127, 64, 96], [128, 0, 61, 64, 2, 64, 127, 1]),
    (torch.float16, 8, 16, 8, 128, 4, 40, 512, 1500, [64, 0, 128, 30, 64, 64, 100, 64], [1, 64, 2, 3, 128, 64, 0, 64]),
    (torch.bfloat16, 3, 8, 2, 128, 4, 32, 256, 700, [64, 40], [64, 96]),         # matrix cores, merge as a launch of its own
    (torch.bfloat16, 2, 16, 4, 128, 4, 32, 2048, 4500, [64] * 4, [30, 64, 0, 100]),   # 1024 frequencies, two passes
    (torch.bfloat16, 4, 24, 8, 128, 4, 40, 2048, 6000, U, U),                    # ... whose value pass merges (V: own launch)
    (torch.float32, 2, 8, 2, 64, 4, 16, 256, 420, [10, 30], [3, 64]),            # fp32 storage: the any-shape kernels
]


def _pair(case):
    from fourierattention_amd import DynamicCache
    dtype, B, Hq, Hkv, D, I, W, M, prompt, kcnt, vcnt = CASES[case]
    masks = _masks(1, Hkv, D, kcnt, vcnt, seed=case)
    cfg = _cfg(masks, numinittokens=I, maxlocallen=W, maxmidstates=M, num_key_value_heads=Hkv, max_new_tokens=32)
    a, b = DynamicCache(cfg), DynamicCache(cfg)
    a.defer_coef_update, b.defer_coef_update = True, False
    r = np.random.default_rng(300 + case)
    k0 = H.to_gpu(H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)), dtype), dtype)
    v0 = H.to_gpu(H.to_dtype_np(r.standard_normal((B, Hkv, prompt, D)) + 0.1, dtype), dtype)
    for c in (a, b):
        c.update(k0, v0, 0)
    return a, b, r, (dtype, B, Hq, Hkv, D)


def _token(r, dtype, B, Hq, Hkv, D):
    kn = H.to_gpu(H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype), dtype)
    vn = H.to_gpu(H.to_dtype_np(r.standard_normal((B, Hkv, 1, D)), dtype), dtype)
    q = H.to_gpu(H.to_dtype_np(r.standard_normal((B, Hq, 1, D)) * 1.5, dtype), dtype)
    return kn, vn, q


def _close(x, y, what):
    x, y = x.float().cpu().numpy(), y.float().cpu().numpy()
    scale = max(1.0, float(np.abs(y).max()))
    assert np.abs(x - y).max() <= 2e-6 * scale, (what, float(np.abs(x - y).max()), scale)


@pytest.mark.parametrize("case", range(len(CASES)))
def test_update_inside_the_attention_equals_update_at_once(case):
    a, b, r, shape = _pair(case)
    dtype, B, Hq, Hkv, D = shape
    for step in range(5):
        kn, vn, q = _token(r, *shape)
        print(f"case {case} step {step}", flush=True)
        pa, pb = a.update(kn, vn, 0), b.update(kn, vn, 0)
        assert a._layers[0].owed is not None and b._layers[0].owed is None
        oa = a.decode_attention(q, 0, Hq, Hkv)
        ob = b.decode_attention(q, 0, Hq, Hkv)
        assert a._layers[0].owed is None                      # applied by the call, exactly once
        assert torch.isfinite(oa).all()
        # the attention has seen the updated coefficients (the two calls may cut the work the same way or not:
        # both are the same launches on the same numbers up to the rounding of the update itself)
        assert float((oa - ob).abs().max()) <= 1e-4, float((oa - ob).abs().max())
        for tag, p_a, p_b in (("k", pa[0], pb[0]), ("v", pa[1], pb[1])):
            _close(p_a[f"{tag}_compressed"], p_b[f"{tag}_compressed"], (tag, step))
        # a second attention over the same state leaves the coefficients alone
        oa2 = a.decode_attention(q, 0, Hq, Hkv)
        assert torch.equal(oa2, a.decode_attention(q, 0, Hq, Hkv))
        _close(pa[0]["k_compressed"], pb[0]["k_compressed"], ("k again", step))
        _close(pa[1]["v_compressed"], pb[1]["v_compressed"], ("v again", step))


def test_owed_update_is_settled_when_nobody_attends():
    """Two updates in a row, and a read of the coefficients right after an update: the owed term goes in through a
    launch of its own before the window slot of the evicted row is written again."""
    a, b, r, shape = _pair(0)
    dtype, B, Hq, Hkv, D = shape
    for step in range(3):
        kn, vn, q = _token(r, *shape)
        pa, pb = a.update(kn, vn, 0), b.update(kn, vn, 0)
    assert a._layers[0].owed is not None
    _close(pa[0]["k_compressed"], pb[0]["k_compressed"], "k")      # the read settles it
    assert a._layers[0].owed is None
    _close(pa[1]["v_compressed"], pb[1]["v_compressed"], "v")
    oa, ob = a.decode_attention(q, 0, Hq, Hkv), b.decode_attention(q, 0, Hq, Hkv)
    assert float((oa - ob).abs().max()) <= 1e-4


def test_pending_update_through_the_c_abi_is_validated():
    from fourierattention_amd import _lib
    import ctypes
    a = _lib.DecodeArgs()
    a.q_len, a.B, a.Hq, a.Hkv, a.D = 1, 1, 4, 2, 128
    a.il_rows[0] = 8
    q = torch.zeros(1, 1, 512, dtype=torch.bfloat16, device="cuda")
    kv = torch.zeros(1, 8, 256, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(1, 4, 1, 128, device="cuda")
    a.q, a.out, a.dtype = q.data_ptr(), out.data_ptr(), _lib.FA_BF16
    a.k_il[0], a.v_il[0], a.il_batch_stride[0], a.il_row_stride[0] = kv.data_ptr(), kv.data_ptr(), 8 * 256, 256
    a.upd_k_row, a.upd_T, a.N = kv.data_ptr(), 0, 128                # a pending update without a period
    assert _lib.load().fa_decode_attn(ctypes.byref(a), None) == -2     # FA_ERR_BAD_SHAPE
    a.upd_T, a.Ck = 100, 64                                          # ... without coefficients to apply it to
    assert _lib.load().fa_decode_attn(ctypes.byref(a), None) == -1     # FA_ERR_NULL_POINTER
